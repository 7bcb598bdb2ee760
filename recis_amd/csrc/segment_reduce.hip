// Ragged gather + segment reduce (pooling) forward and backward for gfx950.
//
// Design (differs from the reference's one-atomic-per-element kernels,
// csrc/ops/embedding_segment_reduce_kernel.cu:23-120):
//   * a power-of-two "team" of lanes owns one segment; the team is split into
//     row groups of LPR lanes, each lane moving one 16-byte vector of a row, so
//     a 64-lane wave streams TEAM/LPR rows per step with fully coalesced
//     16-byte accesses
//   * partial sums stay in registers (fp32) and the row groups are combined
//     with wave shuffles; each output row is written exactly once, with no
//     atomics and no pre-zeroed output
//   * segment offsets of the segments a workgroup owns are staged in LDS once
//   * the backward pass walks segments the same way: the pooled gradient row is
//     read once per segment and fanned out to its occurrences, by plain stores
//     when the caller guarantees distinct rows, by fp32 atomics otherwise
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.cuh"

namespace recis_hip {
namespace {

__device__ __forceinline__ float load_weight(const void* w, int wdt, int64_t i) {
  if (wdt == RECIS_F32) return static_cast<const float*>(w)[i];
  if (wdt == RECIS_BF16) return to_float(static_cast<const bf16_t*>(w)[i]);
  return to_float(static_cast<const f16_t*>(w)[i]);
}

struct SegArgs {
  const void* weight;
  const void* rev;
  const void* offs;
  int64_t B, U, S;
  int D;
  int wdt, rev64, off64;
  int lpr_log2, team_log2;
  int mean;
  int nt_out;  // output larger than the caches can hold: write it with non-temporal stores
  int nt_in;   // likewise for the rows read
  int* err;
  // rows addressed through a table instead of a dense [U, D] array (BLK kernels): row u is row
  // row_index[u] of the block list (blocks of block_rows rows); a negative row_index reads as zeros
  const int64_t* row_index;
  const void* const* blocks;
  int64_t block_rows, n_blocks;
  int64_t pitch;  // elements from one row of a block to the next
};

// Address of unique row idx (idx < U checked by the caller) in the block list, nullptr = zero row.
template <typename TIn>
__device__ __forceinline__ const TIn* block_row(const SegArgs& a, int64_t idx) {
  const int64_t ri = a.row_index[idx];
  if (ri < 0) return nullptr;  // key not in the table (read-only lookup)
  int64_t b = 0, r = ri;
  if (a.n_blocks > 1) {
    b = ri / a.block_rows;
    r = ri - b * a.block_rows;
  }
  if (b >= a.n_blocks || r >= a.block_rows) {
    raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
    return nullptr;
  }
  return static_cast<const TIn*>(a.blocks[b]) + r * a.pitch;
}

// Stage offsets[s0 .. s0 + teams_per_block] into LDS and return this team's
// [start, end). Returns false for teams beyond the last segment.
__device__ __forceinline__ bool team_segment(const SegArgs& a, int64_t* s_off,
                                             int64_t& s, int64_t& start,
                                             int64_t& end) {
  const int tid = threadIdx.x;
  const int teams_per_block = kBlock >> a.team_log2;
  const int64_t s0 = static_cast<int64_t>(blockIdx.x) * teams_per_block;
  for (int i = tid; i <= teams_per_block; i += kBlock) {
    int64_t si = s0 + i;
    if (si <= a.S) s_off[i] = load_index(a.offs, a.off64, si);
  }
  __syncthreads();
  const int team = tid >> a.team_log2;
  s = s0 + team;
  if (s >= a.S) return false;
  start = s_off[team];
  end = s_off[team + 1];
  if (start < 0 || end > a.B || end < start) {
    raise_device_error(a.err, RECIS_DEVERR_OFFSETS);
    start = end = 0;
  }
  return true;
}

// ------------------------------------------------------------------ forward
// KIND selects what a row fetch has to do, so that the common cases keep few registers live
// (the kernel is bound by the number of waves a CU can hold):
//   kFwdGeneric   weights and/or 64-bit reverse indices, all checked at run time
//   kFwdPlain     no reverse indices, no weights: rows of a segment are contiguous in emb
//   kFwdRev32     int32 reverse indices, no weights
enum { kFwdGeneric = 0, kFwdPlain = 1, kFwdRev32 = 2 };

template <typename TIn, typename TOut, int VEC, int KIND, bool BLK>
__global__ void __launch_bounds__(kBlock)
seg_pool_fwd_kernel(const TIn* __restrict__ emb, TOut* __restrict__ out, SegArgs a) {
  __shared__ int64_t s_off[kBlock + 1];
  int64_t s, start, end;
  if (!team_segment(a, s_off, s, start, end)) return;

  const int lane_t = threadIdx.x & ((1 << a.team_log2) - 1);
  const int rg = lane_t >> a.lpr_log2;
  const int cl = lane_t & ((1 << a.lpr_log2) - 1);
  const int step = 1 << (a.team_log2 - a.lpr_log2);
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;
  const float scale = (a.mean && end > start) ? 1.0f / static_cast<float>(end - start) : 1.0f;

  auto fetch = [&](int64_t r, int c0, float (&v)[VEC], float& w) {
    int64_t idx;
    if constexpr (KIND == kFwdPlain) {
      idx = r;
      w = 1.0f;
    } else if constexpr (KIND == kFwdRev32) {
      idx = static_cast<const int32_t*>(a.rev)[r];
      w = 1.0f;
    } else {
      idx = a.rev ? load_index(a.rev, a.rev64, r) : r;
      w = a.weight ? load_weight(a.weight, a.wdt, r) : 1.0f;
    }
    if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
      raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = 0.f;
      w = 0.f;
      return;
    }
    if constexpr (BLK) {
      const TIn* row = block_row<TIn>(a, idx);
      if (row) {
        load_pack<TIn, VEC>(row + c0, v);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 0.f;
      }
    } else {
      load_pack<TIn, VEC>(emb + idx * D + c0, v);
    }
  };
  auto add = [&](float (&acc)[VEC], const float (&v)[VEC], float w) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      if constexpr (KIND == kFwdGeneric) {
        acc[j] = fmaf(v[j], w, acc[j]);
      } else {
        acc[j] = fmaf(v[j], w, acc[j]);  // w is 1 or 0 here; same rounding as the generic path
      }
    }
  };

  for (int c0 = cl * VEC; c0 < D; c0 += col_stride) {
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;

    int64_t r = start + rg;
    for (; r + 3 * step < end; r += 4 * step) {
      float v0[VEC], v1[VEC], v2[VEC], v3[VEC];
      float w0, w1, w2, w3;
      fetch(r, c0, v0, w0);
      fetch(r + step, c0, v1, w1);
      fetch(r + 2 * step, c0, v2, w2);
      fetch(r + 3 * step, c0, v3, w3);
      add(acc, v0, w0);
      add(acc, v1, w1);
      add(acc, v2, w2);
      add(acc, v3, w3);
    }
    for (; r < end; r += step) {
      float v0[VEC];
      float w0;
      fetch(r, c0, v0, w0);
      add(acc, v0, w0);
    }
    // combine the row groups of the team (partners share cl, hence c0)
    for (int off = 1 << a.lpr_log2; off < (1 << a.team_log2); off <<= 1) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += __shfl_xor(acc[j], off, kWave);
    }
    if (rg == 0) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] *= scale;
      store_pack<TOut, VEC>(out + s * D + c0, acc);
    }
  }
}

// Unweighted pooling of segments of several rows, built to keep many bytes in flight per wave: the
// kernel is bound by memory latency x resident waves, so
//   * the two offsets of a segment are read directly (no LDS staging, no barrier)
//   * the reverse indices of up to TEAM rows are read by ONE coalesced load (a lane each) and
//     handed to the lanes that need them with shuffles, instead of one dependent load per row
//   * every lane then has up to eight independent row loads in flight
// Rows are summed per row group in increasing order, like the generic kernel. Requires U < 2^31.
enum { kFastPlain = 0, kFastRev32 = 1, kFastRev64 = 2 };

// A row of zeros, as long as any row these kernels take (D <= 8192 of at most 4 bytes). The fast
// kernels keep several row loads in flight per lane; a lane with no row to read in some round reads
// this one instead, so that the loads of a round stay one straight run of instructions (a branch
// around each makes the compiler wait for every outstanding load before it issues the next).
__device__ __align__(256) const unsigned char g_zero_row[8192 * 4] = {};

template <typename T, int VEC, bool NT>
__device__ __forceinline__ void load_row_pack(const T* p, float (&v)[VEC]) {
  if constexpr (NT) {
    load_pack_stream<T, VEC>(p, v);
  } else {
    load_pack<T, VEC>(p, v);
  }
}

// WG: long segments (behaviour sequences of hundreds of rows): a whole workgroup per segment, each
// of its waves sums a contiguous quarter of the rows and the quarters meet in LDS. With a wave per
// segment the launch lasts as long as its longest segment takes one wave.
template <typename TIn, typename TOut, int VEC, int KIND, bool BLK, bool WG = false>
__global__ void __launch_bounds__(kBlock)
seg_pool_fwd_fast_kernel(const TIn* __restrict__ emb, TOut* __restrict__ out, SegArgs a) {
  extern __shared__ float s_wave_part[];  // WG only: [waves][D]
  const int64_t s = WG ? static_cast<int64_t>(blockIdx.x)
                       : static_cast<int64_t>(blockIdx.x) * (kBlock >> a.team_log2) + (threadIdx.x >> a.team_log2);
  if (s >= a.S) return;  // whole teams leave together
  int64_t start = load_index(a.offs, a.off64, s);
  int64_t end = load_index(a.offs, a.off64, s + 1);
  if (start < 0 || end > a.B || end < start) {
    raise_device_error(a.err, RECIS_DEVERR_OFFSETS);
    start = end = 0;
  }
  const int64_t seg_len = end - start;
  const int wave = threadIdx.x / kWave;
  if constexpr (WG) {  // this wave's share of the rows
    constexpr int n_waves = kBlock / kWave;
    const int64_t share = (seg_len + n_waves - 1) / n_waves;
    start = min(end, start + wave * share);
    end = min(end, start + share);
  }
  const int team = 1 << a.team_log2;
  const int lane = threadIdx.x & (kWave - 1);
  const int lane_t = lane & (team - 1);
  const int team_lane0 = lane - lane_t;
  const int rg = lane_t >> a.lpr_log2;
  const int cl = lane_t & ((1 << a.lpr_log2) - 1);
  const int step = team >> a.lpr_log2;
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;
  const float scale = (a.mean && seg_len > 0) ? 1.0f / static_cast<float>(seg_len) : 1.0f;

  const TIn* zero_row = reinterpret_cast<const TIn*>(g_zero_row);
  const int64_t zero_at = BLK ? 0 : zero_row - emb;
  // rows read once, or too many to stay cached: streaming loads (picked here, outside the loops)
  const bool nt = (KIND == kFastPlain && !BLK) || a.nt_in;
  for (int cbase = 0; cbase < D; cbase += col_stride) {  // uniform: every lane takes part in the shuffles
    const int c0 = cbase + cl * VEC;
    const bool col_ok = c0 < D;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
    auto sum_rows = [&](auto nt_tag) {
      constexpr bool NT = decltype(nt_tag)::value;
      for (int64_t base = start; base < end; base += team) {
        const int n_here = static_cast<int>(min(static_cast<int64_t>(team), end - base));
        int32_t mine = -1;       // row of occurrence base + lane_t in emb ...
        uint64_t mine_addr = 0;  // ... or its address in the block list (BLK), 0 = zero row
        if (lane_t < n_here) {
          int64_t idx;
          if constexpr (KIND == kFastPlain) {
            idx = base + lane_t;
          } else if constexpr (KIND == kFastRev32) {
            idx = static_cast<const int32_t*>(a.rev)[base + lane_t];
          } else {
            idx = static_cast<const int64_t*>(a.rev)[base + lane_t];
          }
          if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
            raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
          } else if constexpr (BLK) {
            mine_addr = reinterpret_cast<uint64_t>(block_row<TIn>(a, idx));
          } else {
            mine = static_cast<int32_t>(idx);
          }
        }
        constexpr int kFly = VEC >= 8 ? 4 : 8;  // row loads in flight per lane
        for (int q0 = 0; q0 < n_here; q0 += kFly * step) {  // same trip count for the whole team (shuffles inside)
          const int q = q0 + rg;
          float v[kFly][VEC];
#pragma unroll
          for (int k = 0; k < kFly; ++k) {  // no branches in here: see g_zero_row
            const int src = q + k * step;
            const int from = (team_lane0 + src) & (kWave - 1);  // past the team: some other lane's row, not used
            const bool want = src < n_here && col_ok;
            const TIn* row;
            if constexpr (BLK) {
              const uint32_t lo = __shfl(static_cast<uint32_t>(mine_addr), from, kWave);
              const uint32_t hi = __shfl(static_cast<uint32_t>(mine_addr >> 32), from, kWave);
              const uint64_t addr = (static_cast<uint64_t>(hi) << 32) | lo;
              row = (want && addr != 0) ? reinterpret_cast<const TIn*>(addr) + c0 : zero_row;
            } else {
              // (the row of zeros as an offset from emb: one global pointer for every load; a choice
              // between two pointers makes the loads generic ones)
              const int32_t id = __shfl(mine, from, kWave);
              row = emb + ((want && id >= 0) ? static_cast<int64_t>(id) * D + c0 : zero_at);
            }
            load_row_pack<TIn, VEC, NT>(row, v[k]);
          }
#pragma unroll
          for (int k = 0; k < kFly; ++k) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] += v[k][j];
          }
        }
      }
    };
    if (nt) {
      sum_rows(std::true_type{});
    } else {
      sum_rows(std::false_type{});
    }
    for (int off = 1 << a.lpr_log2; off < team; off <<= 1) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += __shfl_xor(acc[j], off, kWave);
    }
    if constexpr (WG) {
      constexpr int n_waves = kBlock / kWave;
      if (rg == 0 && col_ok) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) s_wave_part[wave * D + c0 + j] = acc[j];
      }
      __syncthreads();
      if (wave == 0 && rg == 0 && col_ok) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          float sum = s_wave_part[c0 + j];
          for (int w = 1; w < n_waves; ++w) sum += s_wave_part[w * D + c0 + j];
          acc[j] = sum * scale;
        }
        store_pack<TOut, VEC>(out + s * D + c0, acc);
      }
      __syncthreads();
    } else if (rg == 0 && col_ok) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] *= scale;
      store_pack<TOut, VEC>(out + s * D + c0, acc);
    }
  }
}

// MAX combiner: element-wise maximum and the occurrence that produced it.
// Value and occurrence travel as one 64-bit key: the high word is the float
// mapped to an order-preserving unsigned integer (any NaN maps to the top, so it
// propagates), the low word is 0xFFFFFFFF - occurrence, so that among equal
// values the earliest occurrence is the largest key. Key 0 = "no row yet".
__device__ __forceinline__ uint64_t max_key(float v, int64_t r) {
  uint32_t b = (v == 0.f) ? 0u : __float_as_uint(v);  // -0 and +0 tie
  uint32_t m = (v != v) ? 0xFFFFFFFFu : ((b & 0x80000000u) ? ~b : (b | 0x80000000u));
  return (static_cast<uint64_t>(m) << 32) | (0xFFFFFFFFu - static_cast<uint32_t>(r));
}
__device__ __forceinline__ float max_key_value(uint64_t k) {
  uint32_t m = static_cast<uint32_t>(k >> 32);
  if (m == 0xFFFFFFFFu) return __uint_as_float(0x7FC00000u);
  return __uint_as_float((m & 0x80000000u) ? (m & 0x7FFFFFFFu) : ~m);
}

template <typename TIn, typename TOut, int VEC>
__global__ void __launch_bounds__(kBlock)
seg_max_fwd_kernel(const TIn* __restrict__ emb, TOut* __restrict__ out,
                   int32_t* __restrict__ argmax, SegArgs a) {
  __shared__ int64_t s_off[kBlock + 1];
  int64_t s, start, end;
  if (!team_segment(a, s_off, s, start, end)) return;

  const int lane_t = threadIdx.x & ((1 << a.team_log2) - 1);
  const int rg = lane_t >> a.lpr_log2;
  const int cl = lane_t & ((1 << a.lpr_log2) - 1);
  const int64_t step = int64_t(1) << (a.team_log2 - a.lpr_log2);
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;

  for (int c0 = cl * VEC; c0 < D; c0 += col_stride) {
    uint64_t key[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) key[j] = 0;
    for (int64_t r = start + rg; r < end; r += step) {
      int64_t idx = a.rev ? load_index(a.rev, a.rev64, r) : r;
      if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
        raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
        continue;
      }
      float v[VEC];
      load_pack<TIn, VEC>(emb + idx * D + c0, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        uint64_t k = max_key(v[j], r);
        key[j] = k > key[j] ? k : key[j];
      }
    }
    for (int off = 1 << a.lpr_log2; off < (1 << a.team_log2); off <<= 1) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        uint32_t lo = __shfl_xor(static_cast<uint32_t>(key[j]), off, kWave);
        uint32_t hi = __shfl_xor(static_cast<uint32_t>(key[j] >> 32), off, kWave);
        uint64_t other = (static_cast<uint64_t>(hi) << 32) | lo;
        key[j] = other > key[j] ? other : key[j];
      }
    }
    if (rg == 0) {
      float best[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) best[j] = key[j] ? max_key_value(key[j]) : 0.f;
      store_pack<TOut, VEC>(out + s * D + c0, best);
      if (argmax) {  // one store per lane, like the values (the host picks VEC so that it is aligned)
        Pack<int32_t, VEC> am;
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          am.v[j] = key[j] ? static_cast<int32_t>(0xFFFFFFFFu - static_cast<uint32_t>(key[j])) : -1;
        *reinterpret_cast<Pack<int32_t, VEC>*>(argmax + s * D + c0) = am;
      }
    }
  }
}

// MAX forward with the memory behaviour of seg_pool_fwd_fast_kernel (indices by one coalesced
// load + shuffles, four row loads in flight per lane). Requires U < 2^31 and B < 2^31.
template <typename TIn, typename TOut, int VEC, int KIND>
__global__ void __launch_bounds__(kBlock)
seg_max_fwd_fast_kernel(const TIn* __restrict__ emb, TOut* __restrict__ out, int32_t* __restrict__ argmax,
                        SegArgs a) {
  const int64_t s = static_cast<int64_t>(blockIdx.x) * (kBlock >> a.team_log2) + (threadIdx.x >> a.team_log2);
  if (s >= a.S) return;  // whole teams leave together
  int64_t start = load_index(a.offs, a.off64, s);
  int64_t end = load_index(a.offs, a.off64, s + 1);
  if (start < 0 || end > a.B || end < start) {
    raise_device_error(a.err, RECIS_DEVERR_OFFSETS);
    start = end = 0;
  }
  const int team = 1 << a.team_log2;
  const int lane = threadIdx.x & (kWave - 1);
  const int lane_t = lane & (team - 1);
  const int team_lane0 = lane - lane_t;
  const int rg = lane_t >> a.lpr_log2;
  const int cl = lane_t & ((1 << a.lpr_log2) - 1);
  const int step = team >> a.lpr_log2;
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;
  const TIn* zero_row = reinterpret_cast<const TIn*>(g_zero_row);

  for (int cbase = 0; cbase < D; cbase += col_stride) {  // uniform: every lane takes part in the shuffles
    const int c0 = cbase + cl * VEC;
    const bool col_ok = c0 < D;
    // Inside a lane the occurrences come in ascending order, so a strict float comparison keeps
    // the first of equal values (-0 == +0) and costs less than building a key per element. The
    // running best starts at -inf with no row; the first NaN of the data wins over every number
    // and is kept from then on (nothing is taken once the best is a NaN). A lane whose values are
    // all -inf never takes one: its first row is put in afterwards. No arrays of bool in here:
    // those live in vector registers as bytes, and the selects and tests that go with them were
    // two thirds of the loop's instructions (the vector units, not the memory, then set the pace:
    // 3.4e8 vector instructions per launch of the 16 M row workload, 0.64 ms of SIMD time).
    float best_v[VEC];
    int32_t best_r[VEC];
    auto scan_rows = [&](auto nt_tag) {
      constexpr bool NT = decltype(nt_tag)::value;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        best_v[j] = -__builtin_huge_valf();
        best_r[j] = -1;
      }
      // the row of zeros as an offset from emb, so that every load goes through the one global
      // pointer (see the sum kernel)
      const int64_t zero_at = zero_row - emb;
      for (int64_t base = start; base < end; base += team) {
        const int n_here = static_cast<int>(min(static_cast<int64_t>(team), end - base));
        int32_t mine = -1;  // row of occurrence base + lane_t
        if (lane_t < n_here) {
          int64_t idx;
          if constexpr (KIND == kFastPlain) {
            idx = base + lane_t;
          } else if constexpr (KIND == kFastRev32) {
            idx = static_cast<const int32_t*>(a.rev)[base + lane_t];
          } else {
            idx = static_cast<const int64_t*>(a.rev)[base + lane_t];
          }
          if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
            raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
          } else {
            mine = static_cast<int32_t>(idx);
          }
        }
        constexpr int kFly = 4;  // row loads in flight per lane (8 was measured: slower, fewer resident waves)
        for (int q0 = 0; q0 < n_here; q0 += kFly * step) {  // same trip count for the whole team
          float v[kFly][VEC];
          int32_t id[kFly];  // -1: nothing to read (a row of zeros is loaded and not looked at)
#pragma unroll
          for (int k = 0; k < kFly; ++k) {  // no branches in here: see g_zero_row
            const int src = q0 + rg + k * step;
            const int32_t got = __shfl(mine, (team_lane0 + src) & (kWave - 1), kWave);
            id[k] = (src < n_here && col_ok) ? got : -1;
            const int64_t at = id[k] >= 0 ? static_cast<int64_t>(id[k]) * D + c0 : zero_at;
            load_row_pack<TIn, VEC, NT>(emb + at, v[k]);
          }
#pragma unroll
          for (int k = 0; k < kFly; ++k) {
            const int32_t r = static_cast<int32_t>(base) + q0 + rg + k * step;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              const float x = v[k][j];
              // & not &&: no branches (the values are all at hand)
              const bool take = (id[k] >= 0) & !(x <= best_v[j]) & (best_v[j] == best_v[j]);
              best_v[j] = take ? x : best_v[j];
              best_r[j] = take ? r : best_r[j];
            }
          }
        }
      }
    };
    if (KIND == kFastPlain || a.nt_in) {
      scan_rows(std::true_type{});
    } else {
      scan_rows(std::false_type{});
    }
    // a lane that read rows and took none (all -inf): its first row holds the first -inf
    const int64_t lane_first = start + rg;
    uint64_t key[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      if (best_r[j] < 0 && lane_first < end && col_ok) best_r[j] = static_cast<int32_t>(lane_first);
      key[j] = best_r[j] >= 0 ? max_key(best_v[j], best_r[j]) : 0;
    }
    for (int off = 1 << a.lpr_log2; off < team; off <<= 1) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        uint32_t lo = __shfl_xor(static_cast<uint32_t>(key[j]), off, kWave);
        uint32_t hi = __shfl_xor(static_cast<uint32_t>(key[j] >> 32), off, kWave);
        uint64_t other = (static_cast<uint64_t>(hi) << 32) | lo;
        key[j] = other > key[j] ? other : key[j];
      }
    }
    if (rg == 0 && col_ok) {
      float best[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) best[j] = key[j] ? max_key_value(key[j]) : 0.f;
      store_pack<TOut, VEC>(out + s * D + c0, best);
      if (argmax) {  // one store per lane, like the values (the host picks VEC so that it is aligned)
        Pack<int32_t, VEC> am;
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          am.v[j] = key[j] ? static_cast<int32_t>(0xFFFFFFFFu - static_cast<uint32_t>(key[j])) : -1;
        *reinterpret_cast<Pack<int32_t, VEC>*>(argmax + s * D + c0) = am;
      }
    }
  }
}

// TILE combiner forward: one row group per occurrence, out[i] = w_i * emb[rev_i];
// occurrences outside [offsets[0], offsets[S]) produce zero rows.
template <typename TIn, typename TOut, int VEC, bool BLK>
__global__ void __launch_bounds__(kBlock)
seg_tile_fwd_kernel(const TIn* __restrict__ emb, TOut* __restrict__ out, SegArgs a) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t r = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  if (r >= a.B) return;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;
  const int64_t lo = load_index(a.offs, a.off64, 0);
  const int64_t hi = load_index(a.offs, a.off64, a.S);
  bool live = r >= lo && r < hi;
  int64_t idx = 0;
  float w = 0.f;
  if (live) {
    idx = a.rev ? load_index(a.rev, a.rev64, r) : r;
    w = a.weight ? load_weight(a.weight, a.wdt, r) : 1.0f;
    if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
      raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
      live = false;
    }
  }
  const TIn* row = nullptr;
  if (live) {
    if constexpr (BLK) {
      row = block_row<TIn>(a, idx);
    } else {
      row = emb + idx * D;
    }
    live = row != nullptr;
  }
  for (int c0 = cl * VEC; c0 < D; c0 += col_stride) {
    float v[VEC];
    if (live) {
      load_pack<TIn, VEC>(row + c0, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] *= w;
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = 0.f;
    }
    store_pack<TOut, VEC>(out + r * D + c0, v);
  }
}

// ----------------------------------------------------------------- backward
template <typename TOut, int VEC>
__global__ void __launch_bounds__(kBlock)
fill_zero_rows_kernel(TOut* __restrict__ p, int64_t n_packs) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  float z[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) z[j] = 0.f;
  for (; i < n_packs; i += stride) store_pack<TOut, VEC>(p + i * VEC, z);
}

// SUM / MEAN backward, segment-major. ATOMIC=false writes each touched row once.
// Unweighted backward onto distinct rows (no atomics): the pooled gradient row of a segment is
// read once and stored to every row of the segment. As in the forward, the reverse indices of
// up to TEAM rows come from one coalesced load and travel by shuffles, so the stores of a lane
// follow each other without a dependent index load in between. Requires U < 2^31.
template <typename TG, typename TOut, int VEC, int KIND>
__global__ void __launch_bounds__(kBlock)
seg_pool_bwd_fast_kernel(const TG* __restrict__ grad_out, TOut* __restrict__ grad_unique, SegArgs a) {
  const int64_t s = static_cast<int64_t>(blockIdx.x) * (kBlock >> a.team_log2) + (threadIdx.x >> a.team_log2);
  if (s >= a.S) return;  // whole teams leave together
  int64_t start = load_index(a.offs, a.off64, s);
  int64_t end = load_index(a.offs, a.off64, s + 1);
  if (start < 0 || end > a.B || end < start) {
    raise_device_error(a.err, RECIS_DEVERR_OFFSETS);
    start = end = 0;
  }
  const int team = 1 << a.team_log2;
  const int lane = threadIdx.x & (kWave - 1);
  const int lane_t = lane & (team - 1);
  const int team_lane0 = lane - lane_t;
  const int rg = lane_t >> a.lpr_log2;
  const int cl = lane_t & ((1 << a.lpr_log2) - 1);
  const int step = team >> a.lpr_log2;
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;
  const float scale = (a.mean && end > start) ? 1.0f / static_cast<float>(end - start) : 1.0f;

  for (int cbase = 0; cbase < D; cbase += col_stride) {  // uniform: every lane takes part in the shuffles
    const int c0 = cbase + cl * VEC;
    const bool col_ok = c0 < D;
    float g[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) g[j] = 0.f;
    if (col_ok) load_pack<TG, VEC>(grad_out + s * D + c0, g);
#pragma unroll
    for (int j = 0; j < VEC; ++j) g[j] *= scale;
    for (int64_t base = start; base < end; base += team) {
      const int n_here = static_cast<int>(min(static_cast<int64_t>(team), end - base));
      int32_t mine = -1;  // row of occurrence base + lane_t
      if (lane_t < n_here) {
        int64_t idx;
        if constexpr (KIND == kFastPlain) {
          idx = base + lane_t;
        } else if constexpr (KIND == kFastRev32) {
          idx = static_cast<const int32_t*>(a.rev)[base + lane_t];
        } else {
          idx = static_cast<const int64_t*>(a.rev)[base + lane_t];
        }
        if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
          raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
        } else {
          mine = static_cast<int32_t>(idx);
        }
      }
      for (int q0 = 0; q0 < n_here; q0 += 4 * step) {  // same trip count for the whole team
        int32_t id[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int src = q0 + rg + k * step;
          id[k] = __shfl(mine, team_lane0 + min(src, team - 1), kWave);
          if (src >= n_here || !col_ok) id[k] = -1;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (id[k] >= 0) {
            TOut* dst = grad_unique + static_cast<int64_t>(id[k]) * D + c0;
            if (KIND == kFastPlain || a.nt_out) {
              store_pack_stream<TOut, VEC>(dst, g);
            } else {
              store_pack<TOut, VEC>(dst, g);  // a small gradient is read again by the next kernel
            }
          }
        }
      }
    }
  }
}

template <typename TG, typename TOut, int VEC, bool ATOMIC>
__global__ void __launch_bounds__(kBlock)
seg_pool_bwd_kernel(const TG* __restrict__ grad_out, TOut* __restrict__ grad_unique, SegArgs a) {
  __shared__ int64_t s_off[kBlock + 1];
  int64_t s, start, end;
  if (!team_segment(a, s_off, s, start, end)) return;

  const int lane_t = threadIdx.x & ((1 << a.team_log2) - 1);
  const int rg = lane_t >> a.lpr_log2;
  const int cl = lane_t & ((1 << a.lpr_log2) - 1);
  const int64_t step = int64_t(1) << (a.team_log2 - a.lpr_log2);
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;
  const float scale = (a.mean && end > start) ? 1.0f / static_cast<float>(end - start) : 1.0f;

  for (int c0 = cl * VEC; c0 < D; c0 += col_stride) {
    float g[VEC];
    load_pack<TG, VEC>(grad_out + s * D + c0, g);
#pragma unroll
    for (int j = 0; j < VEC; ++j) g[j] *= scale;
    for (int64_t r = start + rg; r < end; r += step) {
      int64_t idx = a.rev ? load_index(a.rev, a.rev64, r) : r;
      float w = a.weight ? load_weight(a.weight, a.wdt, r) : 1.0f;
      if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
        raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
        continue;
      }
      float v[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = g[j] * w;
      if constexpr (ATOMIC) {
        float* dst = reinterpret_cast<float*>(grad_unique) + idx * D + c0;
#pragma unroll
        for (int j = 0; j < VEC; ++j) unsafeAtomicAdd(dst + j, v[j]);
      } else {
        store_pack<TOut, VEC>(grad_unique + idx * D + c0, v);
      }
    }
  }
}

// Rows of occurrences that no segment covers (before offsets[0], after
// offsets[S]) when the caller promised a bijection occurrence <-> row and no
// zero fill was done.
template <typename TOut, int VEC>
__global__ void __launch_bounds__(kBlock)
seg_bwd_zero_uncovered_kernel(TOut* __restrict__ grad_unique, SegArgs a) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t lo = load_index(a.offs, a.off64, 0);
  const int64_t hi = load_index(a.offs, a.off64, a.S);
  const int64_t head = lo < 0 ? 0 : (lo > a.B ? a.B : lo);
  const int64_t tail_begin = hi < head ? head : (hi > a.B ? a.B : hi);
  const int64_t n_uncovered = head + (a.B - tail_begin);
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int col_stride = VEC << a.lpr_log2;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * rows_per_block;
  float z[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) z[j] = 0.f;
  for (int64_t k = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
       k < n_uncovered; k += stride) {
    int64_t r = k < head ? k : tail_begin + (k - head);
    int64_t idx = a.rev ? load_index(a.rev, a.rev64, r) : r;
    if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) continue;
    for (int c0 = cl * VEC; c0 < a.D; c0 += col_stride)
      store_pack<TOut, VEC>(grad_unique + idx * a.D + c0, z);
  }
}

// TILE backward: one row group per occurrence.
template <typename TG, typename TOut, int VEC, bool ATOMIC>
__global__ void __launch_bounds__(kBlock)
seg_tile_bwd_kernel(const TG* __restrict__ grad_out, TOut* __restrict__ grad_unique, SegArgs a) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t r = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  if (r >= a.B) return;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;
  const int64_t lo = load_index(a.offs, a.off64, 0);
  const int64_t hi = load_index(a.offs, a.off64, a.S);
  const bool live = r >= lo && r < hi;
  int64_t idx = a.rev ? load_index(a.rev, a.rev64, r) : r;
  if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
    raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  if (ATOMIC && !live) return;
  const float w = live ? (a.weight ? load_weight(a.weight, a.wdt, r) : 1.0f) : 0.f;
  for (int c0 = cl * VEC; c0 < D; c0 += col_stride) {
    float v[VEC];
    if (live) {
      load_pack<TG, VEC>(grad_out + r * D + c0, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] *= w;
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = 0.f;
    }
    if constexpr (ATOMIC) {
      float* dst = reinterpret_cast<float*>(grad_unique) + idx * D + c0;
#pragma unroll
      for (int j = 0; j < VEC; ++j) unsafeAtomicAdd(dst + j, v[j]);
    } else {
      store_pack<TOut, VEC>(grad_unique + idx * D + c0, v);
    }
  }
}

// MAX backward: route each pooled-gradient element to the winning occurrence.
// grad_unique is zero-filled by the caller. One thread per (segment, column).
// MAX backward onto distinct rows that are all reached (a bijection between occurrences and
// rows): segment-major, every row of the segment is written in full -- the gradient where the
// row won the column, zero elsewhere -- so no zero fill of the output and no scatter are needed.
// Requires U < 2^31.
template <typename TG, typename TOut, int VEC, int KIND>
__global__ void __launch_bounds__(kBlock)
seg_max_bwd_rows_kernel(const TG* __restrict__ grad_out, const int32_t* __restrict__ argmax,
                        TOut* __restrict__ grad_unique, SegArgs a) {
  const int64_t s = static_cast<int64_t>(blockIdx.x) * (kBlock >> a.team_log2) + (threadIdx.x >> a.team_log2);
  if (s >= a.S) return;  // whole teams leave together
  int64_t start = load_index(a.offs, a.off64, s);
  int64_t end = load_index(a.offs, a.off64, s + 1);
  if (start < 0 || end > a.B || end < start) {
    raise_device_error(a.err, RECIS_DEVERR_OFFSETS);
    start = end = 0;
  }
  const int team = 1 << a.team_log2;
  const int lane = threadIdx.x & (kWave - 1);
  const int lane_t = lane & (team - 1);
  const int team_lane0 = lane - lane_t;
  const int rg = lane_t >> a.lpr_log2;
  const int cl = lane_t & ((1 << a.lpr_log2) - 1);
  const int step = team >> a.lpr_log2;
  const int col_stride = VEC << a.lpr_log2;
  const int D = a.D;

  for (int cbase = 0; cbase < D; cbase += col_stride) {  // uniform: every lane takes part in the shuffles
    const int c0 = cbase + cl * VEC;
    const bool col_ok = c0 < D;
    float g[VEC];
    int32_t win[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      g[j] = 0.f;
      win[j] = -1;
    }
    if (col_ok) {
      load_pack<TG, VEC>(grad_out + s * D + c0, g);
#pragma unroll
      for (int j = 0; j < VEC; ++j) win[j] = argmax[s * D + c0 + j];
    }
    for (int64_t base = start; base < end; base += team) {
      const int n_here = static_cast<int>(min(static_cast<int64_t>(team), end - base));
      int32_t mine = -1;  // row of occurrence base + lane_t
      if (lane_t < n_here) {
        int64_t idx;
        if constexpr (KIND == kFastPlain) {
          idx = base + lane_t;
        } else if constexpr (KIND == kFastRev32) {
          idx = static_cast<const int32_t*>(a.rev)[base + lane_t];
        } else {
          idx = static_cast<const int64_t*>(a.rev)[base + lane_t];
        }
        if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
          raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
        } else {
          mine = static_cast<int32_t>(idx);
        }
      }
      for (int q0 = 0; q0 < n_here; q0 += 4 * step) {  // same trip count for the whole team
        int32_t id[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int src = q0 + rg + k * step;
          id[k] = __shfl(mine, team_lane0 + min(src, team - 1), kWave);
          if (src >= n_here || !col_ok) id[k] = -1;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (id[k] < 0) continue;
          const int32_t r = static_cast<int32_t>(base) + q0 + rg + k * step;
          float v[VEC];
#pragma unroll
          for (int j = 0; j < VEC; ++j) v[j] = win[j] == r ? g[j] : 0.f;
          TOut* dst = grad_unique + static_cast<int64_t>(id[k]) * D + c0;
          if (a.nt_out) {
            store_pack_stream<TOut, VEC>(dst, v);
          } else {
            store_pack<TOut, VEC>(dst, v);
          }
        }
      }
    }
  }
}

template <typename TG, typename TOut, bool ATOMIC>
__global__ void __launch_bounds__(kBlock)
seg_max_bwd_kernel(const TG* __restrict__ grad_out, const int32_t* __restrict__ argmax,
                   TOut* __restrict__ grad_unique, SegArgs a) {
  const int64_t total = a.S * a.D;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < total; e += stride) {
    const int32_t r = argmax[e];
    if (r < 0) continue;
    if (static_cast<int64_t>(r) >= a.B) {
      raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
      continue;
    }
    const int d = static_cast<int>(e % a.D);
    int64_t idx = a.rev ? load_index(a.rev, a.rev64, r) : r;
    if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(a.U)) {
      raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
      continue;
    }
    const float g = to_float(grad_out[e]);
    if constexpr (ATOMIC) {
      unsafeAtomicAdd(reinterpret_cast<float*>(grad_unique) + idx * a.D + d, g);
    } else {
      grad_unique[idx * a.D + d] = from_float<TOut>(g);
    }
  }
}

// ------------------------------------------------------------ host dispatch
// Team size: enough row groups to cover about half the average segment, so that
// each group still has a few rows to pipeline.
int pick_team_log2(int64_t B, int64_t S, int lpr_log2) {
  int64_t avg = S > 0 ? B / S : 1;
  int rows_log2 = 0;
  while ((int64_t(2) << rows_log2) <= avg / 2 && rows_log2 + lpr_log2 < 6) ++rows_log2;
  return lpr_log2 + rows_log2;
}

template <typename F>
int dispatch_vec(int vec, F&& f) {
  switch (vec) {
    case 8: return f(std::integral_constant<int, 8>{});
    case 4: return f(std::integral_constant<int, 4>{});
    case 2: return f(std::integral_constant<int, 2>{});
    case 1: return f(std::integral_constant<int, 1>{});
    default: return fail(RECIS_ERR_ARG, "unsupported vector width %d", vec);
  }
}

// Calls f(TIn tag, TOut tag) for the supported (in, out) storage pairs:
// same type, or any type widened to fp32.
template <typename F>
int dispatch_types(int in_dt, int out_dt, F&& f) {
  if (in_dt == RECIS_F32 && out_dt == RECIS_F32) return f(float{}, float{});
  if (in_dt == RECIS_BF16 && out_dt == RECIS_BF16) return f(bf16_t{}, bf16_t{});
  if (in_dt == RECIS_BF16 && out_dt == RECIS_F32) return f(bf16_t{}, float{});
  if (in_dt == RECIS_F16 && out_dt == RECIS_F16) return f(f16_t{}, f16_t{});
  if (in_dt == RECIS_F16 && out_dt == RECIS_F32) return f(f16_t{}, float{});
  if (in_dt == RECIS_F32 && out_dt == RECIS_BF16) return f(float{}, bf16_t{});
  if (in_dt == RECIS_F32 && out_dt == RECIS_F16) return f(float{}, f16_t{});
  return fail(RECIS_ERR_ARG, "unsupported dtype pair (in=%d, out=%d)", in_dt, out_dt);
}

int check_common(const void* offsets, int64_t B, int64_t U, int64_t S, int64_t D,
                 int mode, int wdt, const void* weight) {
  RECIS_REQUIRE(B >= 0 && U >= 0 && S >= 0, "negative size (B=%lld U=%lld S=%lld)",
                (long long)B, (long long)U, (long long)S);
  RECIS_REQUIRE(D >= 1 && D <= (1 << 20), "embedding dim %lld out of range", (long long)D);
  RECIS_REQUIRE(offsets != nullptr, "offsets must not be NULL");
  RECIS_REQUIRE(mode >= RECIS_SUM && mode <= RECIS_MAX, "invalid mode %d", mode);
  RECIS_REQUIRE(weight == nullptr || dtype_size(wdt) > 0, "invalid weight dtype %d", wdt);
  RECIS_REQUIRE(B < (int64_t(1) << 31) || mode != RECIS_MAX,
                "MAX combiner supports fewer than 2^31 occurrences");
  return RECIS_OK;
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

// Where the unique rows live when they are not a dense [U, D] array.
struct BlockSource {
  const int64_t* row_index;
  const void* const* blocks;
  int64_t block_rows, n_blocks;
  int64_t row_pitch_bytes;  // 0: rows lie back to back
};

static int forward_impl(const void* unique_emb, const BlockSource* blk, int emb_dtype, const void* weight,
                        int weight_dtype, const void* reverse_indices, int rev_is64, const void* offsets,
                        int off_is64, void* out, int out_dtype, int32_t* argmax_out, int64_t B, int64_t U,
                        int64_t S, int64_t D, int mode, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = check_common(offsets, B, U, S, D, mode, weight_dtype, weight)) return rc;
  RECIS_REQUIRE(reverse_indices != nullptr || U == B,
                "reverse_indices == NULL (identity) needs U == B (U=%lld, B=%lld)",
                (long long)U, (long long)B);
  const int64_t out_rows = (mode == RECIS_TILE) ? B : S;
  if (out_rows == 0) return RECIS_OK;
  RECIS_REQUIRE(out != nullptr, "out must not be NULL");
  RECIS_REQUIRE(unique_emb != nullptr || U == 0 || blk != nullptr, "unique_emb must not be NULL");
  const int in_sz = dtype_size(emb_dtype), out_sz = dtype_size(out_dtype);
  RECIS_REQUIRE(in_sz && out_sz, "invalid dtype (emb=%d out=%d)", emb_dtype, out_dtype);

  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");

  // vector width in elements, limited by both row widths and pointer alignment
  // (blocks are 16-byte aligned by contract)
  const int vb_in = pick_vec_bytes(D * in_sz, blk ? 16 : reinterpret_cast<uintptr_t>(unique_emb));
  const int vb_out = pick_vec_bytes_max(D * out_sz, reinterpret_cast<uintptr_t>(out), 32);
  int vec = std::min(vb_in / in_sz, vb_out / out_sz);
  if (vec < 1) vec = 1;
  if (mode == RECIS_MAX && argmax_out)  // the winners' occurrences leave as packs of VEC 32-bit words
    vec = std::min(vec, pick_vec_bytes(D * 4, reinterpret_cast<uintptr_t>(argmax_out)) / 4);
  RowGeom geom;
  geom.vec = vec;
  geom.lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));

  SegArgs a;
  a.weight = weight;
  a.rev = reverse_indices;
  a.offs = offsets;
  a.B = B;
  a.U = U;
  a.S = S;
  a.D = static_cast<int>(D);
  a.wdt = weight_dtype;
  a.rev64 = rev_is64;
  a.off64 = off_is64;
  a.lpr_log2 = geom.lpr_log2;
  a.team_log2 = pick_team_log2(B, S, geom.lpr_log2);
  a.mean = (mode == RECIS_MEAN);
  a.nt_out = 0;
  a.nt_in = !blk && U * D * static_cast<int64_t>(dtype_size(emb_dtype)) >= (int64_t(1) << 30);
  a.err = err;
  a.row_index = blk ? blk->row_index : nullptr;
  a.blocks = blk ? blk->blocks : nullptr;
  a.block_rows = blk ? blk->block_rows : 1;
  a.n_blocks = blk ? blk->n_blocks : 0;
  a.pitch = D;
  if (blk && blk->row_pitch_bytes) {
    RECIS_REQUIRE(blk->row_pitch_bytes >= D * in_sz && blk->row_pitch_bytes % in_sz == 0 &&
                      blk->row_pitch_bytes % vb_in == 0,
                  "row pitch of %lld bytes does not fit rows of %lld elements", (long long)blk->row_pitch_bytes,
                  (long long)D);
    a.pitch = blk->row_pitch_bytes / in_sz;
  }

  return dispatch_types(emb_dtype, out_dtype, [&](auto tin, auto tout) {
    using TIn = decltype(tin);
    using TOut = decltype(tout);
    return dispatch_vec(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(TIn) > 16 || VEC * sizeof(TOut) > 32) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        if (mode == RECIS_TILE) {
          const int rows_per_block = kBlock >> a.lpr_log2;
          const int64_t grid = (B + rows_per_block - 1) / rows_per_block;
          RECIS_TIME_KERNEL("seg_tile_fwd_kernel", stream)
          if (blk)
            seg_tile_fwd_kernel<TIn, TOut, VEC, true><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                nullptr, static_cast<TOut*>(out), a);
          else
            seg_tile_fwd_kernel<TIn, TOut, VEC, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                static_cast<const TIn*>(unique_emb), static_cast<TOut*>(out), a);
        } else if (blk) {
          // rows in the table: the int32-index kernels (what a batch plan produces) and the generic one
          const int teams_per_block = kBlock >> a.team_log2;
          const int64_t grid = (S + teams_per_block - 1) / teams_per_block;
          TOut* o = static_cast<TOut*>(out);
          const bool rev32 = a.weight == nullptr && a.rev != nullptr && !a.rev64;
          const bool fast_blk = rev32 && U < (int64_t(1) << 31) && a.team_log2 > a.lpr_log2;
          // segments of hundreds of rows: a workgroup each, as for dense rows below
          const bool wg_blk = fast_blk && a.team_log2 == 6 && S > 0 && B / S >= 128 && D <= 4096;
          RECIS_TIME_KERNEL("seg_pool_fwd_kernel", stream)
          if (wg_blk)
            seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastRev32, true, true><<<dim3(S), dim3(kBlock),
                sizeof(float) * (kBlock / kWave) * static_cast<size_t>(D), stream>>>(nullptr, o, a);
          else if (fast_blk)
            seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastRev32, true><<<dim3(grid), dim3(kBlock), 0, stream>>>(nullptr, o, a);
          else if (rev32)
            seg_pool_fwd_kernel<TIn, TOut, VEC, kFwdRev32, true><<<dim3(grid), dim3(kBlock), 0, stream>>>(nullptr, o, a);
          else
            seg_pool_fwd_kernel<TIn, TOut, VEC, kFwdGeneric, true><<<dim3(grid), dim3(kBlock), 0, stream>>>(nullptr, o, a);
        } else {
          const int teams_per_block = kBlock >> a.team_log2;
          const int64_t grid = (S + teams_per_block - 1) / teams_per_block;
          if (mode == RECIS_MAX) {
            const TIn* e = static_cast<const TIn*>(unique_emb);
            TOut* o = static_cast<TOut*>(out);
            RECIS_TIME_KERNEL("seg_max_fwd_kernel", stream)
            if (U >= (int64_t(1) << 31) || B >= (int64_t(1) << 31))
              seg_max_fwd_kernel<TIn, TOut, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, argmax_out, a);
            else if (a.rev == nullptr)
              seg_max_fwd_fast_kernel<TIn, TOut, VEC, kFastPlain><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, argmax_out, a);
            else if (!a.rev64)
              seg_max_fwd_fast_kernel<TIn, TOut, VEC, kFastRev32><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, argmax_out, a);
            else
              seg_max_fwd_fast_kernel<TIn, TOut, VEC, kFastRev64><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, argmax_out, a);
          } else {
            const TIn* e = static_cast<const TIn*>(unique_emb);
            TOut* o = static_cast<TOut*>(out);
            // several rows per segment: the latency-oriented kernel; about one row: the lean one
            const bool fast = a.weight == nullptr && U < (int64_t(1) << 31) && a.team_log2 > a.lpr_log2;
            // segments of hundreds of rows: a workgroup each (the team is a whole wave already)
            const bool wg = fast && a.team_log2 == 6 && S > 0 && B / S >= 128 && D <= 4096;
            const size_t wg_lds = sizeof(float) * (kBlock / kWave) * static_cast<size_t>(D);
            RECIS_TIME_KERNEL("seg_pool_fwd_kernel", stream)
            if (wg && a.rev == nullptr)
              seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastPlain, false, true><<<dim3(S), dim3(kBlock), wg_lds, stream>>>(e, o, a);
            else if (wg && !a.rev64)
              seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastRev32, false, true><<<dim3(S), dim3(kBlock), wg_lds, stream>>>(e, o, a);
            else if (wg)
              seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastRev64, false, true><<<dim3(S), dim3(kBlock), wg_lds, stream>>>(e, o, a);
            else if (fast && a.rev == nullptr)
              seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastPlain, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, a);
            else if (fast && !a.rev64)
              seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastRev32, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, a);
            else if (fast)
              seg_pool_fwd_fast_kernel<TIn, TOut, VEC, kFastRev64, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, a);
            else if (a.weight == nullptr && a.rev == nullptr)
              seg_pool_fwd_kernel<TIn, TOut, VEC, kFwdPlain, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, a);
            else if (a.weight == nullptr && !a.rev64)
              seg_pool_fwd_kernel<TIn, TOut, VEC, kFwdRev32, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, a);
            else
              seg_pool_fwd_kernel<TIn, TOut, VEC, kFwdGeneric, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(e, o, a);
          }
        }
        RECIS_LAUNCH_CHECK();
        return RECIS_OK;
      }
    });
  });
}

extern "C" int recis_segment_reduce_forward(
    const void* unique_emb, int emb_dtype, const void* weight, int weight_dtype,
    const void* reverse_indices, int rev_is64, const void* offsets, int off_is64,
    void* out, int out_dtype, int32_t* argmax_out, int64_t B, int64_t U, int64_t S,
    int64_t D, int mode, void* stream_) {
  return forward_impl(unique_emb, nullptr, emb_dtype, weight, weight_dtype, reverse_indices, rev_is64, offsets,
                      off_is64, out, out_dtype, argmax_out, B, U, S, D, mode, stream_);
}

extern "C" int recis_segment_reduce_forward_blocks(
    const void* const* emb_blocks_dev, int64_t n_blocks, int64_t block_rows, int64_t row_pitch_bytes,
    const int64_t* row_index, int emb_dtype, const void* weight, int weight_dtype, const void* reverse_indices, int rev_is64,
    const void* offsets, int off_is64, void* out, int out_dtype, int64_t B, int64_t U, int64_t S,
    int64_t D, int mode, void* stream_) {
  RECIS_REQUIRE(mode != RECIS_MAX, "the MAX combiner takes dense rows (recis_segment_reduce_forward)");
  RECIS_REQUIRE(n_blocks >= 0 && block_rows > 0, "bad block list");
  RECIS_REQUIRE(U == 0 || (emb_blocks_dev != nullptr && row_index != nullptr), "NULL block list / row_index");
  BlockSource blk{row_index, emb_blocks_dev, block_rows, n_blocks, row_pitch_bytes};
  return forward_impl(nullptr, &blk, emb_dtype, weight, weight_dtype, reverse_indices, rev_is64, offsets, off_is64,
                      out, out_dtype, nullptr, B, U, S, D, mode, stream_);
}

extern "C" int recis_segment_reduce_backward(
    const void* grad_out, int grad_dtype, const void* weight, int weight_dtype,
    const void* reverse_indices, int rev_is64, const void* offsets, int off_is64,
    const int32_t* argmax, void* grad_unique, int out_dtype, int64_t B, int64_t U,
    int64_t S, int64_t D, int mode, int flags, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = check_common(offsets, B, U, S, D, mode, weight_dtype, weight)) return rc;
  RECIS_REQUIRE(reverse_indices != nullptr || U == B,
                "reverse_indices == NULL (identity) needs U == B (U=%lld, B=%lld)",
                (long long)U, (long long)B);
  if (U == 0) return RECIS_OK;
  RECIS_REQUIRE(grad_unique != nullptr, "grad_unique must not be NULL");
  const int64_t in_rows = (mode == RECIS_TILE) ? B : S;
  RECIS_REQUIRE(grad_out != nullptr || in_rows == 0, "grad_out must not be NULL");
  RECIS_REQUIRE(mode != RECIS_MAX || argmax != nullptr || S == 0,
                "MAX backward needs the argmax written by the forward");
  const int in_sz = dtype_size(grad_dtype), out_sz = dtype_size(out_dtype);
  RECIS_REQUIRE(in_sz && out_sz, "invalid dtype (grad=%d out=%d)", grad_dtype, out_dtype);
  const bool unique = (flags & RECIS_FLAG_REV_UNIQUE) || reverse_indices == nullptr;
  RECIS_REQUIRE(unique || out_dtype == RECIS_F32,
                "accumulating duplicates needs an fp32 grad_unique (got dtype %d); "
                "pass RECIS_FLAG_REV_UNIQUE if reverse_indices has no duplicates",
                out_dtype);

  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");

  const int vb_in = pick_vec_bytes(D * in_sz, reinterpret_cast<uintptr_t>(grad_out));
  const int vb_out = pick_vec_bytes(D * out_sz, reinterpret_cast<uintptr_t>(grad_unique));
  int vec = std::min(vb_in / in_sz, vb_out / out_sz);
  if (vec < 1) vec = 1;
  const int lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));

  SegArgs a;
  a.weight = weight;
  a.rev = reverse_indices;
  a.offs = offsets;
  a.B = B;
  a.U = U;
  a.S = S;
  a.D = static_cast<int>(D);
  a.wdt = weight_dtype;
  a.rev64 = rev_is64;
  a.off64 = off_is64;
  a.lpr_log2 = lpr_log2;
  a.team_log2 = pick_team_log2(B, S, lpr_log2);
  a.mean = (mode == RECIS_MEAN);
  // 1 GiB is far past what L2 and the 256 MB memory-side cache keep for the next kernel
  a.nt_out = U * D * out_sz >= (int64_t(1) << 30);
  a.nt_in = 0;
  a.err = err;

  // Rows no occurrence maps to must read zero. With a promised bijection
  // (unique and U == B) every row is reached through its occurrence, so only
  // occurrences outside the offsets range need clearing; otherwise clear all.
  const bool max_rows = mode == RECIS_MAX && unique && U == B && U < (int64_t(1) << 31) && B < (int64_t(1) << 31);
  const bool bijection = unique && U == B && (mode != RECIS_MAX || max_rows);

  return dispatch_types(grad_dtype, out_dtype, [&](auto tin, auto tout) {
    using TG = decltype(tin);
    using TOut = decltype(tout);
    return dispatch_vec(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(TG) > 16 || VEC * sizeof(TOut) > 16) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        if (!bijection) {
          const int64_t n_packs = U * D / VEC;  // D % VEC == 0 by construction
          int64_t grid = std::min<int64_t>((n_packs + kBlock - 1) / kBlock, 256 * 32);
          if (grid < 1) grid = 1;
          fill_zero_rows_kernel<TOut, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(
              static_cast<TOut*>(grad_unique), n_packs);
          RECIS_LAUNCH_CHECK();
        } else if (mode != RECIS_TILE) {  // bijection: only occurrences outside the offsets range need clearing
          seg_bwd_zero_uncovered_kernel<TOut, VEC><<<dim3(64), dim3(kBlock), 0, stream>>>(
              static_cast<TOut*>(grad_unique), a);
          RECIS_LAUNCH_CHECK();
        }
        if (max_rows) {
          if (S > 0) {
            const int teams_per_block = kBlock >> a.team_log2;
            const int64_t grid = (S + teams_per_block - 1) / teams_per_block;
            const TG* gsrc = static_cast<const TG*>(grad_out);
            TOut* gdst = static_cast<TOut*>(grad_unique);
            RECIS_TIME_KERNEL("seg_max_bwd_kernel", stream)
            if (a.rev == nullptr)
              seg_max_bwd_rows_kernel<TG, TOut, VEC, kFastPlain><<<dim3(grid), dim3(kBlock), 0, stream>>>(gsrc, argmax, gdst, a);
            else if (!a.rev64)
              seg_max_bwd_rows_kernel<TG, TOut, VEC, kFastRev32><<<dim3(grid), dim3(kBlock), 0, stream>>>(gsrc, argmax, gdst, a);
            else
              seg_max_bwd_rows_kernel<TG, TOut, VEC, kFastRev64><<<dim3(grid), dim3(kBlock), 0, stream>>>(gsrc, argmax, gdst, a);
            RECIS_LAUNCH_CHECK();
          }
        } else if (mode == RECIS_MAX) {
          const int64_t total = S * D;
          if (total > 0) {
            int64_t grid = std::min<int64_t>((total + kBlock - 1) / kBlock, 256 * 64);
            if (unique)
              seg_max_bwd_kernel<TG, TOut, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                  static_cast<const TG*>(grad_out), argmax, static_cast<TOut*>(grad_unique), a);
            else
              seg_max_bwd_kernel<TG, TOut, true><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                  static_cast<const TG*>(grad_out), argmax, static_cast<TOut*>(grad_unique), a);
            RECIS_LAUNCH_CHECK();
          }
        } else if (mode == RECIS_TILE) {
          if (B > 0) {
            const int rows_per_block = kBlock >> a.lpr_log2;
            const int64_t grid = (B + rows_per_block - 1) / rows_per_block;
            if (unique)
              seg_tile_bwd_kernel<TG, TOut, VEC, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                  static_cast<const TG*>(grad_out), static_cast<TOut*>(grad_unique), a);
            else
              seg_tile_bwd_kernel<TG, TOut, VEC, true><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                  static_cast<const TG*>(grad_out), static_cast<TOut*>(grad_unique), a);
            RECIS_LAUNCH_CHECK();
          }
        } else if (S > 0) {
          const int teams_per_block = kBlock >> a.team_log2;
          const int64_t grid = (S + teams_per_block - 1) / teams_per_block;
          const TG* gsrc = static_cast<const TG*>(grad_out);
          TOut* gdst = static_cast<TOut*>(grad_unique);
          const bool fast = unique && a.weight == nullptr && U < (int64_t(1) << 31) && a.team_log2 > a.lpr_log2;
          if (fast) {
            RECIS_TIME_KERNEL("seg_pool_bwd_kernel", stream)
            if (a.rev == nullptr)
              seg_pool_bwd_fast_kernel<TG, TOut, VEC, kFastPlain><<<dim3(grid), dim3(kBlock), 0, stream>>>(gsrc, gdst, a);
            else if (!a.rev64)
              seg_pool_bwd_fast_kernel<TG, TOut, VEC, kFastRev32><<<dim3(grid), dim3(kBlock), 0, stream>>>(gsrc, gdst, a);
            else
              seg_pool_bwd_fast_kernel<TG, TOut, VEC, kFastRev64><<<dim3(grid), dim3(kBlock), 0, stream>>>(gsrc, gdst, a);
          } else if (unique)
            RECIS_TIME_KERNEL("seg_pool_bwd_kernel", stream)
            seg_pool_bwd_kernel<TG, TOut, VEC, false><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                static_cast<const TG*>(grad_out), static_cast<TOut*>(grad_unique), a);
          else
            RECIS_TIME_KERNEL("seg_pool_bwd_kernel", stream)
            seg_pool_bwd_kernel<TG, TOut, VEC, true><<<dim3(grid), dim3(kBlock), 0, stream>>>(
                static_cast<const TG*>(grad_out), static_cast<TOut*>(grad_unique), a);
          RECIS_LAUNCH_CHECK();
        }
        return RECIS_OK;
      }
    });
  });
}
