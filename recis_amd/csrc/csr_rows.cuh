// Gather-reduce over the occurrence lists of a batch plan (kernels and their launcher), shared by
// the translation units that instantiate them: out[u] = sum over the list entries k of unique id u
// of coef[k] * rows[src[k]], from one input or from two (the gradients of two outputs of one
// lookup), ending in a store or in the optimizer's update of the table row.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <type_traits>

#include "common.cuh"
#include "optim_rows.cuh"

namespace recis_hip {
namespace {

constexpr int kHotLen = RECIS_PLAN_HOT_LEN;      // rows with more occurrences than this are "hot"
constexpr int kHotChunk = RECIS_PLAN_HOT_CHUNK;  // occurrences per hot work item

__device__ __forceinline__ float load_coef(const void* w, int wdt, int64_t i) {
  if (wdt == RECIS_F32) return static_cast<const float*>(w)[i];
  if (wdt == RECIS_BF16) return to_float(static_cast<const bf16_t*>(w)[i]);
  return to_float(static_cast<const f16_t*>(w)[i]);
}

constexpr int kMaxParts = 8;  // input arrays of one gather-reduce launch (PARTS kernels)

struct CsrArgs {
  const int32_t* row_start;  // [U + 1]
  const int32_t* src;        // [n] input row per list entry (negative = skip)
  const void* coef;          // [n] per list entry, or NULL
  int coef_dt;
  int64_t U, n_rows;
  int D;
  int lpr_log2;
  int accumulate;
  const int32_t* out_rows;  // kEpiStore only: the sum of row u goes to out[out_rows[u]] (NULL: to out[u])
  int nt_in;  // the gathered rows are too many to stay cached: non-temporal loads
  // a second input over the same lists (kernels with TIn2 != void): entry k also adds
  // coef2[k] * rows2[src2[k]]; the cover range does not apply to it
  const void* rows2;
  const int32_t* src2;
  const void* coef2;
  int coef2_dt;
  int nt_in2;
  int64_t n_rows2;
  int* err;
  const void* cover;  // offsets [cover_S + 1] or NULL: entries whose src lies outside
  int cover64;        // [cover[0], cover[cover_S]) are skipped
  int64_t cover_S;
  // hot rows (more than hot_len occurrences): (row, chunk) work items, partial sums per item
  int32_t hot_len;           // INT_MAX when the caller brings no work items: every row is "cold"
  const int32_t* hot_items;  // [2 * hot_cap]
  const int64_t* counts;     // counts[1] = number of items
  int64_t hot_cap;
  float* hot_part;           // [hot_cap, D]
  int64_t cold_blocks;       // the last cold_blocks workgroups work per row, the ones before per hot item
  // PARTS kernels: the input rows as n_parts arrays laid end to end in src's numbering; part f
  // holds rows from part_lo32[f] on (INT32_MAX for an unused part). Of the one input; in kernels
  // with two inputs, of the SECOND.
  int n_parts;
  const void* part_rows[kMaxParts];
  int32_t part_lo32[kMaxParts];
};

// What a gather-reduce launch does with the finished sum of row u (template parameter EPI):
//   kEpiStore    out[u] (+)= sum
//   kEpiAdam     the sum is the gradient of table row row_index[u]: the Adam-family update of that
//                row (parameter and both moments) is applied at once, the gradient never written
//   kEpiAdagrad  the same with the Adagrad update
//   kEpiAdamCached  kEpiAdam without the streaming hint on the table rows: what the host launches
//                for a kEpiAdam request on a table small enough to stay in the caches (see
//                stream_table_rows); a kernel of its own, because one kernel holding both kinds of
//                access costs registers (measured: 126 -> 219 us)
enum { kEpiStore = 0, kEpiAdam = 1, kEpiAdagrad = 2, kEpiAdamCached = 3 };
constexpr bool epi_is_adam(int epi) { return epi == kEpiAdam || epi == kEpiAdamCached; }
struct FuseArgs {
  const int64_t* row_index;  // [U]; a negative index skips the row
  void* const* emb;          // block tables (device arrays of block pointers)
  void* const* s0;           // exp_avg / the Adagrad accumulator
  void* const* s1;           // exp_avg_sq
  RowBlocks rb;
  AdamCoef adam;
  float lr, eps;             // Adagrad
  // Adam without a cal_alpha launch in front (adam.alpha == NULL in the row kernel): every thread
  // works alpha out from the running powers as they stand (nobody writes them while the row
  // kernel runs) and leaves it in alpha_ws; the finish kernel, which runs afterwards, reads alpha
  // from there (its adam.alpha) and its first thread advances the powers (advance_powers).
  void* beta1_t;
  void* beta2_t;
  int beta_is_f64;
  int advance_powers;
  double adam_lr;
  double* alpha_ws;
};

// alpha of this step from the running powers before the step; the advanced powers in b1 / b2 (as doubles).
__device__ __forceinline__ double alpha_from_powers(const FuseArgs& f, double& b1, double& b2) {
  if (f.beta_is_f64) {
    return cal_alpha_step<double>(static_cast<const double*>(f.beta1_t)[0], static_cast<const double*>(f.beta2_t)[0],
                                  f.adam_lr, f.adam.beta1, f.adam.beta2, b1, b2);
  }
  float n1, n2;
  const double alpha = cal_alpha_step<float>(static_cast<const float*>(f.beta1_t)[0],
                                             static_cast<const float*>(f.beta2_t)[0], f.adam_lr, f.adam.beta1,
                                             f.adam.beta2, n1, n2);
  b1 = n1;
  b2 = n2;
  return alpha;
}

// Where table row idx lies in the parameter and state blocks, for a caller that asks as soon as
// idx is known (see csr_rows_kernel).
template <typename T>
struct RowPlaces {
  T* w;   // NULL: no update (a key the table does not hold, or an index out of range: flagged)
  T* s0;
  T* s1;
};
template <typename T, int EPI>
__device__ __forceinline__ RowPlaces<T> row_places(const FuseArgs& f, int* err, int64_t idx) {
  RowPlaces<T> p{nullptr, nullptr, nullptr};
  int64_t b, off;
  if (idx < 0) return p;
  if (!block_row(f.rb, idx, b, off)) {
    raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
    return p;
  }
  const int64_t at = off * f.rb.pitch;
  p.w = static_cast<T*>(f.emb[b]) + at;
  p.s0 = static_cast<T*>(f.s0[b]) + at;
  if constexpr (epi_is_adam(EPI)) p.s1 = static_cast<T*>(f.s1[b]) + at;
  return p;
}
template <typename T, int VEC, int EPI>
__device__ __forceinline__ void fused_row_update_at(const FuseArgs& f, const RowPlaces<T>& p, int c0,
                                                    const float (&acc)[VEC], double alpha) {
  if (p.w == nullptr) return;
  if constexpr (epi_is_adam(EPI)) {
    // kEpiAdam: streaming accesses to the table rows (see load_row_pack_of_table)
    adam_update_pack<T, VEC, EPI == kEpiAdam>(p.w + c0, p.s0 + c0, p.s1 + c0, acc, alpha, f.adam);
  } else {
    adagrad_update_pack<T, VEC>(p.w + c0, p.s0 + c0, acc, f.lr, f.eps);
  }
}

// The epilogue of one pack of one finished row; T = the table's row type for the optimizer kinds.
// idx = row_index[u] of the finished row (callers load it early: it heads a chain of dependent
// accesses); alpha: of this step (Adam only).
template <typename T, int VEC, int EPI>
__device__ __forceinline__ void fused_row_update(const FuseArgs& f, int* err, int64_t idx, int c0,
                                                 const float (&acc)[VEC], double alpha) {
  // (a key the table does not hold, idx < 0, takes no gradient)
  fused_row_update_at<T, VEC, EPI>(f, row_places<T, EPI>(f, err, idx), c0, acc, alpha);
}


// A row of zeros as long as any row (D <= 8192 of at most 4 bytes): what a list entry reads that
// has nothing to add (outside the cover, past the end of a round), so that the gathers need no
// branch around a load. With a branch around each load the compiler waits for the loads in flight
// before the next one goes out, and the gathers of a round run one after the other.
__device__ __align__(256) const unsigned char g_csr_zero_row[8192 * 4] = {};

// One input as a kernel sees it: entries whose src lies outside [lo, hi) are skipped, those at or
// past n_rows raise the index-range error.
template <typename T>
struct SrcView {
  const T* rows;
  const int32_t* src;
  const void* coef;
  int coef_dt;
  int nt;
  int64_t n_rows, lo, hi;
};

// Row s of the input: of the one array (PARTS == false), or of the part that holds it. No
// branches: the callers keep several of these loads in flight.
template <typename TIn, bool PARTS>
__device__ __forceinline__ const TIn* src_row(const TIn* rows, const CsrArgs& a, int64_t s) {
  if constexpr (!PARTS) {
    return rows + s * a.D;
  } else {
    const TIn* base = static_cast<const TIn*>(a.part_rows[0]);
    int32_t lo = 0;
    const int32_t s32 = static_cast<int32_t>(s);  // src entries are 32-bit, and so are the parts' first rows
#pragma unroll
    for (int k = 1; k < kMaxParts; ++k) {
      const bool past = s32 >= a.part_lo32[k];  // the first row of an unused part is past every row
      base = past ? static_cast<const TIn*>(a.part_rows[k]) : base;
      lo = past ? a.part_lo32[k] : lo;
    }
    return base + static_cast<int64_t>(s32 - lo) * a.D;
  }
}

__device__ __forceinline__ void cover_range(const CsrArgs& a, int64_t& lo, int64_t& hi) {
  lo = 0;
  hi = a.n_rows;
  if (a.cover) {
    lo = max(lo, load_index(a.cover, a.cover64, 0));
    hi = min(hi, load_index(a.cover, a.cover64, a.cover_S));
  }
}

// A whole wave works the list entries [e_begin, e_end) (uniform arguments, every lane calls):
// `src` and `coef` of 64 entries come from one coalesced load, a lane each, and reach the lanes
// that gather the rows through shuffles; lane group g of `groups` takes entries g, g + groups,
// ... with several row loads in flight. acc: this group's partial sum for columns
// c0 .. c0 + VEC (the caller folds the groups).
template <typename TIn, int VEC, bool PARTS, bool NT>
__device__ __forceinline__ void wave_gather_range_nt(const SrcView<TIn>& s, const CsrArgs& a, int32_t e_begin,
                                                     int32_t e_end, int c0, bool col_ok, int g, int groups,
                                                     float (&acc)[VEC]) {
  constexpr int kFly = 4;  // row loads in flight per lane, all of them at once (no branches below)
  const int lane = threadIdx.x & (kWave - 1);
  const TIn* zero_row = reinterpret_cast<const TIn*>(g_csr_zero_row);
  const int64_t zero_at = PARTS ? 0 : zero_row - s.rows;  // the row of zeros as an offset from the input
  bool beyond = false;
  for (int32_t cb = e_begin; cb < e_end; cb += kWave) {
    const int n_here = min(kWave, e_end - cb);
    // the row this lane's entry reads (none: -1 / NULL). With parts, where it lies is worked out once
    // per entry, here, not by every lane that gathers it, and the address travels to those lanes.
    int32_t s_mine = -1;
    const TIn* p_mine = nullptr;
    float w_mine = 0.f;
    if (lane < n_here) {
      const int32_t sv = s.src[cb + lane];
      if (sv >= s.lo && sv < s.hi) {
        s_mine = sv;
        if constexpr (PARTS) p_mine = src_row<TIn, true>(s.rows, a, sv);
        w_mine = s.coef ? load_coef(s.coef, s.coef_dt, cb + lane) : 1.0f;
      } else {
        beyond = beyond | (static_cast<int64_t>(sv) >= s.n_rows);
      }
    }
    for (int q0 = 0; q0 < n_here; q0 += kFly * groups) {  // same trip count for the whole wave (shuffles inside)
      float v[kFly][VEC];
      float w[kFly];
#pragma unroll
      for (int k = 0; k < kFly; ++k) {  // no branches in here: see g_csr_zero_row
        const int first = q0 + k * groups;  // this round's entries: first + 0 .. first + groups - 1, one per group
        const int e = first + g;
        const int from = min(e, kWave - 1);
        const bool in_round = (e < n_here) & col_ok;
        const float w_got = s.coef ? __shfl(w_mine, from, kWave) : 1.0f;  // every lane takes part in the shuffle
        const TIn* row;
        if constexpr (PARTS) {
          const uintptr_t bits = reinterpret_cast<uintptr_t>(p_mine);
          const uint32_t p_lo = __shfl(static_cast<uint32_t>(bits), from, kWave);
          const uint32_t p_hi = __shfl(static_cast<uint32_t>(bits >> 32), from, kWave);
          const uintptr_t got = (static_cast<uintptr_t>(p_hi) << 32) | p_lo;
          const bool have = in_round & (got != 0);
          row = have ? reinterpret_cast<const TIn*>(got) + c0 : zero_row;
          w[k] = have ? w_got : 0.f;
        } else {
          const int32_t id = __shfl(s_mine, from, kWave);
          const bool have = in_round & (id >= 0);
          row = s.rows + (have ? static_cast<int64_t>(id) * a.D + c0 : zero_at);
          w[k] = have ? w_got : 0.f;
        }
        if constexpr (NT) {
          load_pack_stream<TIn, VEC>(row, v[k]);
        } else {
          load_pack<TIn, VEC>(row, v[k]);
        }
      }
#pragma unroll
      for (int k = 0; k < kFly; ++k) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = fmaf(v[k][j], w[k], acc[j]);
      }
    }
  }
  if (beyond) raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
}
template <typename TIn, int VEC, bool PARTS>
__device__ __forceinline__ void wave_gather_range(const SrcView<TIn>& s, const CsrArgs& a, int32_t e_begin,
                                                  int32_t e_end, int c0, bool col_ok, int g, int groups,
                                                  float (&acc)[VEC]) {
  if (s.nt) {  // uniform; picked here, outside the loops
    wave_gather_range_nt<TIn, VEC, PARTS, true>(s, a, e_begin, e_end, c0, col_ok, g, groups, acc);
  } else {
    wave_gather_range_nt<TIn, VEC, PARTS, false>(s, a, e_begin, e_end, c0, col_ok, g, groups, acc);
  }
}

// Workgroups of kBlock threads that a row kernel which strides over its rows launches on the current
// device: 32 per compute unit (four times what a unit holds at once, so that the workgroups that finish
// early leave their place to others; 4 - 96 were measured), RECIS_COLD_GRID_PER_CU to try another number.
inline int64_t cold_grid_blocks() {
  static const int64_t n = [] {
    int cus = 256;
    (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, current_device());
    const char* s = std::getenv("RECIS_COLD_GRID_PER_CU");
    const int per = s != nullptr && *s ? std::atoi(s) : 32;
    return static_cast<int64_t>(cus) * std::max(1, per);
  }();
  return n;
}

constexpr int kCoopLen = 8;  // longer lists are shared among the lane groups of a wave

// One launch for all rows. The last cold_blocks workgroups: one group of LPR lanes per unique row
// with at most hot_len occurrences ("cold"); a wave that holds a row with more than kCoopLen
// occurrences works that row with all its lane groups striding over the list (a row of 200
// occurrences would otherwise be 50 dependent gathers of one group). The first workgroups
// walk the hot work items (row, chunk of kHotChunk occurrences): four waves share the chunk,
// fold their sums through LDS and store ONE partial row per item; csr_hot_finish_kernel adds up
// the partial rows of every hot row in chunk order. No atomics anywhere.
// SHUFFLE: long lists go through wave_gather_range (pays off when a wave has at most eight lane
// groups, i.e. rows of 128 bytes and more); otherwise every group loads its own entries.
// TIn2 != void: every list entry adds a row of a second input as well (see CsrArgs); PARTS then
// says that the second input comes in parts.
template <typename TIn, typename TOut, int VEC, bool SHUFFLE, bool PARTS = false, int EPI = kEpiStore,
          typename TIn2 = void>
// Register budgets of the variants that end in a row update, found by measurement: 64 registers (8
// waves per SIMD) for the one-input kernels, also for those that hand list entries round by
// shuffle (config 3: 187 us with no bound and 92 registers, 178 at 80, 170 at 72; with four
// branch-free gathers in flight the kernel needs 65, and 64 with 44 bytes spilled reads 161 us
// against 168 at 72); no bound for those with two inputs (a bound of 80 registers spills 24-60
// bytes and costs 20 us in config 5).
__global__ void __launch_bounds__(kBlock, (!SHUFFLE && EPI != kEpiStore && (std::is_void<TIn2>::value || sizeof(TOut) == 4))
                                              ? 8 : (SHUFFLE && EPI != kEpiStore && std::is_void<TIn2>::value) ? 8 : 1)
csr_rows_kernel(const TIn* __restrict__ rows, TOut* __restrict__ out, CsrArgs a, FuseArgs f) {
  constexpr bool TWO = !std::is_void<TIn2>::value;
  using TSecond = typename std::conditional<TWO, TIn2, TIn>::type;
  extern __shared__ float s_part[];  // [waves][D], hot part only
  const int D = a.D;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int lane = threadIdx.x & (kWave - 1);
  const int groups = kWave >> a.lpr_log2;  // lane groups of a wave
  const int g = lane >> a.lpr_log2;        // this lane's group in its wave
  // The grid is sized for the caller's bound on the number of unique rows (the host need not know the
  // count): a cold workgroup past the plan's own count leaves at once, before anything else is asked
  // for (two thirds of the workgroups of a typical batch; measured with the exact count as the
  // bound: 12 - 15 us of the update kernel were theirs).
  // Likewise a workgroup of the hot part that no work item is left for (block 0 stays: it leaves
  // alpha behind for the finish kernel).
  {
    const int64_t first_cold = static_cast<int64_t>(gridDim.x) - a.cold_blocks;
    const int64_t b = static_cast<int64_t>(blockIdx.x);
    if (b >= first_cold ? (b - first_cold) * (kBlock >> a.lpr_log2) >= min(a.U, a.counts[0])
                        : (b > 0 && b >= min(a.counts[1], a.hot_cap)))
      return;
  }
  __shared__ double s_alpha;  // Adam: alpha of this step, worked out once per workgroup
  if constexpr (epi_is_adam(EPI)) {
    if (threadIdx.x == 0) {
      double b1, b2;
      s_alpha = f.adam.alpha != nullptr ? f.adam.alpha[0] : alpha_from_powers(f, b1, b2);
      if (f.adam.alpha == nullptr && blockIdx.x == 0) f.alpha_ws[0] = s_alpha;  // for the finish kernel
    }
    __syncthreads();
  }
  SrcView<TIn> in1{rows, a.src, a.coef, a.coef_dt, a.nt_in, a.n_rows, 0, 0};
  cover_range(a, in1.lo, in1.hi);
  const SrcView<TSecond> in2{static_cast<const TSecond*>(a.rows2), a.src2, a.coef2, a.coef2_dt, a.nt_in2,
                             a.n_rows2, 0, a.n_rows2};

  auto fetch = [&](const auto& in, auto parts, int32_t k, int c0, float (&v)[VEC], float& w) {
    using T = typename std::remove_cv<typename std::remove_pointer<decltype(in.rows)>::type>::type;
    const int32_t s = in.src[k];
    w = in.coef ? load_coef(in.coef, in.coef_dt, k) : 1.0f;
    if (s < in.lo || s >= in.hi) {
      if (static_cast<int64_t>(s) >= in.n_rows) raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = 0.f;
      w = 0.f;
      return;
    }
    const T* row = src_row<T, decltype(parts)::value>(in.rows, a, s);
    if (in.nt) {
      load_pack_stream<T, VEC>(row + c0, v);
    } else {
      load_pack<T, VEC>(row + c0, v);
    }
  };
  // acc += sum over list entries k = first, first + step, ... < last of one input (4 gathers in flight)
  // (short lists, a lane group each: the entries are taken as they come, with a branch for the
  // ones that add nothing; making these loads branch-free like those of wave_gather_range was
  // measured and lost, 167 -> 199 us in config 3, where most lists hold one entry)
  auto gather_one = [&](const auto& in, auto parts, int32_t first, int32_t last, int32_t step, int c0,
                        float (&acc)[VEC]) {
    int32_t k = first;
    for (; k + 3 * step < last; k += 4 * step) {
      float v0[VEC], v1[VEC], v2[VEC], v3[VEC];
      float w0, w1, w2, w3;
      fetch(in, parts, k, c0, v0, w0);
      fetch(in, parts, k + step, c0, v1, w1);
      fetch(in, parts, k + 2 * step, c0, v2, w2);
      fetch(in, parts, k + 3 * step, c0, v3, w3);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        acc[j] = fmaf(v0[j], w0, acc[j]);
        acc[j] = fmaf(v1[j], w1, acc[j]);
        acc[j] = fmaf(v2[j], w2, acc[j]);
        acc[j] = fmaf(v3[j], w3, acc[j]);
      }
    }
    for (; k < last; k += step) {
      float v0[VEC];
      float w0;
      fetch(in, parts, k, c0, v0, w0);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = fmaf(v0[j], w0, acc[j]);
    }
  };
  // the first input's entries, then the second's: one fixed order of summation
  auto gather_sum = [&](int32_t first, int32_t last, int32_t step, int c0, float (&acc)[VEC]) {
    gather_one(in1, std::integral_constant<bool, PARTS && !TWO>{}, first, last, step, c0, acc);
    if constexpr (TWO) gather_one(in2, std::integral_constant<bool, PARTS>{}, first, last, step, c0, acc);
  };
  // the wave's sum over the list entries [first, last) for columns c0.., the same in every group
  auto wave_sum = [&](int32_t first, int32_t last, int c0, bool col_ok, float (&acc)[VEC]) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
    if constexpr (SHUFFLE) {
      wave_gather_range<TIn, VEC, PARTS && !TWO>(in1, a, first, last, c0, col_ok, g, groups, acc);
      if constexpr (TWO) wave_gather_range<TSecond, VEC, PARTS>(in2, a, first, last, c0, col_ok, g, groups, acc);
    } else {
      if (col_ok) gather_sum(first + g, last, groups, c0, acc);
    }
    for (int off = 1 << a.lpr_log2; off < kWave; off <<= 1) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += __shfl_xor(acc[j], off, kWave);
    }
  };

  const int64_t hot_blocks = static_cast<int64_t>(gridDim.x) - a.cold_blocks;
  if (static_cast<int64_t>(blockIdx.x) < hot_blocks) {
    // ---- hot work items (the first workgroups: the longest-running ones start first)
    int64_t n_items = a.counts[1];
    if (n_items > a.hot_cap) n_items = a.hot_cap;
    const int wave = threadIdx.x / kWave;
    constexpr int n_waves = kBlock / kWave;
    for (int64_t item = blockIdx.x; item < n_items; item += hot_blocks) {
      const int32_t u = a.hot_items[2 * item];
      const int32_t chunk = a.hot_items[2 * item + 1];
      const int32_t start = a.row_start[u] + chunk * kHotChunk;
      const int32_t end = min(a.row_start[u + 1], start + kHotChunk);
      const int32_t per_wave = (end - start + n_waves - 1) / n_waves;  // a contiguous share per wave
      const int32_t w_begin = min(end, start + wave * per_wave), w_end = min(end, w_begin + per_wave);
      for (int cbase = 0; cbase < D; cbase += VEC << a.lpr_log2) {  // uniform: shuffles inside
        const int c0 = cbase + cl * VEC;
        const bool col_ok = c0 < D;
        float acc[VEC];
        wave_sum(w_begin, w_end, c0, col_ok, acc);
        if (g == 0 && col_ok) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) s_part[wave * D + c0 + j] = acc[j];
        }
      }
      __syncthreads();
      for (int d = threadIdx.x; d < D; d += kBlock) {
        float sum = 0.f;
        for (int w = 0; w < n_waves; ++w) sum += s_part[w * D + d];
        a.hot_part[item * D + d] = sum;
      }
      __syncthreads();
    }
    return;
  }

  // ---- cold rows
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t u = (static_cast<int64_t>(blockIdx.x) - hot_blocks) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  // a.U may be an upper bound (a caller that has not read the plan's count back passes the number of
  // ids): rows at and past the count the plan left on the device have no list
  const bool valid = u < a.U && u < a.counts[0];
  const int32_t start = valid ? a.row_start[u] : 0;
  int32_t end = valid ? a.row_start[u + 1] : 0;
  const bool hot = end - start > a.hot_len;  // left to the work items and the finish kernel
  if (hot) end = start;
  // The table row of this group's unique id is asked for before the gathers; the kernel with
  // registers to spare (one input, no shuffles) also asks where that row lies in the blocks, so
  // that the block-table reads run under the gathers instead of heading the row update (config 4:
  // 146 -> 136 us; the other kernels spill with six registers more and lose 10 %).
  constexpr bool kEarlyPlaces = EPI != kEpiStore && !SHUFFLE && !TWO;
  using TRow = typename std::conditional<EPI != kEpiStore, TOut, float>::type;
  RowPlaces<TRow> places{nullptr, nullptr, nullptr};
  int64_t idx_mine = -1;
  if constexpr (EPI != kEpiStore) {
    if (valid) idx_mine = f.row_index[u];  // (under the same test as the list bounds: the three loads go out together)
    if constexpr (kEarlyPlaces) places = row_places<TRow, EPI>(f, a.err, idx_mine);
  }
  // the finished sum of this lane group's own row u
  auto finish = [&](int64_t row, int c0, float (&acc)[VEC]) {
    if constexpr (EPI != kEpiStore) {
      if constexpr (kEarlyPlaces)
        fused_row_update_at<TRow, VEC, EPI>(f, places, c0, acc, epi_is_adam(EPI) ? s_alpha : 0.0);
      else
        fused_row_update<TOut, VEC, EPI>(f, a.err, idx_mine, c0, acc, epi_is_adam(EPI) ? s_alpha : 0.0);
    } else {
      TOut* dst = out + (a.out_rows ? static_cast<int64_t>(a.out_rows[row]) : row) * D + c0;
      if (a.accumulate) {
        float old[VEC];
        load_pack<TOut, VEC>(dst, old);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += old[j];
      }
      store_pack<TOut, VEC>(dst, acc);
    }
  };
  // short rows: every lane group works its own row
  const bool is_long = a.lpr_log2 < 6 && end - start > kCoopLen;  // with one group per wave there is nobody to share with
  if (valid && !is_long && !hot) {
    // (Asking for the row's parameter and state packs before the gradient is gathered, to run their
    // latency under that of the gathers, was measured and lost: 150 -> 205 us in config 4. The packs
    // cost registers, hence resident waves, and the gathers then queue behind the table reads.)
    for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
      float acc[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
      gather_sum(start, end, 1, c0, acc);
      finish(u, c0, acc);
    }
  }
  // long rows of this wave, one after the other, summed by all its lane groups; the owning group
  // keeps the sum and every group finishes its row afterwards, all at once (a finish that updates
  // the table row is a chain of dependent accesses: one per row in a row would leave the wave
  // waiting on it with three quarters of its lanes idle). A wave with several groups has lanes for
  // all of D (lpr_log2 < 6), so a long row is one pack per lane.
  uint64_t todo = __ballot(is_long);
  if (todo == 0) return;
  const int c0 = cl * VEC;
  const bool col_ok = c0 < D;
  float keep[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) keep[j] = 0.f;
  while (todo) {
    const int owner = __ffsll(static_cast<unsigned long long>(todo)) - 1;  // first lane of the owning group
    todo &= ~(((uint64_t(1) << (1 << a.lpr_log2)) - 1) << owner);  // the group's lanes (fewer than 64 here)
    const int r = owner >> a.lpr_log2;
    const int32_t r_start = __shfl(start, owner, kWave), r_end = __shfl(end, owner, kWave);
    float acc[VEC];
    wave_sum(r_start, r_end, c0, col_ok, acc);
    if (g == r) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) keep[j] = acc[j];
    }
  }
  if (is_long && col_ok) finish(u, c0, keep);
}

// out[u] (+)= sum of the partial rows of hot row u (or the optimizer's update of the row with that
// sum). One wave per work item with chunk 0 (the items of a row are consecutive): its lane groups
// share the row's partials out among themselves (an id that makes up a tenth of the batch has a
// hundred of them) and fold their sums with shuffles, always in the same order.
template <typename TOut, int VEC, int EPI = kEpiStore>
__global__ void __launch_bounds__(kBlock)
csr_hot_finish_kernel(TOut* __restrict__ out, CsrArgs a, FuseArgs f) {
  double alpha = 0;
  if constexpr (epi_is_adam(EPI)) {
    alpha = f.adam.alpha[0];
    if (f.advance_powers && blockIdx.x == 0 && threadIdx.x == 0) {  // nobody reads them in this kernel
      double b1, b2;
      alpha_from_powers(f, b1, b2);
      if (f.beta_is_f64) {
        static_cast<double*>(f.beta1_t)[0] = b1;
        static_cast<double*>(f.beta2_t)[0] = b2;
      } else {
        static_cast<float*>(f.beta1_t)[0] = static_cast<float>(b1);
        static_cast<float*>(f.beta2_t)[0] = static_cast<float>(b2);
      }
    }
  }
  int64_t n_items = a.counts[1];
  if (n_items > a.hot_cap) n_items = a.hot_cap;
  const int D = a.D;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int lane = threadIdx.x & (kWave - 1);
  const int groups = kWave >> a.lpr_log2, g = lane >> a.lpr_log2;
  const int64_t waves_total = static_cast<int64_t>(gridDim.x) * (kBlock / kWave);
  for (int64_t item = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave; item < n_items;
       item += waves_total) {  // uniform in the wave
    if (a.hot_items[2 * item + 1] != 0) continue;
    const int32_t u = a.hot_items[2 * item];
    const int32_t len = a.row_start[u + 1] - a.row_start[u];
    int64_t n_chunks = (len + kHotChunk - 1) / kHotChunk;
    if (item + n_chunks > n_items) n_chunks = n_items - item;  // items cut off by hot_cap (cannot happen with the documented hot_cap)
    for (int cbase = 0; cbase < D; cbase += VEC << a.lpr_log2) {  // uniform: shuffles inside
      const int c0 = cbase + cl * VEC;
      const bool col_ok = c0 < D;
      float acc[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
      if (col_ok) {
        for (int64_t k = g; k < n_chunks; k += groups) {
          float v[VEC];
          load_pack<float, VEC>(a.hot_part + (item + k) * D + c0, v);
#pragma unroll
          for (int j = 0; j < VEC; ++j) acc[j] += v[j];
        }
      }
      for (int off = 1 << a.lpr_log2; off < kWave; off <<= 1) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += __shfl_xor(acc[j], off, kWave);
      }
      if (g != 0 || !col_ok) continue;
      if constexpr (EPI != kEpiStore) {
        fused_row_update<TOut, VEC, EPI>(f, a.err, f.row_index[u], c0, acc, alpha);
      } else {
        TOut* dst = out + static_cast<int64_t>(a.out_rows ? a.out_rows[u] : u) * D + c0;
        if (a.accumulate) {
          float old[VEC];
          load_pack<TOut, VEC>(dst, old);
#pragma unroll
          for (int j = 0; j < VEC; ++j) acc[j] += old[j];
        }
        store_pack<TOut, VEC>(dst, acc);
      }
    }
  }
}

// ------------------------------------------------------------------ expand (transpose of the gather-reduce)
// out[dst[k], :] = w[dst[k]] * row(u) for every list entry k of every unique id u: the forward
// of pooling when every segment holds exactly one id, and of the unpooled (tile) output. Each
// unique row is read ONCE and stored to all its occurrences; stores do not wait for anything,

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

// ------------------------------------------------------------------ host side
// One input of a gather-reduce as the caller describes it.
struct CsrInput {
  const void* rows;
  int dtype;
  int64_t n_rows;
  const int32_t* src;
  const void* coef;  // or NULL
  int coef_dtype;
  // the second of two inputs may come as n_parts arrays laid end to end (rows == NULL then)
  const void* const* part_rows = nullptr;
  const int64_t* part_counts = nullptr;
  int n_parts = 0;
};

struct CsrRequest {
  CsrInput in1;
  const CsrInput* in2 = nullptr;                // the second input, with csr_gather_reduce_run<true>
  const void* const* part_rows = nullptr;       // in1 as n_parts arrays laid end to end (in1.rows is NULL then)
  const int64_t* part_counts = nullptr;
  int n_parts = 0;
  const int32_t* row_start = nullptr;
  const int32_t* hot_items = nullptr;
  int64_t hot_cap = 0;
  const int64_t* counts_dev = nullptr;
  void* out = nullptr;                          // NULL when epi != kEpiStore
  int out_dtype = RECIS_F32;                    // the table's row type when epi != kEpiStore
  int64_t U = 0, D = 0;
  int accumulate = 0;
  const int32_t* out_rows = nullptr;            // kEpiStore only: where the sum of row u goes (see CsrArgs)
  const void* cover = nullptr;
  int cover64 = 0;
  int64_t cover_S = 0;
  hipStream_t stream = nullptr;
  int epi = kEpiStore;
  const FuseArgs* fuse = nullptr;               // where the table rows are, when epi != kEpiStore
  size_t extra_ws = 0;                          // bytes of the stream's workspace (after the partial rows of the
  void** extra_out = nullptr;                   // hot items) handed to the caller before anything is launched
};

// Checks, geometry, workspace and the launches of one gather-reduce. TWO picks the family of
// kernels this translation unit instantiates: one input (any supported pair of input and output
// types, PARTS included) or two inputs (each fp32 or the half type of the other / of the table).
// ONLY_EPI >= 0: only the kernels with that ending are instantiated here (the others are refused),
// so that the families can be compiled side by side.
template <bool TWO, int ONLY_EPI = -1>
int csr_gather_reduce_run(const CsrRequest& r) {
  const int64_t U = r.U, D = r.D, hot_cap = r.hot_cap;
  const int epi = r.epi, n_parts = r.n_parts;
  hipStream_t stream = r.stream;
  RECIS_REQUIRE(U >= 0 && r.in1.n_rows >= 0, "negative size");
  RECIS_REQUIRE(D >= 1 && D <= 8192, "embedding dim %lld out of range", (long long)D);
  RECIS_REQUIRE(U == 0 || (r.in1.src && r.row_start && (r.out || epi != kEpiStore) && r.counts_dev), "NULL argument");
  RECIS_REQUIRE(n_parts > 0 || r.in1.rows != nullptr || r.in1.n_rows == 0, "rows must not be NULL");
  RECIS_REQUIRE(hot_cap == 0 || r.hot_items, "hot_items must not be NULL");
  const int in_sz = dtype_size(r.in1.dtype), out_sz = dtype_size(r.out_dtype);
  RECIS_REQUIRE(in_sz && out_sz, "invalid dtype");
  RECIS_REQUIRE(r.in1.coef == nullptr || dtype_size(r.in1.coef_dtype), "invalid coef dtype");
  uintptr_t align_of = reinterpret_cast<uintptr_t>(r.in1.rows);
  for (int f = 0; f < n_parts; ++f) align_of |= reinterpret_cast<uintptr_t>(r.part_rows[f]);  // the coarsest alignment
  // with two inputs an fp32 one may go in 32-byte packs, so that a half-precision partner (or
  // table row) still gets its 16 bytes per lane
  const int vb_in = (TWO && in_sz == 4) ? pick_vec_bytes_max(D * in_sz, align_of, 32) : pick_vec_bytes(D * in_sz, align_of);
  // table blocks are allocator-aligned and are read and written in 16-byte packs at most
  const int vb_out = epi != kEpiStore ? pick_vec_bytes(D * out_sz, 16)
                                      : pick_vec_bytes_max(D * out_sz, reinterpret_cast<uintptr_t>(r.out), 32);
  int vec = std::max(1, std::min(vb_in / in_sz, vb_out / out_sz));
  CsrArgs a{};
  if constexpr (TWO) {
    RECIS_REQUIRE(r.in2 != nullptr && n_parts == 0, "two inputs: the second must be given, the first one array");
    const CsrInput& b = *r.in2;
    const int in2_sz = dtype_size(b.dtype);
    RECIS_REQUIRE(in2_sz, "invalid dtype of the second input");
    RECIS_REQUIRE(b.n_parts >= 0 && b.n_parts <= kMaxParts, "second input: at most %d parts (got %d)", kMaxParts,
                  b.n_parts);
    int64_t n_rows2 = b.n_rows;
    uintptr_t align2 = reinterpret_cast<uintptr_t>(b.rows);
    if (b.n_parts > 0) {
      RECIS_REQUIRE(b.part_rows && b.part_counts, "second input: NULL part tables");
      n_rows2 = 0;
      align2 = 0;
      for (int f = 0; f < b.n_parts; ++f) {
        RECIS_REQUIRE(b.part_counts[f] >= 0 && (b.part_rows[f] != nullptr || b.part_counts[f] == 0),
                      "second input: bad part %d", f);
        n_rows2 += b.part_counts[f];
        align2 |= reinterpret_cast<uintptr_t>(b.part_rows[f]);
      }
    }
    RECIS_REQUIRE(n_rows2 >= 0 && (U == 0 || b.src), "second input: src must not be NULL");
    RECIS_REQUIRE(b.n_parts > 0 || b.rows != nullptr || n_rows2 == 0, "second input: rows must not be NULL");
    RECIS_REQUIRE(b.coef == nullptr || dtype_size(b.coef_dtype), "invalid coef dtype of the second input");
    const int vb2 = in2_sz == 4 ? pick_vec_bytes_max(D * in2_sz, align2, 32) : pick_vec_bytes(D * in2_sz, align2);
    const int widest = 16 / std::min(std::min(in_sz, in2_sz), out_sz);  // 16 bytes of the narrowest type
    vec = std::max(1, std::min(std::min(vec, widest), vb2 / in2_sz));
    a.rows2 = b.rows;
    a.src2 = b.src;
    a.coef2 = b.coef;
    a.coef2_dt = b.coef_dtype;
    a.n_rows2 = n_rows2;
    a.nt_in2 = n_rows2 * D * in2_sz >= (int64_t(1) << 30);
  }
  a.row_start = r.row_start;
  a.src = r.in1.src;
  a.coef = r.in1.coef;
  a.coef_dt = r.in1.coef_dtype;
  a.U = U;
  a.n_rows = r.in1.n_rows;
  a.cover = r.cover;
  a.cover64 = r.cover64;
  a.cover_S = r.cover_S;
  a.D = static_cast<int>(D);
  a.lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  a.accumulate = r.accumulate;
  a.out_rows = r.out_rows;
  a.nt_in = r.in1.n_rows * D * in_sz >= (int64_t(1) << 30);
  a.err = device_error_word(current_device());
  RECIS_REQUIRE(a.err != nullptr, "could not reach the device error word");
  const int rows_per_block = kBlock >> a.lpr_log2;
  a.cold_blocks = (U + rows_per_block - 1) / rows_per_block;
  a.hot_len = hot_cap > 0 ? kHotLen : INT_MAX;
  a.hot_items = r.hot_items;
  a.counts = r.counts_dev;
  a.hot_cap = hot_cap;
  a.hot_part = nullptr;
  // the part table: of the one input, or of the second of two; the kernels find a row's part by
  // comparing with the parts' first rows, so an unused part starts past every row
  const void* const* parts_of = TWO ? r.in2->part_rows : r.part_rows;
  const int64_t* counts_of = TWO ? r.in2->part_counts : r.part_counts;
  a.n_parts = TWO ? r.in2->n_parts : n_parts;
  int64_t part_first = 0;
  for (int f = 0; f < kMaxParts; ++f) {
    a.part_rows[f] = f < a.n_parts ? parts_of[f] : nullptr;
    a.part_lo32[f] = f < a.n_parts ? static_cast<int32_t>(part_first) : INT32_MAX;
    if (f < a.n_parts) part_first += counts_of[f];
  }
  RECIS_REQUIRE(part_first <= INT32_MAX, "the parts hold %lld rows, more than 32-bit src entries name",
                (long long)part_first);
  int64_t hot_blocks = 0;
  if (hot_cap > 0 || r.extra_ws > 0) {
    void* ws = nullptr;
    const size_t hot_bytes = (sizeof(float) * static_cast<size_t>(hot_cap) * static_cast<size_t>(D) + 255) & ~size_t(255);
    if (int rc = get_workspace(stream, hot_bytes + r.extra_ws, &ws)) return rc;
    a.hot_part = static_cast<float*>(ws);
    if (r.extra_out) *r.extra_out = static_cast<char*>(ws) + hot_bytes;
    if (hot_cap > 0) hot_blocks = std::min<int64_t>(hot_cap, 4096);
  }
  if (U == 0) return RECIS_OK;
  const FuseArgs f = r.fuse ? *r.fuse : FuseArgs{};
  const size_t lds = sizeof(float) * (kBlock / kWave) * static_cast<size_t>(D);
  auto with_types = [&](auto tin, auto tout, auto tin2) {
    using TIn = decltype(tin);
    using TOut = decltype(tout);
    using TIn2 = typename std::conditional<TWO, decltype(tin2), void>::type;
    constexpr size_t in2_bytes = TWO ? sizeof(decltype(tin2)) : 1;
    return dispatch_vec(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(TIn) > (TWO ? 32 : 16) || VEC * in2_bytes > 32 || VEC * sizeof(TOut) > 32) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        const TIn* rin = static_cast<const TIn*>(r.in1.rows);
        TOut* o = static_cast<TOut*>(r.out);
        const bool shuffle = a.lpr_log2 >= 3;  // at most eight lane groups per wave
        const dim3 grid(a.cold_blocks + hot_blocks), block(kBlock);
        const int64_t fin = std::min<int64_t>((hot_cap + kBlock / kWave - 1) / (kBlock / kWave), 2048);  // a wave per item
        auto launch = [&](auto epi_tag) {
          constexpr int EPI = decltype(epi_tag)::value;
          {
            RECIS_TIME_KERNEL(EPI == kEpiStore ? "csr_rows_kernel" : epi_is_adam(EPI) ? "csr_rows_adam_kernel"
                                                                                      : "csr_rows_adagrad_kernel", stream)
            if (a.n_parts > 0) {
              if constexpr (TWO) {  // the second input in parts
                if (shuffle)
                  csr_rows_kernel<TIn, TOut, VEC, true, true, EPI, TIn2><<<grid, block, lds, stream>>>(rin, o, a, f);
                else
                  csr_rows_kernel<TIn, TOut, VEC, false, true, EPI, TIn2><<<grid, block, lds, stream>>>(rin, o, a, f);
              } else if constexpr (sizeof(TOut) == 4 && EPI == kEpiStore) {  // parts go to fp32 rows only
                if (shuffle)
                  csr_rows_kernel<TIn, TOut, VEC, true, true><<<grid, block, lds, stream>>>(rin, o, a, f);
                else
                  csr_rows_kernel<TIn, TOut, VEC, false, true><<<grid, block, lds, stream>>>(rin, o, a, f);
              }
            } else if (shuffle) {
              csr_rows_kernel<TIn, TOut, VEC, true, false, EPI, TIn2><<<grid, block, lds, stream>>>(rin, o, a, f);
            } else {
              csr_rows_kernel<TIn, TOut, VEC, false, false, EPI, TIn2><<<grid, block, lds, stream>>>(rin, o, a, f);
            }
            RECIS_LAUNCH_CHECK();
          }
          if (hot_cap > 0) {
            FuseArgs f_fin = f;
            if (epi_is_adam(EPI) && f.adam.alpha == nullptr) {  // the row kernel worked alpha out itself
              f_fin.adam.alpha = f.alpha_ws;
              f_fin.advance_powers = 1;
            }
            csr_hot_finish_kernel<TOut, VEC, EPI><<<dim3(fin), block, 0, stream>>>(o, a, f_fin);
            RECIS_LAUNCH_CHECK();
          }
          return RECIS_OK;
        };
        constexpr bool all = ONLY_EPI < 0;
        if (epi == kEpiAdam) {
          if constexpr ((all || ONLY_EPI == kEpiAdam) && VEC * sizeof(TOut) <= 16) {
            if (stream_table_rows(f.rb, sizeof(TOut), 3)) return launch(std::integral_constant<int, kEpiAdam>{});
            return launch(std::integral_constant<int, kEpiAdamCached>{});
          }
        } else if (epi == kEpiAdagrad) {
          if constexpr ((all || ONLY_EPI == kEpiAdagrad) && VEC * sizeof(TOut) <= 16)
            return launch(std::integral_constant<int, kEpiAdagrad>{});
        } else {
          if constexpr (all || ONLY_EPI == kEpiStore) return launch(std::integral_constant<int, kEpiStore>{});
        }
        return fail(RECIS_ERR_ARG, "internal: no kernel for this ending and vector width here");
      }
    });
  };
  const int rows_dtype = r.in1.dtype, out_dtype = r.out_dtype;
  if constexpr (!TWO) {
    if (rows_dtype == RECIS_F32 && out_dtype == RECIS_F32) return with_types(float{}, float{}, 0);
    if (rows_dtype == RECIS_BF16 && out_dtype == RECIS_F32) return with_types(bf16_t{}, float{}, 0);
    if (rows_dtype == RECIS_F16 && out_dtype == RECIS_F32) return with_types(f16_t{}, float{}, 0);
    if (rows_dtype == RECIS_BF16 && out_dtype == RECIS_BF16) return with_types(bf16_t{}, bf16_t{}, 0);
    if (rows_dtype == RECIS_F16 && out_dtype == RECIS_F16) return with_types(f16_t{}, f16_t{}, 0);
    if (epi != kEpiStore) {  // fp32 gradients onto half-precision rows
      if (rows_dtype == RECIS_F32 && out_dtype == RECIS_BF16) return with_types(float{}, bf16_t{}, 0);
      if (rows_dtype == RECIS_F32 && out_dtype == RECIS_F16) return with_types(float{}, f16_t{}, 0);
    }
    return fail(RECIS_ERR_ARG, "unsupported dtype pair (rows=%d, out=%d)", rows_dtype, out_dtype);
  } else {
    // each input fp32 or a half type; two half inputs of one type; with a fused row update a
    // half input has the table's type
    const int d2 = r.in2->dtype;
    auto second = [&](auto tin, auto tout) {
      using TIn = decltype(tin);
      using TOut = decltype(tout);
      constexpr bool half_in = sizeof(TIn) == 2, half_out = sizeof(TOut) == 2;
      if (d2 == RECIS_F32) return with_types(tin, tout, float{});
      if constexpr (half_in) {
        if (d2 == rows_dtype) return with_types(tin, tout, tin);
      } else if constexpr (half_out) {
        if (d2 == out_dtype) return with_types(tin, tout, tout);
      } else {
        if (epi == kEpiStore) {
          if (d2 == RECIS_BF16) return with_types(tin, tout, bf16_t{});
          if (d2 == RECIS_F16) return with_types(tin, tout, f16_t{});
        }
      }
      return fail(RECIS_ERR_ARG, "unsupported dtypes (inputs=%d and %d, out=%d)", rows_dtype, d2, out_dtype);
    };
    if (out_dtype == RECIS_F32) {
      if (rows_dtype == RECIS_F32) return second(float{}, float{});
      if (epi == kEpiStore) {
        if (rows_dtype == RECIS_BF16) return second(bf16_t{}, float{});
        if (rows_dtype == RECIS_F16) return second(f16_t{}, float{});
      }
    } else if (epi != kEpiStore) {
      if (out_dtype == RECIS_BF16 && rows_dtype == RECIS_F32) return second(float{}, bf16_t{});
      if (out_dtype == RECIS_BF16 && rows_dtype == RECIS_BF16) return second(bf16_t{}, bf16_t{});
      if (out_dtype == RECIS_F16 && rows_dtype == RECIS_F32) return second(float{}, f16_t{});
      if (out_dtype == RECIS_F16 && rows_dtype == RECIS_F16) return second(f16_t{}, f16_t{});
    }
    return fail(RECIS_ERR_ARG, "unsupported dtypes (inputs=%d and %d, out=%d)", rows_dtype, d2, out_dtype);
  }
}

// Shared front of the fused entry points: argument checks and the table description.
inline int fill_fuse_args(FuseArgs& f, const int64_t* row_index, void* const* emb, void* const* s0, void* const* s1,
                          bool need_s1, int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes, int64_t D,
                          int row_dtype) {
  RECIS_REQUIRE(row_index && emb && s0 && (s1 || !need_s1), "row_index and the block tables must not be NULL");
  RECIS_REQUIRE(n_blocks >= 1 && block_size >= 1, "bad block geometry (n_blocks=%lld block_size=%lld)",
                (long long)n_blocks, (long long)block_size);
  RECIS_REQUIRE(dtype_size(row_dtype), "invalid row dtype");
  f = FuseArgs{};
  f.row_index = row_index;
  f.emb = emb;
  f.s0 = s0;
  f.s1 = s1;
  f.rb.n_blocks = n_blocks;
  f.rb.block_size = block_size;
  f.rb.D = static_cast<int>(D);
  // block bases and the pitch are required to be aligned like the row width allows
  f.rb.pitch = pitch_elements(row_pitch_bytes, D, dtype_size(row_dtype), pick_vec_bytes(D * dtype_size(row_dtype), 16));
  RECIS_REQUIRE(f.rb.pitch >= D, "row pitch of %lld bytes does not fit rows of %lld elements", (long long)row_pitch_bytes,
                (long long)D);
  return RECIS_OK;
}


// The Adam-family variant of a request (r.epi == kEpiAdam, r.fuse == &f). alpha lives in the stream's
// workspace behind the partial rows of the hot items, so a first pass with U = 0 reserves the
// workspace and learns where alpha goes, launching nothing. With hot work items (every batch plan
// brings them) the kernels work alpha out and advance the running powers themselves (see
// FuseArgs); otherwise, and when no row is touched (the powers advance all the same), cal_alpha
// runs in front as in recis_block_apply_adamw.
template <bool TWO, int ONLY_EPI = -1>
int run_with_alpha(CsrRequest& r, FuseArgs& f, void* beta1_t, void* beta2_t, int beta_is_f64, double lr,
                   double beta1, double beta2, double weight_decay, double eps) {
  void* alpha = nullptr;
  CsrRequest probe = r;
  probe.U = 0;
  probe.extra_ws = 256;
  probe.extra_out = &alpha;
  if (int rc = csr_gather_reduce_run<TWO, ONLY_EPI>(probe)) return rc;
  const bool in_kernel = r.U > 0 && r.hot_cap > 0;
  if (!in_kernel) {
    if (int rc = launch_cal_alpha(beta1_t, beta2_t, beta_is_f64, static_cast<double*>(alpha), lr, beta1, beta2, r.stream))
      return rc;
    if (r.U == 0) return RECIS_OK;
  }
  f.adam.alpha = in_kernel ? nullptr : static_cast<const double*>(alpha);
  f.adam.beta1 = beta1;
  f.adam.beta2 = beta2;
  f.adam.decay = weight_decay;
  f.adam.eps = eps;
  f.beta1_t = beta1_t;
  f.beta2_t = beta2_t;
  f.beta_is_f64 = beta_is_f64;
  f.advance_powers = 0;
  f.adam_lr = lr;
  f.alpha_ws = static_cast<double*>(alpha);
  r.extra_ws = 256;
  r.extra_out = &alpha;
  return csr_gather_reduce_run<TWO, ONLY_EPI>(r);
}

// The request of an entry point with two inputs; `second` must outlive the request.
inline CsrRequest two_input_request(const recis_csr_input* a, const recis_csr_input* b, CsrInput& second,
                             const int32_t* row_start, const int32_t* hot_items, int64_t hot_cap,
                             const int64_t* counts_dev, int64_t U, int64_t D, void* stream_) {
  CsrRequest r;
  r.in1 = CsrInput{a->rows, a->rows_dtype, a->n_rows, a->src, a->coef, a->coef_dtype};
  second = CsrInput{b->rows, b->rows_dtype, b->n_rows, b->src, b->coef, b->coef_dtype};
  second.part_rows = b->part_rows;
  second.part_counts = b->part_counts;
  second.n_parts = b->n_parts;
  r.in2 = &second;
  r.row_start = row_start;
  r.hot_items = hot_items;
  r.hot_cap = hot_cap;
  r.counts_dev = counts_dev;
  r.U = U;
  r.D = D;
  r.stream = static_cast<hipStream_t>(stream_);
  return r;
}


}  // namespace
}  // namespace recis_hip
