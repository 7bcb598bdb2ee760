// The per-row arithmetic of the sparse optimizers, shared by the stand-alone row kernels
// (optim.hip) and the gather-reduce kernels that apply the update as soon as a row's gradient is
// summed (plan.hip).
//
// Adam family: what block_apply_adamw does per element (csrc/ops/block_apply_adamw_op.cc:32-58):
// products and sums in double, sqrtf in float, every assignment rounded to the storage type, no
// fused multiply-add. The kernels are bound by memory traffic, so the arithmetic is free, and
// doing it this way reproduces the reference's CPU path bit for bit.
// Adagrad has no reference counterpart; it is the textbook update in float.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "common.cuh"

namespace recis_hip {

// Where the rows of the table live and which of them a launch touches.
struct RowBlocks {
  int64_t n_blocks;
  int64_t block_size;
  int D;
  int64_t pitch;  // elements from one row of a block to the next (D when rows lie back to back)
};

// The row pitch in elements of a row_pitch_bytes argument (0 = rows lie back to back); negative
// when the pitch does not fit rows of D elements of elem_size bytes moved vec_bytes at a time.
inline int64_t pitch_elements(int64_t row_pitch_bytes, int64_t D, int elem_size, int vec_bytes) {
  if (row_pitch_bytes == 0) return D;
  if (row_pitch_bytes < D * elem_size || row_pitch_bytes % elem_size || row_pitch_bytes % vec_bytes) return -1;
  return row_pitch_bytes / elem_size;
}

// Block and row-in-block of table row idx; false when idx is negative or beyond the blocks.
__device__ __forceinline__ bool block_row(const RowBlocks& r, int64_t idx, int64_t& b, int64_t& off) {
  if (idx < 0) return false;
  if (r.n_blocks == 1) {
    b = 0;
    off = idx;
    return idx < r.block_size;
  }
  if ((static_cast<uint64_t>(idx) | static_cast<uint64_t>(r.block_size)) >> 32) {
    b = idx / r.block_size;
    off = idx - b * r.block_size;
  } else {
    const uint32_t bs = static_cast<uint32_t>(r.block_size);
    const uint32_t q = static_cast<uint32_t>(idx) / bs;
    b = q;
    off = static_cast<uint32_t>(idx) - q * bs;
  }
  return b < r.n_blocks;
}

// Whether a row update should touch the table rows with the streaming (non-temporal) hint: yes
// when the `slots` arrays it works on (parameter and state) are together larger than what the
// caches keep from one step to the next (the 256 MB of memory-side cache; RECIS_STREAM_ROWS_MIN_MB
// in the environment moves the line, 0 = always stream), no for a small table, whose rows the
// next step would otherwise have to fetch from memory again.
inline bool stream_table_rows(const RowBlocks& rb, size_t elem_size, int slots) {
  static const int64_t min_bytes = [] {
    const char* s = std::getenv("RECIS_STREAM_ROWS_MIN_MB");
    return (s != nullptr && *s ? std::atoll(s) : 256) << 20;
  }();
  return rb.n_blocks * rb.block_size * rb.pitch * static_cast<int64_t>(elem_size) * (rb.pitch > rb.D ? 1 : slots) >= min_bytes;
}

struct AdamCoef {
  const double* alpha;  // device word left by cal_alpha: -lr / (1 - beta1^t) * sqrtf(1 - beta2^t)
  double beta1, beta2, decay, eps;
};

// cal_alpha (block_apply_adamw_op.cc:77-85) on values: the running powers advance in their own
// precision and alpha comes out of the advanced powers. One definition for the one-thread kernel
// and for the kernels that work alpha out themselves, so both give the same bits.
template <typename beta_t>
__device__ __forceinline__ double cal_alpha_step(beta_t b1_old, beta_t b2_old, double lr, double beta1, double beta2,
                                                 beta_t& b1_new, beta_t& b2_new) {
  // no fused multiply-add: with double powers `1 - b1_old * beta1` would otherwise skip the rounding of
  // the product that the reference's `beta1_t[0] *= beta1` makes
#pragma clang fp contract(off)
  b1_new = static_cast<beta_t>(b1_old * beta1);
  b2_new = static_cast<beta_t>(b2_old * beta2);
  const beta_t bc1 = 1 - b1_new;
  const beta_t bc2 = 1 - b2_new;
  const beta_t alpha = static_cast<beta_t>(-lr / bc1 * sqrtf(static_cast<float>(bc2)));
  return static_cast<double>(alpha);
}

// One pack of VEC elements of one row, in registers: g = gradient (fp32); w / m / v updated in place.
template <typename T, int VEC>
__device__ __forceinline__ void adam_compute_pack(Pack<T, VEC>& w, Pack<T, VEC>& m, Pack<T, VEC>& v,
                                                  const float (&g)[VEC], double alpha, const AdamCoef& c) {
#pragma clang fp contract(off)
  const double omb1 = 1 - c.beta1, omb2 = 1 - c.beta2;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    // every line: double arithmetic, then one rounding to the storage type
    float we = to_float(w.v[j]), me = to_float(m.v[j]), ve = to_float(v.v[j]);
    const float ge = g[j];
    we = to_float(from_float<T>(static_cast<float>(we * c.decay)));
    me = to_float(from_float<T>(static_cast<float>(me * c.beta1 + ge * omb1)));
    ve = to_float(from_float<T>(static_cast<float>(ve * c.beta2 + omb2 * ge * ge)));
    if constexpr (sizeof(T) == 2) {
      // 16-bit rows: `emb_elem += <double>` (block_apply_adamw_op.cc:55-56) converts the step to the row
      // type first and adds the two in float (c10::Half has no += for a double): two roundings
      const float upd = to_float(from_float<T>(static_cast<float>(alpha * (me / (sqrtf(ve) + c.eps)))));
      we = to_float(from_float<T>(we + upd));
    } else {
      we = to_float(from_float<T>(static_cast<float>(we + alpha * (me / (sqrtf(ve) + c.eps)))));
    }
    w.v[j] = from_float<T>(we);
    m.v[j] = from_float<T>(me);
    v.v[j] = from_float<T>(ve);
  }
}

// One pack of a table row read or written. STREAM: with the streaming (non-temporal) hint, for
// 16-byte packs: the rows of a table far larger than the caches are not touched again before they
// are evicted anyway, and without the hint they push out what the step does read again (its
// lists, the gradient rows): the fused update of a 340 MB-per-slot table ran 8 % faster with it,
// and so did the kernels after it.
template <typename T, int VEC, bool STREAM>
__device__ __forceinline__ Pack<T, VEC> load_row_pack_of_table(const T* p) {
  if constexpr (STREAM && sizeof(T) * VEC == 16) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const u4 raw = __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    Pack<T, VEC> pk;
    __builtin_memcpy(&pk, &raw, 16);
    return pk;
  } else {
    return *reinterpret_cast<const Pack<T, VEC>*>(p);
  }
}
template <typename T, int VEC, bool STREAM>
__device__ __forceinline__ void store_row_pack_of_table(T* p, const Pack<T, VEC>& pk) {
  if constexpr (STREAM && sizeof(T) * VEC == 16) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 raw;
    __builtin_memcpy(&raw, &pk, 16);
    __builtin_nontemporal_store(raw, reinterpret_cast<u4*>(p));
  } else {
    *reinterpret_cast<Pack<T, VEC>*>(p) = pk;
  }
}

// The same on memory: read, update, write.
template <typename T, int VEC, bool STREAM = false>
__device__ __forceinline__ void adam_update_pack(T* w_ptr, T* m_ptr, T* v_ptr, const float (&g)[VEC], double alpha,
                                                 const AdamCoef& c) {
  Pack<T, VEC> w = load_row_pack_of_table<T, VEC, STREAM>(w_ptr);
  Pack<T, VEC> m = load_row_pack_of_table<T, VEC, STREAM>(m_ptr);
  Pack<T, VEC> v = load_row_pack_of_table<T, VEC, STREAM>(v_ptr);
  adam_compute_pack<T, VEC>(w, m, v, g, alpha, c);
  store_row_pack_of_table<T, VEC, STREAM>(w_ptr, w);
  store_row_pack_of_table<T, VEC, STREAM>(m_ptr, m);
  store_row_pack_of_table<T, VEC, STREAM>(v_ptr, v);
}

template <typename T, int VEC>
__device__ __forceinline__ void adagrad_compute_pack(Pack<T, VEC>& w, Pack<T, VEC>& s, const float (&g)[VEC], float lr,
                                                     float eps) {
#pragma clang fp contract(off)
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    float we = to_float(w.v[j]), se = to_float(s.v[j]);
    const float ge = g[j];
    se = to_float(from_float<T>(se + ge * ge));
    we = we - lr * (ge / (sqrtf(se) + eps));
    w.v[j] = from_float<T>(we);
    s.v[j] = from_float<T>(se);
  }
}

template <typename T, int VEC, bool STREAM = false>
__device__ __forceinline__ void adagrad_update_pack(T* w_ptr, T* s_ptr, const float (&g)[VEC], float lr, float eps) {
  Pack<T, VEC> w = load_row_pack_of_table<T, VEC, STREAM>(w_ptr);
  Pack<T, VEC> s = load_row_pack_of_table<T, VEC, STREAM>(s_ptr);
  adagrad_compute_pack<T, VEC>(w, s, g, lr, eps);
  store_row_pack_of_table<T, VEC, STREAM>(w_ptr, w);
  store_row_pack_of_table<T, VEC, STREAM>(s_ptr, s);
}

// cal_alpha (block_apply_adamw_op.cc:77-85) as a one-thread launch on `stream`: advances the
// running powers in place, in their own precision, and leaves alpha (as double) in alpha_out.
int launch_cal_alpha(void* beta1_t, void* beta2_t, int beta_is_f64, double* alpha_out, double lr, double beta1,
                     double beta2, hipStream_t stream);

}  // namespace recis_hip
