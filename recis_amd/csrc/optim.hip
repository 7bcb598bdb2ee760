// Fused sparse optimizer row updates for gfx950.
//
// Adam family: stands in for block_apply_adamw (csrc/ops/block_apply_adamw_op.cc:114-132,
// device kernels csrc/ops/block_apply_adamw_op_kernel.cu:12-171). The row kernel
// is bound by HBM traffic (grad read + read-modify-write of three rows), so the
// arithmetic is free: it is done exactly as the reference's CPU functor does it
// (block_apply_adamw_op.cc:32-58: products and sums in double, sqrtf in float,
// every assignment rounded to the storage type, no fused multiply-add), which
// makes the result reproducible against the CPU path bit for bit.
//
// Adagrad has no reference counterpart; it is the textbook update in float.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.cuh"
#include "optim_rows.cuh"

#pragma clang fp contract(off)

namespace recis_hip {
namespace {

struct OptArgs {
  const int64_t* index;
  int64_t n;
  int64_t n_blocks;
  int64_t block_size;
  int64_t pitch;
  int D;
  int lpr_log2;
  int* err;
};

__device__ __forceinline__ bool row_offset(const OptArgs& a, int64_t idx, int64_t& b, int64_t& off) {
  const RowBlocks r{a.n_blocks, a.block_size, a.D, a.pitch};
  return block_row(r, idx, b, off);
}

// cal_alpha (block_apply_adamw_op.cc:77-85): advances the running powers in
// place, in their own precision, and leaves alpha (as double) for the row kernel.
template <typename beta_t>
__global__ void cal_alpha_kernel(beta_t* beta1_t, beta_t* beta2_t, double* alpha_out, double lr,
                                 double beta1, double beta2) {
  beta_t b1, b2;
  alpha_out[0] = cal_alpha_step<beta_t>(beta1_t[0], beta2_t[0], lr, beta1, beta2, b1, b2);
  beta1_t[0] = b1;
  beta2_t[0] = b2;
}

template <typename T, typename TG, int VEC>
__global__ void __launch_bounds__(kBlock)
adamw_rows_kernel(OptArgs a, const TG* __restrict__ grad, T* const* __restrict__ emb_blocks,
                  T* const* __restrict__ m_blocks, T* const* __restrict__ v_blocks,
                  const double* __restrict__ alpha_ptr, double beta1, double beta2, double decay,
                  double eps) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  if (i >= a.n) return;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  int64_t b, off;
  if (!row_offset(a, a.index[i], b, off)) {
    raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  const double alpha = alpha_ptr[0];
  const AdamCoef coef{alpha_ptr, beta1, beta2, decay, eps};
  T* w_row = emb_blocks[b] + off * a.pitch;
  T* m_row = m_blocks[b] + off * a.pitch;
  T* v_row = v_blocks[b] + off * a.pitch;
  const TG* g_row = grad + i * a.D;
  for (int c0 = cl * VEC; c0 < a.D; c0 += VEC << a.lpr_log2) {
    float g[VEC];
    load_pack<TG, VEC>(g_row + c0, g);
    adam_update_pack<T, VEC>(w_row + c0, m_row + c0, v_row + c0, g, alpha, coef);
  }
}

// Rows of doubles (the functor with TEmb = double, block_apply_adamw_op.cc:32-58): an element per
// thread, everything in double but the square root (sqrtf of the value converted to float).
__global__ void __launch_bounds__(kBlock)
adamw_rows_f64_kernel(OptArgs a, const double* __restrict__ grad, double* const* __restrict__ emb_blocks,
                      double* const* __restrict__ m_blocks, double* const* __restrict__ v_blocks,
                      const double* __restrict__ alpha_ptr, double beta1, double beta2, double decay, double eps) {
#pragma clang fp contract(off)
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (e >= a.n * a.D) return;
  const int64_t i = e / a.D;
  const int d = static_cast<int>(e - i * a.D);
  int64_t b, off;
  if (!row_offset(a, a.index[i], b, off)) {
    if (d == 0) raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  const int64_t at = off * a.pitch + d;
  const double g = grad[e], alpha = alpha_ptr[0];
  double w = emb_blocks[b][at], m = m_blocks[b][at], v = v_blocks[b][at];
  w = w * decay;
  m = m * beta1 + g * (1 - beta1);
  v = v * beta2 + (1 - beta2) * g * g;
  w += alpha * (m / (sqrtf(static_cast<float>(v)) + eps));
  emb_blocks[b][at] = w;
  m_blocks[b][at] = m;
  v_blocks[b][at] = v;
}

template <typename T, typename TG, int VEC>
__global__ void __launch_bounds__(kBlock)
adagrad_rows_kernel(OptArgs a, const TG* __restrict__ grad, T* const* __restrict__ emb_blocks,
                    T* const* __restrict__ acc_blocks, float lr, float eps) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  if (i >= a.n) return;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  int64_t b, off;
  if (!row_offset(a, a.index[i], b, off)) {
    raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  T* w_row = emb_blocks[b] + off * a.pitch;
  T* s_row = acc_blocks[b] + off * a.pitch;
  const TG* g_row = grad + i * a.D;
  for (int c0 = cl * VEC; c0 < a.D; c0 += VEC << a.lpr_log2) {
    float g[VEC];
    load_pack<TG, VEC>(g_row + c0, g);
    adagrad_update_pack<T, VEC>(w_row + c0, s_row + c0, g, lr, eps);
  }
}

template <typename F>
int dispatch_row_types(int row_dt, int grad_dt, F&& f) {
  if (row_dt == RECIS_F32 && grad_dt == RECIS_F32) return f(float{}, float{});
  if (row_dt == RECIS_BF16 && grad_dt == RECIS_BF16) return f(bf16_t{}, bf16_t{});
  if (row_dt == RECIS_BF16 && grad_dt == RECIS_F32) return f(bf16_t{}, float{});
  if (row_dt == RECIS_F16 && grad_dt == RECIS_F16) return f(f16_t{}, f16_t{});
  if (row_dt == RECIS_F16 && grad_dt == RECIS_F32) return f(f16_t{}, float{});
  return fail(RECIS_ERR_ARG, "unsupported (row dtype %d, grad dtype %d)", row_dt, grad_dt);
}

template <typename F>
int dispatch_vec4(int vec, F&& f) {
  switch (vec) {
    case 8: return f(std::integral_constant<int, 8>{});
    case 4: return f(std::integral_constant<int, 4>{});
    case 2: return f(std::integral_constant<int, 2>{});
    case 1: return f(std::integral_constant<int, 1>{});
    default: return fail(RECIS_ERR_ARG, "bad vector width %d", vec);
  }
}

int fill_opt_args(OptArgs& a, const int64_t* index, const void* grad, int64_t n, int64_t n_blocks,
                  int64_t block_size, int64_t row_pitch_bytes, int64_t D, int row_dtype, int grad_dtype, int& vec) {
  RECIS_REQUIRE(n >= 0 && n_blocks >= 1 && block_size >= 1, "bad sizes (n=%lld n_blocks=%lld block_size=%lld)",
                (long long)n, (long long)n_blocks, (long long)block_size);
  RECIS_REQUIRE(D >= 1 && D <= (1 << 20), "embedding dim %lld out of range", (long long)D);
  RECIS_REQUIRE(index != nullptr && grad != nullptr, "index / grad must not be NULL");
  const int rsz = dtype_size(row_dtype), gsz = dtype_size(grad_dtype);
  RECIS_REQUIRE(rsz && gsz, "invalid dtype");
  // block bases are required to be aligned like the row width allows
  const int vb_row = pick_vec_bytes(D * rsz, 16);
  const int vb_g = pick_vec_bytes(D * gsz, reinterpret_cast<uintptr_t>(grad));
  vec = std::max(1, std::min(vb_row / rsz, vb_g / gsz));
  a.index = index;
  a.n = n;
  a.n_blocks = n_blocks;
  a.block_size = block_size;
  a.pitch = pitch_elements(row_pitch_bytes, D, rsz, vb_row);
  RECIS_REQUIRE(a.pitch >= D, "row pitch of %lld bytes does not fit rows of %lld elements", (long long)row_pitch_bytes,
                (long long)D);
  a.D = static_cast<int>(D);
  a.lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  a.err = device_error_word(current_device());
  RECIS_REQUIRE(a.err != nullptr, "could not reach the device error word");
  return RECIS_OK;
}

}  // namespace

int launch_cal_alpha(void* beta1_t, void* beta2_t, int beta_is_f64, double* alpha_out, double lr, double beta1,
                     double beta2, hipStream_t stream) {
  if (beta_is_f64)
    cal_alpha_kernel<double><<<1, 1, 0, stream>>>(static_cast<double*>(beta1_t), static_cast<double*>(beta2_t),
                                                   alpha_out, lr, beta1, beta2);
  else
    cal_alpha_kernel<float><<<1, 1, 0, stream>>>(static_cast<float*>(beta1_t), static_cast<float*>(beta2_t), alpha_out,
                                                  lr, beta1, beta2);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

int recis_block_apply_adamw(const int64_t* index, const void* grad, int grad_dtype,
                            void* const* emb_blocks_dev, void* const* exp_avg_blocks_dev,
                            void* const* exp_avg_sq_blocks_dev, int64_t n_blocks, int64_t block_size,
                            int64_t row_pitch_bytes, int row_dtype, void* beta1_t, void* beta2_t, int beta_is_f64, double lr,
                            double beta1, double beta2, double weight_decay, double eps, int64_t n,
                            int64_t D, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(beta1_t != nullptr && beta2_t != nullptr, "beta1_t / beta2_t must not be NULL");
  // the running powers advance even when no row is touched (cal_alpha runs first)
  void* ws = nullptr;
  if (int rc = get_workspace(stream, 256, &ws)) return rc;
  double* alpha = static_cast<double*>(ws);
  if (int rc = launch_cal_alpha(beta1_t, beta2_t, beta_is_f64, alpha, lr, beta1, beta2, stream)) return rc;
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(emb_blocks_dev && exp_avg_blocks_dev && exp_avg_sq_blocks_dev, "block tables must not be NULL");
  if (row_dtype == RECIS_F64) {
    RECIS_REQUIRE(grad_dtype == RECIS_F64, "rows of doubles take gradients of doubles");
    RECIS_REQUIRE(n >= 0 && n_blocks >= 1 && block_size >= 1 && D >= 1 && D <= (1 << 20) && index && grad, "bad arguments");
    RECIS_REQUIRE(row_pitch_bytes == 0 || (row_pitch_bytes >= D * 8 && row_pitch_bytes % 8 == 0),
                  "row pitch of %lld bytes does not fit rows of %lld doubles", (long long)row_pitch_bytes, (long long)D);
    OptArgs a{};
    a.index = index;
    a.n = n;
    a.n_blocks = n_blocks;
    a.block_size = block_size;
    a.pitch = row_pitch_bytes ? row_pitch_bytes / 8 : D;
    a.D = static_cast<int>(D);
    a.err = device_error_word(current_device());
    RECIS_REQUIRE(a.err != nullptr, "could not reach the device error word");
    const int64_t grid = (n * D + kBlock - 1) / kBlock;
    RECIS_TIME_KERNEL("adamw_rows_kernel", stream)
    adamw_rows_f64_kernel<<<dim3(grid), dim3(kBlock), 0, stream>>>(
        a, static_cast<const double*>(grad), reinterpret_cast<double* const*>(emb_blocks_dev),
        reinterpret_cast<double* const*>(exp_avg_blocks_dev), reinterpret_cast<double* const*>(exp_avg_sq_blocks_dev),
        alpha, beta1, beta2, weight_decay, eps);
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  }
  OptArgs a;
  int vec = 1;
  if (int rc = fill_opt_args(a, index, grad, n, n_blocks, block_size, row_pitch_bytes, D, row_dtype, grad_dtype, vec)) return rc;
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t grid = (n + rows_per_block - 1) / rows_per_block;
  return dispatch_row_types(row_dtype, grad_dtype, [&](auto t, auto tg) {
    using T = decltype(t);
    using TG = decltype(tg);
    return dispatch_vec4(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(T) > 16 || VEC * sizeof(TG) > 16) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        RECIS_TIME_KERNEL("adamw_rows_kernel", stream)
        adamw_rows_kernel<T, TG, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(
            a, static_cast<const TG*>(grad), reinterpret_cast<T* const*>(emb_blocks_dev),
            reinterpret_cast<T* const*>(exp_avg_blocks_dev), reinterpret_cast<T* const*>(exp_avg_sq_blocks_dev),
            alpha, beta1, beta2, weight_decay, eps);
        RECIS_LAUNCH_CHECK();
        return RECIS_OK;
      }
    });
  });
}

int recis_block_apply_adagrad(const int64_t* index, const void* grad, int grad_dtype,
                              void* const* emb_blocks_dev, void* const* accum_blocks_dev,
                              int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes, int row_dtype, double lr,
                              double eps,
                              int64_t n, int64_t D, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(emb_blocks_dev && accum_blocks_dev, "block tables must not be NULL");
  OptArgs a;
  int vec = 1;
  if (int rc = fill_opt_args(a, index, grad, n, n_blocks, block_size, row_pitch_bytes, D, row_dtype, grad_dtype, vec)) return rc;
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t grid = (n + rows_per_block - 1) / rows_per_block;
  return dispatch_row_types(row_dtype, grad_dtype, [&](auto t, auto tg) {
    using T = decltype(t);
    using TG = decltype(tg);
    return dispatch_vec4(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(T) > 16 || VEC * sizeof(TG) > 16) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        RECIS_TIME_KERNEL("adagrad_rows_kernel", stream)
        adagrad_rows_kernel<T, TG, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(
            a, static_cast<const TG*>(grad), reinterpret_cast<T* const*>(emb_blocks_dev),
            reinterpret_cast<T* const*>(accum_blocks_dev), static_cast<float>(lr), static_cast<float>(eps));
        RECIS_LAUNCH_CHECK();
        return RECIS_OK;
      }
    });
  });
}

}  // extern "C"
