// Gather-reduce over a batch plan's occurrence lists with TWO inputs: the gradients of two outputs
// of one lookup (a pooled output and an unpooled, padded one: the reference adds them with one
// more atomic scatter per output, csrc/ops/embedding_segment_reduce_kernel.cu:79-120 and
// ragged_tile_kernel.cu) are summed into the unique rows in one pass, and the optimizer's update
// of the table row can follow at once. The kernels are those of csr_rows.cuh, instantiated here
// for a second input so that the two families compile side by side.
#include "csr_rows.cuh"

using namespace recis_hip;

namespace {

CsrRequest two_input_request(const recis_csr_input* a, const recis_csr_input* b, CsrInput& second,
                             const int32_t* row_start, const int32_t* hot_items, int64_t hot_cap,
                             const int64_t* counts_dev, int64_t U, int64_t D, void* stream_) {
  CsrRequest r;
  r.in1 = CsrInput{a->rows, a->rows_dtype, a->n_rows, a->src, a->coef, a->coef_dtype};
  second = CsrInput{b->rows, b->rows_dtype, b->n_rows, b->src, b->coef, b->coef_dtype};
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

extern "C" {

int recis_csr_gather_reduce2(const recis_csr_input* a, const recis_csr_input* b, const int32_t* row_start,
                             const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, void* out,
                             int64_t U, int64_t D, int accumulate, void* stream_) {
  RECIS_REQUIRE(a && b, "both inputs must be given");
  CsrInput second;
  CsrRequest r = two_input_request(a, b, second, row_start, hot_items, hot_cap, counts_dev, U, D, stream_);
  r.out = out;
  r.out_dtype = RECIS_F32;
  r.accumulate = accumulate;
  return csr_gather_reduce_run<true>(r);
}

int recis_csr_gather_reduce2_adamw(const recis_csr_input* a, const recis_csr_input* b, const int32_t* row_start,
                                   const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, int64_t U,
                                   int64_t D, const int64_t* row_index, void* const* emb_blocks_dev,
                                   void* const* exp_avg_blocks_dev, void* const* exp_avg_sq_blocks_dev,
                                   int64_t n_blocks, int64_t block_size, int row_dtype, void* beta1_t, void* beta2_t,
                                   int beta_is_f64, double lr, double beta1, double beta2, double weight_decay,
                                   double eps, void* stream_) {
  RECIS_REQUIRE(a && b, "both inputs must be given");
  RECIS_REQUIRE(beta1_t != nullptr && beta2_t != nullptr, "beta1_t / beta2_t must not be NULL");
  FuseArgs f{};
  if (U > 0) {
    if (int rc = fill_fuse_args(f, row_index, emb_blocks_dev, exp_avg_blocks_dev, exp_avg_sq_blocks_dev, true, n_blocks,
                                block_size, D, row_dtype))
      return rc;
  }
  CsrInput second;
  CsrRequest r = two_input_request(a, b, second, row_start, hot_items, hot_cap, counts_dev, U, D, stream_);
  r.out_dtype = row_dtype;
  r.epi = kEpiAdam;
  r.fuse = &f;
  return run_with_alpha<true>(r, f, beta1_t, beta2_t, beta_is_f64, lr, beta1, beta2, weight_decay, eps);
}

int recis_csr_gather_reduce2_adagrad(const recis_csr_input* a, const recis_csr_input* b, const int32_t* row_start,
                                     const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, int64_t U,
                                     int64_t D, const int64_t* row_index, void* const* emb_blocks_dev,
                                     void* const* accum_blocks_dev, int64_t n_blocks, int64_t block_size,
                                     int row_dtype, double lr, double eps, void* stream_) {
  RECIS_REQUIRE(a && b, "both inputs must be given");
  if (U == 0) return RECIS_OK;
  FuseArgs f;
  if (int rc = fill_fuse_args(f, row_index, emb_blocks_dev, accum_blocks_dev, nullptr, false, n_blocks, block_size, D,
                              row_dtype))
    return rc;
  f.lr = static_cast<float>(lr);
  f.eps = static_cast<float>(eps);
  CsrInput second;
  CsrRequest r = two_input_request(a, b, second, row_start, hot_items, hot_cap, counts_dev, U, D, stream_);
  r.out_dtype = row_dtype;
  r.epi = kEpiAdagrad;
  r.fuse = &f;
  return csr_gather_reduce_run<true>(r);
}

}  // extern "C"
