// Gather-reduce over a batch plan's occurrence lists with TWO inputs: the gradients of two outputs
// of one lookup (a pooled output and an unpooled, padded one: the reference adds them with one
// more atomic scatter per output, csrc/ops/embedding_segment_reduce_kernel.cu:79-120 and
// ragged_tile_kernel.cu) are summed into the unique rows in one pass, and the optimizer's update
// of the table row can follow at once. The kernels are those of csr_rows.cuh, instantiated here
// for a second input so that the two families compile side by side.
// (This file: the kernels that end in the Adam-family row update; csr_two.hip holds the ones that store.)
#include "csr_rows.cuh"

using namespace recis_hip;

extern "C" {

int recis_csr_gather_reduce2_adamw(const recis_csr_input* a, const recis_csr_input* b, const int32_t* row_start,
                                   const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, int64_t U,
                                   int64_t D, const int64_t* row_index, void* const* emb_blocks_dev,
                                   void* const* exp_avg_blocks_dev, void* const* exp_avg_sq_blocks_dev,
                                   int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes, int row_dtype,
                                   void* beta1_t, void* beta2_t, int beta_is_f64, double lr, double beta1, double beta2,
                                   double weight_decay, double eps, void* stream_) {
  RECIS_REQUIRE(a && b, "both inputs must be given");
  RECIS_REQUIRE(a->n_parts == 0, "only the second input may come in parts");
  RECIS_REQUIRE(beta1_t != nullptr && beta2_t != nullptr, "beta1_t / beta2_t must not be NULL");
  FuseArgs f{};
  if (U > 0) {
    if (int rc = fill_fuse_args(f, row_index, emb_blocks_dev, exp_avg_blocks_dev, exp_avg_sq_blocks_dev, true, n_blocks,
                                block_size, row_pitch_bytes, D, row_dtype))
      return rc;
  }
  CsrInput second;
  CsrRequest r = two_input_request(a, b, second, row_start, hot_items, hot_cap, counts_dev, U, D, stream_);
  r.out_dtype = row_dtype;
  r.epi = kEpiAdam;
  r.fuse = &f;
  return run_with_alpha<true, kEpiAdam>(r, f, beta1_t, beta2_t, beta_is_f64, lr, beta1, beta2, weight_decay, eps);
}

}  // extern "C"
