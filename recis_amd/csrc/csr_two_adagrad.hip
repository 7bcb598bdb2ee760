// Gather-reduce over a batch plan's occurrence lists with TWO inputs: the gradients of two outputs
// of one lookup (a pooled output and an unpooled, padded one: the reference adds them with one
// more atomic scatter per output, csrc/ops/embedding_segment_reduce_kernel.cu:79-120 and
// ragged_tile_kernel.cu) are summed into the unique rows in one pass, and the optimizer's update
// of the table row can follow at once. The kernels are those of csr_rows.cuh, instantiated here
// for a second input so that the two families compile side by side.
// (This file: the kernels that end in the Adagrad row update; csr_two.hip holds the ones that store.)
#include "csr_rows.cuh"

using namespace recis_hip;

extern "C" {

int recis_csr_gather_reduce2_adagrad(const recis_csr_input* a, const recis_csr_input* b, const int32_t* row_start,
                                     const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, int64_t U,
                                     int64_t D, const int64_t* row_index, void* const* emb_blocks_dev,
                                     void* const* accum_blocks_dev, int64_t n_blocks, int64_t block_size,
                                     int64_t row_pitch_bytes, int row_dtype, double lr, double eps, void* stream_) {
  RECIS_REQUIRE(a && b, "both inputs must be given");
  RECIS_REQUIRE(a->n_parts == 0, "only the second input may come in parts");
  if (U == 0) return RECIS_OK;
  FuseArgs f;
  if (int rc = fill_fuse_args(f, row_index, emb_blocks_dev, accum_blocks_dev, nullptr, false, n_blocks, block_size,
                              row_pitch_bytes, D, row_dtype))
    return rc;
  f.lr = static_cast<float>(lr);
  f.eps = static_cast<float>(eps);
  CsrInput second;
  CsrRequest r = two_input_request(a, b, second, row_start, hot_items, hot_cap, counts_dev, U, D, stream_);
  r.out_dtype = row_dtype;
  r.epi = kEpiAdagrad;
  r.fuse = &f;
  return csr_gather_reduce_run<true, kEpiAdagrad>(r);
}

}  // extern "C"
