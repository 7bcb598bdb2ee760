// Gather-reduce over a batch plan's occurrence lists with TWO inputs: the gradients of two outputs
// of one lookup (a pooled output and an unpooled, padded one: the reference adds them with one
// more atomic scatter per output, csrc/ops/embedding_segment_reduce_kernel.cu:79-120 and
// ragged_tile_kernel.cu) are summed into the unique rows in one pass, and the optimizer's update
// of the table row can follow at once. The kernels are those of csr_rows.cuh, instantiated here
// for a second input so that the two families compile side by side.
#include "csr_rows.cuh"

using namespace recis_hip;

extern "C" {

int recis_csr_gather_reduce2(const recis_csr_input* a, const recis_csr_input* b, const int32_t* row_start,
                             const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, void* out,
                             int64_t U, int64_t D, int accumulate, void* stream_) {
  RECIS_REQUIRE(a && b, "both inputs must be given");
  RECIS_REQUIRE(a->n_parts == 0, "only the second input may come in parts");
  CsrInput second;
  CsrRequest r = two_input_request(a, b, second, row_start, hot_items, hot_cap, counts_dev, U, D, stream_);
  r.out = out;
  r.out_dtype = RECIS_F32;
  r.accumulate = accumulate;
  return csr_gather_reduce_run<true, kEpiStore>(r);
}

}  // extern "C"
