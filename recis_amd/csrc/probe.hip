// Measurement support: what this device does with rows at random places, with nothing else in
// the kernel. No reference counterpart; bench.py's probe workload calls it to state the ceiling
// the row kernels of the training step are held against.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.cuh"

namespace recis_hip {
namespace {

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// A lane group of LPR lanes per row (16 bytes per lane), R rows per group with their loads in
// flight together. Reads: the packs are xor-ed and stored only if they come out as a value no
// input holds, so nothing is written. Writes: every lane stores its lane number.
template <int R, bool WRITE>
__global__ void __launch_bounds__(kBlock)
probe_rows_kernel(u4* __restrict__ table, const int32_t* __restrict__ idx, int64_t n, int lpr_log2, int64_t pitch16,
                  u4* __restrict__ sink) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t r0 = (t >> lpr_log2) * R;
  const int c = static_cast<int>(t & ((1 << lpr_log2) - 1));
  if (r0 >= n) return;
  int32_t s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) s[r] = r0 + r < n ? idx[r0 + r] : idx[r0];
  if constexpr (WRITE) {
    const u4 v = {static_cast<uint32_t>(threadIdx.x), 1u, 2u, 3u};
#pragma unroll
    for (int r = 0; r < R; ++r) __builtin_nontemporal_store(v, table + static_cast<int64_t>(s[r]) * pitch16 + c);
  } else {
    u4 acc = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int r = 0; r < R; ++r) acc ^= __builtin_nontemporal_load(table + static_cast<int64_t>(s[r]) * pitch16 + c);
    if (acc.x == 0x9E3779B9u && acc.y == 0x7F4A7C15u) sink[t & 1023] = acc;
  }
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" int recis_hip_probe_random_rows(void* table, int64_t rows, int64_t row_bytes, const int32_t* idx, int64_t n,
                                           int rows_in_flight, int write, void* sink, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(table && idx && sink, "NULL argument");
  RECIS_REQUIRE(rows >= 1 && rows <= INT32_MAX && n >= 0, "bad sizes");
  RECIS_REQUIRE(row_bytes >= 16 && row_bytes <= 1024 && (row_bytes & (row_bytes - 1)) == 0,
                "row_bytes must be a power of two from 16 to 1024");
  RECIS_REQUIRE(reinterpret_cast<uintptr_t>(table) % 16 == 0, "the table must be 16-byte aligned");
  RECIS_REQUIRE(rows_in_flight == 1 || rows_in_flight == 2 || rows_in_flight == 4, "rows_in_flight: 1, 2 or 4");
  if (n == 0) return RECIS_OK;
  const int lpr_log2 = ilog2_ceil(row_bytes / 16);
  const int64_t groups = (n + rows_in_flight - 1) / rows_in_flight;
  const int64_t threads = groups << lpr_log2;
  const dim3 grid(static_cast<unsigned>((threads + kBlock - 1) / kBlock)), block(kBlock);
  u4* t = static_cast<u4*>(table);
  u4* s = static_cast<u4*>(sink);
  const int64_t pitch16 = row_bytes / 16;
  auto launch = [&](auto rtag) {
    constexpr int R = decltype(rtag)::value;
    if (write)
      probe_rows_kernel<R, true><<<grid, block, 0, stream>>>(t, idx, n, lpr_log2, pitch16, s);
    else
      probe_rows_kernel<R, false><<<grid, block, 0, stream>>>(t, idx, n, lpr_log2, pitch16, s);
  };
  RECIS_TIME_KERNEL("probe_rows_kernel", stream) {
    if (rows_in_flight == 1) launch(std::integral_constant<int, 1>{});
    else if (rows_in_flight == 2) launch(std::integral_constant<int, 2>{});
    else launch(std::integral_constant<int, 4>{});
  }
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}
