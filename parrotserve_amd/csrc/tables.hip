// Device side of the incremental slot tables: a decode iteration appends exactly one slot to the
// suffix list of every request of the batch, so the padded [B, width] table and the length vector
// that the reference rebuilds from Python lists every iteration
// (parrot/engine/builtin/attn_func.py:523-531,553-569) are patched in place instead.
#include "common.hpp"

namespace ph {

__global__ __launch_bounds__(256) void append_slots_kernel(int32_t* __restrict__ table, int64_t stride,
                                                           int32_t* __restrict__ lens,
                                                           const int32_t* __restrict__ rows,
                                                           const int32_t* __restrict__ new_slots, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int r = rows ? rows[i] : i;
  const int l = lens[r];
  if (l < stride) {  // the host grows the table before a row fills up; never write past a row
    table[(int64_t)r * stride + l] = new_slots[i];
    lens[r] = l + 1;
  }
}

}  // namespace ph

extern "C" int ph_suffix_tables_append(int32_t* table, int64_t table_stride, int32_t* lens, const int32_t* rows,
                                       const int32_t* new_slots, int64_t n, void* stream) {
  if (n < 0 || table_stride <= 0) return PH_ERR_ARG;
  if (n == 0) return PH_OK;
  if (!table || !lens || !new_slots) return PH_ERR_ARG;
  hipLaunchKernelGGL(ph::append_slots_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     table, table_stride, lens, rows, new_slots, (int)n);
  return ph::launch_status();
}
