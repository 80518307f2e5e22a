// A toy encoding of positions, for the tests: a learned row per position is added to the embedded
// rows before the first layer.  Which row of the table a row of the step takes is a table of the
// step that the part lays out on the host itself (its StepTables in the test).  This file holds what it brings along to run from C: a kernel, the
// launcher that the host's part calls too, and a runner for the walk of csrc/engine.hip
// (kappai_embedded_fn), which the host registers under a name.  Nothing in the framework's own
// files knows of it.
#include "common.h"
#include "engine.h"

struct toy_learned_positions {    // what the runner reads (mirrored by the test's ctypes struct)
  const void* table;              // [positions, width]
  int table_is_bf16;
  int positions;
  int rows_table;                 // the place in kappai_batch::tables of the part's own table of the
};                                // step: the table's row for every row of the step

template <typename T>
__global__ void toy_add_positions_kernel(float* __restrict__ resid, const T* __restrict__ table,
                                         const int* __restrict__ table_row, int D, int positions) {
  const int t = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= D) return;
  const int p = min(max(table_row[t], 0), positions - 1);
  float v;
  if constexpr (sizeof(T) == 2) v = bf16_to_f32(table[(size_t)p * D + c]);
  else v = table[(size_t)p * D + c];
  resid[(size_t)t * D + c] += v;
}

extern "C" int toy_add_positions_launch(float* resid, const void* table, int table_is_bf16,
                                        const int* table_row, int M, int D, int positions,
                                        hipStream_t stream) {
  if (M < 1 || D < 1 || positions < 1 || M > 65535 || table_row == nullptr)
    return (int)hipErrorInvalidValue;
  const dim3 grid((D + 127) / 128, M), block(128);
  if (table_is_bf16)
    hipLaunchKernelGGL(toy_add_positions_kernel<bf16_t>, grid, block, 0, stream, resid,
                       (const bf16_t*)table, table_row, D, positions);
  else
    hipLaunchKernelGGL(toy_add_positions_kernel<float>, grid, block, 0, stream, resid,
                       (const float*)table, table_row, D, positions);
  return (int)hipGetLastError();
}

extern "C" void toy_learned_positions_run(kappai_step* s, const void* desc, float* resid, int M) {
  const kappai_step_api& api = *s->api;
  const toy_learned_positions& d = *static_cast<const toy_learned_positions*>(desc);
  if (api.dry(s) || !api.ok(s)) return;
  const kappai_batch& b = *api.batch(s);
  if (d.rows_table < 0 || d.rows_table >= KAPPAI_MAX_TABLES || b.tables[d.rows_table] == nullptr ||
      b.table_rows[d.rows_table] != M) {
    api.fail(s, "the toy positions did not get their table of the step");
    return;
  }
  api.launched(s, toy_add_positions_launch(resid, d.table, d.table_is_bf16, b.tables[d.rows_table],
                                           M, api.model(s)->width, d.positions, api.stream(s)));
}

extern "C" int toy_learned_positions_desc_bytes(void) { return (int)sizeof(toy_learned_positions); }
