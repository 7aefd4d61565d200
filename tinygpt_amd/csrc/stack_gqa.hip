// stack_gqa.hip — launches of the matrix-core grouped-query attention of layered models (kernels/stack_gqa_mfma.h); a translation unit of its own so that
// its template instances compile beside stack.hip.
#include "stack.h"

#include "kernels/stack_gqa_mfma.h"

namespace {
template <int DT, int ND, bool SPLIT>
void launch_nt(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaMfmaArgs& a, dim3 grid) {
  if (a.vdim <= 128) hipLaunchKernelGGL((tgx::gqa_attn_mfma_kernel<DT, ND, 1, SPLIT>), grid, dim3(256), 0, c->stream, m, a);
  else hipLaunchKernelGGL((tgx::gqa_attn_mfma_kernel<DT, ND, 2, SPLIT>), grid, dim3(256), 0, c->stream, m, a);
}
template <int DT, bool SPLIT>
void launch_nd(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaMfmaArgs& a, dim3 grid) {
  switch (a.dim / 64) {
    case 1: launch_nt<DT, 1, SPLIT>(c, m, a, grid); break;
    case 2: launch_nt<DT, 2, SPLIT>(c, m, a, grid); break;
    default: launch_nt<DT, 4, SPLIT>(c, m, a, grid); break;
  }
}
}  // namespace

bool gqa_mfma_shapes_ok(int dt, int dim, int vdim, int page_shift, long long ldq) {
  return dt != tgx::DT_F32 && (dim == 64 || dim == 128 || dim == 256) && vdim % 32 == 0 && vdim >= 32 && vdim <= 256 && page_shift >= 6 && ldq % 4 == 0;
}

void launch_gqa_mfma(tgx_ctx* c, const tgx::StepMeta& m, const tgx::GqaMfmaArgs& a, dim3 grid, bool split) {
  if (!gqa_mfma_shapes_ok(c->dt, a.dim, a.vdim, m.page_shift, a.ldq)) { c->launch_fault = "matrix-core attention: head sizes or storage dtype it does not take"; return; }
  TGX_DT16_SWITCH(c->dt, if (split) launch_nd<DT, true>(c, m, a, grid); else launch_nd<DT, false>(c, m, a, grid);)
}
