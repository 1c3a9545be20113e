// Package oe.mma.lds: the matrix role of the one-epilogue example with its accumulator in an LDS tile.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mma_body.hpp"
extern "C" __device__ int pipelink_oe_acc_tile();  // byte offset of the four waves' tiles in dynamic LDS
extern "C" __device__ void oe_mma_lds_role_mma(const void* params, unsigned variant) {
  (void)variant;
  const int wave = (int)(threadIdx.x >> 6) - pipelink_oe_warp_mma();
  oe_mma::role<2>(params, pipelink_smem + pipelink_oe_acc_tile() + wave * (64 * OE_LDS_PITCH));
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.mma.lds", "0.1.0");
PL_PARAMS(OeMmaParams);
PL_ROLE(mma, oe_mma_lds_role_mma, 4);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_RING(ab_ring, "consume", mma, "bf16", 16, 256, 64, "pipelink_gs_depth", 32768, "pipelink_gs_full", "warps(load)", load,
        "pipelink_gs_empty", "warps(mma)", mma, load);
PL_CLAIM_WARPS("pipelink_oe_warp_mma", mma, 4);
PL_CLAIM("pipelink_oe_acc_tile", "smem", 4 * 64 * OE_LDS_PITCH, 16, "kernel");
PL_USES("pipelink_oe_acc_tile");
PL_CALL(epilogue, "oe_epilogue_store",
        "extern \"C\" __device__ void pipelink_call_epilogue(const void* view, const OeTile* tile, const void* source);");
PL_EXPORT_TENSOR(acc, "gemm_accumulator", "f32", 64, 64, "lds", "row_major", OE_LDS_PITCH);
PL_USES("pipelink_gs_depth");
PL_USES("pipelink_gs_ring");
PL_USES("pipelink_gs_full");
PL_USES("pipelink_gs_empty");
PL_USES("pipelink_oe_warp_mma");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
