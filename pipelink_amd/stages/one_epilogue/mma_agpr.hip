// Package oe.mma.agpr: the matrix role of the one-epilogue example with its accumulator in AGPRs.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mma_body.hpp"

extern "C" __device__ void oe_mma_agpr_role_mma(const void* params, unsigned variant) {
  (void)variant;
  oe_mma::role<0>(params, nullptr);
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.mma.agpr", "0.1.0");
PL_PARAMS(OeMmaParams);
PL_ROLE(mma, oe_mma_agpr_role_mma, 4);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_RING(ab_ring, "consume", mma, "bf16", 16, 256, 64, "pipelink_gs_depth", 32768, "pipelink_gs_full", "warps(load)", load,
        "pipelink_gs_empty", "warps(mma)", mma, load);
PL_CLAIM_WARPS("pipelink_oe_warp_mma", mma, 4);

PL_CALL(epilogue, "oe_epilogue_store",
        "extern \"C\" __device__ void pipelink_call_epilogue(const void* view, const OeTile* tile, const void* source);");
PL_EXPORT_TENSOR(acc, "gemm_accumulator", "f32", 64, 64, "agpr", "mfma32x32c", 0);
PL_USES("pipelink_gs_depth");
PL_USES("pipelink_gs_ring");
PL_USES("pipelink_gs_full");
PL_USES("pipelink_gs_empty");
PL_USES("pipelink_oe_warp_mma");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
