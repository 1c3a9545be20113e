// Package oe.mma.wide: the matrix role of the one-epilogue example with a 256 x 128 workgroup tile, each of the four
// waves holding 128 x 64 in 128 AGPRs.  Per 64 contraction elements a workgroup moves 48 KB through L2 and LDS for
// 4.2 MFLOP, against 32 KB for 2.1 MFLOP with the 128 x 128 tile of the three homes: a quarter fewer operand bytes
// per flop -- what bounds those -- and three stages of 48 KB fit the LDS, so half as many bytes again are in flight.
// (A 256 x 256 tile would halve the bytes, but its waves need all 512 registers of a SIMD lane, and a kernel's waves
// all get the same allocation: the loader waves could not share the SIMDs.)
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mma_body.hpp"

extern "C" __device__ void oe_mma_wide_role_mma(const void* params, unsigned variant) {
  (void)variant;
  oe_mma::role<0, 4, 2>(params, nullptr);
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.mma.wide", "0.1.0");
PL_PARAMS(OeMmaParams);
PL_ROLE(mma, oe_mma_wide_role_mma, 4);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_RING(ab_ring, "consume", mma, "bf16", 16, 384, 64, "pipelink_gs_depth", OE_WIDE_STAGE_BYTES, "pipelink_gs_full", "warps(load)", load,
        "pipelink_gs_empty", "warps(mma)", mma, load);
PL_CLAIM_WARPS("pipelink_oe_warp_mma", mma, 4);

PL_CALL(epilogue, "oe_epilogue_wide_store",
        "extern \"C\" __device__ void pipelink_call_epilogue(const void* view, const OeTile* tile, const void* source);");
PL_EXPORT_TENSOR(acc, "gemm_accumulator", "f32", 128, 64, "agpr", "mfma32x32c", 0);
PL_USES("pipelink_gs_depth");
PL_USES("pipelink_gs_ring");
PL_USES("pipelink_gs_full");
PL_USES("pipelink_gs_empty");
PL_USES("pipelink_oe_warp_mma");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
