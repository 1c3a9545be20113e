/* Shared declarations of the one-epilogue-many-producers example: C = (A . B) * scale[col] + bias[col],
 * bf16 operands, fp32 accumulate, bf16 out; A [M, K] row-major, B handed over as B^T [N, K] row-major.
 *
 * Three matrix packages keep a wave's 64 x 64 accumulator in three different homes -- accumulation
 * registers (AGPRs), vector registers (VGPRs), a tile in LDS -- and export it as tensor "acc"; ONE
 * epilogue package imports "acc" through a function the linker generates for the home it is linked
 * against, and is never rebuilt (examples/one-epilogue-many-producers in the reference: providers/
 * accumulator/*, consumer/epilogue.cu).  The loader is the gs.loader package of the three-package GEMM
 * example, unchanged: same ring contract. */
#ifndef PIPELINK_OE_ABI_H
#define PIPELINK_OE_ABI_H

#include <stdint.h>
#include <pipelink/host_view.h>

#define OE_TILE 128
#define OE_TILE_K 64
#define OE_STAGE_BYTES (2 * 128 * 128)
#define OE_LOAD_WAVES 2 /* the loader's waves: arrivals on a stage's `full` counter per fill (GS_LOAD_WAVES) */
#define OE_LDS_PITCH (64 * 4 + 16) /* bytes between rows of a wave's 64 x 64 fp32 tile in LDS */

typedef struct OeMmaParams {
  uint32_t* status;
  int32_t n, k;
} OeMmaParams;

typedef struct OeEpilogueParams {
  const float* bias;  /* [N] */
  const float* scale; /* [N] */
  uint16_t* c;        /* [M, N] bf16 */
  int32_t m, n;
} OeEpilogueParams;

typedef struct OeTile {
  int32_t row0, col0; /* first row / column of the calling wave's 64 x 64 share */
} OeTile;

#endif
