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
/* the wide trio (oe.loader.wide, oe.mma.wide, oe.epilogue.wide): a 256 x 128 workgroup tile, a wave's share 128 x 64 */
#define OE_WIDE_TILE_M 256
#define OE_WIDE_TILE_N 128
#define OE_WIDE_STAGE_BYTES ((256 + 128) * 128) /* 64 contraction elements of 256 A rows, then of 128 B^T rows */
#define OE_WIDE_LOAD_WAVES 3                    /* 128 rows each: upper A, lower A, B^T */

/* the 256 x 256 pair (oe.mma.full, which brings its own operands, and oe.epilogue.full): a wave's share 128 x 128 */
#define OE_FULL_TILE 256
#define OE_FULL_BUFFERS 5 /* 16 KB buffers (32 contraction elements of 256 rows) per operand ring */

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
  int32_t row0, col0; /* first row / column of the calling wave's share (64 x 64; 128 x 64 in the wide trio) */
} OeTile;

/* the wide loader's params: the layout of the three-package example's GsLoaderParams */
typedef struct OeLoaderParams {
  const uint16_t* a;  /* [M, K] bf16 */
  const uint16_t* bt; /* [N, K] bf16 */
  uint32_t* status;   /* [1], set to non-zero by a wait that gave up */
  int32_t m, n, k;    /* multiples of 256, 128, 64 */
  int32_t reserved;
} OeLoaderParams;

/* params of oe.mma.full: operands and extents */
typedef struct OeFullParams {
  const uint16_t* a;  /* [M, K] bf16 */
  const uint16_t* bt; /* [N, K] bf16 */
  uint32_t* status;   /* [1]; this package has no wait that can give up and leaves it alone */
  int32_t m, n, k;    /* m, n multiples of 256; k a multiple of 64, at least 256; m * k and n * k below 2^31 elements */
  int32_t reserved;
} OeFullParams;

#endif
