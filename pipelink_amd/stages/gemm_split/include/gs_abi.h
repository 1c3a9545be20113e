/* Shared declarations of the three-package GEMM example: C = GELU(A . B + bias), bf16 in, fp32
 * accumulate, bf16 out.  A is [M, K] row-major; B is handed over as B^T, [N, K] row-major (the
 * contraction index contiguous in both operands).
 *
 * The split follows the reference's three-package GEMM (examples/hopper-gemm-split: loader /
 * MMA / epilogue; contracts in src/channels.cuh:33-71) with GELU in place of its ReLU:
 *   gs.loader    role `load`, 2 waves (one for the A rows, one for the B rows): global -> LDS ring, one ring
 *                stage = 64 contraction elements of the tile's 128 A rows and 128 B rows (2 x 16 KB)
 *   gs.mma       role `mma`, 4 waves as 2 x 2, 64 x 64 outputs each: LDS -> MFMA 32x32x16 bf16
 *   gs.epilogue  an export the mma role calls with its accumulator: + bias, GELU, bf16 store */
#ifndef PIPELINK_GS_ABI_H
#define PIPELINK_GS_ABI_H

#include <stdint.h>
#include <pipelink/host_view.h>

#define GS_TILE_M 128
#define GS_TILE_N 128
#define GS_TILE_K 64                    /* contraction elements per ring stage */
#define GS_STAGE_BYTES (2 * 128 * 128)  /* A rows then B rows, 128 bytes each */
#define GS_LOAD_WAVES 2                 /* arrivals on a stage's `full` counter per fill: one per loader wave */

typedef struct GsLoaderParams {
  const uint16_t* a;  /* [M, K] bf16 */
  const uint16_t* bt; /* [N, K] bf16 */
  uint32_t* status;   /* [1], set to non-zero by a wait that gave up */
  int32_t m, n, k;    /* multiples of 128, 128, 64 */
  int32_t reserved;
} GsLoaderParams;

typedef struct GsMmaParams {
  uint32_t* status;
  int32_t n, k;
} GsMmaParams;

typedef struct GsEpilogueParams {
  const float* bias; /* [N] */
  uint16_t* c;       /* [M, N] bf16 */
  int32_t m, n;
} GsEpilogueParams;

/* which 128 x 128 tile a workgroup owns */
typedef struct GsTile {
  int32_t row0, col0;
} GsTile;

#ifdef __HIPCC__
/* Accumulator of one mma wave: [row fragment][column fragment] MFMA 32x32 C tiles.  Element
 * (register r, lane l) of tile (i, j) is
 *   row    = row0 + 64 * (wave / 2) + 32 * i + 8 * (r / 4) + 4 * (l / 32) + r % 4
 *   column = col0 + 64 * (wave % 2) + 32 * j + l % 32                                        */
typedef float gs_v16f __attribute__((ext_vector_type(16)));
struct GsAcc {
  gs_v16f v[2][2];
};
#endif

#endif
