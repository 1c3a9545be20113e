/* Shared declarations of the flash-attention prefill example: O = softmax(scale * Q K^T + mask) V per
 * head, bf16 in, fp32 accumulate, bf16 out, grouped-query (several query heads share a KV head).
 *
 *   fa.core         role `core`, 4 waves: one workgroup owns 128 consecutive queries of one query head;
 *                   a wave owns 32 of them.  Streams 64-key blocks of K and V through LDS (V read
 *                   column-wise with the transposing LDS read), online softmax in registers, MFMA 32x32x16 bf16.
 *   fa.mask.causal  exports that say which keys a query may see; the core calls them through call
 *                   channels, so another mask is another package (campaigns/attention/src/sm90 in the
 *                   reference: stage_core.cu, stage_mask_default.cu / stage_mask_window.cu).
 * The output projection runs as a second linked pipeline (bf16 GEMM packages) on the [B * S, Hq * D]
 * matrix this stage writes. */
#ifndef PIPELINK_FA_ABI_H
#define PIPELINK_FA_ABI_H

#include <stdint.h>
#include <pipelink/host_view.h>

#define FA_D 128        /* head dimension */
#define FA_Q_TILE 128   /* queries per workgroup */
#define FA_K_BLOCK 64   /* keys per streamed block */

typedef struct FaCoreParams {
  const uint16_t* q; /* [B, Hq, S, D] bf16 */
  const uint16_t* k; /* [B, Hkv, S, D] */
  const uint16_t* v; /* [B, Hkv, S, D] */
  uint16_t* o;       /* [B, S, Hq * D] */
  int32_t batch, q_heads, kv_heads, seq; /* seq % 128 == 0 */
  float scale_log2e; /* softmax scale * log2(e) */
  int32_t reserved;
} FaCoreParams;

typedef struct FaMaskParams {
  int32_t seq;
  int32_t window; /* unused by the causal mask */
} FaMaskParams;

#endif
