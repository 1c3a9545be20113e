/* Shared declarations of the decode megakernel example: one persistent kernel runs a whole decoding
 * step of a Llama-shaped model (RMSNorm, fused QKV matvec, RoPE, attention over the KV cache, output
 * projection, gate/up matvec + SwiGLU, down matvec, LM head) for one token.
 *
 * Packages (campaigns/megakernel/port/src in the reference: interpreter.cu + ops/*.cu wrapped as opcode
 * slots): mk.interp -- the persistent role: every workgroup walks the same instruction stream, calls the
 * op an instruction names through a call channel with its share of the work, and meets the others at a
 * grid barrier where an instruction asks for one (arriving after the op, waiting inside the next one: MkPending
 * below) -- and eight op packages: mk.rmsnorm, mk.qkv, mk.rope,
 * mk.attn, mk.oproj, mk.upgate, mk.down, mk.lmhead.  Swapping the attention package (mk.attn for
 * mk.attn.wide) and relinking changes nothing else.
 *
 * Everything an op needs is in MkModel, the interpreter's params; ops have no params of their own and
 * receive the interpreter's view. */
#ifndef PIPELINK_MK_ABI_H
#define PIPELINK_MK_ABI_H

#include <stdint.h>
#include <pipelink/host_view.h>

#define MK_THREADS 256
#define MK_HEAD_DIM 64
// floats per (head, context chunk) of the attention partials: 64 unnormalised outputs, the chunk's maximum (log2
// units), its sum of exponentials, two floats of padding (rows stay 16-byte aligned)
#define MK_PARTIAL_STRIDE (MK_HEAD_DIM + 4)

/* Opcodes are not constants of this header: each op package claims one number in the link's "opcode" domain
 * (pipelink_mk_opcode_<op>), the pipeline binds the numbers, the interpreter and the ops read them through the
 * handle functions, and the host takes them from link.json ("bindings") when it writes the instruction stream.
 * An opcode nobody claimed is a no-op.  The ops:
 *   rmsnorm_attn   x * rsqrt(mean x^2 + eps) * attn_norm[layer]  -> LDS vector      (rmsnorm_ffn, rmsnorm_final alike)
 *   qkv            qkv = Wqkv[layer] . vector
 *   attn           RoPE, append to the cache, partial attention of (head, chunk)
 *   oproj          combine the partials; x += Wo[layer] . attention
 *   upgate         h = silu(Wgate . vector) * (Wup . vector)
 *   down           x += Wdown . h
 *   lmhead         logits = Wlm . vector */

/* one instruction: 4 x int32 */
typedef struct MkInstr {
  int32_t opcode, layer, barrier_after, reserved;
} MkInstr;

/* What stands between an op and its inputs when the interpreter calls it.  A grid barrier is in two halves: a
 * workgroup arrives when it has finished an op, and waits for the others only when the next op needs what they
 * wrote.  An op therefore first asks for what depends on nobody -- its first rows of weights, its first stretch of
 * the cache -- and then calls the interpreter's `op_inputs` channel once, which waits for the barrier (if one is
 * open) and runs the normalisation that fills the workgroup's LDS vector (if the instruction before was one).
 * Before that call an op may read only what no op writes during the step and may not touch the LDS vector.  An op
 * that returns without the call has the interpreter make it. */
typedef struct MkPending {
  const MkInstr* norm; /* an rmsnorm instruction whose result the op needs, or null */
  uint32_t barrier;    /* the barrier of this launch to wait for (1, 2, ...), 0: none */
} MkPending;

typedef struct MkModel {
  const uint16_t* weights; /* bf16; per layer: attn_norm[D], wqkv[(HQ+2HKV)*64][D], wo[D][HQ*64], ffn_norm[D], wgate[DFF][D],
                              wup[DFF][D], wdown[D][DFF]; then final_norm[D], lm_head[V][D] */
  uint16_t* kv_cache;      /* bf16 [L][2][SMAX][HKV][64] */
  float* x;                /* [D] residual stream, in and out */
  float* qkv;              /* [(HQ + 2 HKV) * 64] */
  float* attn_partial;     /* [HQ][chunks][MK_PARTIAL_STRIDE]: unnormalised output, maximum (log2 units), sum */
  float* h;                /* [DFF] */
  float* logits;           /* [V] */
  const float* rope;       /* [2][32]: cos, sin of pos * theta^(-2 i / 64) */
  const MkInstr* program;
  uint32_t* sync;          /* 1024 words, all zero before the first launch.  [0] grid barrier arrivals, [1] status (bit 0: a
                              wait gave up; sticky, the host clears it), [2] count of workgroups that have finished,
                              [3] launches closed so far, [32 * (1 + xcd)] arrivals of one XCD's workgroups, [.. + 1] the
                              generation its leader passed on, [.. + 2] its workgroups that have finished, [512 + b]
                              0x100 | the XCC workgroup b ran on (written by the first launch).  A launch leaves
                              every word but [1], [3] and [512 ..] at zero. */
  int32_t num_instr, layers, d, hq, hkv, dff, vocab, pos, smax, chunks;
  float eps, attn_scale_log2e;
} MkModel;

#ifdef __cplusplus
#ifdef __HIPCC__
__host__ __device__
#endif
static inline int64_t mk_layer_elems(const MkModel* m) {
  const int64_t d = m->d, qkv = (int64_t)(m->hq + 2 * m->hkv) * MK_HEAD_DIM;
  return d + qkv * d + d * (int64_t)m->hq * MK_HEAD_DIM + d + 2 * (int64_t)m->dff * d + d * (int64_t)m->dff;
}
#endif

#endif
