/* C ABI of the routed-expert MXFP8 FFN forward (the "MoK" hot path) on gfx950.
 *
 * What the reference reaches through MoKHost.forward -> HostSession.launch
 * (campaigns/mok/host/mok_port_host.py:185-205, pipec/src/pipec2/host/broker.py:741-751)
 * with the residues its owner providers build
 * (campaigns/mok/port/gemm/provider.cu:217-303, campaigns/mok/port/act_gptoss/provider.cu),
 * is reached here through plk_mok_session_create + plk_mok_forward: the session owns one
 * loaded pipeline image (linked or one-unit build) and its device-resident params images;
 * forward fills the framework / GEMM / activation params and launches the gate-up pass
 * and the down pass on the caller's stream.  All tensor arguments are device addresses
 * owned by the caller; nothing is allocated per call.
 *
 * Operand layouts.  Activations are row-major; a code row may be padded to a pitch ld_q >= K,
 * a multiple of 16 -- a pitch that is a multiple of 128 makes every 128-byte piece of a row
 * one aligned cache line, which is what the loader is fastest on:
 *   x_q [T,ld_q_h] e4m3, x_sc [T,ld_sc_h] e8m0 (one byte per 32 elements of H; ld_sc_h % 16 == 0)
 * Weights are stored the way the GEMM streams them; convert once, when the weights are loaded:
 *   w_gate_q / w_up_q (N = I, K = H), w_down_q (N = H, K = I): K-TILED codes [E, K/64, N, 64]
 *   (64 contraction bytes of consecutive rows are contiguous) -- plk_mxfp8_codes_to_k64_tiled
 *   weight scales SLOT-MAJOR [E, ceil(K/128), N, 4] (the 4 scale bytes of 128 contraction
 *   elements of one row are a dword, and one slot's dwords of consecutive rows are
 *   contiguous) -- plk_mxfp8_scales_to_slot_major
 *   tokens_per_expert [E] i32, row_token [R] i32 (routed row -> token; 0 = rows are tokens)
 *   hidden_q [R,I] e4m3 + hidden_sc [R,ld_sc_i] (written by pass 1, read by pass 2)
 *   y [R,H] bf16 */
#ifndef PLK_MOK_H
#define PLK_MOK_H

#include "plk_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* what link.json says about the image (pipec link output: params.entries, threads, dyn_smem_bytes) */
typedef struct plk_mok_link_info {
  uint32_t struct_bytes;       /* sizeof(plk_mok_link_info) */
  uint32_t params_bytes;       /* total size of the params image */
  uint32_t framework_offset;   /* offset of MokFrameworkParams in the image */
  uint32_t gemm_offset;        /* offset of MokGemmResidue */
  uint32_t act_offset;         /* offset of MokActResidue */
  uint32_t threads;            /* workgroup size */
  uint32_t dyn_lds_bytes;      /* dynamic LDS per workgroup */
  uint32_t workgroups_per_cu;  /* occupancy the image was solved for */
} plk_mok_link_info;

typedef struct plk_mok_problem {
  uint32_t struct_bytes; /* sizeof(plk_mok_problem) */
  int32_t num_tokens;    /* T */
  int32_t hidden;        /* H = d_model */
  int32_t intermediate;  /* I = d_ff */
  int32_t num_experts;   /* E */
  int32_t routed_rows;   /* R = sum(tokens_per_expert) */
  int32_t ld_sc_h;       /* scale row pitch for K = H operands */
  int32_t ld_sc_i;       /* scale row pitch for K = I operands */
  int32_t ld_q_h;        /* code row pitch in bytes of x; 0 = H */
  int32_t ld_q_i;        /* code row pitch in bytes of hidden; 0 = I */
  float swiglu_limit;
  int32_t reserved;
  uint64_t x_q, x_sc, row_token, tokens_per_expert;
  uint64_t w_gate_q, w_gate_sc, w_up_q, w_up_sc, w_down_q, w_down_sc;
  uint64_t hidden_q, hidden_sc, y;
} plk_mok_problem;

typedef struct plk_mok_session plk_mok_session;

int plk_mok_session_create(const void* image, size_t image_bytes, const plk_mok_link_info* link, plk_mok_session** out);
int plk_mok_session_destroy(plk_mok_session* s);
/* The forward.  plk_mok_forward runs both GEMMs in ONE launch when every row of hidden_q is a whole number of
 * 128-byte cache lines (hidden_q and ld_q_i multiples of 128): down tiles wait on per-row-tile readiness counters that
 * the gate/up tiles bump (campaigns/mok/port/framework/interp_fwd.cu:174-213, gemm/gemm.cu:364-382 in the reference).
 * With any other pitch it is two launches, pass 1 then pass 2.  plk_mok_forward_pass runs one of them (pass 1 = gate/up
 * + SwiGLU + requant, pass 2 = down).  The session keeps the params image of the last problem per kind of launch on
 * the device: a call with the same problem only launches (and can be captured into a graph); a call with another
 * problem first uploads its image, which synchronises the stream -- on a stream that is being captured that call
 * returns PLK_E_CONTRACT.  A problem with more routed-row tiles than any before also makes the session replace its
 * launch workspace (device synchronisation, same rule under capture).
 * The one-launch forward counts on its workgroups (one per CU) all running at once, and its counters belong to the
 * session: forwards of one session must not overlap (one stream, or streams ordered by events).  A forward launched
 * while another kernel holds CUs may see a down tile give up its bounded wait: the first wait that gives up takes 2^14
 * polls (a few tens of milliseconds), every other wait of that launch then ends at once, the launch completes, the call
 * has long returned PLK_OK, and `y` of that forward is void -- plk_mok_status tells, and from the first give-up it
 * reports the session runs every later forward as two launches.  A caller that shares the GPU with other work asks for
 * that from the start: plk_mok_session_launches(s, 2); plk_mok_forward_pass 1 then 2 has no dependency inside a launch
 * either. */
int plk_mok_forward(plk_mok_session* s, const plk_mok_problem* p, void* stream);
int plk_mok_forward_pass(plk_mok_session* s, const plk_mok_problem* p, int pass, void* stream);
/* How plk_mok_forward and plk_mok_forward_static launch from now on: 1 = one launch whenever hidden_q allows it (the
 * default), 2 = always pass 1 then pass 2.  No counterpart in the reference, whose cluster launch has no such choice. */
int plk_mok_session_launches(plk_mok_session* s, int launches);

/* Waits for the stream, then returns and clears the sticky status of the session's launches: 0, or MOK_STATUS_* bits
 * (bit 0: a down tile gave up waiting for its rows of `hidden` after 2^14 polls and multiplied what was there --
 * the outputs of that forward are not to be trusted; the session switches to two launches per forward).  The waits are
 * bounded so that a launch always ends.  Forwards through plk_mok_forward_static keep their status in the library's
 * per-GPU area, which every session on that GPU shares: the session that asks first gets (and clears) the bit. */
int plk_mok_status(plk_mok_session* s, void* stream, uint32_t* status);

/* plk_mok_forward for callers that cannot allocate or wait: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  It calls no hipMalloc / hipFree and no
 * allocating library routine, copies nothing from host memory and never synchronises: what plk_mok_forward keeps in
 * session-owned device buffers -- the launches' params images (at most PLK_MOK_STATIC_IMAGE_BYTES each, else
 * PLK_E_CAPACITY) and the launch workspace of readiness counters (32 + ceil(routed_rows / 256) +
 * num_experts words, at most PLK_MOK_STATIC_WORKSPACE_WORDS, else PLK_E_CAPACITY) -- lives in a fixed area of device
 * memory that belongs to the library (66 KB per GPU, held until the process ends; its address is resolved when a
 * session is created on that GPU) and is written by a small kernel ahead of the launches in stream order, which also
 * clears the workspace.  The session's device must be the current one.  Every call on a GPU shares that GPU's area:
 * calls that overlap on one GPU (two streams, two threads) race on it; calls in one stream do not.
 * Results are byte for byte those of plk_mok_forward. */
#define PLK_MOK_STATIC_IMAGE_BYTES 1024
#define PLK_MOK_STATIC_WORKSPACE_WORDS 16384
int plk_mok_forward_static(plk_mok_session* s, const plk_mok_problem* p, void* stream);

/* MXFP8 block quantiser on the device (what ops.mxfp8_quantize does for the reference's
 * harness, campaigns/mok/host/mok_port_host.py:122): src is fp32 (src_is_bf16 = 0) or bf16
 * [rows, k], dst_q [rows, ld_q] e4m3 (ld_q >= k; pad bytes untouched), dst_sc [rows, ld_sc] e8m0
 * (padding bytes zeroed). */
int plk_mxfp8_quantize(uint64_t src, int src_is_bf16, int64_t rows, int32_t k, uint64_t dst_q, int32_t ld_q,
                       uint64_t dst_sc, int32_t ld_sc, void* stream);

/* Row-major e8m0 scales src [rows, ld_sc] -> slot-major dst [ceil(k/128), rows, 4] (pad bytes 0).
 * For a weight tensor [E, N, K] call it once per expert (or once with rows = E*N when the
 * caller wants one slot-major block per expert, use rows = N and offset the pointers). */
int plk_mxfp8_scales_to_slot_major(uint64_t src, int64_t rows, int32_t k, int32_t ld_sc, uint64_t dst, void* stream);

/* Row-major e4m3 codes src [rows, ld_q] -> K-tiled dst [k/64, rows, 64] (k % 64 == 0, ld_q % 16 == 0,
 * 16-byte aligned addresses).  For a weight tensor [E, N, K] call it once per expert with rows = N. */
int plk_mxfp8_codes_to_k64_tiled(uint64_t src, int64_t rows, int32_t k, int64_t ld_q, uint64_t dst, void* stream);

#ifdef __cplusplus
}
#endif
#endif
