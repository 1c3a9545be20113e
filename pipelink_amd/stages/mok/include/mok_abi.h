/* MoK (routed-expert FFN) call ABI shared by the framework, GEMM and activation owners,
 * host and device.  Plain C structs only; tile geometry of one owner reaches another only
 * through the task records the framework fills in.
 *
 * Mirrors the role of campaigns/mok/port/include/mok_abi.h:15-17 (MokCounters),
 * campaigns/mok/port/gemm/gemm_abi.h:7-13 (MokGemmTask) and
 * campaigns/mok/port/act_gptoss/act_abi.h:8-15 (MokActTask).  Field sets differ: TMA
 * descriptors and CLC/cluster ranks have no gfx950 counterpart, and one task here is one
 * workgroup tile whose gate and up halves are produced together so that the activation
 * runs on the accumulator instead of on a bf16 round trip through HBM. */
#ifndef PIPELINK_MOK_ABI_H
#define PIPELINK_MOK_ABI_H

#include <stdint.h>

#ifndef MOKCOUNTERS_DEFINED
#define MOKCOUNTERS_DEFINED
typedef struct MokCounters {
  int32_t* base; /* dependency counters lent by the framework to every op call: base[t] counts the gate/up tiles of
                    routed-row tile t whose `hidden` columns are in memory (campaigns/mok/port/gemm/gemm.cu:364-382:
                    the reference's readiness counts); null when the launch runs one GEMM only */
  uint32_t* status; /* sticky word of the launch: MOK_STATUS_* bits, raised by a wait that gave up */
} MokCounters;
#endif
enum { MOK_STATUS_WAIT_GAVE_UP = 1 };

/* op codes keep the reference's names; GATE and UP of one tile are issued as one task */
enum {
  MOK_FWD_BOTH = 0,                /* framework params only: gate/up tiles, then down tiles, in one launch */
  MOK_GEMM_FWD_ROUTED_GATE_UP = 3, /* = MOK_GEMM_FWD_ROUTED_GATE of the reference */
  MOK_GEMM_FWD_ROUTED_DOWN = 5
};
enum { MOK_ACT_FWD_ROUTED = 1 };

#ifndef MOKGEMMTASK_DEFINED
#define MOKGEMMTASK_DEFINED
typedef struct MokGemmTask {
  int32_t op;        /* MOK_GEMM_FWD_ROUTED_GATE_UP or MOK_GEMM_FWD_ROUTED_DOWN */
  int32_t expert;    /* local expert whose weights this tile multiplies */
  int32_t row_begin; /* first routed row of the tile */
  int32_t row_end;   /* one past the expert's last routed row; rows >= row_end are padding */
  int32_t col_begin; /* first output column of the tile (per weight matrix) */
  int32_t task_idx;  /* running index of the tile in the schedule */
  int32_t counter_idx; /* readiness counter of the tile's routed-row tile (a launch of both GEMMs), or -1 */
  int32_t wait_target; /* down op: value that counter must have reached before the tile's rows of `hidden` are read
                          (the number of gate/up column tiles); 0 = the tile waits for nothing */
  uint32_t flags;
} MokGemmTask;
#endif

#ifndef MOKACTTASK_DEFINED
#define MOKACTTASK_DEFINED
typedef struct MokActTask {
  int32_t op;        /* MOK_ACT_FWD_ROUTED */
  int32_t row_begin, row_end, col_begin;
  int32_t task_idx;
  int32_t counter_idx; /* counter to bump once the tile's `hidden` columns are in memory, or -1 */
  uint32_t flags;
} MokActTask;
#endif

/* One MXFP8 operand: e4m3 codes [rows, k] (row pitch ld_q bytes) and e8m0 scales, one byte
 * per 32 k-elements.  Activations keep their scales row-major [rows, ld_sc] with ld_sc a
 * multiple of 16 (one 16-byte piece = the scales of four 128-element ring slots).  Weights
 * keep them slot-major, [ceil(k/128), rows, 4] per expert, so the scales one workgroup tile
 * needs for one ring slot are contiguous; ld_sc is unused for them.  Weights carry an expert
 * pitch on both arrays. */
typedef struct MokMxView {
  const uint8_t* q;
  const uint8_t* sc;
  int64_t expert_pitch_q;
  int64_t expert_pitch_sc;
  int32_t rows; /* rows per expert for weights, total rows for activations */
  int32_t k;
  int32_t ld_q;
  int32_t ld_sc;
} MokMxView;

/* Residue of the GEMM owner: every device address and extent its exports read. */
typedef struct MokGemmResidue {
  MokMxView x;       /* activations in token order [T, H] */
  MokMxView hidden;  /* SwiGLU output in routed-row order [R, I] (read by the down GEMM) */
  MokMxView w_gate;  /* [E, I, H] */
  MokMxView w_up;    /* [E, I, H] */
  MokMxView w_down;  /* [E, H, I] */
  const int32_t* row_token; /* [R] routed row -> token row of x; null = identity */
  uint16_t* y;       /* bf16 [R, H] */
  int32_t ld_y;      /* elements */
  int32_t reserved;
} MokGemmResidue;

/* Residue of the activation owner. */
typedef struct MokActResidue {
  uint8_t* hidden_q;  /* e4m3 [R, I] */
  uint8_t* hidden_sc; /* e8m0 [R, ld_sc] */
  int32_t rows, cols, ld_q, ld_sc;
  float swiglu_limit;
  int32_t reserved;
} MokActResidue;

/* Params of the framework role: the schedule. */
typedef struct MokFrameworkParams {
  const int32_t* tokens_per_expert; /* [E] */
  uint32_t* workspace;              /* MOK_WS_* words + one counter per routed-row tile; all zero before a launch,
                                       and the launch leaves them zero (except the status word and the poll limit) */
  int32_t num_experts;
  int32_t op;                       /* which GEMM this launch runs, or MOK_FWD_BOTH */
  int32_t num_col_tiles_gate_up;    /* column tiles of the gate/up GEMM (128 gate + 128 up columns each) */
  int32_t num_col_tiles_down;       /* column tiles of the down GEMM (256 columns each) */
} MokFrameworkParams;
/* workspace words */
enum {
  MOK_WS_STATUS = 0,    /* sticky MOK_STATUS_* bits; the host reads and clears it */
  MOK_WS_FINISHED = 1,  /* workgroups that have left the launch; the last one clears the counters */
  MOK_WS_POLL_LIMIT = 2, /* 0, or the number of polls after which a dependency wait gives up instead of the default 2^14
                            (for tests of the give-up path: the kernels never write it) */
  MOK_WS_GAVE_UP = 3,   /* non-zero once a dependency wait of the running launch has given up: every later wait of that
                            launch gives up at once; the launch's last workgroup puts it back to zero */
  MOK_WS_QUEUE = 8,     /* eight words, one per tile list: how many of the list's tiles have been handed out beyond the two
                            every workgroup starts with; the launch's last workgroup puts them back to zero */
  MOK_WS_COUNTERS = 32  /* first readiness counter */
};

/* The shared scalars every owner of this pipeline is handed (ids of include/plk_host_abi_v2.h); a stage source
 * invokes this among its annotations, after <pipelink/stage.hpp>. */
#define MOK_HOST_SCALARS()                                \
  PL_HOST_SCALAR(1, "mok.num_local_tokens", "i64");       \
  PL_HOST_SCALAR(2, "mok.hidden", "i64");                 \
  PL_HOST_SCALAR(3, "mok.intermediate", "i64");           \
  PL_HOST_SCALAR(4, "mok.num_local_experts", "i64");      \
  PL_HOST_SCALAR(10, "mok.swiglu_limit", "f64");          \
  PL_HOST_SCALAR(11, "mok.pass", "i64");                  \
  PL_HOST_SCALAR(12, "mok.precision", "i64");             \
  PL_HOST_SCALAR(60, "mok.routed_rows", "i64");           \
  PL_HOST_SCALAR(61, "mok.ld_q_h", "i64");                \
  PL_HOST_SCALAR(62, "mok.ld_q_i", "i64");                \
  PL_HOST_SCALAR(63, "mok.ld_sc_h", "i64");               \
  PL_HOST_SCALAR(64, "mok.ld_sc_i", "i64");               \
  PL_HOST_SCALAR(65, "mok.workspace_words", "i64")

/* First argument of every owner export (pack/include/pipelink/host_view.h in the reference). */
#ifndef PIPELINK_HOST_VIEW_DEFINED
#define PIPELINK_HOST_VIEW_DEFINED
typedef struct pipelink_host_view {
  const void* residue;
  const void* scalars;
} pipelink_host_view;
#endif

#endif
