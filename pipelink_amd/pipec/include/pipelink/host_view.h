/* First argument of every export of a stage that has a params blob: where the stage's own
 * params ("residue") and the pipeline's shared scalars are.  The link-generated trampoline
 * re-bases a caller's view onto the callee's params inside the shared image.
 * (pack/include/pipelink/host_view.h in the reference.) */
#ifndef PIPELINK_HOST_VIEW_DEFINED
#define PIPELINK_HOST_VIEW_DEFINED
typedef struct pipelink_host_view {
  const void* residue;
  const void* scalars;
} pipelink_host_view;
#endif
