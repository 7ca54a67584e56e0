// lr_ladder_decode_step_fp8: the one-kernel decode step of ladder_step.hip for weight-only e4m3 projections
// (see LR_STEP_W8 there).  Workspace size, layout and initialisation are those of the bf16 step
// (lr_ladder_step_workspace_bytes / lr_ladder_step_init / lr_ladder_step_fail_offset).
#define LR_STEP_W8 1
#include "ladder_step.hip"
