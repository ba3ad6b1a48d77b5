// ws_fused.hip once more, as the build that can write the kept-set dump (ws_batch.kept_ids).
#define WS_KEPT_BUILD true
#define WS_LAUNCH launch_fused_kept
#define WS_PREPARE prepare_fused_kept
#include "ws_fused.hip"
