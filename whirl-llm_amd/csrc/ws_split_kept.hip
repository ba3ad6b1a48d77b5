// ws_split.hip once more, as the build that can write the kept-set dump (ws_batch.kept_ids).
#define WS_KEPT_BUILD true
#define WS_LAUNCH launch_split_kept
#define WS_PREPARE prepare_split_kept
#include "ws_split.hip"
