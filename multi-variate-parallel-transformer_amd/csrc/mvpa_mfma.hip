// placeholder until the tiled kernel lands
#include "mvpa_common.h"
int mvpa_mfma_supported(const mvpa_fwd_args*) { return 0; }
int mvpa_launch_mfma(const mvpa_fwd_args*, hipStream_t) { return MVPA_ERR_UNSUPPORTED; }
