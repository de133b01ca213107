// placeholder until the fp8 kernel lands
#include "hdit_common.h"
extern "C" __attribute__((visibility("default"))) int hdit_attn_absmax(const hdit_attn_args*, float*, void*) { return HDIT_EUNSUPPORTED; }
extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_fp8(const hdit_attn_args*, const float*, void*) { return HDIT_EUNSUPPORTED; }
