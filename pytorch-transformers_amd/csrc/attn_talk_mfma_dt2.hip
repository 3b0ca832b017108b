// The attention with mixed heads on the matrix cores for heads of 32 elements (see attn_talk_mfma_impl.h).
#include "attn_talk_mfma_impl.h"

template bool talk_launch_head<2>(const TalkLaunch&, int);
