// The attention with mixed heads on the matrix cores for heads of 16 elements (see attn_talk_mfma_impl.h).
#include "attn_talk_mfma_impl.h"

template bool talk_launch_head<1>(const TalkLaunch&, int);
