// The attention with mixed heads on the matrix cores for heads of 112 elements (see attn_talk_mfma_impl.h).
#include "attn_talk_mfma_impl.h"

template bool talk_launch_head<7>(const TalkLaunch&, int);
