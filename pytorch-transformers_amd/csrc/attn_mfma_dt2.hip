// The attention on the matrix cores for heads of 32 elements (see attn_mfma_impl.h).
#include "attn_mfma_impl.h"

template int attn_launch_head<2>(const AttnLaunch&, bool, bool, bool, int);
