// The attention on the matrix cores for heads of 48 elements (see attn_mfma_impl.h).
#include "attn_mfma_impl.h"

template int attn_launch_head<3>(const AttnLaunch&, bool, bool, bool, int);
