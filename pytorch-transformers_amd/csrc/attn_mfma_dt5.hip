// The attention on the matrix cores for heads of 80 elements (see attn_mfma_impl.h).
#include "attn_mfma_impl.h"

template int attn_launch_head<5>(const AttnLaunch&, bool, bool, bool, int);
