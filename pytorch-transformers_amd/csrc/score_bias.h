// What the attention launches make of a PtaScoreBias (pta_kernels.h): one of the three ways the kernels form the
// bias, or a refusal by name.
#pragma once

#include "common.h"
#include "pta_kernels.h"

// mode: 0 slope x key position with the position and the product rounded to bfloat16, 1 the same exact, 2 slope x
// (key position - query position) exact.  Returns 0, or nonzero with the reason in pta_last_error.
static inline int pta_score_bias_mode(const char* what, const PtaScoreBias* b, int* mode) {
    *mode = 1;
    if (!b || !b->slopes) return 0;
    PTA_REQUIRE(b->of == PTA_BIAS_KEY || b->of == PTA_BIAS_DISTANCE,
                "%s: a score bias of kind %d is not built; built are slope x key position and slope x (key position - "
                "query position), one slope per head", what, b->of);
    PTA_REQUIRE(!b->bf16 || b->of == PTA_BIAS_KEY,
                "%s: rounding to bfloat16 as the reference rounds is built for slope x key position only", what);
    *mode = b->of == PTA_BIAS_DISTANCE ? 2 : b->bf16 ? 0 : 1;
    return 0;
}
