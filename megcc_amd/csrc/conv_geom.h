// Geometry of one ConvBias call, derived on the host from the Tensor layouts the way the reference
// kernel derives it at run time (BareMetal/ConvKernel.cpp:269-287), and handed to the kernels by
// value.
#pragma once
#include <stdint.h>

#include "megcc_gfx950.h"

namespace mg {

struct ConvGeom {
    int n, ic, ih, iw, oc, oh, ow;
    int fh, fw, sh, sw, ph, pw, dh, dw;
    int groups;  // 1 for DENSE
    int fmt;     // MegccFormat
    int act;     // MegccNonline
    int has_bias;
    float s_src, s_flt, s_dst;
};

}  // namespace mg
