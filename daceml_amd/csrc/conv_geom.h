// Geometry of a 2-D convolution after validation (all extents fit an int): shared by the convolution sources.
#pragma once

namespace dml {

struct ConvGeom {
    int n, c, h, w, m, kh, kw, sh, sw, ph, pw, dh, dw, group, oh, ow, cg, mg, act;
};

}  // namespace dml
