#include "common.h"
extern "C" int mjt_conv2d_meta(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y, const mjt_conv_params* p) {
    return mjt::guarded([&] { MJT_FAIL(MJT_ERR_UNSUPPORTED, "conv2d_meta: not built yet"); });
}
