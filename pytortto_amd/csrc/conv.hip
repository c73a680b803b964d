#include "tt_common.h"
extern "C" {
int tt_conv2d_fwd_f32(const float*, const float*, const float*, float*, int, int, int, int, int, int, int, int, int,
                      int, int, int, int, int) { return tt::fail(-1, "tt_conv2d_fwd_f32: not implemented"); }
int tt_conv2d_dgrad_f32(const float*, const float*, const float*, float*, int, int, int, int, int, int, int, int,
                        int, int, int, int, int, int, int, int) { return tt::fail(-1, "tt_conv2d_dgrad_f32: not implemented"); }
int tt_conv2d_wgrad_f32(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int, int,
                        int, int, int, int, int) { return tt::fail(-1, "tt_conv2d_wgrad_f32: not implemented"); }
}
