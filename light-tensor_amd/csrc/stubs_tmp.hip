#include "common.h"
extern "C" {
#define STUB(name, ...) int name(__VA_ARGS__) { lten_hip::set_error(#name ": not built yet"); return 3; }
STUB(lten_hip_sgemm, int, int, uint64_t, uint64_t, uint64_t, float, const float*, uint64_t, const float*, uint64_t, float, float*, uint64_t)
STUB(lten_hip_sgemm_strided_batched, int, int, uint64_t, uint64_t, uint64_t, float, const float*, uint64_t, int64_t, const float*, uint64_t, int64_t, float, float*, uint64_t, int64_t, uint64_t)
STUB(lten_hip_fc_forward_f32, uint64_t, uint64_t, uint64_t, const float*, const float*, const float*, float*)
STUB(lten_hip_fc_backward_f32, uint64_t, uint64_t, uint64_t, const float*, const float*, const float*, float*, float*, float*)
STUB(lten_hip_im2col_f32, const float*, int, int, int, int, int, int, int, int, int, int, int, float*)
STUB(lten_hip_im2col_u8, const uint8_t*, int, int, int, int, int, int, int, int, int, int, int, uint8_t*)
STUB(lten_hip_col2im_f32, const float*, int, int, int, int, int, int, int, int, int, int, int, float*)
STUB(lten_hip_conv2d_forward_f32, uint64_t, uint64_t, uint64_t, uint64_t, uint64_t, int, int, int, int, int, int, const float*, const float*, const float*, float*)
STUB(lten_hip_conv2d_wgrad_f32, uint64_t, uint64_t, uint64_t, uint64_t, uint64_t, int, int, int, int, int, int, const float*, const float*, float*, void*)
uint64_t lten_hip_conv2d_wgrad_workspace_bytes(uint64_t, uint64_t, uint64_t, uint64_t, uint64_t, int, int, int, int, int, int) { return 0; }
}
