// The norm of a decoder layer that norms every sublayer's input AND output in groups of channels.
//   group_norm_add: N(u; w) cuts a row into `groups` equal runs, divides each run by its own root mean square
//     and multiplies the row by w.  One launch takes a sublayer's output into the fp32 stream,
//         stream += layer_scale * N(s1 * y1 + s2 * y2; post_w),
//     and writes the next sublayer's (or the model's last) norm N(stream; w) of the new stream.
// All arithmetic is fp32.
#include "mixers_common.cuh"

namespace swm {

// One wave per (row, run of channels): no barrier anywhere.  The addend's norm, the stream update and the next norm
// of the same run all stay in the wave; values are read again where they are needed a second time (they sit in the
// cache: a run is a few KB).
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void group_norm_add_kernel(
    float* __restrict__ stream, const void* __restrict__ y1, int64_t y1_stride, float s1, const void* __restrict__ y2,
    int64_t y2_stride, float s2, const float* __restrict__ post_w, const float* __restrict__ layer_scale,
    const float* __restrict__ w, void* __restrict__ out, int groups, float eps, int64_t rows, int width) {
  const int64_t unit = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= rows * groups) return;                         // uniform over the wave
  const int lane = threadIdx.x & 63;
  const int64_t t = unit / groups;
  const int g = (int)(unit % groups), size = width / groups, c0 = g * size;
  float* x = stream + t * (int64_t)width + c0;
  if (y1 != nullptr) {
    float ss = 0.0f;
    for (int c = lane; c < size; c += 64) {
      float v = s1 * ld<TY>(y1, t * y1_stride + c0 + c);
      if (y2 != nullptr) v += s2 * ld<TY>(y2, t * y2_stride + c0 + c);
      ss += v * v;
    }
    ss = sw::wave_sum(ss);
    const float f = 1.0f / sqrtf(ss / (float)size + eps);
    for (int c = lane; c < size; c += 64) {
      float v = s1 * ld<TY>(y1, t * y1_stride + c0 + c);
      if (y2 != nullptr) v += s2 * ld<TY>(y2, t * y2_stride + c0 + c);
      v = v * f * post_w[c0 + c];
      if (layer_scale != nullptr) v *= layer_scale[c0 + c];
      x[c] += v;
    }
  }
  if (out == nullptr) return;
  float ss = 0.0f;
  for (int c = lane; c < size; c += 64) ss += x[c] * x[c];   // a lane reads back what it wrote itself
  ss = sw::wave_sum(ss);
  const float f = 1.0f / sqrtf(ss / (float)size + eps);
  for (int c = lane; c < size; c += 64) st<TO>(out, t * (int64_t)width + c0 + c, x[c] * f * w[c0 + c]);
}

}  // namespace swm

extern "C" int swm_group_norm_add(float* residual, const void* y1, int64_t y1_stride, float s1, const void* y2,
                                  int64_t y2_stride, float s2, int y_dtype, const float* post_w,
                                  const float* layer_scale, const float* w, void* out, int out_dtype, int groups,
                                  float eps, int64_t rows, int width, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(y_dtype) && act_ok(out_dtype), "group_norm_add: unsupported dtype %d / %d", y_dtype, out_dtype);
  SW_CHECK_ARG(width > 0 && groups > 0 && width % groups == 0 && rows * groups < (1ll << 32),
               "group_norm_add: width %d in %d groups", width, groups);
  SW_CHECK_ARG((y1 == nullptr && y2 == nullptr) || (y1 != nullptr && post_w != nullptr),
               "group_norm_add: an addend needs its norm's weight (and a second addend a first)");
  SW_CHECK_ARG(out == nullptr || w != nullptr, "group_norm_add: an output needs its norm's weight");
  const int waves = 4;
  const dim3 grid((unsigned)((rows * groups + waves - 1) / waves));
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SWM_GN_LAUNCH(TY, TO)                                                                                          \
  hipLaunchKernelGGL((group_norm_add_kernel<TY, TO>), grid, dim3(64 * waves), 0, s, residual, y1, y1_stride, s1, y2,   \
                     y2_stride, s2, post_w, layer_scale, w, out, groups, eps, rows, width)
  if (y_dtype == SW_F32) {
    if (out_dtype == SW_F32) SWM_GN_LAUNCH(float, float); else SWM_GN_LAUNCH(float, sw::bf16_t);
  } else {
    if (out_dtype == SW_F32) SWM_GN_LAUNCH(sw::bf16_t, float); else SWM_GN_LAUNCH(sw::bf16_t, sw::bf16_t);
  }
#undef SWM_GN_LAUNCH
  SW_CHECK_LAUNCH();
  return SW_OK;
}
