// Pieces of a decoder layer whose sublayer outputs enter an fp32 stream through a learned gate and whose layers
// receive a weighted mix of the outputs of ALL earlier layers:
//   * gated_stream_step: v = stream + mult * y * sigmoid(gate); optionally v is filed as the newest entry of a
//     history of layer outputs and replaced by the history's weighted sum; optionally the next norm of v, an
//     element-wise tanh norm tanh(alpha v) w + b (no statistics of the row), leaves in the activation dtype;
//   * poly_norm: a feed-forward activation a U(z) + b U(z^2) + c U(z^3) + e, U = division of the row by its root
//     mean square;
//   * gate_mul: y * sigmoid(gate) or y * silu(gate) between two library GEMMs;
//   * latent_rope_cache: the cache write and the query layout of attention whose keys and values are one low-rank
//     latent per token plus one rotated key part shared by all heads.
// All arithmetic is fp32; activations are read and written in the model's dtype.
#include "mixers_common.cuh"

namespace swm {

constexpr int kGsThreads = 256;

template <typename T>
__global__ __launch_bounds__(kGsThreads) void gated_stream_step_kernel(
    float* __restrict__ stream, const void* __restrict__ y, int64_t y_stride, const void* __restrict__ gate,
    int64_t gate_stride, float mult, float* __restrict__ history, int64_t layer_stride,
    const float* __restrict__ depth_weights, int entries, const float* __restrict__ norm_alpha,
    const float* __restrict__ norm_weight, const float* __restrict__ norm_bias, void* __restrict__ out, int width) {
  const int64_t t = blockIdx.x;
  const float alpha = out != nullptr ? norm_alpha[0] : 0.0f;
  for (int i = blockIdx.y * kGsThreads + threadIdx.x; i < width; i += gridDim.y * kGsThreads) {
    const int64_t at = t * (int64_t)width + i;
    float v = stream[at];
    if (y != nullptr) {
      float add = ld<T>(y, t * y_stride + i);
      if (gate != nullptr) add *= sigmoidf_(ld<T>(gate, t * gate_stride + i));
      v += mult * add;
    }
    if (history != nullptr) {
      history[(int64_t)(entries - 1) * layer_stride + at] = v;
      float mix = 0.0f;
      for (int j = 0; j + 1 < entries; ++j) mix += depth_weights[j] * history[(int64_t)j * layer_stride + at];
      v = mix + depth_weights[entries - 1] * v;
    }
    if (y != nullptr || history != nullptr) stream[at] = v;
    if (out != nullptr) st<T>(out, at, tanhf(alpha * v) * norm_weight[i] + norm_bias[i]);
  }
}

// one workgroup per row: the three mean squares in one pass, the combination in a second
template <typename T>
__global__ __launch_bounds__(kGsThreads) void poly_norm_kernel(void* __restrict__ out, const void* __restrict__ z,
                                                               int64_t z_stride, const float* __restrict__ coef,
                                                               float eps, int ff) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  for (int i = threadIdx.x; i < ff; i += kGsThreads) {
    const float v = ld<T>(z, t * z_stride + i);
    const float v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  s3 = block_sum(s3, red);
  const float n = (float)ff;
  const float f1 = coef[0] / sqrtf(s1 / n + eps), f2 = coef[1] / sqrtf(s2 / n + eps),
              f3 = coef[2] / sqrtf(s3 / n + eps), e = coef[3];
  for (int i = threadIdx.x; i < ff; i += kGsThreads) {
    const float v = ld<T>(z, t * z_stride + i);
    st<T>(out, t * (int64_t)ff + i, f1 * v + f2 * (v * v) + f3 * (v * v * v) + e);
  }
}

// y [rows, heads, size] with strides -> out [rows, heads * size] = y * (silu ? gate sigmoid(gate) : sigmoid(gate))
template <typename T>
__global__ __launch_bounds__(kGsThreads) void gate_mul_kernel(void* __restrict__ out, const void* __restrict__ y,
                                                              int64_t y_row_stride, int64_t y_head_stride,
                                                              const void* __restrict__ gate, int64_t gate_stride,
                                                              int heads, int size, int silu) {
  const int64_t t = blockIdx.x;
  const int n = heads * size;
  for (int i = blockIdx.y * kGsThreads + threadIdx.x; i < n; i += gridDim.y * kGsThreads) {
    const int h = i / size, c = i % size;
    const float g = ld<T>(gate, t * gate_stride + i);
    const float f = silu ? g * sigmoidf_(g) : sigmoidf_(g);
    st<T>(out, t * (int64_t)n + i, ld<T>(y, t * y_row_stride + h * y_head_stride + c) * f);
  }
}

// one workgroup per row.  Queries: q_out[t, h] = q_latent[t, h, :rank] | rotate(q_rot[t, h, :rot]);
// cache[slot] = down[t, :rank] / rms * norm_weight | rotate(down[t, rank:rank + rot]); pairs are neighbours.
template <typename T>
__global__ __launch_bounds__(kGsThreads) void latent_rope_cache_kernel(
    float* __restrict__ q_out, const void* __restrict__ q_latent, int64_t ql_row_stride, int64_t ql_head_stride,
    const void* __restrict__ q_rot, int64_t qr_row_stride, int64_t qr_head_stride, const void* __restrict__ down,
    int64_t down_stride, const float* __restrict__ norm_weight, float eps, const int64_t* __restrict__ positions,
    const float* __restrict__ inv_freq, void* __restrict__ cache, const int64_t* __restrict__ slot_mapping, int heads,
    int rank, int rot) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int row = rank + rot, pairs = rot / 2;
  for (int e = threadIdx.x; e < heads * rank; e += kGsThreads) {
    const int h = e / rank, c = e % rank;
    q_out[(t * heads + h) * (int64_t)row + c] = ld<T>(q_latent, t * ql_row_stride + h * ql_head_stride + c);
  }
  for (int e = threadIdx.x; e < heads * pairs; e += kGsThreads) {
    const int h = e / pairs, i = e % pairs;
    const int64_t src = t * qr_row_stride + h * qr_head_stride + 2 * i;
    const float a = ld<T>(q_rot, src), b = ld<T>(q_rot, src + 1);
    float s, c;
    sincosf(pos * inv_freq[i], &s, &c);
    float* dst = q_out + (t * heads + h) * (int64_t)row + rank + 2 * i;
    dst[0] = a * c - b * s;
    dst[1] = b * c + a * s;
  }
  if (down == nullptr) return;
  const int64_t slot = slot_mapping[t];                      // uniform over the workgroup
  float ss = 0.0f;
  for (int c = threadIdx.x; c < rank; c += kGsThreads) {
    const float v = ld<T>(down, t * down_stride + c);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  if (slot < 0) return;
  const float f = 1.0f / sqrtf(ss / (float)rank + eps);
  for (int c = threadIdx.x; c < rank; c += kGsThreads)
    st<T>(cache, slot * (int64_t)row + c, ld<T>(down, t * down_stride + c) * f * norm_weight[c]);
  for (int i = threadIdx.x; i < pairs; i += kGsThreads) {
    const float a = ld<T>(down, t * down_stride + rank + 2 * i), b = ld<T>(down, t * down_stride + rank + 2 * i + 1);
    float s, c;
    sincosf(pos * inv_freq[i], &s, &c);
    st<T>(cache, slot * (int64_t)row + rank + 2 * i, a * c - b * s);
    st<T>(cache, slot * (int64_t)row + rank + 2 * i + 1, b * c + a * s);
  }
}

}  // namespace swm

extern "C" {

int swm_gated_stream_step(float* stream, const void* y, int64_t y_stride, const void* gate, int64_t gate_stride,
                          float mult, float* history, int64_t layer_stride, const float* depth_weights, int entries,
                          const float* norm_alpha, const float* norm_weight, const float* norm_bias, void* out,
                          int64_t rows, int width, int act_dtype, void* stream_handle) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "gated_stream_step: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(width > 0 && rows < (1ll << 31), "gated_stream_step: bad shape");
  SW_CHECK_ARG(history == nullptr || (entries >= 1 && depth_weights != nullptr && layer_stride >= rows * width),
               "gated_stream_step: a history needs its weights and at least one entry");
  SW_CHECK_ARG(out == nullptr || (norm_alpha != nullptr && norm_weight != nullptr && norm_bias != nullptr),
               "gated_stream_step: a norm needs alpha, weight and bias");
  const unsigned per_row = (unsigned)std::min(8, (width + 4 * kGsThreads - 1) / (4 * kGsThreads));
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(gated_stream_step_kernel<T>, dim3((unsigned)rows, per_row),
                                                 dim3(kGsThreads), 0, static_cast<hipStream_t>(stream_handle), stream, y,
                                                 y_stride, gate, gate_stride, mult, history, layer_stride, depth_weights,
                                                 entries, norm_alpha, norm_weight, norm_bias, out, width););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_poly_norm(void* out, const void* z, int64_t z_stride, const float* coef, float eps, int64_t rows, int ff,
                  int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "poly_norm: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(ff > 0 && rows < (1ll << 31), "poly_norm: bad shape");
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(poly_norm_kernel<T>, dim3((unsigned)rows), dim3(kGsThreads), 0,
                                                 static_cast<hipStream_t>(stream), out, z, z_stride, coef, eps, ff););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_gate_mul(void* out, const void* y, int64_t y_row_stride, int64_t y_head_stride, const void* gate,
                 int64_t gate_stride, int64_t rows, int heads, int size, int silu, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "gate_mul: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && size > 0 && rows < (1ll << 31), "gate_mul: bad shape");
  const unsigned per_row = (unsigned)std::min(8, (heads * size + 4 * kGsThreads - 1) / (4 * kGsThreads));
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(gate_mul_kernel<T>, dim3((unsigned)rows, per_row), dim3(kGsThreads), 0,
                                                 static_cast<hipStream_t>(stream), out, y, y_row_stride, y_head_stride,
                                                 gate, gate_stride, heads, size, silu););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_latent_rope_cache(float* q_out, const void* q_latent, int64_t ql_row_stride, int64_t ql_head_stride,
                          const void* q_rot, int64_t qr_row_stride, int64_t qr_head_stride, const void* down,
                          int64_t down_stride, const float* norm_weight, float eps, const int64_t* positions,
                          const float* inv_freq, void* cache, const int64_t* slot_mapping, int64_t rows, int heads,
                          int rank, int rot, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "latent_rope_cache: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && rank > 0 && rot >= 0 && rot % 2 == 0 && rows < (1ll << 31),
               "latent_rope_cache: %d heads, rank %d, %d rotated coordinates (an even number)", heads, rank, rot);
  SW_CHECK_ARG(down == nullptr || (cache != nullptr && slot_mapping != nullptr && norm_weight != nullptr),
               "latent_rope_cache: a cache write needs the cache, the slots and the norm weight");
  SWM_DISPATCH_ACT(act_dtype,
                   hipLaunchKernelGGL(latent_rope_cache_kernel<T>, dim3((unsigned)rows), dim3(kGsThreads), 0,
                                      static_cast<hipStream_t>(stream), q_out, q_latent, ql_row_stride, ql_head_stride,
                                      q_rot, qr_row_stride, qr_head_stride, down, down_stride, norm_weight, eps,
                                      positions, inv_freq, cache, slot_mapping, heads, rank, rot););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // extern "C"
