// Norms with a single gain on an fp32 residual stream, the whole-projection query / key norm with its
// cache write, the per-head output norm with a sigmoid gate, and the short causal convolution with its
// carried inputs.  All arithmetic is fp32; activations are read and written in the model's dtype.
#include <string>

#include "mixers_common.cuh"

namespace sw {
static thread_local std::string g_mixers_error;
void set_error(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_mixers_error = buf;
}
}  // namespace sw

namespace swm {

constexpr int kRowThreads = 256;

// ------------------------------------------------------------------- single-gain norms
// TY: type of the sublayer output y; T: the activation type of cast_out
template <typename TY, typename T>
__global__ __launch_bounds__(kRowThreads) void scalar_norm_add_kernel(
    float* __restrict__ residual, const void* __restrict__ y, const float* __restrict__ gain, float eps,
    void* __restrict__ cast_out, int width, int64_t y_stride) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const char* yrow = static_cast<const char*>(y) + t * y_stride * sizeof(typename Conv<TY>::store_t);
  float ss = 0.0f;
  for (int c = threadIdx.x; c < width; c += kRowThreads) {
    const float v = ld<TY>(yrow, c);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float f = gain[0] / sqrtf(ss / (float)width + eps);
  float* r = residual + t * (int64_t)width;
  for (int c = threadIdx.x; c < width; c += kRowThreads) {
    const float v = r[c] + ld<TY>(yrow, c) * f;
    r[c] = v;
    if (cast_out != nullptr) st<T>(cast_out, t * (int64_t)width + c, v);
  }
}

template <typename T>
__global__ __launch_bounds__(kRowThreads) void scalar_norm_kernel(
    void* __restrict__ out, const float* __restrict__ x, const float* __restrict__ gain, float eps, int width) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float* r = x + t * (int64_t)width;
  float ss = 0.0f;
  for (int c = threadIdx.x; c < width; c += kRowThreads) ss += r[c] * r[c];
  ss = block_sum(ss, red);
  const float f = gain[0] / sqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += kRowThreads) st<T>(out, t * (int64_t)width + c, r[c] * f);
}

// ------------------------------------------------- query / key norm over the projection + cache write
template <typename T>
__global__ __launch_bounds__(kRowThreads) void qk_norm_cache_kernel(
    float* __restrict__ q_out, const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    int64_t in_stride, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    void* __restrict__ key_cache, void* __restrict__ value_cache, const int64_t* __restrict__ slot_mapping,
    int q_size, int k_size, int v_size) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int64_t row = t * in_stride;
  float ss = 0.0f;
  for (int c = threadIdx.x; c < q_size; c += kRowThreads) {
    const float x = ld<T>(q, row + c);
    ss += x * x;
  }
  ss = block_sum(ss, red);
  const float fq = 1.0f / sqrtf(ss / (float)q_size + eps);
  for (int c = threadIdx.x; c < q_size; c += kRowThreads)
    q_out[t * (int64_t)q_size + c] = ld<T>(q, row + c) * fq * q_gain[c];
  if (k == nullptr) return;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;                       // uniform over the workgroup
  float sk = 0.0f;
  for (int c = threadIdx.x; c < k_size; c += kRowThreads) {
    const float x = ld<T>(k, row + c);
    sk += x * x;
  }
  sk = block_sum(sk, red);
  const float fk = 1.0f / sqrtf(sk / (float)k_size + eps);
  for (int c = threadIdx.x; c < k_size; c += kRowThreads)
    st<T>(key_cache, slot * (int64_t)k_size + c, ld<T>(k, row + c) * fk * k_gain[c]);
  for (int c = threadIdx.x; c < v_size; c += kRowThreads)
    st<T>(value_cache, slot * (int64_t)v_size + c, ld<T>(v, row + c));
}

// ------------------------------------------------------------ per-head output norm with a sigmoid gate
// one wave per (row, head)
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(
    void* __restrict__ out, const float* __restrict__ o, const void* __restrict__ gate, int64_t gate_stride,
    const float* __restrict__ weight, int weight_head_stride, float eps, int64_t rows, int heads, int vdim,
    int gate_silu) {
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= rows * heads) return;           // uniform over the wave
  const int lane = threadIdx.x & 63;
  const int64_t t = unit / heads;
  const int h = (int)(unit % heads);
  const float* src = o + (t * heads + h) * (int64_t)vdim;
  float ss = 0.0f;
  for (int c = lane; c < vdim; c += 64) ss += src[c] * src[c];
  ss = sw::wave_sum(ss);
  const float f = 1.0f / sqrtf(ss / (float)vdim + eps);
  for (int c = lane; c < vdim; c += 64) {
    const float gv = ld<T>(gate, t * gate_stride + h * vdim + c);
    const float g = gate_silu ? gv * sigmoidf_(gv) : sigmoidf_(gv);
    st<T>(out, (t * heads + h) * (int64_t)vdim + c, src[c] * f * weight[h * weight_head_stride + c] * g);
  }
}

// ------------------------------------------------------------------------- short convolution + silu
constexpr int kMaxTaps = 16;

// TX: type of the inputs x, TO: type of the outputs.  silu: the activation after the sum; residual: the input
// itself is added to its convolution (out = x + conv(x)).
// advance: the launch also moves the state past the step's tokens.  Only a sequence's first num_taps - 1 rows read
// the state, so the workgroup of the FIRST row works all of them out (the workgroups of the others leave at once) and
// then writes the new state; a thread owns its channel in both, so nothing is read after it was overwritten.
template <typename TX, typename TO>
__global__ __launch_bounds__(kRowThreads) void short_conv_kernel(
    void* __restrict__ out, const void* __restrict__ x, int64_t x_stride, const float* __restrict__ taps,
    float* __restrict__ state, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ token_seq, const int32_t* __restrict__ state_slot, int channels, int num_taps, int silu,
    int residual, int advance) {
  const int64_t t0 = blockIdx.x;
  const int c = blockIdx.y * kRowThreads + threadIdx.x;
  const int s = token_seq[t0];
  const int first = q_start[s], n = q_start[s + 1] - first, keep = num_taps - 1;
  const int rel = (int)t0 - first;
  int count = 1;
  if (advance && keep > 0) {
    if (rel > 0 && rel < keep) return;                  // the whole workgroup: the first row's workgroup does this row
    if (rel == 0) count = min(keep, n);
  }
  if (c >= channels) return;
  const bool carried = ctx_len[s] > 0;
  float* carry = state + (int64_t)state_slot[s] * keep * channels;
  for (int64_t t = t0; t < t0 + count; ++t) {
    float acc = 0.0f;
    for (int j = 0; j < num_taps; ++j) {
      const int back = num_taps - 1 - j;                // tokens before the current one
      const int64_t src = t - back;
      float xv;
      if (src >= first) {
        xv = ld<TX>(x, src * x_stride + c);
      } else if (carried) {
        // the input `first - src` tokens before this step's first one: the state's row (num_taps-1) - that
        xv = carry[(int64_t)(num_taps - 1 - (first - (int)src)) * channels + c];
      } else {
        xv = 0.0f;
      }
      acc += taps[(int64_t)c * num_taps + j] * xv;
    }
    if (residual) acc += ld<TX>(x, t * x_stride + c);
    st<TO>(out, t * (int64_t)channels + c, silu ? acc * sigmoidf_(acc) : acc);
  }
  if (!advance || keep == 0 || rel != 0) return;
  float fresh[kMaxTaps];
  for (int p = 0; p < keep; ++p) {
    // new row p holds the input (keep - p) tokens before the END of this step
    const int off = n - (keep - p);                     // index among this step's tokens; < 0: before them
    float v;
    if (off >= 0) v = ld<TX>(x, (int64_t)(first + off) * x_stride + c);
    else if (carried && keep + off >= 0) v = carry[(int64_t)(keep + off) * channels + c];
    else v = 0.0f;
    fresh[p] = v;
  }
  for (int p = 0; p < keep; ++p) carry[(int64_t)p * channels + c] = fresh[p];
}

// one thread per (sequence, channel): reads what it needs of the old state, then writes the new one
template <typename T>
__global__ __launch_bounds__(kRowThreads) void short_conv_advance_kernel(
    float* __restrict__ state, const void* __restrict__ x, int64_t x_stride, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot, int channels, int num_taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * kRowThreads + threadIdx.x;
  if (c >= channels) return;
  const int first = q_start[s], n = q_start[s + 1] - first, keep = num_taps - 1;
  if (n == 0) return;
  float* carry = state + (int64_t)state_slot[s] * keep * channels;
  const bool carried = ctx_len[s] > 0;
  float fresh[kMaxTaps];
  for (int p = 0; p < keep; ++p) {
    // new row p holds the input (keep - p) tokens before the END of this step
    const int off = n - (keep - p);                     // index among this step's tokens; < 0: before them
    float v;
    if (off >= 0) v = ld<T>(x, (int64_t)(first + off) * x_stride + c);
    else if (carried && keep + off >= 0) v = carry[(int64_t)(keep + off) * channels + c];
    else v = 0.0f;
    fresh[p] = v;
  }
  for (int p = 0; p < keep; ++p) carry[(int64_t)p * channels + c] = fresh[p];
}

}  // namespace swm

extern "C" {

int swm_abi_version(void) { return SWM_ABI_VERSION; }
const char* swm_last_error(void) { return sw::g_mixers_error.c_str(); }

int swm_scalar_norm_add(float* residual, const void* y, const float* gain, float eps, void* cast_out,
                        int64_t rows, int width, int64_t y_stride, int y_dtype, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype) && act_ok(y_dtype), "scalar_norm_add: unsupported dtype %d / %d", y_dtype, act_dtype);
  SW_CHECK_ARG(width > 0 && y_stride >= width && rows < (1ll << 31), "scalar_norm_add: bad shape");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (y_dtype == SW_F32) {
    SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL((scalar_norm_add_kernel<float, T>), dim3((unsigned)rows),
                                                   dim3(kRowThreads), 0, s, residual, y, gain, eps, cast_out, width,
                                                   y_stride););
  } else {
    SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL((scalar_norm_add_kernel<sw::bf16_t, T>), dim3((unsigned)rows),
                                                   dim3(kRowThreads), 0, s, residual, y, gain, eps, cast_out, width,
                                                   y_stride););
  }
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_scalar_norm(void* out, const float* x, const float* gain, float eps, int64_t rows, int width,
                    int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "scalar_norm: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(width > 0 && rows < (1ll << 31), "scalar_norm: bad shape");
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(scalar_norm_kernel<T>, dim3((unsigned)rows), dim3(kRowThreads), 0,
                                                 static_cast<hipStream_t>(stream), out, x, gain, eps, width););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_qk_norm_cache(float* q_out, const void* q, const void* k, const void* v, int64_t in_stride,
                      const float* q_gain, const float* k_gain, float eps, void* key_cache, void* value_cache,
                      const int64_t* slot_mapping, int64_t rows, int q_size, int k_size, int v_size,
                      int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "qk_norm_cache: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(q_size > 0 && rows < (1ll << 31), "qk_norm_cache: bad shape");
  SW_CHECK_ARG(k == nullptr || (v != nullptr && k_gain != nullptr && key_cache != nullptr && value_cache != nullptr &&
                                slot_mapping != nullptr && k_size > 0 && v_size > 0),
               "qk_norm_cache: keys without values, gains, caches or slots");
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(qk_norm_cache_kernel<T>, dim3((unsigned)rows), dim3(kRowThreads), 0,
                                                 static_cast<hipStream_t>(stream), q_out, q, k, v, in_stride, q_gain,
                                                 k_gain, eps, key_cache, value_cache, slot_mapping, q_size, k_size,
                                                 v_size););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_head_norm_gate(void* out, const float* o, const void* gate, int64_t gate_stride, const float* weight,
                       int weight_head_stride, float eps, int64_t rows, int heads, int vdim, int act_dtype,
                       void* stream) {
  return swm_head_norm_gate_act(out, o, gate, gate_stride, weight, weight_head_stride, eps, rows, heads, vdim, 0,
                                act_dtype, stream);
}

int swm_head_norm_gate_act(void* out, const float* o, const void* gate, int64_t gate_stride, const float* weight,
                           int weight_head_stride, float eps, int64_t rows, int heads, int vdim, int gate_silu,
                           int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "head_norm_gate: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && vdim > 0 && rows * heads < (1ll << 32), "head_norm_gate: bad shape");
  const unsigned blocks = (unsigned)((rows * heads + 3) / 4);
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(head_norm_gate_kernel<T>, dim3(blocks), dim3(256), 0,
                                                 static_cast<hipStream_t>(stream), out, o, gate, gate_stride, weight,
                                                 weight_head_stride, eps, rows, heads, vdim, gate_silu););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_short_conv(float* out, const void* x, int64_t x_stride, const float* taps, const float* state,
                   const int32_t* q_start, const int32_t* ctx_len, const int32_t* token_seq,
                   const int32_t* state_slot, int64_t rows, int channels, int num_taps, int act_dtype,
                   void* stream) {
  return swm_causal_conv(out, SW_F32, x, act_dtype, x_stride, taps, const_cast<float*>(state), q_start, ctx_len, token_seq,
                         state_slot, rows, channels, num_taps, 1, 0, 0, stream);
}

int swm_causal_conv(void* out, int out_dtype, const void* x, int x_dtype, int64_t x_stride, const float* taps,
                    float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* token_seq,
                    const int32_t* state_slot, int64_t rows, int channels, int num_taps, int silu, int residual,
                    int advance, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(x_dtype) && act_ok(out_dtype), "causal_conv: unsupported dtype %d / %d", x_dtype, out_dtype);
  SW_CHECK_ARG(channels > 0 && num_taps >= 1 && num_taps <= kMaxTaps && rows < (1ll << 31),
               "causal_conv: %d taps (1..%d supported), %d channels", num_taps, kMaxTaps, channels);
  const dim3 grid((unsigned)rows, (unsigned)((channels + kRowThreads - 1) / kRowThreads));
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SWM_CONV_LAUNCH(TX, TO)                                                                                       \
  hipLaunchKernelGGL((short_conv_kernel<TX, TO>), grid, dim3(kRowThreads), 0, s, out, x, x_stride, taps, state,       \
                     q_start, ctx_len, token_seq, state_slot, channels, num_taps, silu, residual, advance)
  if (x_dtype == SW_F32) {
    if (out_dtype == SW_F32) SWM_CONV_LAUNCH(float, float); else SWM_CONV_LAUNCH(float, sw::bf16_t);
  } else {
    if (out_dtype == SW_F32) SWM_CONV_LAUNCH(sw::bf16_t, float); else SWM_CONV_LAUNCH(sw::bf16_t, sw::bf16_t);
  }
#undef SWM_CONV_LAUNCH
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_short_conv_advance(float* state, const void* x, int64_t x_stride, const int32_t* q_start,
                           const int32_t* ctx_len, const int32_t* state_slot, int num_seqs, int channels,
                           int num_taps, int act_dtype, void* stream) {
  using namespace swm;
  if (num_seqs == 0 || num_taps <= 1) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "short_conv_advance: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(channels > 0 && num_taps <= kMaxTaps, "short_conv_advance: %d taps (1..%d supported)", num_taps,
               kMaxTaps);
  const dim3 grid((unsigned)num_seqs, (unsigned)((channels + kRowThreads - 1) / kRowThreads));
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(short_conv_advance_kernel<T>, grid, dim3(kRowThreads), 0,
                                                 static_cast<hipStream_t>(stream), state, x, x_stride, q_start,
                                                 ctx_len, state_slot, channels, num_taps););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // extern "C"
