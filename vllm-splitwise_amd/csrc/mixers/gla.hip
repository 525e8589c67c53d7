// Gated linear attention with a decay per head and key channel:  S_t = diag(a_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t,
// a_t = sigmoid(z_t)^(1 / tau) from a projection z of the layer's input, the state S [key size, value size] carried
// in fp32 per sequence.  Decays are handled as logarithms, log a_t = logsigmoid(z_t) / tau, in fp32.
//
// One wave owns (sequence, head, 32 value channels) and keeps its slice of the state in registers across the whole
// run, in the matrix cores' accumulator layout (lane l: value channel l % 32; element r of block b: key coordinate
// 32 b + 8 (r / 4) + 4 (l / 32) + r % 4).  The waves of a workgroup share a chunk's queries, keys, decays and values,
// staged once in LDS.  A chunk of up to 32 tokens is taken token by token: every lane multiplies its state elements by
// the token's decays, adds k v, and the two lanes of a value channel join their halves of S^T q.
#include "mixers_common.cuh"

namespace swm {

using f32x16 = __attribute__((ext_vector_type(16))) float;
constexpr int kGlaChunk = 32;

// log(sigmoid(x)) = min(x, 0) - log1p(exp(-|x|))
__device__ __forceinline__ float logsigmoidf_(float x) { return fminf(x, 0.0f) - log1pf(expf(-fabsf(x))); }

template <typename T, int NDB>
__global__ __launch_bounds__(512) void gla_kernel(
    float* __restrict__ out, const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    int64_t in_stride, const void* __restrict__ decay_pre, int64_t decay_stride, const float* __restrict__ decay_bias,
    float inv_tau, float q_scale, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot, int heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int DS = NDB * 32 + 4;                           // row stride of the staged tiles
  const int nw = blockDim.x >> 6;
  const int VS = nw * 32;
  float* Qs = lds;                                           // [32][DS] queries, scaled
  float* Ks = Qs + kGlaChunk * DS;                           // [32][DS] keys
  float* As = Ks + kGlaChunk * DS;                           // [32][DS] decays
  float* Vs = As + kGlaChunk * DS;                           // [32][VS] values of this workgroup's channels
  const int seq = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 31, hl = lane >> 5;
  const int vb0 = blockIdx.z * nw;                           // first block of 32 value channels of the workgroup
  const int n = q_start[seq + 1] - q_start[seq];
  if (n <= 0) return;                                        // the whole workgroup
  const int row0 = q_start[seq];
  const int vc = (vb0 + wave) * 32 + li;                     // this lane's value channel
  const bool vc_ok = vc < vdim;
  float* sp = state + ((int64_t)state_slot[seq] * heads + h) * (int64_t)dim * vdim;

  f32x16 S[NDB];
  const bool fresh = ctx_len[seq] == 0;
#pragma unroll
  for (int b = 0; b < NDB; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
      S[b][r] = (!fresh && vc_ok && c < dim) ? sp[(int64_t)c * vdim + vc] : 0.0f;
    }

  const int64_t qk_col = (int64_t)h * dim, v_col = (int64_t)h * vdim;
  for (int c0 = 0; c0 < n; c0 += kGlaChunk) {
    const int cn = min(kGlaChunk, n - c0);
    const int64_t base = (int64_t)(row0 + c0) * in_stride, dbase = (int64_t)(row0 + c0) * decay_stride;
    __syncthreads();                                         // the last chunk's tiles have been read
    for (int e = threadIdx.x; e < cn * NDB * 32; e += blockDim.x) {
      const int r = e / (NDB * 32), c = e % (NDB * 32);
      float qv = 0.0f, kv = 0.0f, av = 1.0f;
      if (c < dim) {
        qv = ld<T>(q, base + r * in_stride + qk_col + c) * q_scale;
        kv = ld<T>(k, base + r * in_stride + qk_col + c);
        float z = ld<T>(decay_pre, dbase + r * decay_stride + qk_col + c);
        if (decay_bias != nullptr) z += decay_bias[qk_col + c];
        av = expf(logsigmoidf_(z) * inv_tau);
      }
      Qs[r * DS + c] = qv;
      Ks[r * DS + c] = kv;
      As[r * DS + c] = av;
    }
    for (int e = threadIdx.x; e < cn * VS; e += blockDim.x) {
      const int r = e / VS, c = vb0 * 32 + e % VS;
      Vs[r * VS + e % VS] = c < vdim ? ld<T>(v, base + r * in_stride + v_col + c) : 0.0f;
    }
    __syncthreads();
    for (int j = 0; j < cn; ++j) {
      const float vj = Vs[j * VS + wave * 32 + li];
      float acc = 0.0f;
#pragma unroll
      for (int b = 0; b < NDB; ++b) {
        if (32 * b < dim) {
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            const int c = 32 * b + 8 * g4 + 4 * hl;
            const float4 qv = *reinterpret_cast<const float4*>(Qs + j * DS + c);
            const float4 kv = *reinterpret_cast<const float4*>(Ks + j * DS + c);
            const float4 av = *reinterpret_cast<const float4*>(As + j * DS + c);
            S[b][4 * g4] = av.x * S[b][4 * g4] + kv.x * vj;
            S[b][4 * g4 + 1] = av.y * S[b][4 * g4 + 1] + kv.y * vj;
            S[b][4 * g4 + 2] = av.z * S[b][4 * g4 + 2] + kv.z * vj;
            S[b][4 * g4 + 3] = av.w * S[b][4 * g4 + 3] + kv.w * vj;
            acc += S[b][4 * g4] * qv.x + S[b][4 * g4 + 1] * qv.y + S[b][4 * g4 + 2] * qv.z + S[b][4 * g4 + 3] * qv.w;
          }
        }
      }
      acc += __shfl_xor(acc, 32, 64);
      if (hl == 0 && vc_ok) out[(int64_t)(row0 + c0 + j) * heads * vdim + v_col + vc] = acc;
    }
  }
  if (vc_ok) {
#pragma unroll
    for (int b = 0; b < NDB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
        if (c < dim) sp[(int64_t)c * vdim + vc] = S[b][r];
      }
  }
}

template <typename T, int NDB>
int launch_gla(float* out, const void* q, const void* k, const void* v, int64_t in_stride, const void* decay_pre,
               int64_t decay_stride, const float* decay_bias, float tau, float q_scale, float* state,
               const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int num_seqs, int heads,
               int dim, int vdim, hipStream_t stream) {
  const int vblocks = (vdim + 31) / 32;
  const int waves = std::min(vblocks, 8);
  const size_t lds_bytes = (size_t)(3 * kGlaChunk * (NDB * 32 + 4) + kGlaChunk * waves * 32) * sizeof(float);
  auto kernel = gla_kernel<T, NDB>;
  static size_t allowed = 64 * 1024;                         // per instantiation
  if (lds_bytes > allowed) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds_bytes));
    allowed = lds_bytes;
  }
  const unsigned zgroups = (unsigned)((vblocks + waves - 1) / waves);
  hipLaunchKernelGGL(kernel, dim3((unsigned)num_seqs, (unsigned)heads, zgroups), dim3(64 * waves), lds_bytes, stream,
                     out, q, k, v, in_stride, decay_pre, decay_stride, decay_bias, 1.0f / tau, q_scale, state, q_start,
                     ctx_len, state_slot, heads, dim, vdim);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // namespace swm

extern "C" int swm_gla(float* out, const void* q, const void* k, const void* v, int64_t in_stride,
                       const void* decay_pre, int64_t decay_stride, const float* decay_bias, float tau, float q_scale,
                       float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot,
                       int64_t rows, int num_seqs, int max_query_len, int heads, int dim, int vdim, int act_dtype,
                       void* stream) {
  using namespace swm;
  if (rows == 0 || num_seqs == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "gla: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && heads < 65536 && dim > 0 && dim <= 256 && vdim > 0 && (vdim + 255) / 256 < 65536,
               "gla: %d heads, key size %d (at most 256), value size %d", heads, dim, vdim);
  SW_CHECK_ARG(tau > 0.0f, "gla: tau must be positive");
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SWM_GLA_CASE(N)                                                                                             \
  case N:                                                                                                           \
    SWM_DISPATCH_ACT(act_dtype, return (launch_gla<T, N>(out, q, k, v, in_stride, decay_pre, decay_stride,          \
                                                         decay_bias, tau, q_scale, state, q_start, ctx_len,         \
                                                         state_slot, num_seqs, heads, dim, vdim, s)););             \
    break;
  switch ((dim + 31) / 32) {
    SWM_GLA_CASE(1)
    SWM_GLA_CASE(2)
    SWM_GLA_CASE(3)
    SWM_GLA_CASE(4)
    SWM_GLA_CASE(5)
    SWM_GLA_CASE(6)
    SWM_GLA_CASE(7)
    SWM_GLA_CASE(8)
  }
#undef SWM_GLA_CASE
  return SW_OK;
}
