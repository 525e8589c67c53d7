// Delta-rule recurrences with an fp32 state per (sequence slot, head): S is [dim, vdim], keys index rows.
//
// Two launches per layer.  A PROLOGUE, parallel over tokens, computes everything of a token that does not depend
// on the state (unit vectors, decays with their softplus / exponentials, removal rates, beta) into one fp32
// operand block per (token, head).  The RECURRENCE then only multiplies and adds.
//
// Work split of the recurrence for wave64: one wave owns 16 columns of one head's state; a column is spread over
// 4 lanes that each hold a quarter of its rows in registers (lane = 4 * column + row group).  A product with a
// key-side vector (S^T k, S^T q) is a per-lane partial sum over its rows plus two xor-shuffles; no LDS, no
// barriers, so the only serial dependence is the recurrence itself.  The state is read once at the first token
// of the step (not at all when the sequence starts here) and written once after the last: a decode step moves
// exactly the state, a prompt portion moves it once per portion.  Operands of the next 8 tokens are in flight
// while the current 8 are worked through (see delta_recurrence_kernel).
#include "mixers_common.cuh"

namespace swm {

constexpr int kColsPerWave = 16;
constexpr int kPrepThreads = 256;

// sum over the 4 lanes of a column (a quad): DPP quad permutes, no trip through the LDS crossbar
__device__ __forceinline__ float quad_swap(float v, int ctrl_is_xor2) {
  const int x = __float_as_int(v);
  // quad_perm [1,0,3,2] = 0xB1 swaps neighbours, [2,3,0,1] = 0x4E swaps pairs
  const int y = ctrl_is_xor2 ? __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true)
                             : __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true);
  return __int_as_float(y);
}
__device__ __forceinline__ float group_sum(float v) {
  v += quad_swap(v, 0);
  v += quad_swap(v, 1);
  return v;
}

// ---------------------------------------------------------------------------------------- prologues
// Everything of a token that does not depend on the state is computed once, in parallel over tokens, into
// an fp32 operand block per (token, head): the recurrence then only multiplies and adds.
//
// channel rule: ops[t, h] = { q (unit, times dim^-1/2) | k (unit) | g (decay) }, beta[t, h]
template <typename T>
__global__ __launch_bounds__(kPrepThreads) void channel_delta_prep_kernel(
    float* __restrict__ ops, float* __restrict__ beta, const float* __restrict__ qkv,
    const void* __restrict__ beta_pre, int64_t beta_stride, const void* __restrict__ decay_pre, int64_t decay_stride,
    int decay_per_head, const float* __restrict__ dt_bias, const float* __restrict__ a_log, int heads, int kv_heads,
    int dim, int vdim) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row_w = 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim;
  const float* row = qkv + t * row_w;
  const int group = heads / kv_heads;
  const float qscale = 1.0f / sqrtf((float)dim);
  for (int h = wave; h < heads; h += kPrepThreads / 64) {
    const int c = h / group;
    const float* q = row + c * dim;
    const float* k = row + (int64_t)kv_heads * dim + c * dim;
    float qq = 0.0f, kk = 0.0f;
    for (int i = lane; i < dim; i += 64) {
      qq += q[i] * q[i];
      kk += k[i] * k[i];
    }
    qq = sw::wave_sum(qq);
    kk = sw::wave_sum(kk);
    const float qf = qscale / sqrtf(qq + 1e-6f), kf = 1.0f / sqrtf(kk + 1e-6f);
    const float rate = expf(a_log[h]);
    // one decay for the whole head (every key channel gets the same number), or one per key channel
    const float head_decay =
        decay_per_head ? expf(-rate * softplusf_(ld<T>(decay_pre, t * decay_stride + h) + dt_bias[h])) : 0.0f;
    const int dimp = (dim + 3) & ~3;                     // operand rows are padded to whole 16-byte pieces
    float* o = ops + (t * heads + h) * 3 * (int64_t)dimp;
    for (int i = lane; i < dimp; i += 64) {
      const bool in = i < dim;
      o[i] = in ? q[i] * qf : 0.0f;
      o[dimp + i] = in ? k[i] * kf : 0.0f;
      float gdec = head_decay;
      if (in && !decay_per_head)
        gdec = expf(-rate * softplusf_(ld<T>(decay_pre, t * decay_stride + (int64_t)h * dim + i) + dt_bias[h * dim + i]));
      o[2 * dimp + i] = in ? gdec : 0.0f;
    }
    if (lane == 0) beta[t * heads + h] = sigmoidf_(ld<T>(beta_pre, t * beta_stride + h));
  }
}

// general rule: ops[t, h] = { r | k | w (decay) | a k / (|k|^2 + 1e-6) }: with u = k / |k| the removal term
// (a * u)(u^T S) equals (a k / |k|^2)(k^T S)
template <typename T>
__global__ __launch_bounds__(kPrepThreads) void general_delta_prep_kernel(
    float* __restrict__ ops, const void* __restrict__ rp, const void* __restrict__ kp, int64_t rkv_stride,
    const void* __restrict__ decay_pre, int64_t decay_stride, const float* __restrict__ w0,
    const void* __restrict__ rate_pre, int64_t rate_stride, const float* __restrict__ a_bias, int heads, int dim) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float kDecay = 0.60653065971263342f;            // exp(-1/2)
  for (int h = wave; h < heads; h += kPrepThreads / 64) {
    float kk = 0.0f;
    for (int i = lane; i < dim; i += 64) {
      const float k = ld<T>(kp, t * rkv_stride + h * dim + i);
      kk += k * k;
    }
    kk = sw::wave_sum(kk);
    const float inv = 1.0f / (kk + 1e-6f);
    const int dimp = (dim + 3) & ~3;
    float* o = ops + (t * heads + h) * 4 * (int64_t)dimp;
    for (int i = lane; i < dimp; i += 64) {
      const bool in = i < dim;
      const float k = in ? ld<T>(kp, t * rkv_stride + h * dim + i) : 0.0f;
      o[i] = in ? ld<T>(rp, t * rkv_stride + h * dim + i) : 0.0f;
      o[dimp + i] = k;
      o[2 * dimp + i] = in ? expf(-kDecay * sigmoidf_(ld<T>(decay_pre, t * decay_stride + h * dim + i) + w0[h * dim + i])) : 0.0f;
      o[3 * dimp + i] = in ? sigmoidf_(ld<T>(rate_pre, t * rate_stride + h * dim + i) + a_bias[h * dim + i]) * k * inv : 0.0f;
    }
  }
}

// ---------------------------------------------------------------------------------------- recurrences
// RQ rows per lane (a multiple of 4; dim <= 4 * RQ): lane group rg holds rows [rg * RQ, (rg + 1) * RQ).
// One recurrence kernel for both rules.  MODE 0 (channel): operands {q, k, g}, v fp32 from the convolution's
// output, beta;  MODE 1 (general): operands {r, k, w, a k / |k|^2}, v in the activation type TV.
//
// Operands reach the lanes through LDS in chunks of kChunk (a multiple of 4) tokens: while the wave works through one chunk, the
// loads of the next are in flight (each lane fetches a different 16-byte piece, so a chunk costs a handful of
// loads per lane instead of a broadcast load per operand row), and a token step reads its rows from LDS.
constexpr int kChunk = 4;

template <int RQ, int NOPS, int MODE, typename TV>
__global__ __launch_bounds__(64) void delta_recurrence_kernel(
    float* __restrict__ out, const float* __restrict__ ops, const float* __restrict__ beta, const void* __restrict__ vsrc,
    int64_t v_stride, int64_t v_off, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot, int heads, int dim, int vdim) {
  constexpr int PIECES = (kChunk * NOPS * RQ + 63) / 64;        // 16-byte pieces of a chunk per lane (dim <= 4 RQ)
  extern __shared__ float lds[];
  constexpr int RQ4 = 4 * RQ;                                    // an operand row in LDS: padded with zeros
  const int dimp = (dim + 3) & ~3;
  const int tok_floats = NOPS * dimp;                            // operand floats of one (token, head) in memory
  constexpr int lds_floats = NOPS * RQ4;                         // ... and in LDS
  constexpr int tok_stride = lds_floats + 20;                    // + 16 values + beta, kept on 16 bytes
  const int lane = threadIdx.x, rg = lane & 3, row0 = rg * RQ;
  if (dimp < RQ4) {                                              // rows shorter than their LDS slot: the padding is
    for (int e = lane; e < 2 * kChunk * tok_stride; e += 64) lds[e] = 0.0f;    // zeroed once and never written
    __syncthreads();
  }
  const int cw = lane >> 2;
  const int col = blockIdx.x * kColsPerWave + cw;
  const int h = blockIdx.y, s = blockIdx.z;
  const int first = q_start[s], n = q_start[s + 1] - first;
  if (n == 0) return;
  const bool col_ok = col < vdim;
  const int colc = col_ok ? col : vdim - 1;             // out-of-range lanes shadow the last column, never store
  float* S = state + ((int64_t)state_slot[s] * heads + h) * dim * vdim;
  float Sr[RQ];
#pragma unroll
  for (int i = 0; i < RQ; ++i) Sr[i] = (ctx_len[s] > 0 && row0 + i < dim) ? S[(int64_t)(row0 + i) * vdim + colc] : 0.0f;
  const int pieces_per_tok = tok_floats / 4;
  float4 held[PIECES];
  float vheld[kChunk / 4] = {0.0f}, bheld = 0.0f;
  // a lane's share of chunk `c`: global -> registers
  auto fetch = [&](int c) {
    const int t0 = first + c * kChunk, left = min(kChunk, first + n - t0);
    const int count = left * pieces_per_tok;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      const int idx = lane + 64 * j;
      if (idx < count)
        held[j] = *reinterpret_cast<const float4*>(ops + ((int64_t)(t0 + idx / pieces_per_tok) * heads + h) * tok_floats +
                                                   4 * (idx % pieces_per_tok));
    }
#pragma unroll
    for (int j = 0; j < kChunk / 4; ++j) {
      const int tk = (lane >> 4) + 4 * j, cc = min((int)blockIdx.x * kColsPerWave + (lane & 15), vdim - 1);
      if (tk < left) vheld[j] = ld<TV>(vsrc, (int64_t)(t0 + tk) * v_stride + v_off + (int64_t)h * vdim + cc);
    }
    if (MODE == 0 && lane < left) bheld = beta[(int64_t)(t0 + lane) * heads + h];
  };
  // registers -> LDS buffer
  auto park = [&](int c, float* buf) {
    const int t0 = first + c * kChunk, left = min(kChunk, first + n - t0);
    const int count = left * pieces_per_tok;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      const int idx = lane + 64 * j;
      if (idx < count) {
        const int off = idx % pieces_per_tok, per_row = dimp / 4;
        *reinterpret_cast<float4*>(buf + (idx / pieces_per_tok) * tok_stride + (off / per_row) * RQ4 + 4 * (off % per_row)) =
            held[j];
      }
    }
#pragma unroll
    for (int j = 0; j < kChunk / 4; ++j) {
      const int tk = (lane >> 4) + 4 * j;
      if (tk < left) buf[tk * tok_stride + lds_floats + (lane & 15)] = vheld[j];
    }
    if (MODE == 0 && lane < left) buf[lane * tok_stride + lds_floats + 16] = bheld;
  };
  const int chunks = (n + kChunk - 1) / kChunk;
  const int buf_floats = kChunk * tok_stride;          // two buffers, used in turn
  fetch(0);
  park(0, lds);
  __syncthreads();
#pragma unroll 1
  for (int c = 0; c < chunks; ++c) {
    if (c + 1 < chunks) fetch(c + 1);
    const float* buf = lds + (c & 1) * buf_floats;
    const int t0 = first + c * kChunk, left = min(kChunk, first + n - t0);
    // Two register sets take turns: while one token is worked through, the next one's operand rows are on
    // their way from LDS (the reads are issued first and waited for a whole token step later).
    auto rows_in = [&](float4 (&dst)[NOPS][RQ / 4], float& v, float& b, int tk) {
      const float* op = buf + tk * tok_stride + row0;
#pragma unroll
      for (int a = 0; a < NOPS; ++a)
#pragma unroll
        for (int i = 0; i < RQ / 4; ++i)
          dst[a][i] = *reinterpret_cast<const float4*>(op + a * RQ4 + 4 * i);
      v = buf[tk * tok_stride + lds_floats + cw];
      if (MODE == 0) b = buf[tk * tok_stride + lds_floats + 16];
    };
    auto step = [&](const float4 (&x)[NOPS][RQ / 4], float v, float b, int tk) {
      float o = 0.0f, ks = 0.0f;
      if (MODE == 0) {                                   // x: q, k, g
#pragma unroll
        for (int i = 0; i < RQ / 4; ++i) {
          {
            const float4 k4 = x[1][i], g4 = x[2][i];
            Sr[4 * i] *= g4.x; Sr[4 * i + 1] *= g4.y; Sr[4 * i + 2] *= g4.z; Sr[4 * i + 3] *= g4.w;
            ks += k4.x * Sr[4 * i] + k4.y * Sr[4 * i + 1] + k4.z * Sr[4 * i + 2] + k4.w * Sr[4 * i + 3];
          }
        }
        ks = group_sum(ks);
        const float u = b * (v - ks);
#pragma unroll
        for (int i = 0; i < RQ / 4; ++i) {
          {
            const float4 q4 = x[0][i], k4 = x[1][i];
            Sr[4 * i] += k4.x * u; Sr[4 * i + 1] += k4.y * u; Sr[4 * i + 2] += k4.z * u; Sr[4 * i + 3] += k4.w * u;
            o += q4.x * Sr[4 * i] + q4.y * Sr[4 * i + 1] + q4.z * Sr[4 * i + 2] + q4.w * Sr[4 * i + 3];
          }
        }
      } else {                                           // x: r, k, w, a k / |k|^2
#pragma unroll
        for (int i = 0; i < RQ / 4; ++i) {
          {
            const float4 k4 = x[1][i];
            ks += k4.x * Sr[4 * i] + k4.y * Sr[4 * i + 1] + k4.z * Sr[4 * i + 2] + k4.w * Sr[4 * i + 3];
          }
        }
        ks = group_sum(ks);                              // k^T S of the OLD state
#pragma unroll
        for (int i = 0; i < RQ / 4; ++i) {
          {
            const float4 r4 = x[0][i], k4 = x[1][i], w4 = x[2][i], a4 = x[NOPS - 1][i];
            Sr[4 * i] = w4.x * Sr[4 * i] - a4.x * ks + k4.x * v;
            Sr[4 * i + 1] = w4.y * Sr[4 * i + 1] - a4.y * ks + k4.y * v;
            Sr[4 * i + 2] = w4.z * Sr[4 * i + 2] - a4.z * ks + k4.z * v;
            Sr[4 * i + 3] = w4.w * Sr[4 * i + 3] - a4.w * ks + k4.w * v;
            o += r4.x * Sr[4 * i] + r4.y * Sr[4 * i + 1] + r4.z * Sr[4 * i + 2] + r4.w * Sr[4 * i + 3];
          }
        }
      }
      o = group_sum(o);
      if (rg == 0 && col_ok) out[((int64_t)(t0 + tk) * heads + h) * vdim + col] = o;
    };
    float4 xa[NOPS][RQ / 4], xb[NOPS][RQ / 4];
    float va = 0.0f, vb = 0.0f, ba = 0.0f, bb = 0.0f;
    rows_in(xa, va, ba, 0);
#pragma unroll 1
    for (int tk = 0; tk < left; tk += 2) {
      if (tk + 1 < left) rows_in(xb, vb, bb, tk + 1);
      step(xa, va, ba, tk);
      if (tk + 1 < left) {
        if (tk + 2 < left) rows_in(xa, va, ba, tk + 2);
        step(xb, vb, bb, tk + 1);
      }
    }
    if (c + 1 < chunks) park(c + 1, lds + ((c + 1) & 1) * buf_floats);
    __syncthreads();
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RQ; ++i)
      if (row0 + i < dim) S[(int64_t)(row0 + i) * vdim + col] = Sr[i];
  }
}

inline size_t recurrence_lds_bytes(int nops, int rq) { return sizeof(float) * 2 * kChunk * (size_t)(nops * 4 * rq + 20); }

// launches above 64 KiB of LDS (key sizes near 256) have to be allowed first
template <typename K>
inline hipError_t allow_lds(K kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

}  // namespace swm

// rows per lane for a key size: 4, 8, 16, 32 or 64 (key sizes up to 256)
#define SWM_DISPATCH_ROWS(dim, ...)                       \
  do {                                                    \
    if ((dim) <= 16) { constexpr int RQ = 4; __VA_ARGS__ }        \
    else if ((dim) <= 32) { constexpr int RQ = 8; __VA_ARGS__ }   \
    else if ((dim) <= 64) { constexpr int RQ = 16; __VA_ARGS__ }  \
    else if ((dim) <= 128) { constexpr int RQ = 32; __VA_ARGS__ } \
    else { constexpr int RQ = 64; __VA_ARGS__ }                   \
  } while (0)

extern "C" {

int64_t swm_channel_delta_workspace_floats(int64_t rows, int heads, int dim) {
  return rows * heads * (3 * (int64_t)((dim + 3) & ~3) + 1);
}
int64_t swm_general_delta_workspace_floats(int64_t rows, int heads, int dim) {
  return rows * heads * 4 * (int64_t)((dim + 3) & ~3);
}

static int delta_with_decay(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride,
                            const void* decay_pre, int64_t decay_stride, int decay_per_head, const float* dt_bias,
                            const float* a_log, float* state, const int32_t* q_start, const int32_t* ctx_len,
                            const int32_t* state_slot, int64_t rows, int num_seqs, int heads, int kv_heads, int dim,
                            int vdim, float* workspace, int act_dtype, void* stream) {
  using namespace swm;
  if (num_seqs == 0 || rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "channel_delta: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 256 && vdim > 0 &&
                   workspace != nullptr && rows < (1ll << 31),
               "channel_delta: heads %d, kv heads %d, key size %d (up to 256), value size %d", heads, kv_heads, dim,
               vdim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ops = workspace;
  float* beta = workspace + rows * heads * 3 * (int64_t)((dim + 3) & ~3);
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(channel_delta_prep_kernel<T>, dim3((unsigned)rows), dim3(kPrepThreads), 0,
                                                 s, ops, beta, qkv, beta_pre, beta_stride, decay_pre, decay_stride,
                                                 decay_per_head, dt_bias, a_log, heads, kv_heads, dim, vdim););
  SW_CHECK_LAUNCH();
  const dim3 grid((unsigned)((vdim + kColsPerWave - 1) / kColsPerWave), (unsigned)heads, (unsigned)num_seqs);
  const int64_t row_w = 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim;
  SWM_DISPATCH_ROWS(dim, SW_CHECK_HIP(allow_lds(delta_recurrence_kernel<RQ, 3, 0, float>, recurrence_lds_bytes(3, RQ))););
  SWM_DISPATCH_ROWS(dim, hipLaunchKernelGGL((delta_recurrence_kernel<RQ, 3, 0, float>), grid, dim3(64),
                                            recurrence_lds_bytes(3, RQ), s, out, ops, beta, qkv, row_w,
                                            2 * (int64_t)kv_heads * dim, state, q_start, ctx_len, state_slot, heads, dim,
                                            vdim););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_channel_delta(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride,
                      const void* decay_pre, const float* dt_bias, const float* a_log, float* state,
                      const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows,
                      int num_seqs, int heads, int kv_heads, int dim, int vdim, float* workspace, int act_dtype,
                      void* stream) {
  return delta_with_decay(out, qkv, beta_pre, beta_stride, decay_pre, (int64_t)heads * dim, 0, dt_bias, a_log, state,
                          q_start, ctx_len, state_slot, rows, num_seqs, heads, kv_heads, dim, vdim, workspace, act_dtype,
                          stream);
}

int swm_gated_delta(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride, const void* decay_pre,
                    int64_t decay_stride, const float* dt_bias, const float* a_log, float* state,
                    const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows,
                    int num_seqs, int heads, int kv_heads, int dim, int vdim, float* workspace, int act_dtype,
                    void* stream) {
  return delta_with_decay(out, qkv, beta_pre, beta_stride, decay_pre, decay_stride, 1, dt_bias, a_log, state, q_start,
                          ctx_len, state_slot, rows, num_seqs, heads, kv_heads, dim, vdim, workspace, act_dtype, stream);
}

int swm_general_delta(float* out, const void* r, const void* k, const void* v, int64_t rkv_stride,
                      const void* decay_pre, int64_t decay_stride, const float* w0, const void* rate_pre,
                      int64_t rate_stride, const float* a_bias, float* state, const int32_t* q_start,
                      const int32_t* ctx_len, const int32_t* state_slot, int64_t rows, int num_seqs, int heads,
                      int dim, float* workspace, int act_dtype, void* stream) {
  using namespace swm;
  if (num_seqs == 0 || rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "general_delta: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && dim > 0 && dim <= 256 && workspace != nullptr && rows < (1ll << 31),
               "general_delta: heads %d, key size %d (up to 256)", heads, dim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(general_delta_prep_kernel<T>, dim3((unsigned)rows), dim3(kPrepThreads), 0,
                                                 s, workspace, r, k, rkv_stride, decay_pre, decay_stride, w0, rate_pre,
                                                 rate_stride, a_bias, heads, dim););
  SW_CHECK_LAUNCH();
  const dim3 grid((unsigned)((dim + kColsPerWave - 1) / kColsPerWave), (unsigned)heads, (unsigned)num_seqs);
  SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_ROWS(dim, SW_CHECK_HIP(allow_lds(delta_recurrence_kernel<RQ, 4, 1, T>,
                                                                            recurrence_lds_bytes(4, RQ)));););
  SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_ROWS(dim, hipLaunchKernelGGL(
      (delta_recurrence_kernel<RQ, 4, 1, T>), grid, dim3(64), recurrence_lds_bytes(4, RQ), s, out, workspace, nullptr, v,
      rkv_stride, (int64_t)0, state, q_start, ctx_len, state_slot, heads, dim, dim);););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // extern "C"
