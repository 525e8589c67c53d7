// Gated linear attention with a decay per head and key channel:  S_t = diag(a_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t,
// a_t = sigmoid(z_t)^(1 / tau) from a projection z of the layer's input, the state S [key size, value size] carried
// in fp32 per sequence.  Decays are handled as logarithms, g_t = log a_t = logsigmoid(z_t) / tau, in fp32.
//
// One wave owns (sequence, head, 32 value channels) and keeps its slice of the state in registers across the whole
// run, in the matrix cores' accumulator layout (lane l: value channel l % 32; element r of block b: key coordinate
// 32 b + 8 (r / 4) + 4 (l / 32) + r % 4).  The waves of a workgroup share a chunk's queries, keys, decays and values,
// staged once in LDS.  A chunk of up to 32 tokens takes one of two routes, chosen per chunk for the whole workgroup:
//
//  * matrix route.  With G_t = g_1 + ... + g_t inside the chunk (<= 0), q~_t = q_t e^(G_t), k~_t = k_t e^(-G_t):
//        A[i, j] = q~_i . k~_j  (j <= i),   O = A V + Q~ S,   S <- diag(e^(G_n)) (S + K~^T V)
//    three fp32 products on the matrix cores (v_mfma_f32_32x32x2_f32), which is the recurrence with its sums
//    reordered.  e^(-G_t) grows as the chunk's decays multiply up, so this route is taken only while every channel's
//    G_n stays above -kSafeLog: the factors then stay within e^(+-kSafeLog) and nothing over- or underflows.
//  * token route: every lane multiplies its state elements by the token's decays, adds k v, and the two lanes of a
//    value channel join their halves of S^T q.  Exact for any decay (a product of decays that underflows is a state
//    that has been forgotten), and the cheaper route for runs of a few tokens (a decoded token is a chunk of one).
//
// Long runs are cut into segments of kGlaSegment tokens that run side by side: a first launch takes every segment but a
// sequence's last from the EMPTY state and leaves its end state and its summed log decays; a scan turns these into the
// states at the segments' ends, S_end(j) = diag(e^(D_j)) S_end(j - 1) + local(j); a second launch runs every segment
// from its true start state and writes the outputs.
#include "mixers_common.cuh"

namespace swm {

using f32x16 = __attribute__((ext_vector_type(16))) float;
constexpr int kGlaChunk = 32;
constexpr int kGlaSegment = 128;       // tokens per segment of a long run (a multiple of kGlaChunk)
constexpr float kSafeLog = 24.0f;      // the matrix route needs every channel's summed log-decay of a chunk above -this
constexpr int kTokenRouteBelow = 6;    // chunks shorter than this go token by token without asking
constexpr int kGlaWhole = 0, kGlaLocal = 1, kGlaFinal = 2;

// log(sigmoid(x)) = min(x, 0) - log1p(exp(-|x|))
__device__ __forceinline__ float logsigmoidf_(float x) { return fminf(x, 0.0f) - log1pf(expf(-fabsf(x))); }

// mode kGlaWhole: blockIdx.x is a sequence and its whole run goes from the slot's state to the slot's state.
// kGlaLocal / kGlaFinal: blockIdx.x is a segment (see the head of the file); seg_state [segments, heads, dim, vdim],
// seg_decay [segments, heads, dim].
template <typename T, int NDB>
__global__ __launch_bounds__(512) void gla_kernel(
    float* __restrict__ out, const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    int64_t in_stride, const void* __restrict__ decay_pre, int64_t decay_stride, const float* __restrict__ decay_bias,
    float inv_tau, float q_scale, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot, int num_seqs, int heads, int dim,
    int vdim, int mode, float* __restrict__ seg_state, float* __restrict__ seg_decay) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int DS = NDB * 32 + 4;                           // row stride of the staged tiles
  constexpr int CH = NDB * 32;                               // key channels, padded
  const int nw = blockDim.x >> 6;
  const int VS = nw * 32;
  float* Qs = lds;                                           // [32][DS] queries, scaled
  float* Ks = Qs + kGlaChunk * DS;                           // [32][DS] keys
  float* Gs = Ks + kGlaChunk * DS;                           // [32][DS] log decays, then their running sums or the decays
  float* Vs = Gs + kGlaChunk * DS;                           // [32][VS] values of this workgroup's channels
  float* part = Vs + kGlaChunk * VS;                         // [8][CH] sums of the log decays over groups of tokens
  float* dsum = part + 8 * CH;                               // [CH] summed log decays of the whole segment
  float* red = dsum + CH;                                    // [nw] workgroup minimum
  const int h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 31, hl = lane >> 5;
  const int vb0 = blockIdx.z * nw;                           // first block of 32 value channels of the workgroup
  int seq = blockIdx.x, tok0 = 0, n;
  if (mode == kGlaWhole) {
    n = q_start[seq + 1] - q_start[seq];
  } else {
    n = find_query_tile(q_start, num_seqs, blockIdx.x, kGlaSegment, &seq, &tok0);
  }
  if (n <= 0) return;                                        // the whole workgroup
  const int row0 = q_start[seq] + tok0;
  const bool last_seg = tok0 + n == q_start[seq + 1] - q_start[seq];
  if (mode == kGlaLocal && last_seg) return;
  const int vc = (vb0 + wave) * 32 + li;                     // this lane's value channel
  const bool vc_ok = vc < vdim;
  float* sp = state + ((int64_t)state_slot[seq] * heads + h) * (int64_t)dim * vdim;
  float* seg_out = seg_state + ((int64_t)blockIdx.x * heads + h) * (int64_t)dim * vdim;      // segment modes only
  const float* start = (mode == kGlaFinal && tok0 > 0) ? seg_out - (int64_t)heads * dim * vdim : sp;

  // token groups for the sums down a chunk: `groups` threads per channel, each with 32 / groups tokens
  int groups = 1;
  while (groups < 8 && 2 * groups * CH <= (int)blockDim.x) groups <<= 1;
  const int per = kGlaChunk / groups;

  f32x16 S[NDB];
  const bool fresh = mode == kGlaLocal || (tok0 == 0 && ctx_len[seq] == 0);
#pragma unroll
  for (int b = 0; b < NDB; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
      S[b][r] = (!fresh && vc_ok && c < dim) ? start[(int64_t)c * vdim + vc] : 0.0f;
    }
  if (mode == kGlaLocal)
    for (int c = threadIdx.x; c < CH; c += blockDim.x) dsum[c] = 0.0f;

  const int64_t qk_col = (int64_t)h * dim, v_col = (int64_t)h * vdim;
  for (int c0 = 0; c0 < n; c0 += kGlaChunk) {
    const int cn = min(kGlaChunk, n - c0);
    const int64_t base = (int64_t)(row0 + c0) * in_stride, dbase = (int64_t)(row0 + c0) * decay_stride;
    const bool ask = cn >= kTokenRouteBelow || mode == kGlaLocal;     // uniform over the workgroup
    const int stage_rows = ask ? kGlaChunk : cn;             // the matrix route reads all 32 rows: the rest are zeros
    __syncthreads();                                         // the last chunk's tiles have been read
    for (int e = threadIdx.x; e < stage_rows * CH; e += blockDim.x) {
      const int r = e / CH, c = e % CH;
      float qv = 0.0f, kv = 0.0f, gv = 0.0f;
      if (r < cn && c < dim) {
        if (mode != kGlaLocal) qv = ld<T>(q, base + r * in_stride + qk_col + c) * q_scale;
        kv = ld<T>(k, base + r * in_stride + qk_col + c);
        float z = ld<T>(decay_pre, dbase + r * decay_stride + qk_col + c);
        if (decay_bias != nullptr) z += decay_bias[qk_col + c];
        gv = logsigmoidf_(z) * inv_tau;
      }
      Qs[r * DS + c] = qv;
      Ks[r * DS + c] = kv;
      Gs[r * DS + c] = gv;
    }
    for (int e = threadIdx.x; e < stage_rows * VS; e += blockDim.x) {
      const int r = e / VS, c = vb0 * 32 + e % VS;
      Vs[r * VS + e % VS] = (r < cn && c < vdim) ? ld<T>(v, base + r * in_stride + v_col + c) : 0.0f;
    }
    __syncthreads();
    bool matrix_route = false;
    if (ask) {
      // sums of the log decays over each group of tokens (rows beyond the chunk hold 0), then the smallest sum over
      // the whole chunk of any channel
      for (int u = threadIdx.x; u < CH * groups; u += blockDim.x) {
        const int c = u % CH, gi = u / CH;
        float total = 0.0f;
        for (int r = gi * per; r < (gi + 1) * per; ++r) total += Gs[r * DS + c];
        part[gi * CH + c] = total;
      }
      __syncthreads();
      float lowest = 0.0f;
      for (int c = threadIdx.x; c < CH; c += blockDim.x) {
        float total = 0.0f;
        for (int gi = 0; gi < groups; ++gi) total += part[gi * CH + c];
        lowest = fminf(lowest, total);
        if (mode == kGlaLocal) dsum[c] += total;
      }
#pragma unroll
      for (int step = 32; step >= 1; step >>= 1) lowest = fminf(lowest, __shfl_xor(lowest, step, 64));
      if (lane == 0) red[wave] = lowest;
      __syncthreads();
      for (int w = 0; w < nw; ++w) lowest = fminf(lowest, red[w]);
      matrix_route = lowest >= -kSafeLog;
    }
    if (matrix_route) {
      // ---- running sums of the log decays down the chunk; q~ = q e^G, k~ = k e^(-G); rows beyond the chunk stay zero
      for (int u = threadIdx.x; u < CH * groups; u += blockDim.x) {
        const int c = u % CH, gi = u / CH;
        float run = 0.0f;
        for (int g2 = 0; g2 < gi; ++g2) run += part[g2 * CH + c];
        for (int r = gi * per; r < min((gi + 1) * per, cn); ++r) {
          run += Gs[r * DS + c];
          Gs[r * DS + c] = run;
          Qs[r * DS + c] *= expf(run);
          Ks[r * DS + c] *= expf(-run);
        }
      }
      __syncthreads();
      // ---- values of the chunk: channel vc of token (r, hl)
      float vt[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) vt[r] = Vs[(8 * (r / 4) + 4 * hl + (r % 4)) * VS + wave * 32 + li];
      if (mode != kGlaLocal) {
        // ---- A^T = K~ Q~^T (rows: keys, columns: queries); this lane: token li of the chunk as key and as query
        f32x16 a;
#pragma unroll
        for (int r = 0; r < 16; ++r) a[r] = 0.0f;
#pragma unroll
        for (int b = 0; b < NDB; ++b) {
          if (32 * b < dim) {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              const int c = 32 * b + 8 * g4 + 4 * hl;
              const float4 qv = *reinterpret_cast<const float4*>(Qs + li * DS + c);
              const float4 kv = *reinterpret_cast<const float4*>(Ks + li * DS + c);
              a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qv.x, a, 0, 0, 0);
              a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qv.y, a, 0, 0, 0);
              a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qv.z, a, 0, 0, 0);
              a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qv.w, a, 0, 0, 0);
            }
          }
        }
        // element r: key j = 8 (r / 4) + 4 hl + r % 4, query i = li; a key counts for the queries from itself on
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = 8 * (r / 4) + 4 * hl + (r % 4);
          a[r] = (j <= li && li < cn) ? a[r] : 0.0f;
        }
        // ---- O^T = V^T A^T + S^T Q~^T
        f32x16 o;
#pragma unroll
        for (int r = 0; r < 16; ++r) o[r] = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) o = __builtin_amdgcn_mfma_f32_32x32x2f32(vt[r], a[r], o, 0, 0, 0);
#pragma unroll
        for (int b = 0; b < NDB; ++b) {
          if (32 * b < dim) {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              const float4 qv = *reinterpret_cast<const float4*>(Qs + li * DS + 32 * b + 8 * g4 + 4 * hl);
              o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4], qv.x, o, 0, 0, 0);
              o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4 + 1], qv.y, o, 0, 0, 0);
              o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4 + 2], qv.z, o, 0, 0, 0);
              o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4 + 3], qv.w, o, 0, 0, 0);
            }
          }
        }
        if (li < cn && (vb0 + wave) * 32 < vdim) {
          float* dst = out + (int64_t)(row0 + c0 + li) * heads * vdim + v_col + (vb0 + wave) * 32;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int c = 8 * (r / 4) + 4 * hl + (r % 4);
            if ((vb0 + wave) * 32 + c < vdim) dst[c] = o[r];
          }
        }
      }
      // ---- S <- diag(e^(G_n)) (S + K~^T V): A = keys transposed (coordinate li of block b, token (r, hl))
      const float* last = Gs + (cn - 1) * DS;
#pragma unroll
      for (int b = 0; b < NDB; ++b) {
        if (32 * b < dim) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int j = 8 * (r / 4) + 4 * hl + (r % 4);
            S[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(Ks[j * DS + 32 * b + li], vt[r], S[b], 0, 0, 0);
          }
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            const float4 gl = *reinterpret_cast<const float4*>(last + 32 * b + 8 * g4 + 4 * hl);
            S[b][4 * g4] *= expf(gl.x);
            S[b][4 * g4 + 1] *= expf(gl.y);
            S[b][4 * g4 + 2] *= expf(gl.z);
            S[b][4 * g4 + 3] *= expf(gl.w);
          }
        }
      }
      continue;
    }
    // ---- token route: the decays themselves
    for (int e = threadIdx.x; e < cn * CH; e += blockDim.x) {
      const int at = (e / CH) * DS + e % CH;
      Gs[at] = expf(Gs[at]);
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
            const float4 av = *reinterpret_cast<const float4*>(Gs + j * DS + c);
            S[b][4 * g4] = av.x * S[b][4 * g4] + kv.x * vj;
            S[b][4 * g4 + 1] = av.y * S[b][4 * g4 + 1] + kv.y * vj;
            S[b][4 * g4 + 2] = av.z * S[b][4 * g4 + 2] + kv.z * vj;
            S[b][4 * g4 + 3] = av.w * S[b][4 * g4 + 3] + kv.w * vj;
            acc += S[b][4 * g4] * qv.x + S[b][4 * g4 + 1] * qv.y + S[b][4 * g4 + 2] * qv.z + S[b][4 * g4 + 3] * qv.w;
          }
        }
      }
      acc += __shfl_xor(acc, 32, 64);
      if (mode != kGlaLocal && hl == 0 && vc_ok) out[(int64_t)(row0 + c0 + j) * heads * vdim + v_col + vc] = acc;
    }
  }
  if (mode == kGlaFinal && !last_seg) return;                // its end state is the next segment's start: known already
  float* end = mode == kGlaLocal ? seg_out : sp;
  if (vc_ok) {
#pragma unroll
    for (int b = 0; b < NDB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
        if (c < dim) end[(int64_t)c * vdim + vc] = S[b][r];
      }
  }
  if (mode == kGlaLocal && blockIdx.z == 0) {
    __syncthreads();
    for (int c = threadIdx.x; c < dim; c += blockDim.x) seg_decay[((int64_t)blockIdx.x * heads + h) * dim + c] = dsum[c];
  }
}

// seg_state[segment] (its end state from the empty state) -> the state at the segment's end:
// S_end(j) = diag(e^(D_j)) S_end(j - 1) + local(j), S_end(-1) = the slot's state (nothing for a new sequence)
__global__ __launch_bounds__(256) void gla_scan_kernel(
    float* __restrict__ seg_state, const float* __restrict__ seg_decay, const float* __restrict__ state,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot,
    int heads, int dim, int vdim) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  const int size = dim * vdim;
  if (e >= size) return;
  const int c = e / vdim;
  const int n = q_start[seq + 1] - q_start[seq];
  const int segs = (n + kGlaSegment - 1) / kGlaSegment;
  if (segs <= 1) return;
  int first = 0;
  for (int s = 0; s < seq; ++s) first += (q_start[s + 1] - q_start[s] + kGlaSegment - 1) / kGlaSegment;
  float S = ctx_len[seq] == 0 ? 0.0f : state[((int64_t)state_slot[seq] * heads + h) * size + e];
  // eight segments at a time: their loads do not wait for one another
  const int64_t stride = (int64_t)heads * size, dstride = (int64_t)heads * dim;
  float* p = seg_state + ((int64_t)first * heads + h) * size + e;
  const float* d = seg_decay + ((int64_t)first * heads + h) * dim + c;
  for (int j0 = 0; j0 + 1 < segs; j0 += 8) {
    float local[8], keep[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      local[i] = j0 + i + 1 < segs ? p[(j0 + i) * stride] : 0.0f;
      keep[i] = j0 + i + 1 < segs ? expf(d[(j0 + i) * dstride]) : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (j0 + i + 1 < segs) {
        S = keep[i] * S + local[i];
        p[(j0 + i) * stride] = S;
      }
    }
  }
}

template <typename T, int NDB>
int launch_gla(float* out, const void* q, const void* k, const void* v, int64_t in_stride, const void* decay_pre,
               int64_t decay_stride, const float* decay_bias, float tau, float q_scale, float* state,
               const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows, int num_seqs,
               int max_query_len, int heads, int dim, int vdim, float* workspace, hipStream_t stream) {
  const int vblocks = (vdim + 31) / 32;
  const int waves = std::min(vblocks, 8);
  const size_t lds_bytes =
      (size_t)(3 * kGlaChunk * (NDB * 32 + 4) + kGlaChunk * waves * 32 + 9 * NDB * 32 + 16) * sizeof(float);
  auto kernel = gla_kernel<T, NDB>;
  static size_t allowed = 64 * 1024;                         // per instantiation
  if (lds_bytes > allowed) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds_bytes));
    allowed = lds_bytes;
  }
  const unsigned zgroups = (unsigned)((vblocks + waves - 1) / waves);
  const float inv_tau = 1.0f / tau;
  if (workspace == nullptr || max_query_len <= 2 * kGlaSegment) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)num_seqs, (unsigned)heads, zgroups), dim3(64 * waves), lds_bytes, stream,
                       out, q, k, v, in_stride, decay_pre, decay_stride, decay_bias, inv_tau, q_scale, state, q_start,
                       ctx_len, state_slot, num_seqs, heads, dim, vdim, kGlaWhole, (float*)nullptr, (float*)nullptr);
    SW_CHECK_LAUNCH();
    return SW_OK;
  }
  const int64_t items = rows / kGlaSegment + num_seqs;
  float* seg_state = workspace;
  float* seg_decay = workspace + items * heads * (int64_t)dim * vdim;
  hipLaunchKernelGGL(kernel, dim3((unsigned)items, (unsigned)heads, zgroups), dim3(64 * waves), lds_bytes, stream, out,
                     q, k, v, in_stride, decay_pre, decay_stride, decay_bias, inv_tau, q_scale, state, q_start, ctx_len,
                     state_slot, num_seqs, heads, dim, vdim, kGlaLocal, seg_state, seg_decay);
  SW_CHECK_LAUNCH();
  hipLaunchKernelGGL(gla_scan_kernel, dim3((unsigned)num_seqs, (unsigned)heads, (unsigned)((dim * vdim + 255) / 256)),
                     dim3(256), 0, stream, seg_state, seg_decay, state, q_start, ctx_len, state_slot, heads, dim, vdim);
  SW_CHECK_LAUNCH();
  hipLaunchKernelGGL(kernel, dim3((unsigned)items, (unsigned)heads, zgroups), dim3(64 * waves), lds_bytes, stream, out,
                     q, k, v, in_stride, decay_pre, decay_stride, decay_bias, inv_tau, q_scale, state, q_start, ctx_len,
                     state_slot, num_seqs, heads, dim, vdim, kGlaFinal, seg_state, seg_decay);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // namespace swm

extern "C" int64_t swm_gla_workspace_floats(int64_t rows, int num_seqs, int max_query_len, int heads, int dim, int vdim) {
  if (max_query_len <= 2 * swm::kGlaSegment) return 0;
  return (rows / swm::kGlaSegment + num_seqs) * (int64_t)heads * dim * ((int64_t)vdim + 1);
}

extern "C" int swm_gla(float* out, const void* q, const void* k, const void* v, int64_t in_stride,
                       const void* decay_pre, int64_t decay_stride, const float* decay_bias, float tau, float q_scale,
                       float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot,
                       int64_t rows, int num_seqs, int max_query_len, int heads, int dim, int vdim, float* workspace,
                       int act_dtype, void* stream) {
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
                                                         state_slot, rows, num_seqs, max_query_len, heads, dim,     \
                                                         vdim, workspace, s)););                                    \
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
