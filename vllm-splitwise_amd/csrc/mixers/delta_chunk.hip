// The delta rule with a gate and ONE decay per head in chunks of 32 tokens, for steps that bring long runs:
//     S <- g_t S;  u_t = beta_t (v_t - S^T k_t);  S <- S + k_t u_t^T;  o_t = S^T q_t         (S [dim, vdim], fp32)
// With L_t = log g_1 + ... + log g_t inside a chunk (<= 0, so every ratio e^(L_t - L_s), s <= t, is at most 1) and S_0
// the state at the chunk's start, the chunk's u_t solve (I + A) U = diag(beta) (V - diag(e^L) K S_0) with the strict
// lower triangle A[t, s] = beta_t e^(L_t - L_s) (k_t . k_s).  T = (I + A)^-1 does not depend on the state, so
//   a PROLOGUE, parallel over (chunk, head), makes unit q and k, beta, L, inverts the triangle by forward
//   substitution and leaves   Kb = T diag(beta e^L) K,  Vb = T diag(beta) V,  P[t, s] = e^(L_t - L_s) (q_t . k_s) (s <= t),
//   Qg = diag(e^L) Q,  Kg = diag(e^(L_n - L)) K  and  e^(L_n);
//   the SEQUENTIAL kernel walks a sequence's chunks with   U = Vb - Kb S_0,   O = Qg S_0 + P U,   S_n = e^(L_n) S_0 + Kg^T U,
//   four fp32 products on the matrix cores (v_mfma_f32_32x32x2_f32) per chunk, which is the recurrence with its sums
//   reordered.  A workgroup owns (sequence, head, 32 value channels); its wave b keeps the state's key coordinates
//   32 b .. 32 b + 31 in the accumulator layout (lane l: value channel l % 32; element r: key coordinate 32 b +
//   8 (r / 4) + 4 (l / 32) + r % 4) for the whole run; the waves share a chunk's Kb, Qg, Kg and P, staged once in LDS.
// Rows of a last, shorter chunk are padded with beta = 0, k = 0, g = 1: they change nothing and are not stored.
#include "mixers_common.cuh"

namespace swm {

using f32x16 = __attribute__((ext_vector_type(16))) float;
constexpr int kDcChunk = 32;
constexpr int kDcPrepThreads = 256;

// floats of one (chunk, head) in the workspace: Kb | Qg | Kg ([32][dp] each) | P [32][32] | Vb [32][vdim] | e^(L_n), padded
__host__ __device__ inline int64_t dc_record_floats(int dp, int vdim) { return 96 * (int64_t)dp + 1024 + 32 * (int64_t)vdim + 32; }

// (three waves per SIMD: without the bound the compiler spends registers on the unrolled last loop and one workgroup
// fills a compute unit)
template <typename T>
__global__ __launch_bounds__(kDcPrepThreads, 3) void delta_chunk_prep_kernel(
    float* __restrict__ work, const float* __restrict__ qkv, const void* __restrict__ beta_pre, int64_t beta_stride,
    const void* __restrict__ decay_pre, int64_t decay_stride, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const int32_t* __restrict__ q_start, int num_seqs, int heads, int kv_heads, int dim,
    int vdim, int dp) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int KS = dp + 4;                         // rows on 16 bytes
  float* Kn = lds;                               // [32][KS] unit keys
  float* Qn = Kn + kDcChunk * KS;                // [32][KS] unit queries times dim^-1/2
  float* A = Qn + kDcChunk * KS;                 // [32][33] the strict lower triangle, then scratch
  float* Tm = A + kDcChunk * 33;                 // [32][33] (I + A)^-1
  float* beta = Tm + kDcChunk * 33;              // [32]
  float* L = beta + kDcChunk;                    // [32] running sums of the log decays
  float* eL = L + kDcChunk;                      // [32] their exponentials
  int seq = 0, tok0 = 0;
  const int cn = find_query_tile(q_start, num_seqs, blockIdx.x, kDcChunk, &seq, &tok0);
  if (cn <= 0) return;                           // the whole workgroup
  const int h = blockIdx.y, g = h / (heads / kv_heads);
  const int64_t row0 = q_start[seq] + tok0;
  const int64_t row_w = 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float qscale = 1.0f / sqrtf((float)dim);
  // ---- the chunk's raw queries and keys into LDS (every load in flight at once), then unit length in place;
  //      beta and the log decays
  for (int e = threadIdx.x; e < kDcChunk * dp; e += kDcPrepThreads) {
    const int r = e / dp, i = e % dp;
    const bool in = r < cn && i < dim;
    const float* q = qkv + (row0 + r) * row_w + (int64_t)g * dim;
    Qn[r * KS + i] = in ? q[i] : 0.0f;
    Kn[r * KS + i] = in ? q[(int64_t)kv_heads * dim + i] : 0.0f;
  }
  if (threadIdx.x < kDcChunk) {
    const int r = threadIdx.x;
    beta[r] = r < cn ? sigmoidf_(ld<T>(beta_pre, (row0 + r) * beta_stride + h)) : 0.0f;
    L[r] = r < cn ? -expf(a_log[h]) * softplusf_(ld<T>(decay_pre, (row0 + r) * decay_stride + h) + dt_bias[h]) : 0.0f;
  }
  __syncthreads();
  for (int r = wave; r < kDcChunk; r += kDcPrepThreads / 64) {
    float qq = 0.0f, kk = 0.0f;
    for (int i = lane; i < dp; i += 64) {
      qq += Qn[r * KS + i] * Qn[r * KS + i];
      kk += Kn[r * KS + i] * Kn[r * KS + i];
    }
    qq = sw::wave_sum(qq);
    kk = sw::wave_sum(kk);
    const float qf = qscale / sqrtf(qq + 1e-6f), kf = 1.0f / sqrtf(kk + 1e-6f);
    for (int i = lane; i < dp; i += 64) {
      Qn[r * KS + i] *= qf;
      Kn[r * KS + i] *= kf;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = 0.0f;
    for (int r = 0; r < kDcChunk; ++r) {
      run += L[r];
      L[r] = run;
      eL[r] = expf(run);
    }
  }
  __syncthreads();
  float* rec = work + ((int64_t)blockIdx.x * heads + h) * dc_record_floats(dp, vdim);
  float* Kb = rec;
  float* Qg = rec + 32 * (int64_t)dp;
  float* Kg = rec + 64 * (int64_t)dp;
  float* P = rec + 96 * (int64_t)dp;
  float* Vb = P + 1024;
  // ---- A (strict lower) and P (lower with the diagonal)
  for (int e = threadIdx.x; e < kDcChunk * kDcChunk; e += kDcPrepThreads) {
    const int t = e >> 5, s = e & 31;
    float kk = 0.0f, qk = 0.0f;
    if (s <= t) {
      float4 k4 = make_float4(0.f, 0.f, 0.f, 0.f), q4 = k4;
#pragma unroll 4
      for (int i = 0; i < dp; i += 4) {                         // the padding holds zeros
        const float4 ks = *reinterpret_cast<const float4*>(Kn + s * KS + i);
        const float4 kt = *reinterpret_cast<const float4*>(Kn + t * KS + i);
        const float4 qt = *reinterpret_cast<const float4*>(Qn + t * KS + i);
        k4.x += kt.x * ks.x; k4.y += kt.y * ks.y; k4.z += kt.z * ks.z; k4.w += kt.w * ks.w;
        q4.x += qt.x * ks.x; q4.y += qt.y * ks.y; q4.z += qt.z * ks.z; q4.w += qt.w * ks.w;
      }
      kk = (k4.x + k4.y) + (k4.z + k4.w);
      qk = (q4.x + q4.y) + (q4.z + q4.w);
    }
    const float ratio = s <= t ? expf(L[t] - L[s]) : 0.0f;
    A[t * 33 + s] = s < t ? beta[t] * ratio * kk : 0.0f;
    P[e] = ratio * qk;
  }
  __syncthreads();
  // ---- T = (I + A)^-1 row by row: T[t, :] = e_t - sum_{s < t} A[t, s] T[s, :]
  // Eight neighbouring lanes share column j (lane part p takes the rows s = j + p, j + p + 8, ...), a wave holds eight
  // whole columns: a column reads only what its own lanes wrote, so the waves need no barrier between the rows.
  {
    const int j = threadIdx.x >> 3, p = threadIdx.x & 7;
    for (int t = 0; t < kDcChunk; ++t) {
      float part = 0.0f;
      for (int s = j + p; s < t; s += 8) part += A[t * 33 + s] * Tm[s * 33 + j];     // T[s, j] = 0 for s < j
      part = lanes_sum<8>(part);
      if (p == 0) Tm[t * 33 + j] = (t == j ? 1.0f : 0.0f) - part;
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
    }
  }
  __syncthreads();
  // ---- A <- T diag(beta): what V is multiplied with;  Tm <- T diag(beta e^L): what K is multiplied with
  for (int e = threadIdx.x; e < kDcChunk * kDcChunk; e += kDcPrepThreads) {
    const int t = e >> 5, s = e & 31;
    const float tb = s <= t ? Tm[t * 33 + s] * beta[s] : 0.0f;
    A[t * 33 + s] = tb;
    Tm[t * 33 + s] = tb * eL[s];
  }
  __syncthreads();
  const float Ln = L[kDcChunk - 1];
  for (int e = threadIdx.x; e < kDcChunk * dp; e += kDcPrepThreads) {
    const int t = e / dp, i = e % dp;
    float acc = 0.0f;
#pragma unroll 4
    for (int s = 0; s <= t; ++s) acc += Tm[t * 33 + s] * Kn[s * KS + i];
    Kb[e] = acc;
    Qg[e] = eL[t] * Qn[t * KS + i];
    Kg[e] = expf(Ln - L[t]) * Kn[t * KS + i];
  }
  if (threadIdx.x == 0) Vb[32 * (int64_t)vdim] = expf(Ln);
  // ---- Vb = T diag(beta) V, a thread per value channel
  const int64_t v_off = 2 * (int64_t)kv_heads * dim + (int64_t)h * vdim;
  for (int c = threadIdx.x; c < vdim; c += kDcPrepThreads) {
    float vv[kDcChunk];
#pragma unroll
    for (int s = 0; s < kDcChunk; ++s) vv[s] = s < cn ? qkv[(row0 + s) * row_w + v_off + c] : 0.0f;
#pragma unroll
    for (int t = 0; t < kDcChunk; ++t) {
      float acc = 0.0f;
#pragma unroll
      for (int s = 0; s <= t; ++s) acc += A[t * 33 + s] * vv[s];
      Vb[t * (int64_t)vdim + c] = acc;
    }
  }
}

// One workgroup owns (sequence, head, 32 value channels); its wave b owns the state's key coordinates 32 b .. 32 b + 31
// (one accumulator block), so the products over the key size are shared out among the waves: every wave multiplies its
// block of Kb and Qg with its block of S, the partial products meet in LDS, every wave forms the same U from them, the
// chunk's turn-taking wave adds P U to the summed Qg S_0 and stores the outputs, and every wave updates its block of S.
template <int NDB>
__global__ __launch_bounds__(64 * NDB) void delta_chunk_kernel(
    float* __restrict__ out, const float* __restrict__ work, float* __restrict__ state,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot,
    int heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int DP = NDB * 32;
  constexpr int DS = DP + 4;
  float* Kbs = lds;                              // [32][DS]
  float* Qgs = Kbs + kDcChunk * DS;
  float* Kgs = Qgs + kDcChunk * DS;
  float* Ps = Kgs + kDcChunk * DS;               // [32][36]
  float* red = Ps + kDcChunk * 36;               // [NDB][2][16][64]: every wave's Kb S_b and Qg S_b, register by register
  const int seq = blockIdx.x, h = blockIdx.y;
  const int b = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 31, hl = lane >> 5;
  const int n = q_start[seq + 1] - q_start[seq];
  if (n <= 0) return;                            // the whole workgroup
  const int64_t row0 = q_start[seq];
  int chunk0 = 0;                                // this sequence's first chunk among the step's
  for (int s = 0; s < seq; ++s) chunk0 += (q_start[s + 1] - q_start[s] + kDcChunk - 1) / kDcChunk;
  const int vc = blockIdx.z * 32 + li;           // this lane's value channel
  const bool vc_ok = vc < vdim;
  const int vcc = vc_ok ? vc : vdim - 1;
  float* sp = state + ((int64_t)state_slot[seq] * heads + h) * (int64_t)dim * vdim;
  f32x16 S;
  const bool fresh = ctx_len[seq] == 0;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
    S[r] = (!fresh && vc_ok && c < dim) ? sp[(int64_t)c * vdim + vc] : 0.0f;
  }
  const int64_t rec_floats = dc_record_floats(DP, vdim);
  const int chunks = (n + kDcChunk - 1) / kDcChunk;
  for (int ci = 0; ci < chunks; ++ci) {
    const int cn = min(kDcChunk, n - ci * kDcChunk);
    const float* rec = work + ((int64_t)(chunk0 + ci) * heads + h) * rec_floats;
    const float* Vb = rec + 96 * (int64_t)DP + 1024;
    __syncthreads();                             // the last chunk's tiles and partial products have been read
    for (int e = threadIdx.x; e < kDcChunk * DP / 4; e += 64 * NDB) {
      const int r = e / (DP / 4), c = (e % (DP / 4)) * 4;
      *reinterpret_cast<float4*>(Kbs + r * DS + c) = *reinterpret_cast<const float4*>(rec + r * DP + c);
      *reinterpret_cast<float4*>(Qgs + r * DS + c) = *reinterpret_cast<const float4*>(rec + 32 * DP + r * DP + c);
      *reinterpret_cast<float4*>(Kgs + r * DS + c) = *reinterpret_cast<const float4*>(rec + 64 * DP + r * DP + c);
    }
    for (int e = threadIdx.x; e < 1024; e += 64 * NDB) Ps[(e >> 5) * 36 + (e & 31)] = rec[96 * DP + e];
    // this lane's Vb: token (r, hl), channel vc
    float u[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) u[r] = Vb[(int64_t)(8 * (r / 4) + 4 * hl + (r % 4)) * vdim + vcc];
    const float gn = Vb[32 * (int64_t)vdim];
    __syncthreads();
    // ---- this wave's share of Kb S_0 and Qg S_0: A = the staged rows (token li, coordinate), B = the state's block
    f32x16 ks, o;
#pragma unroll
    for (int r = 0; r < 16; ++r) ks[r] = o[r] = 0.0f;
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const int c = 32 * b + 8 * g4 + 4 * hl;
      const float4 kb = *reinterpret_cast<const float4*>(Kbs + li * DS + c);
      const float4 qg = *reinterpret_cast<const float4*>(Qgs + li * DS + c);
      ks = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.x, S[4 * g4], ks, 0, 0, 0);
      ks = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.y, S[4 * g4 + 1], ks, 0, 0, 0);
      ks = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.z, S[4 * g4 + 2], ks, 0, 0, 0);
      ks = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.w, S[4 * g4 + 3], ks, 0, 0, 0);
      o = __builtin_amdgcn_mfma_f32_32x32x2f32(qg.x, S[4 * g4], o, 0, 0, 0);
      o = __builtin_amdgcn_mfma_f32_32x32x2f32(qg.y, S[4 * g4 + 1], o, 0, 0, 0);
      o = __builtin_amdgcn_mfma_f32_32x32x2f32(qg.z, S[4 * g4 + 2], o, 0, 0, 0);
      o = __builtin_amdgcn_mfma_f32_32x32x2f32(qg.w, S[4 * g4 + 3], o, 0, 0, 0);
    }
    if (NDB > 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        red[((b * 2) * 16 + r) * 64 + lane] = ks[r];
        red[((b * 2 + 1) * 16 + r) * 64 + lane] = o[r];
      }
      __syncthreads();
      // ---- U = Vb - Kb S_0 (the waves' shares summed in a fixed order): element r is token (r, hl), channel li
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < NDB; ++w) total += red[((w * 2) * 16 + r) * 64 + lane];
        u[r] -= total;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) u[r] -= ks[r];
    }
    // ---- O = Qg S_0 + P U, by one wave (they take turns): A = P (token li, key token (r, hl)), B = U
    if (b == ci % NDB) {
      if (NDB > 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float total = 0.0f;
#pragma unroll
          for (int w = 0; w < NDB; ++w) total += red[((w * 2 + 1) * 16 + r) * 64 + lane];
          o[r] = total;
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r)
        o = __builtin_amdgcn_mfma_f32_32x32x2f32(Ps[li * 36 + 8 * (r / 4) + 4 * hl + (r % 4)], u[r], o, 0, 0, 0);
      if (vc_ok) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int t = 8 * (r / 4) + 4 * hl + (r % 4);
          if (t < cn) out[((row0 + ci * kDcChunk + t) * heads + h) * (int64_t)vdim + vc] = o[r];
        }
      }
    }
    // ---- S_b <- e^(L_n) S_b + Kg_b^T U: A = Kg transposed (coordinate 32 b + li, token (r, hl)), B = U
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] *= gn;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      S = __builtin_amdgcn_mfma_f32_32x32x2f32(Kgs[(8 * (r / 4) + 4 * hl + (r % 4)) * DS + 32 * b + li], u[r], S, 0, 0, 0);
  }
  if (vc_ok) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
      if (c < dim) sp[(int64_t)c * vdim + vc] = S[r];
    }
  }
}

template <typename K>
inline hipError_t dc_allow_lds(K kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

template <int NDB>
int launch_delta_chunk(float* out, const float* work, float* state, const int32_t* q_start, const int32_t* ctx_len,
                       const int32_t* state_slot, int num_seqs, int heads, int dim, int vdim, hipStream_t stream) {
  const size_t lds_bytes =
      sizeof(float) * (3 * (size_t)kDcChunk * (NDB * 32 + 4) + kDcChunk * 36 + (NDB > 1 ? NDB * 2 * 16 * 64 : 0));
  SW_CHECK_HIP(dc_allow_lds(delta_chunk_kernel<NDB>, lds_bytes));
  const dim3 grid((unsigned)num_seqs, (unsigned)heads, (unsigned)((vdim + 31) / 32));
  hipLaunchKernelGGL(delta_chunk_kernel<NDB>, grid, dim3(64 * NDB), lds_bytes, stream, out, work, state, q_start, ctx_len,
                     state_slot, heads, dim, vdim);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // namespace swm

extern "C" {

int64_t swm_gated_delta_chunked_workspace_floats(int64_t rows, int num_seqs, int heads, int dim, int vdim) {
  const int dp = (dim + 31) / 32 * 32;
  return (rows / swm::kDcChunk + num_seqs) * heads * swm::dc_record_floats(dp, vdim);
}

int swm_gated_delta_chunked(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride,
                            const void* decay_pre, int64_t decay_stride, const float* dt_bias, const float* a_log,
                            float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot,
                            int64_t rows, int num_seqs, int heads, int kv_heads, int dim, int vdim, float* workspace,
                            int act_dtype, void* stream) {
  using namespace swm;
  if (num_seqs == 0 || rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "gated_delta_chunked: unsupported dtype %d", act_dtype);
  // a chunk's staged operands and the waves' partial products fill the LDS of a compute unit at key size 224
  SW_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 224 && vdim > 0 &&
                   workspace != nullptr && rows < (1ll << 31),
               "gated_delta_chunked: heads %d, kv heads %d, key size %d (up to 224), value size %d", heads, kv_heads, dim,
               vdim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int ndb = (dim + 31) / 32, dp = ndb * 32;
  const int64_t chunks = rows / kDcChunk + num_seqs;            // an upper bound: surplus workgroups leave at once
  const size_t prep_lds = sizeof(float) * (2 * (size_t)kDcChunk * (dp + 4) + 2 * kDcChunk * 33 + 3 * kDcChunk);
  SWM_DISPATCH_ACT(act_dtype, SW_CHECK_HIP(dc_allow_lds(delta_chunk_prep_kernel<T>, prep_lds)););
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(delta_chunk_prep_kernel<T>, dim3((unsigned)chunks, (unsigned)heads),
                                                 dim3(kDcPrepThreads), prep_lds, s, workspace, qkv, beta_pre, beta_stride,
                                                 decay_pre, decay_stride, dt_bias, a_log, q_start, num_seqs, heads,
                                                 kv_heads, dim, vdim, dp););
  SW_CHECK_LAUNCH();
  switch (ndb) {
    case 1: return launch_delta_chunk<1>(out, workspace, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, s);
    case 2: return launch_delta_chunk<2>(out, workspace, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, s);
    case 3: return launch_delta_chunk<3>(out, workspace, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, s);
    case 4: return launch_delta_chunk<4>(out, workspace, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, s);
    case 5: return launch_delta_chunk<5>(out, workspace, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, s);
    case 6: return launch_delta_chunk<6>(out, workspace, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, s);
    default: return launch_delta_chunk<7>(out, workspace, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, s);
  }
}

}  // extern "C"
