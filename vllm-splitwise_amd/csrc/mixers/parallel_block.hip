// Pieces of a decoder layer whose two sublayers read ONE norm of an fp32 residual stream:
//   * stream_add_norm: the sublayers' outputs are summed into the stream and the next layer's norm (per-channel
//     weight with an offset, so that a weight stored around zero is offset + w) is taken in the same pass;
//   * clamped_glu / relu2: activations between the library GEMMs of a feed-forward;
//   * rope_cache: partial rotary embedding on neighbouring pairs from a table of per-pair frequencies (angles
//     from fp32 positions), rotated queries out in fp32, rotated keys and values into the paged cache;
//   * group_router: the choice of a sigmoid router from its fp32 logits: a selection bias, a limit to the best
//     groups of experts and weights normalised over the chosen ones.
// All arithmetic is fp32; activations are read and written in the model's dtype.
#include "mixers_common.cuh"

namespace swm {

constexpr int kPbThreads = 256;
constexpr int kMaxNormHeads = 1024;     // query plus key heads of a layer whose rotation kernel also norms them

// residual += (a + b + c);  out = residual / sqrt(mean(residual^2) + eps) * (offset + weight)
template <typename T>
__global__ __launch_bounds__(kPbThreads) void stream_add_norm_kernel(
    float* __restrict__ residual, const void* __restrict__ a, int64_t a_stride, const void* __restrict__ b,
    int64_t b_stride, const float* __restrict__ c, const float* __restrict__ weight, float offset, float eps,
    void* __restrict__ out, int width) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float* r = residual + t * (int64_t)width;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < width; i += kPbThreads) {
    float v = r[i];
    if (a != nullptr || b != nullptr || c != nullptr) {
      float add = 0.0f;
      if (a != nullptr) add += ld<T>(a, t * a_stride + i);
      if (b != nullptr) add += ld<T>(b, t * b_stride + i);
      if (c != nullptr) add += c[t * (int64_t)width + i];
      v += add;
      r[i] = v;
    }
    ss += v * v;
  }
  if (out == nullptr) return;
  ss = block_sum(ss, red);
  const float f = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += kPbThreads)
    st<T>(out, t * (int64_t)width + i, r[i] * f * (offset + weight[i]));
}

// in [rows, 2 * ff] (gate | up):  g = min(gate, limit), u = clamp(up, -limit, limit);  out = g sigmoid(alpha g) (u + shift)
template <typename T>
__global__ __launch_bounds__(kPbThreads) void clamped_glu_kernel(void* __restrict__ out, const void* __restrict__ in,
                                                                 int64_t in_stride, int ff, float alpha, float limit,
                                                                 float shift) {
  const int64_t t = blockIdx.x;
  for (int i = blockIdx.y * kPbThreads + threadIdx.x; i < ff; i += gridDim.y * kPbThreads) {
    const float g = fminf(ld<T>(in, t * in_stride + i), limit);
    const float u = fminf(fmaxf(ld<T>(in, t * in_stride + ff + i), -limit), limit);
    st<T>(out, t * (int64_t)ff + i, g * sigmoidf_(alpha * g) * (u + shift));
  }
}

template <typename T>
__global__ __launch_bounds__(kPbThreads) void relu2_kernel(void* __restrict__ out, const void* __restrict__ in,
                                                           int64_t in_stride, int ff) {
  const int64_t t = blockIdx.x;
  for (int i = blockIdx.y * kPbThreads + threadIdx.x; i < ff; i += gridDim.y * kPbThreads) {
    const float z = fmaxf(ld<T>(in, t * in_stride + i), 0.0f);
    st<T>(out, t * (int64_t)ff + i, z * z);
  }
}

// one workgroup per row; a thread per (head, pair) or per passed-through coordinate
template <typename T>
__global__ __launch_bounds__(kPbThreads) void rope_cache_kernel(
    float* __restrict__ q_out, const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    int64_t in_stride, const int64_t* __restrict__ positions, const float* __restrict__ inv_freq, int rot_dims,
    void* __restrict__ key_cache, void* __restrict__ value_cache, const int64_t* __restrict__ slot_mapping, int heads,
    int kv_heads, int dim, int vdim, int pair_halves, const float* __restrict__ q_norm,
    const float* __restrict__ k_norm, float norm_eps) {
  const int64_t t = blockIdx.x;
  const int64_t row = t * in_stride;
  const float pos = (float)positions[t];
  // optional RMS norm of every query and key head over its coordinates (one weight [dim] for all heads), before
  // the rotation: a wave per head works out the head's factor
  __shared__ float fac[kMaxNormHeads];
  const bool normed = q_norm != nullptr;
  if (normed) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int all = heads + (k != nullptr ? kv_heads : 0);
    for (int h = wave; h < all; h += kPbThreads / 64) {
      const void* src = h < heads ? q : k;
      const int64_t off = row + (int64_t)(h < heads ? h : h - heads) * dim;
      float ss = 0.0f;
      for (int i = lane; i < dim; i += 64) {
        const float x = ld<T>(src, off + i);
        ss += x * x;
      }
      ss = sw::wave_sum(ss);
      if (lane == 0) fac[h] = 1.0f / sqrtf(ss / (float)dim + norm_eps);
    }
    __syncthreads();
  }
  auto lq = [&](int h, int i) {
    const float x = ld<T>(q, row + (int64_t)h * dim + i);
    return normed ? x * fac[h] * q_norm[i] : x;
  };
  auto lk = [&](int h, int i) {
    const float x = ld<T>(k, row + (int64_t)h * dim + i);
    return normed ? x * fac[heads + h] * k_norm[i] : x;
  };
  if (pair_halves) {
    // coordinate i < rot_dims / 2 turns with coordinate i + rot_dims / 2; those from rot_dims on pass
    const int hf = rot_dims / 2, units = dim - hf;            // a unit: one pair, or one passed-through coordinate
    for (int e = threadIdx.x; e < heads * units; e += kPbThreads) {
      const int h = e / units, u = e % units;
      const int64_t src = row + h * dim, dst = t * (int64_t)heads * dim + h * dim;
      if (u < hf) {
        const float a = lq(h, u), b = lq(h, u + hf);
        float s, c;
        sincosf(pos * inv_freq[u], &s, &c);
        q_out[dst + u] = a * c - b * s;
        q_out[dst + u + hf] = b * c + a * s;
      } else {
        q_out[dst + u + hf] = lq(h, u + hf);
      }
    }
    if (k == nullptr) return;
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    for (int e = threadIdx.x; e < kv_heads * units; e += kPbThreads) {
      const int h = e / units, u = e % units;
      const int64_t src = row + h * dim, dst = slot * (int64_t)kv_heads * dim + h * dim;
      if (u < hf) {
        const float a = lk(h, u), b = lk(h, u + hf);
        float s, c;
        sincosf(pos * inv_freq[u], &s, &c);
        st<T>(key_cache, dst + u, a * c - b * s);
        st<T>(key_cache, dst + u + hf, b * c + a * s);
      } else {
        st<T>(key_cache, dst + u + hf, lk(h, u + hf));
      }
    }
    for (int e = threadIdx.x; e < kv_heads * vdim; e += kPbThreads)
      st<T>(value_cache, slot * (int64_t)kv_heads * vdim + e, ld<T>(v, row + e));
    return;
  }
  const int half = rot_dims / 2, pairs = dim / 2;          // pairs beyond `half` pass through; so does an odd last one
  // queries
  for (int e = threadIdx.x; e < heads * pairs; e += kPbThreads) {
    const int h = e / pairs, i = e % pairs;
    const int64_t src = row + h * dim + 2 * i, dst = t * (int64_t)heads * dim + h * dim + 2 * i;
    const float a = lq(h, 2 * i), b = lq(h, 2 * i + 1);
    if (i < half) {
      float s, c;
      sincosf(pos * inv_freq[i], &s, &c);
      q_out[dst] = a * c - b * s;
      q_out[dst + 1] = b * c + a * s;
    } else {
      q_out[dst] = a;
      q_out[dst + 1] = b;
    }
  }
  if (dim & 1)
    for (int h = threadIdx.x; h < heads; h += kPbThreads)
      q_out[t * (int64_t)heads * dim + h * dim + dim - 1] = lq(h, dim - 1);
  if (k == nullptr) return;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  for (int e = threadIdx.x; e < kv_heads * pairs; e += kPbThreads) {
    const int h = e / pairs, i = e % pairs;
    const int64_t src = row + h * dim + 2 * i, dst = slot * (int64_t)kv_heads * dim + h * dim + 2 * i;
    const float a = lk(h, 2 * i), b = lk(h, 2 * i + 1);
    if (i < half) {
      float s, c;
      sincosf(pos * inv_freq[i], &s, &c);
      st<T>(key_cache, dst, a * c - b * s);
      st<T>(key_cache, dst + 1, b * c + a * s);
    } else {
      st<T>(key_cache, dst, a);
      st<T>(key_cache, dst + 1, b);
    }
  }
  if (dim & 1)
    for (int h = threadIdx.x; h < kv_heads; h += kPbThreads)
      st<T>(key_cache, slot * (int64_t)kv_heads * dim + h * dim + dim - 1, lk(h, dim - 1));
  for (int e = threadIdx.x; e < kv_heads * vdim; e += kPbThreads)
    st<T>(value_cache, slot * (int64_t)kv_heads * vdim + e, ld<T>(v, row + e));
}

// The choice of one row by one wave: scores by the lanes, the choice by lane 0 (a few hundred LDS reads for the usual
// sizes).  logits: the row's `experts` numbers (global or LDS); score, choice: LDS scratch of the wave.
constexpr int kMaxRouterExperts = 256;

__device__ __forceinline__ void router_choice(int lane, const float* __restrict__ logits, float* score, float* choice,
                                              const float* __restrict__ correction, int experts, int top, int groups,
                                              int keep, float scale, int softmax, int group_best_one, int normalize,
                                              int32_t* __restrict__ chosen, float* __restrict__ weights) {
  float top_logit = 0.0f, inv_sum = 1.0f;
  if (softmax) {                                             // scores: the softmax over ALL experts
    float m = -INFINITY;
    for (int e = lane; e < experts; e += 64) m = fmaxf(m, logits[e]);
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    float sum = 0.0f;
    for (int e = lane; e < experts; e += 64) sum += expf(logits[e] - m);
    top_logit = m;
    inv_sum = 1.0f / sw::wave_sum(sum);
  }
  for (int e = lane; e < experts; e += 64) {
    const float z = logits[e];
    const float s = softmax ? expf(z - top_logit) * inv_sum : sigmoidf_(z);
    score[e] = s;
    choice[e] = s + (correction != nullptr ? correction[e] : 0.0f);
  }
  __builtin_amdgcn_wave_barrier();
  __threadfence_block();
  // Lane l holds the candidates e = l + 64 k (and the groups g = l + 64 k); every pick is an arg-max over the wave.
  constexpr int PER = kMaxRouterExperts / 64;
  const float kOut = -INFINITY;
  float cand[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) cand[k] = lane + 64 * k < experts ? choice[lane + 64 * k] : kOut;
  if (groups > 1 && keep < groups) {
    const int size = experts / groups;
    // a group's score: its two largest choice scores (or its largest); the groups outside the best `keep` leave the choice
    float gs[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int g = lane + 64 * k;
      gs[k] = INFINITY;                                      // no such group, or one already dropped: never the worst
      if (g < groups) {
        float first = kOut, second = kOut;
        for (int j = 0; j < size; ++j) {
          const float c = choice[g * size + j];
          if (c > first) { second = first; first = c; }
          else if (c > second) second = c;
        }
        gs[k] = (size > 1 && !group_best_one) ? first + second : first;
      }
    }
    for (int drop = 0; drop < groups - keep; ++drop) {
      float lv = INFINITY;
      int lg = -1;
#pragma unroll
      for (int k = 0; k < PER; ++k)                          // ties: the later group goes first
        if (lane + 64 * k < groups && gs[k] <= lv && gs[k] != INFINITY) { lv = gs[k]; lg = lane + 64 * k; }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(lv, off, 64);
        const int og = __shfl_xor(lg, off, 64);
        if (og >= 0 && (lg < 0 || ov < lv || (ov == lv && og > lg))) { lv = ov; lg = og; }
      }
#pragma unroll
      for (int k = 0; k < PER; ++k) {
        if (lane + 64 * k == lg) gs[k] = INFINITY;
        if (lane + 64 * k < experts && (lane + 64 * k) / size == lg) cand[k] = kOut;
      }
    }
  }
  float total = 0.0f;
  for (int n = 0; n < top; ++n) {
    float lv = kOut;
    int le = 1 << 30;
#pragma unroll
    for (int k = 0; k < PER; ++k)                            // ties: the earlier expert
      if (lane + 64 * k < experts && (cand[k] > lv || le == (1 << 30))) { lv = cand[k]; le = lane + 64 * k; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(lv, off, 64);
      const int oe = __shfl_xor(le, off, 64);
      if (ov > lv || (ov == lv && oe < le)) { lv = ov; le = oe; }
    }
#pragma unroll
    for (int k = 0; k < PER; ++k)
      if (lane + 64 * k == le) cand[k] = kOut;
    if (lane == 0) {
      chosen[n] = le;
      weights[n] = score[le];
    }
    total += score[le];
  }
  if (lane != 0) return;
  const float f = normalize ? scale / (total + 1e-20f) : scale;
  for (int n = 0; n < top; ++n) weights[n] *= f;
}

// one wave per row, logits given
__global__ __launch_bounds__(256) void group_router_kernel(
    int32_t* __restrict__ chosen, float* __restrict__ weights, const float* __restrict__ logits,
    const float* __restrict__ correction, int64_t rows, int experts, int top, int groups, int keep, float scale,
    int softmax, int group_best_one, int normalize) {
  __shared__ float s_score[4][kMaxRouterExperts];
  __shared__ float s_choice[4][kMaxRouterExperts];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  if (t >= rows) return;                                     // uniform over the wave; no workgroup barrier below
  router_choice(lane, logits + t * experts, s_score[wave], s_choice[wave], correction, experts, top, groups, keep, scale,
                softmax, group_best_one, normalize, chosen + t * top, weights + t * top);
}

// (row, choice) pairs grouped by expert in ONE launch of one workgroup: a histogram of the chosen experts in LDS, its
// running sum = every expert's first sorted pair, then every pair takes the next place of its expert.  The order
// inside an expert is whatever the LDS counters hand out: the experts' rows are independent, so it does not matter.
constexpr int kPairThreads = 1024;

__global__ __launch_bounds__(kPairThreads) void group_pairs_kernel(int32_t* __restrict__ order,
                                                                   int32_t* __restrict__ expert_start,
                                                                   const int32_t* __restrict__ chosen, int64_t pairs,
                                                                   int experts) {
  __shared__ int count[kMaxRouterExperts + 1];
  __shared__ int cursor[kMaxRouterExperts];
  for (int e = threadIdx.x; e <= experts; e += kPairThreads) count[e] = 0;
  __syncthreads();
  for (int64_t p = threadIdx.x; p < pairs; p += kPairThreads) atomicAdd(&count[chosen[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < experts; ++e) {
      const int n = count[e];
      expert_start[e] = run;
      cursor[e] = run;
      run += n;
    }
    expert_start[experts] = run;
  }
  __syncthreads();
  for (int64_t p = threadIdx.x; p < pairs; p += kPairThreads) order[atomicAdd(&cursor[chosen[p]], 1)] = (int32_t)p;
}

}  // namespace swm

extern "C" {

int swm_stream_add_norm(float* residual, const void* a, int64_t a_stride, const void* b, int64_t b_stride,
                        const float* c, const float* weight, float offset, float eps, void* out, int64_t rows,
                        int width, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "stream_add_norm: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(width > 0 && rows < (1ll << 31) && (out == nullptr || weight != nullptr), "stream_add_norm: bad shape");
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(stream_add_norm_kernel<T>, dim3((unsigned)rows), dim3(kPbThreads), 0,
                                                 static_cast<hipStream_t>(stream), residual, a, a_stride, b, b_stride, c,
                                                 weight, offset, eps, out, width););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_clamped_glu(void* out, const void* in, int64_t in_stride, int64_t rows, int ff, float alpha, float limit,
                    float shift, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "clamped_glu: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(ff > 0 && rows < (1ll << 31) && limit > 0.0f, "clamped_glu: bad shape or limit");
  const dim3 grid((unsigned)rows, (unsigned)std::min(8, (ff + kPbThreads - 1) / kPbThreads));
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(clamped_glu_kernel<T>, grid, dim3(kPbThreads), 0,
                                                 static_cast<hipStream_t>(stream), out, in, in_stride, ff, alpha, limit,
                                                 shift););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_relu2(void* out, const void* in, int64_t in_stride, int64_t rows, int ff, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "relu2: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(ff > 0 && rows < (1ll << 31), "relu2: bad shape");
  const dim3 grid((unsigned)rows, (unsigned)std::min(8, (ff + kPbThreads - 1) / kPbThreads));
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(relu2_kernel<T>, grid, dim3(kPbThreads), 0,
                                                 static_cast<hipStream_t>(stream), out, in, in_stride, ff););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_rope_cache(float* q_out, const void* q, const void* k, const void* v, int64_t in_stride,
                   const int64_t* positions, const float* inv_freq, int rot_dims, int pair_halves, void* key_cache,
                   void* value_cache, const int64_t* slot_mapping, int64_t rows, int heads, int kv_heads, int dim,
                   int vdim, int act_dtype, void* stream) {
  return swm_norm_rope_cache(q_out, q, k, v, in_stride, nullptr, nullptr, 0.0f, positions, inv_freq, rot_dims,
                             pair_halves, key_cache, value_cache, slot_mapping, rows, heads, kv_heads, dim, vdim,
                             act_dtype, stream);
}

int swm_norm_rope_cache(float* q_out, const void* q, const void* k, const void* v, int64_t in_stride,
                        const float* q_norm, const float* k_norm, float norm_eps, const int64_t* positions,
                        const float* inv_freq, int rot_dims, int pair_halves, void* key_cache, void* value_cache,
                        const int64_t* slot_mapping, int64_t rows, int heads, int kv_heads, int dim, int vdim,
                        int act_dtype, void* stream) {
  using namespace swm;
  SW_CHECK_ARG(q_norm == nullptr || ((k == nullptr || k_norm != nullptr) && heads + kv_heads <= kMaxNormHeads),
               "rope_cache: a query norm needs a key norm, and at most %d heads in all", kMaxNormHeads);
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "rope_cache: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && dim > 0 && rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 && rows < (1ll << 31),
               "rope_cache: %d rotated coordinates of %d", rot_dims, dim);
  SW_CHECK_ARG(rot_dims == 0 || inv_freq != nullptr, "rope_cache: no frequencies");
  SW_CHECK_ARG(k == nullptr || (v != nullptr && key_cache != nullptr && value_cache != nullptr &&
                                slot_mapping != nullptr && kv_heads > 0 && vdim > 0),
               "rope_cache: keys need values, caches and slots");
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(rope_cache_kernel<T>, dim3((unsigned)rows), dim3(kPbThreads), 0,
                                                 static_cast<hipStream_t>(stream), q_out, q, k, v, in_stride, positions,
                                                 inv_freq, rot_dims, key_cache, value_cache, slot_mapping, heads,
                                                 kv_heads, dim, vdim, pair_halves, q_norm, k_norm, norm_eps););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_group_router(int32_t* chosen, float* weights, const float* logits, const float* correction, int64_t rows,
                     int experts, int top, int groups, int keep, float scale, void* stream) {
  return swm_group_router_as(chosen, weights, logits, correction, rows, experts, top, groups, keep, scale, 0, 0, 1,
                             stream);
}

int swm_group_router_as(int32_t* chosen, float* weights, const float* logits, const float* correction, int64_t rows,
                        int experts, int top, int groups, int keep, float scale, int softmax, int group_best_one,
                        int normalize, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(experts > 0 && experts <= kMaxRouterExperts && top > 0 && top <= experts,
               "group_router: %d experts (1..%d supported), top %d", experts, kMaxRouterExperts, top);
  SW_CHECK_ARG(groups >= 1 && keep >= 1 && keep <= groups && experts % groups == 0 &&
                   (int64_t)keep * (experts / groups) >= top,
               "group_router: %d groups, %d kept, %d experts, top %d", groups, keep, experts, top);
  hipLaunchKernelGGL(group_router_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     chosen, weights, logits, correction, rows, experts, top, groups, keep, scale, softmax, group_best_one,
                     normalize);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_group_pairs(int32_t* order, int32_t* expert_start, const int32_t* chosen, int64_t pairs, int experts,
                    void* stream) {
  using namespace swm;
  SW_CHECK_ARG(experts > 0 && experts <= kMaxRouterExperts && pairs >= 0 && pairs < (1ll << 31),
               "group_pairs: %d experts (1..%d supported)", experts, kMaxRouterExperts);
  hipLaunchKernelGGL(group_pairs_kernel, dim3(1), dim3(kPairThreads), 0, static_cast<hipStream_t>(stream), order,
                     expert_start, chosen, pairs, experts);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // extern "C"
