// Causal softmax attention of a ragged step over paged keys with grouped query heads, an optional soft cap on the
// scores (cap * tanh(score / cap)), an optional mask (a sliding window, or chunks counted from position 0 inside which
// a position sees the earlier ones), an optional extra term exp(0) in the softmax's denominator (a key of score 0
// that carries no value) and an optional sigmoid gate on the output.  A cache slot's keys and values are addressed
// by strides, so values may be a part of the key rows (attention over a latent shared by all heads).  Given a bias per
// query head the same kernels run WITHOUT a softmax: a seen key weighs sigmoid(score + bias), nothing is normalised over
// the keys, and parts are joined by plain addition.
// Scores, softmax weights and the weighted sum of values are fp32: both products run on the matrix cores in
// fp32 (v_mfma_f32_32x32x2_f32), keys and values are widened when they come from a bf16 cache.
//
// Work split.  A tile is 32 query rows of ONE sequence and ONE key/value head: the R = heads / kv_heads query heads
// of that group for 32 / R consecutive new tokens (row = token * R + head), so a decode step keeps all heads of a
// group in one tile and a prompt shares every loaded key among R * tokens rows.  In steps of prompt portions every
// wave owns a tile and walks its keys alone.  In steps where no sequence brings more tokens than one tile holds (decode
// steps) a workgroup of NW waves owns a tile; wave w takes the 32-key tiles w, w + NW, ... of the visible keys with a
// running softmax of its own, and the waves are joined through LDS in a fixed order (results do not depend on timing).
//
// Matrix-core layouts (A [32 x 2], B [2 x 32], C [32 x 32] per instruction; lane l, half hl = l / 32):
//   S^T = K Q^T : A = keys (row l % 32), B = queries (column l % 32); the two operands read the SAME coordinates in
//                 the same order, so any order of the reduction is right: each lane reads runs of 16.
//   C element r of lane l is key 8 (r / 4) + 4 hl + r % 4, query l % 32: a lane owns ONE query and 16 of the 32 keys,
//                 its partner lane l ^ 32 the other 16.
//   O^T = V^T P^T: A = values (channel l % 32 of key (r, hl)), B = the lane's own weights p[r]: no shuffle between
//                 the two products.  C element r is channel 8 (r / 4) + 4 hl + r % 4 of the lane's query.
#include "mixers_common.cuh"

namespace swm {

using f32x16 = __attribute__((ext_vector_type(16))) float;

constexpr int kQT = 32;               // query rows and keys per tile
constexpr int kMaxBlocks = 16;        // 32-coordinate blocks of the larger of key and value size

// N consecutive elements of a cache row as they are stored (bf16 two to a register), widened where they are used:
// all loads of a key tile are issued before its first product, so their latencies overlap.
template <typename T, int N> struct Raw;
template <int N> struct Raw<float, N> {
  float f[N];
  __device__ __forceinline__ float get(int j) const { return f[j]; }
};
template <int N> struct Raw<bf16_t, N> {
  uint32_t w[(N + 1) / 2];
  __device__ __forceinline__ float get(int j) const {
    return __uint_as_float((j & 1) ? (w[j / 2] & 0xffff0000u) : (w[j / 2] << 16));
  }
};

// elements [c0, c0 + N) of the row at `row_off` (elements) of `size` coordinates, zeros beyond or when !ok;
// `vec`: N is a power of two, N <= 16 bytes' worth per load piece, and size, row_off are multiples of N
template <int N>
__device__ __forceinline__ void load_raw(Raw<float, N>& out, const void* base, int64_t row_off, int c0, int size,
                                         bool ok, bool vec) {
  const float* p = static_cast<const float*>(base) + row_off + c0;
  if (vec) {
    if constexpr (N % 4 == 0) {
#pragma unroll
      for (int j = 0; j < N / 4; ++j) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ok && c0 + 4 * j < size) v = *reinterpret_cast<const float4*>(p + 4 * j);
        out.f[4 * j] = v.x; out.f[4 * j + 1] = v.y; out.f[4 * j + 2] = v.z; out.f[4 * j + 3] = v.w;
      }
    } else if constexpr (N == 2) {
      float2 v = make_float2(0.f, 0.f);
      if (ok && c0 < size) v = *reinterpret_cast<const float2*>(p);
      out.f[0] = v.x; out.f[1] = v.y;
    } else {
      out.f[0] = (ok && c0 < size) ? p[0] : 0.0f;
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) out.f[j] = (ok && c0 + j < size) ? p[j] : 0.0f;
  }
}
template <int N>
__device__ __forceinline__ void load_raw(Raw<bf16_t, N>& out, const void* base, int64_t row_off, int c0, int size,
                                         bool ok, bool vec) {
  const uint16_t* p = static_cast<const uint16_t*>(base) + row_off + c0;
  if (vec && N % 2 == 0) {
    if constexpr (N % 8 == 0) {
#pragma unroll
      for (int j = 0; j < N / 8; ++j) {
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (ok && c0 + 8 * j < size) v = *reinterpret_cast<const uint4*>(p + 8 * j);
        out.w[4 * j] = v.x; out.w[4 * j + 1] = v.y; out.w[4 * j + 2] = v.z; out.w[4 * j + 3] = v.w;
      }
    } else if constexpr (N == 4) {
      uint2 v = make_uint2(0u, 0u);
      if (ok && c0 < size) v = *reinterpret_cast<const uint2*>(p);
      out.w[0] = v.x; out.w[1] = v.y;
    } else if constexpr (N == 2) {
      out.w[0] = (ok && c0 < size) ? *reinterpret_cast<const uint32_t*>(p) : 0u;
    }
  } else {
#pragma unroll
    for (int j = 0; j < (N + 1) / 2; ++j) {
      const uint32_t lo = (ok && c0 + 2 * j < size) ? p[2 * j] : 0u;
      const uint32_t hi = (2 * j + 1 < N && ok && c0 + 2 * j + 1 < size) ? p[2 * j + 1] : 0u;
      out.w[j] = lo | (hi << 16);
    }
  }
}

constexpr bool is_pow2(int n) { return n > 0 && (n & (n - 1)) == 0; }

// NB: the larger of the numbers of 32-coordinate blocks of the key size and of the value size.  A lane's value
// channels are NB neighbours (channel = NB * (l % 32) + block), so one load brings a key's values for all blocks.
// split != 0 (steps in which no sequence brings more tokens than one tile holds, a decode step above all): a workgroup
//   owns one tile and its waves share the keys out among them, joined through LDS (rows_used query rows are live).
// split == 0: every wave owns a tile of its own and walks all of its keys; nothing is joined.
// Up to 128 coordinates the kernel's registers fit two waves per SIMD (workgroups of up to 8 waves); beyond that a wave
// needs more than 256 registers, so those instantiations are built for workgroups of at most 4 waves (one per SIMD, 512
// registers each) instead of spilling.
constexpr int max_waves_of(int nb) { return nb <= 4 ? 8 : 4; }

template <typename T, int NB>
__global__ __launch_bounds__(64 * max_waves_of(NB)) void capped_attention_kernel(
    void* __restrict__ out, const float* __restrict__ q, const void* __restrict__ key_cache,
    const void* __restrict__ value_cache, const void* __restrict__ gate, int64_t gate_stride,
    const int32_t* __restrict__ block_tables, int table_width, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, int num_seqs, int heads, int kv_heads, int dim, int vdim, int page_size,
    float scale, float softcap, int window, int chunk, int sink, const float* __restrict__ score_bias, int64_t k_stride,
    int64_t v_stride, int tpt, int split, int rows_used, int page_shift, float* __restrict__ partial,
    int64_t total_rows) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int R = heads / kv_heads;
  const int dblocks = (dim + 31) / 32;
  const int qstride = dblocks * 32 + 4;
  const int nw = blockDim.x >> 6;
  constexpr int NVB = NB;
  const int ostride = NVB * 32 + 1;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int qi = lane & 31, hl = lane >> 5;
  // split: Qs [32][qstride] | Ml [nw][32][2] | Os [nw][rows_used][ostride];  else per wave one region for Qs, then Os
  const int region = kQT * max(qstride, ostride);
  float* Qs = split ? lds : lds + wave * region;
  float* Ml = lds + kQT * qstride;
  float* Os = split ? Ml + nw * kQT * 2 + wave * rows_used * ostride : Qs;

  int seq = 0, tok0 = 0;
  const int ntok = find_query_tile(q_start, num_seqs, split ? blockIdx.x : blockIdx.x * nw + wave, tpt, &seq, &tok0);
  const bool live = ntok > 0;                                // uniform over the wave (over the workgroup when split)
  const int g = blockIdx.y;
  const int64_t row0 = live ? q_start[seq] + tok0 : 0;
  const int ctx = live ? ctx_len[seq] : 0;
  const int32_t* table = block_tables + (int64_t)seq * table_width;

  if (live) {
    const int e0 = split ? threadIdx.x : lane, step = split ? blockDim.x : 64;
    for (int e = e0; e < kQT * dblocks * 32; e += step) {
      const int r = e / (dblocks * 32), c = e % (dblocks * 32);
      const int tt = r / R, hh = r % R;
      float v = 0.0f;
      if (tt < ntok && c < dim) v = q[(row0 + tt) * (int64_t)heads * dim + (int64_t)(g * R + hh) * dim + c] * scale;
      Qs[r * qstride + c] = v;
    }
  }
  __syncthreads();

  const int first_pos = ctx + tok0, last_pos = ctx + tok0 + ntok - 1;
  // rows without a token behave like the tile's last token and are never stored
  const int pos_q = first_pos + min(qi / R, max(ntok - 1, 0));
  // keys below every row's window are skipped as whole tiles
  const int lowest = chunk > 0 ? first_pos / chunk * chunk : window > 0 ? max(0, first_pos - window + 1) : 0;
  // the first key that this lane's query sees: its chunk's first position, or the window's
  const int low_q = chunk > 0 ? pos_q / chunk * chunk : window > 0 ? pos_q - window + 1 : 0;
  const int tile_lo = lowest / kQT, tile_hi = live ? last_pos / kQT : -1;
  const bool kvec = dim % 8 == 0 && k_stride % 8 == 0;
  const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
  // score_bias: a seen key weighs sigmoid(score + bias of the query's head) and nothing is normalised over the keys;
  // the running maximum then stays 0 (every part's factor is 1) and the denominator is never used
  const bool sig = score_bias != nullptr;
  const float bias_q = sig ? score_bias[g * R + qi % R] : 0.0f;

  f32x16 o[NVB];
#pragma unroll
  for (int b = 0; b < NVB; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[b][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const bool vvec = is_pow2(NB) && vdim % NB == 0 && v_stride % NB == 0;
  // split: the waves of a workgroup, and with gridDim.z > 1 the workgroups of a tile, share the key tiles out
  const int kstep = split ? nw * (int)gridDim.z : 1;
  // cache slot of key k0 + qi of a tile (-1: beyond the tile's last key)
  auto slot_of = [&](int k0) {
    const int key = k0 + qi;
    if (key > last_pos) return -1;
    if (page_shift >= 0) return (table[key >> page_shift] << page_shift) + (key & (page_size - 1));
    return table[key / page_size] * page_size + key % page_size;
  };
  // loads of one key tile: this lane's key row (runs of 16 per block); the values of keys (r, hl)
  auto issue_keys = [&](int slot, Raw<T, 16> (&kraw)[NB]) {
    const int64_t krow = (int64_t)max(slot, 0) * k_stride + (int64_t)g * dim;
#pragma unroll
    for (int b = 0; b < NB; ++b)
      if (b < dblocks) load_raw(kraw[b], key_cache, krow, b * 32 + hl * 16, dim, slot >= 0, kvec);
  };
  auto issue_values = [&](int slot, Raw<T, NB> (&vraw)[16]) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int vslot = __shfl(slot, 8 * (r / 4) + 4 * hl + (r % 4), 64);
      load_raw(vraw[r], value_cache, (int64_t)max(vslot, 0) * v_stride + (int64_t)g * vdim, qi * NB, vdim, vslot >= 0,
               vvec);
    }
  };
  // A tile's values are asked for before its first product and arrive while it runs.  With a 16-bit cache and heads of
  // up to 128 there are registers for a second set of keys: the NEXT tile's keys are asked for at the same time and
  // arrive during this tile; otherwise a tile's keys are asked for when the tile before it ends.
  constexpr bool kAhead = sizeof(typename Conv<T>::store_t) == 2 && NB <= 4;
  int kt = tile_lo + (split ? (int)blockIdx.z * nw + wave : 0);
  Raw<T, 16> kraw[NB];
  int slot_cur = -1, slot_next = -1;
  if (kt <= tile_hi) {
    slot_cur = slot_of(kt * kQT);
    issue_keys(slot_cur, kraw);
    if (kt + kstep <= tile_hi) slot_next = slot_of((kt + kstep) * kQT);
  }
  for (; kt <= tile_hi; kt += kstep) {
    const int k0 = kt * kQT;
    Raw<T, NB> vraw[16];
    issue_values(slot_cur, vraw);
    Raw<T, 16> kraw2[NB];
    if (kAhead && kt + kstep <= tile_hi) issue_keys(slot_next, kraw2);
    const int slot_next2 = kt + 2 * kstep <= tile_hi ? slot_of((kt + 2 * kstep) * kQT) : -1;
    // ---- S^T = K Q^T
    f32x16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (b < dblocks) {
        const float4* qp = reinterpret_cast<const float4*>(Qs + qi * qstride + b * 32 + hl * 16);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 qv = qp[j];
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(kraw[b].get(4 * j), qv.x, s, 0, 0, 0);
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(kraw[b].get(4 * j + 1), qv.y, s, 0, 0, 0);
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(kraw[b].get(4 * j + 2), qv.z, s, 0, 0, 0);
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(kraw[b].get(4 * j + 3), qv.w, s, 0, 0, 0);
        }
      }
    }
    // ---- cap, mask, running softmax (this lane: query qi, keys (r, hl))
    float p[16];
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kj = k0 + 8 * (r / 4) + 4 * hl + (r % 4);
      float v = s[r];
      if (softcap > 0.0f) v = softcap * fast_tanhf_(v * inv_cap);
      const bool seen = kj <= pos_q && kj >= low_q;
      if (sig) {
        p[r] = seen ? __builtin_amdgcn_rcpf(1.0f + fast_expf_(-(v + bias_q))) : 0.0f;
      } else {
        v = seen ? v : -INFINITY;
        p[r] = v;
        tmax = fmaxf(tmax, v);
      }
    }
    float alpha = 1.0f;
    if (sig) {
      m_run = 0.0f;
    } else {
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run, tmax);
      const float m_use = m_new == -INFINITY ? 0.0f : m_new;
      alpha = fast_expf_(m_run - m_use);                     // 0 while nothing has been seen
      float psum = 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[r] = fast_expf_(p[r] - m_use);
        psum += p[r];
      }
      psum += __shfl_xor(psum, 32, 64);
      l_run = l_run * alpha + psum;
      m_run = m_new;
    }
    // ---- O^T = alpha O^T + V^T P^T
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (b < vdim) {                                          // block b holds the channels NB * lane + b
        if (!sig) {
#pragma unroll
          for (int r = 0; r < 16; ++r) o[b][r] *= alpha;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) o[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vraw[r].get(b), p[r], o[b], 0, 0, 0);
      }
    }
    if (kAhead) {
#pragma unroll
      for (int b = 0; b < NB; ++b) kraw[b] = kraw2[b];
    } else if (kt + kstep <= tile_hi) {
      issue_keys(slot_next, kraw);
    }
    slot_cur = slot_next;
    slot_next = slot_next2;
  }

  if (split) {
    // ---- join the waves
    if (!live) return;                                       // the whole workgroup
    if (hl == 0) {
      Ml[(wave * kQT + qi) * 2] = m_run;
      Ml[(wave * kQT + qi) * 2 + 1] = l_run;
    }
    if (qi < rows_used) {
#pragma unroll
      for (int b = 0; b < NVB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) Os[qi * ostride + (8 * (r / 4) + 4 * hl + (r % 4)) * NB + b] = o[b][r];
    }
    __syncthreads();
    const float* Oall = Ml + nw * kQT * 2;
    for (int e = threadIdx.x; e < rows_used * vdim; e += blockDim.x) {
      const int r = e / vdim, c = e % vdim;
      const int tt = r / R, hh = r % R;
      if (tt >= ntok) continue;
      float m_all = -INFINITY;
      for (int w = 0; w < nw; ++w) m_all = fmaxf(m_all, Ml[(w * kQT + r) * 2]);
      if (sink) m_all = fmaxf(m_all, 0.0f);                  // one more term of score 0 that carries no value
      if (partial != nullptr) {
        // this workgroup saw a part of the keys: its maximum, denominator and unnormalised sums go to the scratch that
        // the join kernel reads; the sink is the join's business
        float m_part = -INFINITY;
        for (int w = 0; w < nw; ++w) m_part = fmaxf(m_part, Ml[(w * kQT + r) * 2]);
        float num = 0.0f, den = 0.0f;
        if (m_part != -INFINITY)
          for (int w = 0; w < nw; ++w) {
            const float f = expf(Ml[(w * kQT + r) * 2] - m_part);
            den += f * Ml[(w * kQT + r) * 2 + 1];
            num += f * Oall[(w * rows_used + r) * ostride + c];
          }
        const int64_t pr = ((int64_t)blockIdx.z * total_rows + row0 + tt) * heads + g * R + hh;
        float* ml = partial;
        float* po = partial + (int64_t)gridDim.z * total_rows * heads * 2;
        if (c == 0) {
          ml[pr * 2] = m_part;
          ml[pr * 2 + 1] = den;
        }
        po[pr * vdim + c] = num;
        continue;
      }
      float num = 0.0f, den = sink ? expf(-m_all) : 0.0f;
      for (int w = 0; w < nw; ++w) {
        const float f = expf(Ml[(w * kQT + r) * 2] - m_all);  // a wave that saw no key: exp(-inf) = 0
        den += f * Ml[(w * kQT + r) * 2 + 1];
        num += f * Oall[(w * rows_used + r) * ostride + c];
      }
      float v = sig ? num : num / den;
      const int64_t col = (int64_t)(g * R + hh) * vdim + c;
      if (gate != nullptr) v *= sigmoidf_(ld<T>(gate, (row0 + tt) * gate_stride + col));
      st<T>(out, (row0 + tt) * (int64_t)heads * vdim + col, v);
    }
    return;
  }
  // ---- every wave for itself: turn O^T round through the wave's own LDS region (its queries are done with)
  __syncthreads();
  if (live) {
    const float m_fin = sink ? fmaxf(m_run, 0.0f) : m_run;
    const float fin = sink ? expf(m_run - m_fin) : 1.0f;
    const float inv = sig ? 1.0f : fin / (l_run * fin + (sink ? expf(-m_fin) : 0.0f));
#pragma unroll
    for (int b = 0; b < NVB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) Os[qi * ostride + (8 * (r / 4) + 4 * hl + (r % 4)) * NB + b] = o[b][r] * inv;
  }
  __syncthreads();
  if (!live) return;
  for (int e = lane; e < kQT * vdim; e += 64) {
    const int r = e / vdim, c = e % vdim;
    const int tt = r / R, hh = r % R;
    if (tt >= ntok) continue;
    float v = Os[r * ostride + c];
    const int64_t col = (int64_t)(g * R + hh) * vdim + c;
    if (gate != nullptr) v *= sigmoidf_(ld<T>(gate, (row0 + tt) * gate_stride + col));
    st<T>(out, (row0 + tt) * (int64_t)heads * vdim + col, v);
  }
}

// Steps of very few query rows per sequence and key/value head (a decode step: one token's R query heads) leave a
// 32-row matrix tile mostly empty, so they run on the vector units instead: LK (8 or 16) lanes share a key, each with C
// coordinates of the key, of every query row and of the value; a wave walks 64 / LK keys at a time, a workgroup owns
// (sequence, key/value head).  Every lane group keeps a running softmax of its own; groups are joined by shuffles,
// waves through LDS, both in a fixed order.  RQ: query rows (padded), C: coordinates per lane, U: keys in flight.
template <typename T, int RQ, int C, int LK, int U>
__global__ __launch_bounds__(512) void capped_attention_rows_kernel(
    void* __restrict__ out, const float* __restrict__ q, const void* __restrict__ key_cache,
    const void* __restrict__ value_cache, const void* __restrict__ gate, int64_t gate_stride,
    const int32_t* __restrict__ block_tables, int table_width, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, int heads, int kv_heads, int dim, int vdim, int page_size, int page_shift,
    float scale, float softcap, int window, int chunk, int sink, const float* __restrict__ score_bias, int64_t k_stride,
    int64_t v_stride) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int seq = blockIdx.x, g = blockIdx.y, R = heads / kv_heads;
  const bool sig = score_bias != nullptr;                    // sigmoid weights: see capped_attention_kernel
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, pt = lane % LK, grp = lane / LK, nw = blockDim.x >> 6;
  const int row0 = q_start[seq], n = q_start[seq + 1] - row0;
  if (n <= 0) return;                                        // the whole workgroup
  const int ctx = ctx_len[seq], rows = n * R, last_pos = ctx + n - 1;
  const int32_t* table = block_tables + (int64_t)seq * table_width;
  float* Ml = lds;                                           // [nw][RQ][2]
  float* Os = lds + nw * RQ * 2;                             // [nw][RQ][LK * C]

  float qv[RQ][C], o[RQ][C], m_run[RQ], l_run[RQ], bias[RQ];
  int pos[RQ], low[RQ];
#pragma unroll
  for (int r = 0; r < RQ; ++r) {
    const int tt = r / R, hh = r % R;
    bias[r] = sig ? score_bias[g * R + hh] : 0.0f;
    pos[r] = ctx + min(tt, n - 1);                           // padding rows behave like the last token's
    low[r] = chunk > 0 ? pos[r] / chunk * chunk : window > 0 ? pos[r] - window + 1 : 0;
    m_run[r] = -INFINITY;
    l_run[r] = 0.0f;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int col = pt * C + c;
      qv[r][c] = (r < rows && col < dim) ? q[(int64_t)(row0 + tt) * heads * dim + (int64_t)(g * R + hh) * dim + col] * scale
                                         : 0.0f;
      o[r][c] = 0.0f;
    }
  }
  constexpr int kPiece = C >= 8 ? 8 : 4;
  const bool kvec = dim % kPiece == 0 && k_stride % kPiece == 0, vvec = vdim % kPiece == 0 && v_stride % kPiece == 0;
  const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
  const int lowest = chunk > 0 ? ctx / chunk * chunk : window > 0 ? max(0, ctx - window + 1) : 0;
  constexpr int GW = 64 / LK;                                // lane groups of a wave
  const int groups = nw * GW;
  for (int key0 = lowest + wave * GW + grp; key0 <= last_pos; key0 += groups * U) {
    Raw<T, C> kr[U], vr[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = key0 + u * groups;
      const bool ok = key <= last_pos;
      int slot = 0;
      if (ok) slot = page_shift >= 0 ? (table[key >> page_shift] << page_shift) + (key & (page_size - 1))
                                     : table[key / page_size] * page_size + key % page_size;
      load_raw(kr[u], key_cache, (int64_t)slot * k_stride + (int64_t)g * dim, pt * C, dim, ok, kvec);
      load_raw(vr[u], value_cache, (int64_t)slot * v_stride + (int64_t)g * vdim, pt * C, vdim, ok, vvec);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = key0 + u * groups;
      if (key > last_pos) continue;                          // uniform over the lane group
#pragma unroll
      for (int r = 0; r < RQ; ++r) {
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) s += qv[r][c] * kr[u].get(c);
        s = lanes_sum<LK>(s);
        if (softcap > 0.0f) s = softcap * fast_tanhf_(s * inv_cap);
        const bool seen = key <= pos[r] && key >= low[r];
        if (sig) {
          const float p = seen ? __builtin_amdgcn_rcpf(1.0f + fast_expf_(-(s + bias[r]))) : 0.0f;
          m_run[r] = 0.0f;
#pragma unroll
          for (int c = 0; c < C; ++c) o[r][c] += p * vr[u].get(c);
          continue;
        }
        if (!seen) s = -INFINITY;
        const float m_new = fmaxf(m_run[r], s);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = fast_expf_(m_run[r] - m_use);
        const float p = fast_expf_(s - m_use);
        l_run[r] = l_run[r] * alpha + p;
        m_run[r] = m_new;
#pragma unroll
        for (int c = 0; c < C; ++c) o[r][c] = o[r][c] * alpha + p * vr[u].get(c);
      }
    }
  }
  // ---- join the wave's lane groups
#pragma unroll
  for (int step = LK; step <= 32; step <<= 1) {
#pragma unroll
    for (int r = 0; r < RQ; ++r) {
      const float m_o = __shfl_xor(m_run[r], step, 64), l_o = __shfl_xor(l_run[r], step, 64);
      const float m_new = fmaxf(m_run[r], m_o);
      const float m_use = m_new == -INFINITY ? 0.0f : m_new;
      const float fa = fast_expf_(m_run[r] - m_use), fb = fast_expf_(m_o - m_use);
      l_run[r] = l_run[r] * fa + l_o * fb;
      m_run[r] = m_new;
#pragma unroll
      for (int c = 0; c < C; ++c) o[r][c] = o[r][c] * fa + __shfl_xor(o[r][c], step, 64) * fb;
    }
  }
  // ---- join the waves
  if (grp == 0) {
#pragma unroll
    for (int r = 0; r < RQ; ++r) {
      if (pt == 0) {
        Ml[(wave * RQ + r) * 2] = m_run[r];
        Ml[(wave * RQ + r) * 2 + 1] = l_run[r];
      }
#pragma unroll
      for (int c = 0; c < C; ++c) Os[(wave * RQ + r) * LK * C + pt * C + c] = o[r][c];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < rows * vdim; e += blockDim.x) {
    const int r = e / vdim, c = e % vdim;
    const int tt = r / R, hh = r % R;
    float m_all = -INFINITY;
    for (int w = 0; w < nw; ++w) m_all = fmaxf(m_all, Ml[(w * RQ + r) * 2]);
    if (sink) m_all = fmaxf(m_all, 0.0f);
    float num = 0.0f, den = sink ? expf(-m_all) : 0.0f;
    for (int w = 0; w < nw; ++w) {
      const float f = fast_expf_(Ml[(w * RQ + r) * 2] - m_all);      // a wave that saw no key: 0
      den += f * Ml[(w * RQ + r) * 2 + 1];
      num += f * Os[(w * RQ + r) * LK * C + c];
    }
    float v = sig ? num : num / den;
    const int64_t col = (int64_t)(g * R + hh) * vdim + c;
    if (gate != nullptr) v *= sigmoidf_(ld<T>(gate, (row0 + tt) * gate_stride + col));
    st<T>(out, (int64_t)(row0 + tt) * heads * vdim + col, v);
  }
}

template <typename T, int RQ, int C, int LK>
int launch_capped_rows(void* out, const float* q, const void* key_cache, const void* value_cache, const void* gate,
                       int64_t gate_stride, const int32_t* block_tables, int table_width, const int32_t* q_start,
                       const int32_t* ctx_len, int num_seqs, int heads, int kv_heads, int dim, int vdim, int page_size,
                       float scale, float softcap, int window, int chunk, int sink, const float* score_bias, int64_t k_stride,
                       int64_t v_stride, hipStream_t stream) {
  constexpr bool half = sizeof(typename Conv<T>::store_t) == 2;
  constexpr int U = RQ * C <= 32 ? (half ? 4 : 2) : (half ? 2 : 1);
  const int nw = 8;
  const size_t lds_bytes = (size_t)nw * RQ * (2 + LK * C) * sizeof(float);
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0)
    for (page_shift = 0; (1 << page_shift) < page_size; ++page_shift) {}
  auto kernel = capped_attention_rows_kernel<T, RQ, C, LK, U>;
  static bool raised = false;                                // per instantiation
  if (lds_bytes > 64 * 1024 && !raised) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds_bytes));
    raised = true;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)num_seqs, (unsigned)kv_heads), dim3(64 * nw), lds_bytes, stream, out, q,
                     key_cache, value_cache, gate, gate_stride, block_tables, table_width, q_start, ctx_len, heads,
                     kv_heads, dim, vdim, page_size, page_shift, scale, softcap, window, chunk, sink, score_bias, k_stride,
                     v_stride);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

// -> true when the step was taken by the vector-unit kernel (few rows, lanes' shares small enough for registers)
template <typename T>
bool try_capped_rows(int* status, int rows_used, void* out, const float* q, const void* key_cache,
                     const void* value_cache, const void* gate, int64_t gate_stride, const int32_t* block_tables,
                     int table_width, const int32_t* q_start, const int32_t* ctx_len, int num_seqs, int heads,
                     int kv_heads, int dim, int vdim, int page_size, float scale, float softcap, int window, int chunk,
                     int sink, const float* score_bias, int64_t k_stride, int64_t v_stride, hipStream_t stream) {
  if (rows_used > 8) return false;
  auto pow2 = [](int x) { return x <= 4 ? 4 : x <= 8 ? 8 : x <= 16 ? 16 : x <= 32 ? 32 : 64; };
  const int most = std::max(dim, vdim);
  const int rq = rows_used <= 1 ? 1 : rows_used <= 2 ? 2 : rows_used <= 4 ? 4 : 8;
  // 8 lanes per key while a lane's share of rows x coordinates stays small, else 16
  int lk = 8, c = pow2((most + 7) / 8);
  if (rq * c > 64) {
    lk = 16;
    c = pow2((most + 15) / 16);
  }
  if (rq * c > 64) return false;
#define SWM_ROWS_CASE(RQV, CV, LKV)                                                                                     \
  if (rq == RQV && c == CV && lk == LKV) {                                                                              \
    *status = launch_capped_rows<T, RQV, CV, LKV>(out, q, key_cache, value_cache, gate, gate_stride, block_tables,      \
                                                  table_width, q_start, ctx_len, num_seqs, heads, kv_heads, dim, vdim,  \
                                                  page_size, scale, softcap, window, chunk, sink, score_bias, k_stride, \
                                                  v_stride, stream);                                                              \
    return true;                                                                                                        \
  }
  SWM_ROWS_CASE(1, 4, 8) SWM_ROWS_CASE(1, 8, 8) SWM_ROWS_CASE(1, 16, 8) SWM_ROWS_CASE(1, 32, 8)
  SWM_ROWS_CASE(2, 4, 8) SWM_ROWS_CASE(2, 8, 8) SWM_ROWS_CASE(2, 16, 8) SWM_ROWS_CASE(2, 32, 8)
  SWM_ROWS_CASE(4, 4, 8) SWM_ROWS_CASE(4, 8, 8) SWM_ROWS_CASE(4, 16, 8)
  SWM_ROWS_CASE(8, 4, 8) SWM_ROWS_CASE(8, 8, 8)
  SWM_ROWS_CASE(4, 16, 16) SWM_ROWS_CASE(8, 8, 16)
#undef SWM_ROWS_CASE
  return false;
}

// Joins the parts of a step whose keys were shared out among `parts` workgroups per tile: one workgroup per
// (row, head), parts in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void capped_attention_join_kernel(
    void* __restrict__ out, const float* __restrict__ partial, const void* __restrict__ gate, int64_t gate_stride,
    int64_t total_rows, int heads, int vdim, int parts, int sink, int sig) {
  const int64_t rh = blockIdx.x;                             // row * heads + head
  const float* ml = partial;
  const float* po = partial + (int64_t)parts * total_rows * heads * 2;
  const int64_t part_stride = total_rows * heads;
  float m_all = sink ? 0.0f : -INFINITY;
  for (int z = 0; z < parts; ++z) m_all = fmaxf(m_all, ml[(z * part_stride + rh) * 2]);
  float den = sink ? expf(-m_all) : 0.0f;
  for (int z = 0; z < parts; ++z) {
    const float m = ml[(z * part_stride + rh) * 2];
    if (m != -INFINITY) den += expf(m - m_all) * ml[(z * part_stride + rh) * 2 + 1];
  }
  const int64_t t = rh / heads;
  const int hd = (int)(rh % heads);
  for (int c = threadIdx.x; c < vdim; c += blockDim.x) {
    float num = 0.0f;
    for (int z = 0; z < parts; ++z) {
      const float m = ml[(z * part_stride + rh) * 2];
      if (m != -INFINITY) num += expf(m - m_all) * po[(z * part_stride + rh) * vdim + c];
    }
    float v = sig ? num : num / den;
    if (gate != nullptr) v *= sigmoidf_(ld<T>(gate, t * gate_stride + (int64_t)hd * vdim + c));
    st<T>(out, rh * vdim + c, v);
  }
}

// In how many parts the keys of a tile are shared out among workgroups: steps of few rows per sequence (decode steps)
// of few sequences would otherwise leave most of the GPU idle.  most_keys: an upper bound on the keys a row sees.
inline int key_parts(int num_seqs, int max_query_len, int heads, int kv_heads, int page_size, int table_width, int window,
                     int chunk) {
  const int R = heads / kv_heads, tpt = kQT / R;
  if (max_query_len <= 0 || max_query_len > tpt || max_query_len * R <= 8) return 1;   // not the shared-keys loop
  int64_t most_keys = (int64_t)page_size * table_width;
  if (window > 0) most_keys = std::min<int64_t>(most_keys, window + max_query_len);
  if (chunk > 0) most_keys = std::min<int64_t>(most_keys, chunk);
  const int64_t tiles = (most_keys + kQT - 1) / kQT;
  const int64_t groups = (int64_t)num_seqs * kv_heads;
  int parts = 1;
  while (parts < 16 && groups * parts * 2 <= 512 && tiles >= 8 * parts * 2) parts <<= 1;
  return parts;
}

template <typename T, int NB>
int launch_capped_attention(void* out, const float* q, const void* key_cache, const void* value_cache, const void* gate,
                            int64_t gate_stride, const int32_t* block_tables, int table_width, const int32_t* q_start,
                            const int32_t* ctx_len, int64_t rows, int num_seqs, int max_query_len, int heads,
                            int kv_heads, int dim, int vdim, int page_size, float scale, float softcap, int window,
                            int chunk, int sink, const float* score_bias, int64_t k_stride, int64_t v_stride,
                            float* workspace, hipStream_t stream) {
  const int R = heads / kv_heads;
  const int tpt = kQT / R;
  const int qstride = (dim + 31) / 32 * 32 + 4, ostride = NB * 32 + 1;
  const bool split = max_query_len > 0 && max_query_len <= tpt;
  const int rows_used = split ? max_query_len * R : kQT;
  if (split) {
    int status = SW_OK;
    if (try_capped_rows<T>(&status, rows_used, out, q, key_cache, value_cache, gate, gate_stride, block_tables, table_width,
                           q_start, ctx_len, num_seqs, heads, kv_heads, dim, vdim, page_size, scale, softcap, window,
                           chunk, sink, score_bias, k_stride, v_stride, stream))
      return status;
  }
  auto lds_bytes = [&](int nw) {
    const size_t floats = split ? (size_t)kQT * qstride + (size_t)nw * kQT * 2 + (size_t)nw * rows_used * ostride
                                : (size_t)nw * kQT * std::max(qstride, ostride);
    return floats * sizeof(float);
  };
  const int parts = (split && workspace != nullptr)
                        ? key_parts(num_seqs, max_query_len, heads, kv_heads, page_size, table_width, window, chunk) : 1;
  // two workgroups of a compute unit's 160 KB where the sizes allow it; a launch that cannot fill the compute units
  // twice anyway gives each workgroup as many waves as one unit's LDS holds
  const bool few = split && (int64_t)num_seqs * kv_heads * parts <= 256;
  int nw = split ? max_waves_of(NB) : 4;
  while (nw > 1 && lds_bytes(nw) > (few ? 150 : 72) * 1024) nw >>= 1;
  SW_CHECK_ARG(lds_bytes(nw) <= 160 * 1024, "capped_attention: key size %d with value size %d needs too much LDS", dim,
               vdim);
  auto kernel = capped_attention_kernel<T, NB>;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0)
    for (page_shift = 0; (1 << page_shift) < page_size; ++page_shift) {}
  static size_t allowed = 0;                                 // per instantiation
  if (lds_bytes(nw) > allowed) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds_bytes(nw)));
    allowed = lds_bytes(nw);
  }
  const int64_t tiles = split ? num_seqs : (rows + tpt - 1) / tpt + num_seqs;
  const dim3 grid((unsigned)(split ? tiles : (tiles + nw - 1) / nw), (unsigned)kv_heads, (unsigned)parts);
  hipLaunchKernelGGL(kernel, grid, dim3(64 * nw), lds_bytes(nw), stream, out, q, key_cache, value_cache, gate,
                     gate_stride, block_tables, table_width, q_start, ctx_len, num_seqs, heads, kv_heads, dim, vdim,
                     page_size, scale, softcap, window, chunk, sink, score_bias, k_stride, v_stride, tpt, split ? 1 : 0,
                     rows_used, page_shift, parts > 1 ? workspace : (float*)nullptr, rows);
  SW_CHECK_LAUNCH();
  if (parts > 1) {
    hipLaunchKernelGGL(capped_attention_join_kernel<T>, dim3((unsigned)(rows * heads)), dim3(vdim <= 64 ? 64 : 128), 0,
                       stream, out, workspace, gate, gate_stride, rows, heads, vdim, parts, sink, score_bias != nullptr ? 1 : 0);
    SW_CHECK_LAUNCH();
  }
  return SW_OK;
}

}  // namespace swm

extern "C" int64_t swm_masked_attention_workspace_floats(int64_t rows, int num_seqs, int max_query_len, int heads,
                                                         int kv_heads, int vdim, int page_size, int table_width,
                                                         int window, int chunk) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || heads / kv_heads > swm::kQT) return 0;
  const int parts = swm::key_parts(num_seqs, max_query_len, heads, kv_heads, page_size, table_width, window, chunk);
  return parts > 1 ? (int64_t)parts * rows * heads * (vdim + 2) : 0;
}

static int masked_attention_impl(void* out, const float* q, const void* key_cache, const void* value_cache,
                                 const void* gate, int64_t gate_stride, const int32_t* block_tables, int table_width,
                                 const int32_t* q_start, const int32_t* ctx_len, int64_t rows, int num_seqs,
                                 int max_query_len, int heads, int kv_heads, int dim, int vdim, int page_size,
                                 float scale, float softcap, int window, int chunk, int sink, const float* score_bias,
                                 int64_t k_stride, int64_t v_stride, float* workspace, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0 || num_seqs == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "masked_attention: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && heads / kv_heads <= kQT,
               "masked_attention: %d query heads on %d key/value heads (at most %d per key/value head)", heads, kv_heads,
               kQT);
  SW_CHECK_ARG(dim > 0 && dim <= 32 * kMaxBlocks && vdim > 0 && vdim <= 32 * kMaxBlocks && page_size > 0 &&
                   table_width > 0 && rows < (1ll << 31),
               "masked_attention: key size %d, value size %d (at most %d each)", dim, vdim, 32 * kMaxBlocks);
  SW_CHECK_ARG(!(window > 0 && chunk > 0) && window >= 0 && chunk >= 0,
               "masked_attention: a sliding window (%d) or chunks (%d), not both", window, chunk);
  SW_CHECK_ARG(k_stride >= (int64_t)kv_heads * dim && v_stride >= (int64_t)kv_heads * vdim,
               "masked_attention: a cache slot of %lld / %lld elements cannot hold %d heads", (long long)k_stride,
               (long long)v_stride, kv_heads);
  const int nvb = std::max((vdim + 31) / 32, (dim + 31) / 32);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SWM_CAPPED_CASE(N)                                                                                              \
  case N:                                                                                                               \
    SWM_DISPATCH_ACT(act_dtype, return (launch_capped_attention<T, N>(                                                  \
                                    out, q, key_cache, value_cache, gate, gate_stride, block_tables, table_width,       \
                                    q_start, ctx_len, rows, num_seqs, max_query_len, heads, kv_heads, dim, vdim,        \
                                    page_size, scale, softcap, window, chunk, sink, score_bias, k_stride, v_stride,     \
                                    workspace, s)););                                                                              \
    break;
  switch (nvb) {
    SWM_CAPPED_CASE(1)
    SWM_CAPPED_CASE(2)
    SWM_CAPPED_CASE(3)
    SWM_CAPPED_CASE(4)
    SWM_CAPPED_CASE(5)
    SWM_CAPPED_CASE(6)
    SWM_CAPPED_CASE(7)
    SWM_CAPPED_CASE(8)
    SWM_CAPPED_CASE(9)
    SWM_CAPPED_CASE(10)
    SWM_CAPPED_CASE(11)
    SWM_CAPPED_CASE(12)
    SWM_CAPPED_CASE(13)
    SWM_CAPPED_CASE(14)
    SWM_CAPPED_CASE(15)
    SWM_CAPPED_CASE(16)
  }
#undef SWM_CAPPED_CASE
  return SW_OK;
}

extern "C" int swm_masked_attention(void* out, const float* q, const void* key_cache, const void* value_cache,
                                    const void* gate, int64_t gate_stride, const int32_t* block_tables,
                                    int table_width, const int32_t* q_start, const int32_t* ctx_len, int64_t rows,
                                    int num_seqs, int max_query_len, int heads, int kv_heads, int dim, int vdim,
                                    int page_size, float scale, float softcap, int window, int chunk, int sink,
                                    int64_t k_stride, int64_t v_stride, float* workspace, int act_dtype, void* stream) {
  return masked_attention_impl(out, q, key_cache, value_cache, gate, gate_stride, block_tables, table_width, q_start,
                               ctx_len, rows, num_seqs, max_query_len, heads, kv_heads, dim, vdim, page_size, scale,
                               softcap, window, chunk, sink, nullptr, k_stride, v_stride, workspace, act_dtype, stream);
}

extern "C" int swm_sigmoid_attention(void* out, const float* q, const void* key_cache, const void* value_cache,
                                     const void* gate, int64_t gate_stride, const float* score_bias,
                                     const int32_t* block_tables, int table_width, const int32_t* q_start,
                                     const int32_t* ctx_len, int64_t rows, int num_seqs, int max_query_len, int heads,
                                     int kv_heads, int dim, int vdim, int page_size, float scale, int window,
                                     float* workspace, int act_dtype, void* stream) {
  if (score_bias == nullptr) {
    sw::set_error("sigmoid_attention: the per-head bias is missing (a layer without one passes zeros)");
    return SW_ERR_INVALID;
  }
  return masked_attention_impl(out, q, key_cache, value_cache, gate, gate_stride, block_tables, table_width, q_start,
                               ctx_len, rows, num_seqs, max_query_len, heads, kv_heads, dim, vdim, page_size, scale,
                               0.0f, window, 0, 0, score_bias, (int64_t)kv_heads * dim, (int64_t)kv_heads * vdim,
                               workspace, act_dtype, stream);
}

extern "C" int swm_capped_attention(void* out, const float* q, const void* key_cache, const void* value_cache,
                                    const void* gate, int64_t gate_stride, const int32_t* block_tables,
                                    int table_width, const int32_t* q_start, const int32_t* ctx_len, int64_t rows,
                                    int num_seqs, int max_query_len, int heads, int kv_heads, int dim, int vdim, int page_size,
                                    float scale, float softcap, int window, int act_dtype, void* stream) {
  return swm_masked_attention(out, q, key_cache, value_cache, gate, gate_stride, block_tables, table_width, q_start,
                              ctx_len, rows, num_seqs, max_query_len, heads, kv_heads, dim, vdim, page_size, scale,
                              softcap, window, 0, 0, (int64_t)kv_heads * dim, (int64_t)kv_heads * vdim, nullptr, act_dtype,
                              stream);
}
