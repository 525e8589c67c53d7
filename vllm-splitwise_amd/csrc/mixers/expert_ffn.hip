// Feed-forward experts over rows that were sorted by expert: two grouped "NT" GEMMs (both operands
// contiguous along the reduction), the first with the exact gelu as its epilogue, the second scattering
// its rows back and adding them into an fp32 output.  bf16 runs on the matrix cores (second half of this
// file); fp32 -- true fp32, no reduced-precision matrix mode -- on LDS-tiled vector FMAs.
//
// The host does not know how many rows an expert got (the sort stays on the device), so the grid has the
// upper bound ceil(pairs / TM) + experts row tiles and each workgroup finds its (expert, tile) from the
// prefix sums; surplus workgroups leave at once.  Tiles never straddle two experts.
#include "mixers_common.cuh"

namespace swm {

constexpr int TM = 32, TN = 64, TK = 32, kFfnThreads = 256;

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }
// activation of an expert's hidden layer: SWM_ACT_GELU (exact gelu), SWM_ACT_RELU2 (the square of relu) or
// SWM_ACT_NONE (the products as they are, for a gated unit that a kernel of its own applies)
__device__ __forceinline__ float expert_act(float z, int activation) {
  if (activation == SWM_ACT_NONE) return z;
  if (activation == SWM_ACT_RELU2) {
    const float r = fmaxf(z, 0.0f);
    return r * r;
  }
  return gelu_erf(z);
}

// A gated hidden layer with limits, fused into the up-projection: an expert's matrix then holds, per run of 16 hidden
// channels, the 16 gate rows followed by the 16 up rows (a last, shorter run is padded with zero rows), so that a tile
// of 64 output columns holds gate and up products of the same 32 channels:  g = min(gate, limit),
// u = clamp(up, -limit, limit);  hidden = g * sigmoid(alpha * g) * (u + shift).
struct GluParams {
  float alpha, limit, shift;
};
__device__ __forceinline__ float clamped_glu(float gate, float up, const GluParams& p) {
  const float g = fminf(gate, p.limit), u = fminf(fmaxf(up, -p.limit), p.limit);
  return g * sigmoidf_(p.alpha * g) * (u + p.shift);
}

// -> expert and first sorted row of this workgroup's tile of `tm` rows, rows in it (0: nothing to do)
__device__ __forceinline__ int find_tile(const int32_t* __restrict__ expert_start, int num_experts, int tile,
                                         int* expert, int* row0, int tm = TM) {
  for (int e = 0; e < num_experts; ++e) {
    const int lo = expert_start[e], n = expert_start[e + 1] - lo;
    const int tiles = (n + tm - 1) / tm;
    if (tile < tiles) {
      *expert = e;
      *row0 = lo + tile * tm;
      return min(tm, n - tile * tm);
    }
    tile -= tiles;
  }
  return 0;
}

// acc[2][4] of thread (ty, tx): rows 2 * ty + {0, 1}, columns tx + 16 * {0..3} of the tile
//   A row p: a_base + a_row(p) * K        B row n: b_base + n * K
template <typename T, typename RowOf>
__device__ __forceinline__ void tile_gemm(float (&acc)[2][4], const void* __restrict__ a, RowOf a_row, int rows,
                                          const void* __restrict__ b, int64_t b_off, int n0, int N, int K,
                                          float (*As)[TK + 1], float (*Bs)[TK + 1]) {
  const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
  for (int k0 = 0; k0 < K; k0 += TK) {
    // A tile: 32 x 32 = 1024 values, 4 per thread; B tile: 64 x 32 = 2048 values, 8 per thread
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int e = tid + it * kFfnThreads, r = e >> 5, k = e & 31;
      float v = 0.0f;
      if (r < rows && k0 + k < K) v = ld<T>(a, a_row(r) * (int64_t)K + k0 + k);
      As[r][k] = v;
    }
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int e = tid + it * kFfnThreads, r = e >> 5, k = e & 31;
      float v = 0.0f;
      if (n0 + r < N && k0 + k < K) v = ld<T>(b, b_off + (int64_t)(n0 + r) * K + k0 + k);
      Bs[r][k] = v;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      const float a0 = As[2 * ty][k], a1 = As[2 * ty + 1][k];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float bv = Bs[tx + 16 * j][k];
        acc[0][j] += a0 * bv;
        acc[1][j] += a1 * bv;
      }
    }
    __syncthreads();
  }
}

template <typename T>
__global__ __launch_bounds__(kFfnThreads) void expert_up_gelu_kernel(
    void* __restrict__ hidden, const void* __restrict__ x, const void* __restrict__ up,
    const int32_t* __restrict__ order, const int32_t* __restrict__ expert_start, int num_experts, int width, int ff,
    int top, int activation, int up_rows, GluParams glu) {
  __shared__ float As[TM][TK + 1];
  __shared__ float Bs[TN][TK + 1];
  int e, row0;
  const int rows = find_tile(expert_start, num_experts, blockIdx.x, &e, &row0);
  if (rows == 0) return;
  const int n0 = blockIdx.y * TN;
  float acc[2][4];
  tile_gemm<T>(acc, x, [&](int r) { return (int64_t)(order[row0 + r] / top); }, rows, up, (int64_t)e * up_rows * width, n0,
               up_rows, width, As, Bs);
  const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = 2 * ty + i;
    if (r >= rows) continue;
    if (activation == SWM_ACT_CLAMPED_GLU) {
      // columns tx + 16 j of the tile: j = 0, 2 are gate products, j = 1, 3 the up products of the same channels
#pragma unroll
      for (int j = 0; j < 4; j += 2) {
        const int ch = (n0 / 32 + j / 2) * 16 + tx;
        if (ch < ff) st<T>(hidden, (int64_t)(row0 + r) * ff + ch, clamped_glu(acc[i][j], acc[i][j + 1], glu));
      }
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n < ff) st<T>(hidden, (int64_t)(row0 + r) * ff + n, expert_act(acc[i][j], activation));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kFfnThreads) void expert_down_kernel(
    float* __restrict__ out, const void* __restrict__ hidden, const void* __restrict__ down,
    const int32_t* __restrict__ order, const int32_t* __restrict__ expert_start, int num_experts, int width, int ff,
    int top, float weight, const float* __restrict__ pair_weight) {
  __shared__ float As[TM][TK + 1];
  __shared__ float Bs[TN][TK + 1];
  int e, row0;
  const int rows = find_tile(expert_start, num_experts, blockIdx.x, &e, &row0);
  if (rows == 0) return;
  const int n0 = blockIdx.y * TN;
  float acc[2][4];
  tile_gemm<T>(acc, hidden, [&](int r) { return (int64_t)(row0 + r); }, rows, down, (int64_t)e * width * ff, n0, width,
               ff, As, Bs);
  const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = 2 * ty + i;
    if (r >= rows) continue;
    const int pair = order[row0 + r];
    const int64_t dst = pair / top;
    const float wt = pair_weight != nullptr ? weight * pair_weight[pair] : weight;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= width) continue;
      float* p = out + dst * width + n;
      if (top == 1) *p += wt * acc[i][j];               // a row has one expert: nobody else writes it
      else atomicAdd(p, wt * acc[i][j]);
    }
  }
}


// ------------------------------------------------------------------------------- bf16 on the matrix cores
// 64 x 64 output tile per workgroup, one 32 x 32 quadrant per wave (v_mfma_f32_32x32x16_bf16, fp32 accumulation);
// stages of 64 reduction steps go global -> LDS as 16-byte vectors.  Both operands are contiguous along the
// reduction and are read with the SAME lane -> k mapping (8 consecutive k per lane, the wave's halves 8 apart),
// so only the accumulator's layout matters: element i of lane l is row 8 * (i / 4) + 4 * (l / 32) + i % 4,
// column l % 32.  Needs the reduction size to be a multiple of 8.
constexpr int MM = 64, MN = 64, MK = 64, MPAD = 8;
using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;
using f32x16 = __attribute__((ext_vector_type(16))) float;

template <typename RowOf>
__device__ __forceinline__ void tile_gemm_mfma(f32x16& acc, const uint16_t* __restrict__ a, RowOf a_row, int rows,
                                               const uint16_t* __restrict__ b, int64_t b_off, int n0, int N, int K,
                                               uint16_t (*As)[MK + MPAD], uint16_t (*Bs)[MK + MPAD]) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  for (int k0 = 0; k0 < K; k0 += MK) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int e = tid + it * kFfnThreads, r = e >> 3, k = (e & 7) * 8;
      uint4 va = make_uint4(0u, 0u, 0u, 0u), vb = make_uint4(0u, 0u, 0u, 0u);
      if (r < rows && k0 + k < K) va = *reinterpret_cast<const uint4*>(a + a_row(r) * (int64_t)K + k0 + k);
      if (n0 + r < N && k0 + k < K) vb = *reinterpret_cast<const uint4*>(b + b_off + (int64_t)(n0 + r) * K + k0 + k);
      *reinterpret_cast<uint4*>(&As[r][k]) = va;
      *reinterpret_cast<uint4*>(&Bs[r][k]) = vb;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < MK; ks += 16) {
      const bf16x8 av = *reinterpret_cast<const bf16x8*>(&As[wm * 32 + (lane & 31)][ks + 8 * (lane >> 5)]);
      const bf16x8 bv = *reinterpret_cast<const bf16x8*>(&Bs[wn * 32 + (lane & 31)][ks + 8 * (lane >> 5)]);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
    }
    __syncthreads();
  }
}

// calls f(row in tile, column in tile, value) for the 16 accumulator elements of this lane
template <typename F>
__device__ __forceinline__ void for_each_acc(const f32x16& acc, F&& f) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
  for (int i = 0; i < 16; ++i) f(wm * 32 + 8 * (i / 4) + 4 * (lane >> 5) + (i % 4), wn * 32 + (lane & 31), acc[i]);
}

__global__ __launch_bounds__(kFfnThreads) void expert_up_gelu_mfma_kernel(
    uint16_t* __restrict__ hidden, const uint16_t* __restrict__ x, const uint16_t* __restrict__ up,
    const int32_t* __restrict__ order, const int32_t* __restrict__ expert_start, int num_experts, int width, int ff,
    int top, int activation, int up_rows, GluParams glu) {
  __shared__ __attribute__((aligned(16))) uint16_t As[MM][MK + MPAD];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[MN][MK + MPAD];
  int e, row0;
  const int rows = find_tile(expert_start, num_experts, blockIdx.x, &e, &row0, MM);
  if (rows == 0) return;
  const int n0 = blockIdx.y * MN;
  f32x16 acc;
  tile_gemm_mfma(acc, x, [&](int r) { return (int64_t)(order[row0 + r] / top); }, rows, up, (int64_t)e * up_rows * width,
                 n0, up_rows, width, As, Bs);
  if (activation == SWM_ACT_CLAMPED_GLU) {
    // a lane's column c of the tile: c % 32 < 16 is the gate product of channel (n0 + c) / 32 * 16 + c % 16, and lane
    // + 16 holds the up product of the same channel and rows
    for_each_acc(acc, [&](int r, int c, float v) {
      const float other = __shfl_xor(v, 16, 64);
      const int ch = (n0 + c) / 32 * 16 + c % 16;
      if ((c & 16) == 0 && r < rows && ch < ff)
        hidden[(int64_t)(row0 + r) * ff + ch] = sw::float_to_bf16_bits(clamped_glu(v, other, glu));
    });
    return;
  }
  for_each_acc(acc, [&](int r, int c, float v) {
    if (r < rows && n0 + c < ff) hidden[(int64_t)(row0 + r) * ff + n0 + c] = sw::float_to_bf16_bits(expert_act(v, activation));
  });
}

__global__ __launch_bounds__(kFfnThreads) void expert_down_mfma_kernel(
    float* __restrict__ out, const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ down,
    const int32_t* __restrict__ order, const int32_t* __restrict__ expert_start, int num_experts, int width, int ff,
    int top, float weight, const float* __restrict__ pair_weight) {
  __shared__ __attribute__((aligned(16))) uint16_t As[MM][MK + MPAD];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[MN][MK + MPAD];
  int e, row0;
  const int rows = find_tile(expert_start, num_experts, blockIdx.x, &e, &row0, MM);
  if (rows == 0) return;
  const int n0 = blockIdx.y * MN;
  f32x16 acc;
  tile_gemm_mfma(acc, hidden, [&](int r) { return (int64_t)(row0 + r); }, rows, down, (int64_t)e * width * ff, n0, width,
                 ff, As, Bs);
  for_each_acc(acc, [&](int r, int c, float v) {
    if (r < rows && n0 + c < width) {
      const int pair = order[row0 + r];
      const float wt = pair_weight != nullptr ? weight * pair_weight[pair] : weight;
      float* p = out + (int64_t)(pair / top) * width + n0 + c;
      if (top == 1) *p += wt * v;
      else atomicAdd(p, wt * v);
    }
  });
}

}  // namespace swm

extern "C" {

int swm_expert_up_gelu(void* hidden, const void* x, const void* up, const int32_t* order,
                       const int32_t* expert_start, int num_experts, int64_t sorted_rows, int width, int ff,
                       int top, int act_dtype, void* stream) {
  return swm_expert_up(hidden, x, up, order, expert_start, num_experts, sorted_rows, width, ff, top, SWM_ACT_GELU,
                       act_dtype, stream);
}

int swm_expert_up(void* hidden, const void* x, const void* up, const int32_t* order, const int32_t* expert_start,
                  int num_experts, int64_t sorted_rows, int width, int ff, int top, int activation, int act_dtype,
                  void* stream) {
  return swm_expert_up_as(hidden, x, up, order, expert_start, num_experts, sorted_rows, width, ff, top, activation, 1.0f,
                          INFINITY, 0.0f, act_dtype, stream);
}

int swm_expert_up_as(void* hidden, const void* x, const void* up, const int32_t* order, const int32_t* expert_start,
                     int num_experts, int64_t sorted_rows, int width, int ff, int top, int activation, float glu_alpha,
                     float glu_limit, float glu_shift, int act_dtype, void* stream) {
  using namespace swm;
  if (sorted_rows == 0) return SW_OK;
  const bool gated = activation == SWM_ACT_CLAMPED_GLU;
  const int up_rows = gated ? 32 * ((ff + 15) / 16) : ff;     // runs of 16 gate rows + 16 up rows
  const GluParams glu{glu_alpha, glu_limit, glu_shift};
  SW_CHECK_ARG(activation == SWM_ACT_GELU || activation == SWM_ACT_RELU2 || activation == SWM_ACT_NONE || gated,
               "expert_up: unknown activation %d", activation);
  SW_CHECK_ARG(act_ok(act_dtype), "expert_up_gelu: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(num_experts > 0 && width > 0 && ff > 0 && top > 0 && sorted_rows < (1ll << 30), "expert_up_gelu: bad shape");
  if (act_dtype == SW_BF16 && width % 8 == 0) {
    const dim3 mgrid((unsigned)((sorted_rows + MM - 1) / MM + num_experts), (unsigned)((up_rows + MN - 1) / MN));
    hipLaunchKernelGGL(expert_up_gelu_mfma_kernel, mgrid, dim3(kFfnThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint16_t*>(hidden), static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(up),
                       order, expert_start, num_experts, width, ff, top, activation, up_rows, glu);
    SW_CHECK_LAUNCH();
    return SW_OK;
  }
  const dim3 grid((unsigned)((sorted_rows + TM - 1) / TM + num_experts), (unsigned)((up_rows + TN - 1) / TN));
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(expert_up_gelu_kernel<T>, grid, dim3(kFfnThreads), 0,
                                                 static_cast<hipStream_t>(stream), hidden, x, up, order, expert_start,
                                                 num_experts, width, ff, top, activation, up_rows, glu););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_expert_down(float* out, const void* hidden, const void* down, const int32_t* order,
                    const int32_t* expert_start, int num_experts, int64_t sorted_rows, int width, int ff,
                    int top, float weight, int act_dtype, void* stream) {
  return swm_expert_down_weighted(out, hidden, down, order, expert_start, num_experts, sorted_rows, width, ff, top,
                                  weight, nullptr, act_dtype, stream);
}

int swm_expert_down_weighted(float* out, const void* hidden, const void* down, const int32_t* order,
                             const int32_t* expert_start, int num_experts, int64_t sorted_rows, int width, int ff,
                             int top, float weight, const float* pair_weight, int act_dtype, void* stream) {
  using namespace swm;
  if (sorted_rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "expert_down: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(num_experts > 0 && width > 0 && ff > 0 && top > 0 && sorted_rows < (1ll << 30), "expert_down: bad shape");
  if (act_dtype == SW_BF16 && ff % 8 == 0) {
    const dim3 mgrid((unsigned)((sorted_rows + MM - 1) / MM + num_experts), (unsigned)((width + MN - 1) / MN));
    hipLaunchKernelGGL(expert_down_mfma_kernel, mgrid, dim3(kFfnThreads), 0, static_cast<hipStream_t>(stream), out,
                       static_cast<const uint16_t*>(hidden), static_cast<const uint16_t*>(down), order, expert_start,
                       num_experts, width, ff, top, weight, pair_weight);
    SW_CHECK_LAUNCH();
    return SW_OK;
  }
  const dim3 grid((unsigned)((sorted_rows + TM - 1) / TM + num_experts), (unsigned)((width + TN - 1) / TN));
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(expert_down_kernel<T>, grid, dim3(kFfnThreads), 0,
                                                 static_cast<hipStream_t>(stream), out, hidden, down, order,
                                                 expert_start, num_experts, width, ff, top, weight, pair_weight););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // extern "C"
