// Kernels of a routed feed-forward (a mixture of small gated experts) for gfx950.
//
// moe_route: per token the router's logits z = W_r h in float32, a score per expert
//   (sigmoid(z)), and the `top` experts with the largest scores (ties: the lower index) with
//   their scores as weights.
// moe_gate_up / moe_down: a block a
//   (token, chosen expert) pair and a slab of output channels; the pair's activation row sits in
//   LDS in float32, a wave walks eight weight rows at a time in 16-byte pieces.  The weight of a
//   chosen expert multiplies the expert's INPUT: since the first products are linear,
//   gate(w h) = w gate(h), the weight is applied to the two products in float32 before the
//   activation.  moe_down adds a token's experts in the order of its list, so a token's result
//   does not depend on what else is in the step.
//
// Router, scores, weights and every sum are float32 whatever the storage type.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

constexpr int kRouteWaves = 4;     // tokens a block of the router takes, a wave each
constexpr int kRows = 8;           // weight rows a wave walks at once

template <typename T> struct Vec;
template <> struct Vec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float* o) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// A wave a token: lanes stride the width, one expert after the other.
template <typename T>
__global__ __launch_bounds__(kRouteWaves * kWave) void moe_route_kernel(
    const T* __restrict__ h, const float* __restrict__ router, int* __restrict__ chosen,
    float* __restrict__ weight, int N, int W, int E, int top) {
  extern __shared__ float lds[];       // [kRouteWaves][E]
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int n = blockIdx.x * kRouteWaves + wave;
  if (n >= N) return;                  // nothing below synchronises across waves
  float* score = lds + (size_t)wave * E;
  const T* row = h + (size_t)n * W;
  for (int e = 0; e < E; ++e) {
    const float* r = router + (size_t)e * W;
    float acc = 0.f;
    for (int d = lane; d < W; d += kWave) acc = fmaf(Elem<T>::load(row + d), r[d], acc);
    acc = wave_sum(acc);
    if (lane == 0) score[e] = 1.f / (1.f + expf(-acc));
  }
  wave_lds_sync();
  // the largest `top` scores, one after the other; a lane looks at the experts lane, lane + 64, ...
  for (int k = 0; k < top; ++k) {
    float best = -1.f;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += kWave) {
      const float v = score[e];
      if (v > best) { best = v; at = e; }          // (ascending e: the lower index stays on ties)
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      const float ob = __shfl_xor(best, m, kWave);
      const int oa = __shfl_xor(at, m, kWave);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (lane == 0) {
      chosen[(size_t)n * top + k] = at;
      weight[(size_t)n * top + k] = best;
      score[at] = -2.f;
    }
    wave_lds_sync();
  }
}

// a[p, c] = silu(w g) * (w u), g = Wg[e][c] . h[n], u = Wu[e][c] . h[n]; gate_up [E][2 F][W]
// (an expert's gate rows, then its up rows).  grid (pairs, slabs of channels).
// WIDE: rows are walked in 16-byte pieces (their length fills such pieces), else element by element.
template <typename T, bool WIDE>
__device__ __forceinline__ void load_piece(const T* p, float* o) {
  if constexpr (WIDE) Vec<T>::load(p, o);
  else o[0] = Elem<T>::load(p);
}

template <typename T, bool WIDE>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(
    const T* __restrict__ h, const T* __restrict__ gate_up, const int* __restrict__ chosen,
    const float* __restrict__ weight, T* __restrict__ act, int W, int F, int top, int slab) {
  extern __shared__ float x[];         // [W]
  const int p = blockIdx.x, n = p / top;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  for (int d = threadIdx.x; d < W; d += blockDim.x) x[d] = Elem<T>::load(h + (size_t)n * W + d);
  __syncthreads();
  const int e = chosen[p];
  const float wt = weight[p];
  const T* wg = gate_up + (size_t)e * 2 * F * W;
  const T* wu = wg + (size_t)F * W;
  constexpr int V = WIDE ? Vec<T>::N : 1;
  const int c_end = min(F, (int)(blockIdx.y + 1) * slab);
  for (int c0 = blockIdx.y * slab + wave * kRows; c0 < c_end; c0 += nwaves * kRows) {
    float g[kRows], u[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) g[r] = u[r] = 0.f;
    for (int d = lane * V; d < W; d += kWave * V) {
      float xv[V];
#pragma unroll
      for (int i = 0; i < V; ++i) xv[i] = x[d + i];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const int c = min(c0 + r, F - 1);       // (a row past the end is walked again and not used)
        float a[V], b[V];
        load_piece<T, WIDE>(wg + (size_t)c * W + d, a);
        load_piece<T, WIDE>(wu + (size_t)c * W + d, b);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          g[r] = fmaf(a[i], xv[i], g[r]);
          u[r] = fmaf(b[i], xv[i], u[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      g[r] = wave_sum(g[r]);
      u[r] = wave_sum(u[r]);
    }
    if (lane < kRows && c0 + lane < c_end) {
      float gv = 0.f, uv = 0.f;
#pragma unroll
      for (int r = 0; r < kRows; ++r)
        if (r == lane) { gv = g[r]; uv = u[r]; }
      gv *= wt;
      uv *= wt;
      Elem<T>::store(act + (size_t)p * F + c0 + lane, gv / (1.f + expf(-gv)) * uv);
    }
  }
}

// out[n, c] = sum over the token's chosen experts, in list order, of Wd[e][c] . a[p]; down [E][W][F];
// out float32.  grid (tokens, slabs of columns).
template <typename T, bool WIDE>
__global__ __launch_bounds__(256) void moe_down_kernel(
    const T* __restrict__ act, const T* __restrict__ down, const int* __restrict__ chosen,
    float* __restrict__ out, int W, int F, int top, int slab) {
  extern __shared__ float x[];         // [top][F]
  const int n = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  for (int d = threadIdx.x; d < top * F; d += blockDim.x) x[d] = Elem<T>::load(act + (size_t)n * top * F + d);
  __syncthreads();
  constexpr int V = WIDE ? Vec<T>::N : 1;
  const int c_end = min(W, (int)(blockIdx.y + 1) * slab);
  for (int c0 = blockIdx.y * slab + wave * kRows; c0 < c_end; c0 += nwaves * kRows) {
    float total[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) total[r] = 0.f;
    for (int k = 0; k < top; ++k) {
      const T* wd = down + (size_t)chosen[(size_t)n * top + k] * W * F;
      const float* xk = x + (size_t)k * F;
      float acc[kRows];
#pragma unroll
      for (int r = 0; r < kRows; ++r) acc[r] = 0.f;
      for (int d = lane * V; d < F; d += kWave * V) {
        float xv[V];
#pragma unroll
        for (int i = 0; i < V; ++i) xv[i] = xk[d + i];
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          const int c = min(c0 + r, W - 1);
          float a[V];
          load_piece<T, WIDE>(wd + (size_t)c * F + d, a);
#pragma unroll
          for (int i = 0; i < V; ++i) acc[r] = fmaf(a[i], xv[i], acc[r]);
        }
      }
#pragma unroll
      for (int r = 0; r < kRows; ++r) total[r] += wave_sum(acc[r]);
    }
    if (lane < kRows && c0 + lane < c_end) {
      float v = 0.f;
#pragma unroll
      for (int r = 0; r < kRows; ++r)
        if (r == lane) v = total[r];
      out[(size_t)n * W + c0 + lane] = v;
    }
  }
}

}  // namespace

// h [N, W] in dtype; router [E, W] float32; chosen [N, top] int32 and weight [N, top] float32 out
TK_API int tk_moe_route(int dtype, const void* h, const float* router, int* chosen, float* weight, int N,
                        int W, int E, int top, hipStream_t stream) {
  if (N <= 0) return 0;
  if (E < 1 || top < 1 || top > E || W < 1 || (size_t)E * kRouteWaves * 4 > 64 * 1024) return -1;
  const unsigned blocks = (unsigned)((N + kRouteWaves - 1) / kRouteWaves);
  const size_t lds = (size_t)kRouteWaves * E * sizeof(float);
  if (dtype == 0)
    moe_route_kernel<float><<<blocks, kRouteWaves * kWave, lds, stream>>>((const float*)h, router, chosen, weight, N, W, E, top);
  else
    moe_route_kernel<bf16_t><<<blocks, kRouteWaves * kWave, lds, stream>>>((const bf16_t*)h, router, chosen, weight, N, W, E, top);
  return launch_status();
}

static int slab_for(int channels, long rows) {
  // slabs of channels so that some 1,024 blocks exist, each at least a turn of its four waves
  const long want = (1024 + rows - 1) / rows;
  long slab = (channels + want - 1) / want;
  slab = (slab + 4 * kRows - 1) / (4 * kRows) * (4 * kRows);
  return (int)(slab < 4 * kRows ? 4 * kRows : slab);
}

// act[N * top, F] = silu(w gate) * (w up) of every (token, chosen expert) pair
TK_API int tk_moe_gate_up(int dtype, const void* h, const void* gate_up, const int* chosen, const float* weight,
                          void* act, int N, int W, int F, int top, hipStream_t stream) {
  if (N <= 0) return 0;
  const bool wide = W % (dtype == 0 ? 4 : 8) == 0;
  if ((size_t)W * 4 > 96 * 1024 || (long)N * top > 0x7fffffffL / 2) return -1;
  const int slab = slab_for(F, (long)N * top);
  const dim3 grid(N * top, (F + slab - 1) / slab);
  const size_t lds = (size_t)W * sizeof(float);
#define TK_GU(T_, WIDE_)                                                                               \
  {                                                                                                    \
    static bool allowed = false;                                                                       \
    if (!allowed) {                                                                                    \
      const hipError_t err = hipFuncSetAttribute((const void*)moe_gate_up_kernel<T_, WIDE_>,           \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); \
      if (err != hipSuccess) return (int)err;                                                          \
      allowed = true;                                                                                  \
    }                                                                                                  \
    moe_gate_up_kernel<T_, WIDE_><<<grid, 256, lds, stream>>>((const T_*)h, (const T_*)gate_up, chosen, weight, \
                                                              (T_*)act, W, F, top, slab);              \
  }
  if (dtype == 0 && wide) TK_GU(float, true)
  else if (dtype == 0) TK_GU(float, false)
  else if (wide) TK_GU(bf16_t, true)
  else TK_GU(bf16_t, false)
#undef TK_GU
  return launch_status();
}

// out[N, W] float32 = sum over each token's chosen experts of down[e] act[pair]
TK_API int tk_moe_down(int dtype, const void* act, const void* down, const int* chosen, float* out, int N, int W,
                       int F, int top, hipStream_t stream) {
  if (N <= 0) return 0;
  const bool wide = F % (dtype == 0 ? 4 : 8) == 0;
  if ((size_t)top * F * 4 > 96 * 1024) return -1;
  const int slab = slab_for(W, N);
  const dim3 grid(N, (W + slab - 1) / slab);
  const size_t lds = (size_t)top * F * sizeof(float);
#define TK_DN(T_, WIDE_)                                                                               \
  {                                                                                                    \
    static bool allowed = false;                                                                       \
    if (!allowed) {                                                                                    \
      const hipError_t err = hipFuncSetAttribute((const void*)moe_down_kernel<T_, WIDE_>,              \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); \
      if (err != hipSuccess) return (int)err;                                                          \
      allowed = true;                                                                                  \
    }                                                                                                  \
    moe_down_kernel<T_, WIDE_><<<grid, 256, lds, stream>>>((const T_*)act, (const T_*)down, chosen, out, W, F, top, slab); \
  }
  if (dtype == 0 && wide) TK_DN(float, true)
  else if (dtype == 0) TK_DN(float, false)
  else if (wide) TK_DN(bf16_t, true)
  else TK_DN(bf16_t, false)
#undef TK_DN
  return launch_status();
}

TK_SLOTS(tk_moe_route)
TK_SLOTS(tk_moe_gate_up)
TK_SLOTS(tk_moe_down)
