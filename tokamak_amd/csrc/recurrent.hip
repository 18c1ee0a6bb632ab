// Kernels of recurrent mixers with a matrix-valued state per head (gfx950).
//
// token_shift: per token the interpolations x + (x_prev - x) * mu_s between a row and the row
//   before it in its sequence; the row before a step's first token comes from the request's
//   state, which then takes the step's last row.
// tanh: the activation between the two products of a low-rank decay.
// wkv_scan: per (request, head) the recurrence
//     o_t = (S + diag(u) k_t v_t^T)^T r_t ;  S <- diag(w_t) S + k_t v_t^T ,  w_t = exp(-exp(d_t + w0))
//   over the step's tokens in order, the state S [dim, dim] in float32 registers (a thread owns a
//   column), followed by the head's unit norm, a gain and a SiLU gate.
//
// Decays, exponentials, the state and the norm are float32 whatever the storage type.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

// element idx of a [rows, width] input: T, or float32, or the sum of float32 partial sums
template <typename T>
__device__ __forceinline__ float load_in(const void* p, int f32, int parts, long part_stride, size_t idx) {
  if (!f32) return Elem<T>::load(reinterpret_cast<const T*>(p) + idx);
  const float* f = reinterpret_cast<const float*>(p);
  float s = f[idx];
  for (int i = 1; i < parts; ++i) s += f[idx + (size_t)i * part_stride];
  return s;
}

template <typename T>
__global__ void token_shift_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                   float* __restrict__ last, T* __restrict__ out,
                                   const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                   const int* __restrict__ state_slots, int N, int W, int S) {
  const int n = blockIdx.x;
  const int r = req_of_token[n];
  const int first = q_start[r];
  const int end = q_start[r + 1];
  const bool head = n == first;
  float* mine = last + (size_t)state_slots[r] * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float cur = Elem<T>::load(h + (size_t)n * W + c);
    const float prev = head ? mine[c] : Elem<T>::load(h + (size_t)(n - 1) * W + c);
    const float d = prev - cur;
    for (int s = 0; s < S; ++s)
      Elem<T>::store(out + ((size_t)s * N + n) * W + c, cur + d * mu[(size_t)s * W + c]);
    // the thread that has read the old row of the state is the one that replaces it
    if (head) mine[c] = Elem<T>::load(h + (size_t)(end - 1) * W + c);
  }
}

template <typename T>
__global__ void tanh_kernel(const void* __restrict__ in, int f32, int parts, long part_stride,
                            T* __restrict__ out, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  Elem<T>::store(out + idx, tanhf(load_in<T>(in, f32, parts, part_stride, idx)));
}

constexpr int kScanTokens = 8;   // tokens whose operands are staged in LDS at once

template <typename T, int DMAX>
__global__ __launch_bounds__(DMAX < 64 ? 64 : DMAX) void wkv_scan_kernel(
    const T* __restrict__ r_in, const T* __restrict__ k_in, const T* __restrict__ v_in,
    const T* __restrict__ g_in, const void* __restrict__ d_in, int d_f32, int d_parts, long d_stride,
    const float* __restrict__ w0, const float* __restrict__ u, const float* __restrict__ gain,
    float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ state_slots,
    T* __restrict__ out, int heads, int dim, float eps) {
  constexpr int TB = kScanTokens;
  __shared__ float rr[TB][DMAX], kk[TB][DMAX], ww[TB][DMAX], uk[TB][DMAX], os[TB][DMAX];
  __shared__ float rstd[TB];
  const int req = blockIdx.x, head = blockIdx.y;
  const int j = threadIdx.x;
  const bool live = j < dim;
  const int HD = heads * dim;
  const int col = head * dim + j;
  const int first = q_start[req], end = q_start[req + 1];
  float* S = state + ((size_t)state_slots[req] * heads + head) * dim * dim;
  float s[DMAX];
#pragma unroll
  for (int x = 0; x < DMAX; ++x) s[x] = (live && x < dim) ? S[(size_t)x * dim + j] : 0.f;
  const float w0j = live ? w0[col] : 0.f, uj = live ? u[col] : 0.f, gj = live ? gain[col] : 0.f;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;

  for (int t0 = first; t0 < end; t0 += TB) {
    const int tb = min(TB, end - t0);
    float vloc[TB], gloc[TB];
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      vloc[t] = gloc[t] = 0.f;
      if (t < tb && live) {
        const size_t at = (size_t)(t0 + t) * HD + col;
        const float kv = Elem<T>::load(k_in + at);
        rr[t][j] = Elem<T>::load(r_in + at);
        kk[t][j] = kv;
        uk[t][j] = uj * kv;
        ww[t][j] = expf(-expf(load_in<T>(d_in, d_f32, d_parts, d_stride, at) + w0j));
        vloc[t] = Elem<T>::load(v_in + at);
        gloc[t] = Elem<T>::load(g_in + at);
      }
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      if (t < tb) {
        const float vj = vloc[t];
        float o = 0.f;
#pragma unroll
        for (int x = 0; x < DMAX; ++x) {
          if (x < dim) {
            o = fmaf(rr[t][x], fmaf(uk[t][x], vj, s[x]), o);
            s[x] = fmaf(ww[t][x], s[x], kk[t][x] * vj);
          }
        }
        if (live) os[t][j] = o;
      }
    }
    __syncthreads();
    for (int t = wave; t < tb; t += nwaves) {
      float q = 0.f;
      for (int x = lane; x < dim; x += kWave) q += os[t][x] * os[t][x];
      q = wave_sum(q);
      if (lane == 0) rstd[t] = 1.f / sqrtf(q / (float)dim + eps);
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      if (t < tb && live) {
        const float g = gloc[t];
        const float y = os[t][j] * rstd[t] * gj * (g / (1.f + expf(-g)));
        Elem<T>::store(out + (size_t)(t0 + t) * HD + col, y);
      }
    }
    // (the next round writes rr, kk, ww, uk, which nobody reads after the second barrier, and
    // os and rstd only behind its own barriers)
  }
  if (live) {
#pragma unroll
    for (int x = 0; x < DMAX; ++x)
      if (x < dim) S[(size_t)x * dim + j] = s[x];
  }
}

template <typename T>
int launch_scan(const void* r, const void* k, const void* v, const void* g, const void* d, int d_f32, int d_parts,
                long d_stride, const float* w0, const float* u, const float* gain, float* state,
                const int* q_start, const int* state_slots, void* out, int R, int heads, int dim, float eps,
                hipStream_t stream) {
  const dim3 grid(R, heads);
#define TK_SCAN(DMAX)                                                                                    \
  wkv_scan_kernel<T, DMAX><<<grid, (DMAX < 64 ? 64 : DMAX), 0, stream>>>(                                 \
      (const T*)r, (const T*)k, (const T*)v, (const T*)g, d, d_f32, d_parts, d_stride, w0, u, gain, state, \
      q_start, state_slots, (T*)out, heads, dim, eps)
  if (dim <= 32) TK_SCAN(32);
  else if (dim <= 64) TK_SCAN(64);
  else if (dim <= 128) TK_SCAN(128);
  else TK_SCAN(256);
#undef TK_SCAN
  return launch_status();
}

}  // namespace

// out[s][n] = h[n] + (prev(n) - h[n]) * mu[s]; `last` [slots, W] float32 holds each request's
// newest row.  h, out: dtype (0 float32, 1 bfloat16).
TK_API int tk_token_shift(int dtype, const void* h, const float* mu, float* last, void* out,
                          const int* req_of_token, const int* q_start, const int* state_slots, int N, int W,
                          int S, hipStream_t stream) {
  if (N <= 0 || W <= 0 || S <= 0) return 0;
  const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
  if (dtype == 0)
    token_shift_kernel<float><<<N, threads, 0, stream>>>((const float*)h, mu, last, (float*)out, req_of_token,
                                                         q_start, state_slots, N, W, S);
  else
    token_shift_kernel<bf16_t><<<N, threads, 0, stream>>>((const bf16_t*)h, mu, last, (bf16_t*)out, req_of_token,
                                                          q_start, state_slots, N, W, S);
  return launch_status();
}

TK_API int tk_tanh(int dtype, const void* in, int in_f32, int parts, long part_stride, void* out, long total,
                   hipStream_t stream) {
  if (total <= 0) return 0;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == 0)
    tanh_kernel<float><<<blocks, 256, 0, stream>>>(in, in_f32, parts, part_stride, (float*)out, (size_t)total);
  else
    tanh_kernel<bf16_t><<<blocks, 256, 0, stream>>>(in, in_f32, parts, part_stride, (bf16_t*)out, (size_t)total);
  return launch_status();
}

// r, k, v, g, out: [N, heads * dim] in dtype; d: the decay's pre-activation, dtype or float32
// (partial sums allowed); state [slots, heads, dim, dim] float32.  dim <= 256.
TK_API int tk_wkv_scan(int dtype, const void* r, const void* k, const void* v, const void* g, const void* d,
                       int d_f32, int d_parts, long d_stride, const float* w0, const float* u, const float* gain,
                       float* state, const int* q_start, const int* state_slots, void* out, int R, int heads,
                       int dim, float eps, hipStream_t stream) {
  if (R <= 0 || heads <= 0) return 0;
  if (dim < 1 || dim > 256) return -2;
  if (dtype == 0)
    return launch_scan<float>(r, k, v, g, d, d_f32, d_parts, d_stride, w0, u, gain, state, q_start, state_slots,
                              out, R, heads, dim, eps, stream);
  return launch_scan<bf16_t>(r, k, v, g, d, d_f32, d_parts, d_stride, w0, u, gain, state, q_start, state_slots,
                             out, R, heads, dim, eps, stream);
}

TK_SLOTS(tk_token_shift)
TK_SLOTS(tk_tanh)
TK_SLOTS(tk_wkv_scan)
