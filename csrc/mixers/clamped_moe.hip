// Feed-forward pieces of layers whose experts clamp their gate / up products.
//
//   route_topk_softmax   the `top` largest of E fp32 router logits per token (ties: the lower expert)
//                        and the softmax over those logits only
//   clamped_glu          out = g' * sigmoid(1.702 g') * (u' + 1),  g' = min(g, limit),
//                        u' = clamp(u, -limit, limit); gate and up products side by side [n, F | F]
//                        or alternating in blocks of 16 (the grouped matrix-core GEMMs' layout)
//   gelu_tanh            x <- 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) in place
//   gated_rms_norm       out = o / sqrt(mean(o^2) + eps) * w * sigmoid(g)   (o fp32, one row per token)
//
// (The experts' own products run in sigmoid_moe.hip's grouped kernels with the clamped epilogue.)
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kMaxTop = 64;

__global__ void __launch_bounds__(64)
route_topk_softmax_kernel(int* __restrict__ ids, float* __restrict__ wts, const float* __restrict__ logits,
                          int64_t ld_logits, int E, int top) {
  extern __shared__ float sc[];  // [E]
  __shared__ float chosen[kMaxTop];
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) sc[e] = logits[t * ld_logits + e];
  __syncthreads();
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int bi = E;
    for (int e = lane; e < E; e += 64) {
      const float v = sc[e];
      if (v > best || bi == E) {  // ascending e per lane: the first of equal logits stays
        best = v;
        bi = e;
      }
    }
    // a lane that has no candidate left keeps bi == E and loses every comparison below
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi < E && (bi >= E || ov > best || (ov == best && oi < bi))) {
        best = ov;
        bi = oi;
      }
    }
    if (lane == 0) {
      ids[t * top + k] = bi;
      chosen[k] = best;
      sc[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (lane == 0) {
    const float m = chosen[0];  // the largest
    float sum = 0.f;
    for (int k = 0; k < top; ++k) sum += expf(chosen[k] - m);
    for (int k = 0; k < top; ++k) wts[t * top + k] = expf(chosen[k] - m) / sum;
  }
}

// Router logits of a decode-sized step: out[t, e] = x[t] . w[e] in fp32, one wave per (token, row of
// w), 16-byte loads, a fixed order of sums.  (Prompt-sized steps take an fp32 library GEMM.)
__global__ void __launch_bounds__(256) router_logits_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                            const float* __restrict__ w, int N, int W) {
  const int t = blockIdx.x, e = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (e >= N) return;
  const float* xr = x + static_cast<int64_t>(t) * W;
  const float* wr = w + static_cast<int64_t>(e) * W;
  float a0 = 0.f, a1 = 0.f;
  if ((W & 3) == 0) {
    for (int i = 4 * lane; i < W; i += 256) {
      const float4 xv = *reinterpret_cast<const float4*>(xr + i), wv = *reinterpret_cast<const float4*>(wr + i);
      a0 += xv.x * wv.x + xv.y * wv.y;
      a1 += xv.z * wv.z + xv.w * wv.w;
    }
  } else {
    for (int i = lane; i < W; i += 64) a0 += xr[i] * wr[i];
  }
  const float d = pk::wave_sum(a0 + a1);
  if (lane == 0) out[static_cast<int64_t>(t) * N + e] = d;
}

template <typename T>
__global__ void __launch_bounds__(256) clamped_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, int F,
                                                          float limit, int interleaved) {
  const int r = blockIdx.x;
  const T* src = gu + static_cast<int64_t>(r) * 2 * F;
  for (int i = threadIdx.x; i < F; i += blockDim.x) {
    const int gi = interleaved ? (i >> 4) * 32 + (i & 15) : i;
    const int ui = interleaved ? gi + 16 : F + i;
    const float g = fminf(ld<T>(src + gi), limit);
    const float u = fminf(fmaxf(ld<T>(src + ui), -limit), limit);
    st<T>(out + static_cast<int64_t>(r) * F + i, g * sigmoidf(1.702f * g) * (u + 1.f));
  }
}

// the same on the fp32 split-K slabs [S][n][2F] of a decode GEMM: the slabs are summed on the way in
template <typename T>
__global__ void __launch_bounds__(256) clamped_glu_slabs_kernel(T* __restrict__ out, const float* __restrict__ ws,
                                                                int nslab, int64_t slab_stride, int F, float limit,
                                                                int interleaved) {
  const int r = blockIdx.x;
  const float* src = ws + static_cast<int64_t>(r) * 2 * F;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;  // one output per thread: a decode-sized launch fills the chip
  if (i >= F) return;
  const int gi = interleaved ? (i >> 4) * 32 + (i & 15) : i;
  const int ui = interleaved ? gi + 16 : F + i;
  float g = 0.f, u = 0.f;
  for (int s = 0; s < nslab; ++s) {
    g += src[s * slab_stride + gi];
    u += src[s * slab_stride + ui];
  }
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  st<T>(out + static_cast<int64_t>(r) * F + i, g * sigmoidf(1.702f * g) * (u + 1.f));
}

template <typename T>
__global__ void __launch_bounds__(256) gelu_tanh_kernel(T* __restrict__ x, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float z = ld<T>(x + i);
  st<T>(x + i, 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))));
}

template <typename T, typename G>
__global__ void __launch_bounds__(256) gated_rms_norm_kernel(T* __restrict__ out, const float* __restrict__ o,
                                                             const float* __restrict__ w, const G* __restrict__ g,
                                                             int64_t g_stride, int N, float eps) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const float* row = o + static_cast<int64_t>(t) * N;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += blockDim.x) ss += row[i] * row[i];
  ss = pk::block_sum(ss, red);
  const float k = 1.f / sqrtf(ss / static_cast<float>(N) + eps);
  for (int i = threadIdx.x; i < N; i += blockDim.x)
    st<T>(out + static_cast<int64_t>(t) * N + i, row[i] * k * w[i] * sigmoidf(ld<G>(g + t * g_stride + i)));
}

}  // namespace

PK_EXPORT int pkm_route_topk_softmax(void* ids, void* wts, const void* logits, long long ld_logits, int T, int E, int top,
                                     hipStream_t stream) {
  if (T <= 0) return 0;
  if (top < 1 || top > E || top > kMaxTop || E > 4096 || ld_logits < E) return -1;
  route_topk_softmax_kernel<<<T, 64, E * sizeof(float), stream>>>(static_cast<int*>(ids), static_cast<float*>(wts),
                                                                   static_cast<const float*>(logits), ld_logits, E, top);
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_router_logits(void* out, const void* x, const void* w, int T, int N, int W, hipStream_t stream) {
  if (T <= 0 || N <= 0) return 0;
  const dim3 grid(T, (N + 3) / 4);
  router_logits_kernel<<<grid, 256, 0, stream>>>(static_cast<float*>(out), static_cast<const float*>(x),
                                                 static_cast<const float*>(w), N, W);
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_clamped_glu(void* out, const void* gu, int n, int F, float limit, int interleaved, int dt,
                              hipStream_t stream) {
  if (n <= 0) return 0;
  if (interleaved && F % 16) return -1;
  PKM_DISPATCH(dt, T, clamped_glu_kernel<T><<<n, 256, 0, stream>>>(static_cast<T*>(out), static_cast<const T*>(gu), F,
                                                                   limit, interleaved));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_clamped_glu_slabs(void* out, const void* ws, int nslab, int n, int F, float limit, int interleaved,
                                    int dt, hipStream_t stream) {
  if (n <= 0) return 0;
  if (nslab < 1 || (interleaved && F % 16)) return -1;
  const dim3 grid(n, (F + 255) / 256);
  PKM_DISPATCH(dt, T, clamped_glu_slabs_kernel<T><<<grid, 256, 0, stream>>>(
                          static_cast<T*>(out), static_cast<const float*>(ws), nslab, static_cast<int64_t>(n) * 2 * F, F,
                          limit, interleaved));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_gelu_tanh(void* x, long long n, int dt, hipStream_t stream) {
  if (n <= 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  PKM_DISPATCH(dt, T, gelu_tanh_kernel<T><<<blocks, 256, 0, stream>>>(static_cast<T*>(x), n));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_gated_rms_norm(void* out, const void* o, const void* w, const void* g, long long g_stride, int T,
                                 int N, float eps, int g_dt, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (g_dt != dt) return -1;
  PKM_DISPATCH(dt, E, gated_rms_norm_kernel<E, E><<<T, 256, 0, stream>>>(
                          static_cast<E*>(out), static_cast<const float*>(o), static_cast<const float*>(w),
                          static_cast<const E*>(g), g_stride, N, eps));
  return PK_CHECK_LAUNCH();
}
