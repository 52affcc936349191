// Residual-stream kernels of post-norm layers whose stream stays in fp32:
//
//   embed_rows       x[t] = table[ids[t]]                                    (table bf16 or fp32)
//   token_shift      h[t] = x[t] + (x[t-1] - x[t]) * mu, x[-1] of a sequence's portion taken from
//                    the sequence's state slot (zeros at position 0); h in the activation type
//   save_last_rows   state[slot[s]] = x[last token of sequence s in this step]
//   sum_gain_norm    v = alpha * x + y;  z = v / sqrt(mean(v^2) + eps) * g  (g: ONE number);
//                    optionally z is stored as entry nh-1 of a per-step history of layer outputs
//                    and the kernel hands on  sum_j coef[j] * hist[j]  (the learned average over
//                    all earlier outputs) instead of z; optional copy in the activation type;
//                    optional row gather (the rows whose logits are wanted).
//
// One workgroup per token; sums in fp32; the mean of squares is reduced in a fixed order, so a
// token's result does not depend on the rest of the batch.
#include "mix_common.h"

using namespace pkm;

namespace {

template <typename T>
__global__ void __launch_bounds__(256) embed_rows_kernel(float* __restrict__ out, const T* __restrict__ table,
                                                         const int* __restrict__ ids, int W, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + static_cast<int64_t>(id) * W;
  float* dst = out + static_cast<int64_t>(t) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) dst[i] = ld<T>(src + i);
}

template <typename T>
__global__ void __launch_bounds__(256) token_shift_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                          const float* __restrict__ mu, const float* __restrict__ state,
                                                          const int* __restrict__ token_seq, const int* __restrict__ cu_q,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ slots, int W) {
  const int t = blockIdx.x;
  const int s = token_seq[t];
  const float* cur = x + static_cast<int64_t>(t) * W;
  const float* prev = nullptr;
  if (t > cu_q[s]) {
    prev = cur - W;
  } else if (positions[t] > 0 && slots[s] >= 0) {
    prev = state + static_cast<int64_t>(slots[s]) * W;
  }
  T* dst = out + static_cast<int64_t>(t) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float a = cur[i];
    const float p = prev ? prev[i] : 0.f;
    st<T>(dst + i, a + (p - a) * mu[i]);
  }
}

__global__ void __launch_bounds__(256) save_last_rows_kernel(float* __restrict__ state, const float* __restrict__ x,
                                                             const int* __restrict__ cu_q, const int* __restrict__ slots,
                                                             int W) {
  const int s = blockIdx.x;
  const int end = cu_q[s + 1];
  if (end <= cu_q[s] || slots[s] < 0) return;
  const float* src = x + static_cast<int64_t>(end - 1) * W;
  float* dst = state + static_cast<int64_t>(slots[s]) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) dst[i] = src[i];
}

// Optional fused neighbours:
//   gather (inv, top):  y is a table of expert output rows and the token's y is the plain sum of its
//                       `top` rows y[inv[t * top + j]] (the MoE combine; inv < 0: no row)
//   state (token_seq, cu_q, slots): a token that is the last of its sequence in this step leaves its
//                       x row in the sequence's state slot (the token shift of the NEXT step reads it;
//                       this step's shift has already run)
//   slabs (nslab, slab_stride): y is nslab split-K slabs [nslab][rows][W] of a projection and the
//                       token's y is their sum (the slab reduce of the decode GEMM fused in)
struct NormFusion {
  int nslab;
  int64_t slab_stride;
  const int* inv;
  int top;
  float* state;
  const int* token_seq;
  const int* cu_q;
  const int* slots;
};

template <typename T, typename Y>
__global__ void __launch_bounds__(1024)
sum_gain_norm_kernel(float* __restrict__ out, T* __restrict__ out_act, const float* __restrict__ x,
                     const Y* __restrict__ y, const int* __restrict__ rows, float alpha, const float* __restrict__ gain,
                     float eps, int W, float* __restrict__ hist, int64_t hist_stride, int nh,
                     const float* __restrict__ coef, NormFusion f) {
  __shared__ float red[16];
  extern __shared__ float vbuf[];  // [W] the sum alpha x + y, kept between the two passes
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  const float* xr = x + src * W;
  const Y* yr = (y && !f.inv) ? y + src * W : nullptr;
  float* keep = nullptr;
  if (f.state) {
    const int sq = f.token_seq[r];
    if (r == f.cu_q[sq + 1] - 1 && f.slots[sq] >= 0) keep = f.state + static_cast<int64_t>(f.slots[sq]) * W;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float xv = xr[i];
    float yv = yr ? ld<Y>(yr + i) : 0.f;
    for (int sl = 1; sl < f.nslab; ++sl) yv += ld<Y>(yr + sl * f.slab_stride + i);
    if (f.inv) {
      for (int j = 0; j < f.top; ++j) {
        const int yrow = f.inv[src * f.top + j];
        if (yrow >= 0) yv += ld<Y>(y + static_cast<int64_t>(yrow) * W + i);
      }
    }
    if (keep) keep[i] = xv;
    const float v = alpha * xv + yv;
    vbuf[i] = v;
    ss += v * v;
  }
  ss = pk::block_sum(ss, red);
  const float k = gain[0] / sqrtf(ss / static_cast<float>(W) + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float z = vbuf[i] * k;
    if (hist) {
      const int64_t at = static_cast<int64_t>(r) * W + i;
      hist[(nh - 1) * hist_stride + at] = z;
      float acc = coef[nh - 1] * z;
      for (int j = 0; j < nh - 1; ++j) acc += coef[j] * hist[j * hist_stride + at];
      z = acc;
    }
    if (out) out[static_cast<int64_t>(r) * W + i] = z;
    if (out_act) st<T>(out_act + static_cast<int64_t>(r) * W + i, z);
  }
}

}  // namespace

PK_EXPORT int pkm_embed_rows(void* out, const void* table, const void* ids, int T, int W, int vocab, int dt,
                             hipStream_t stream) {
  if (T <= 0) return 0;
  PKM_DISPATCH(dt, E, embed_rows_kernel<E><<<T, 256, 0, stream>>>(static_cast<float*>(out), static_cast<const E*>(table),
                                                                   static_cast<const int*>(ids), W, vocab));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_token_shift(void* out, const void* x, const void* mu, const void* state, const void* token_seq,
                              const void* cu_q, const void* positions, const void* slots, int T, int W, int dt,
                              hipStream_t stream) {
  if (T <= 0) return 0;
  PKM_DISPATCH(dt, E, token_shift_kernel<E><<<T, 256, 0, stream>>>(
                          static_cast<E*>(out), static_cast<const float*>(x), static_cast<const float*>(mu),
                          static_cast<const float*>(state), static_cast<const int*>(token_seq),
                          static_cast<const int*>(cu_q), static_cast<const int*>(positions),
                          static_cast<const int*>(slots), W));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_save_last_rows(void* state, const void* x, const void* cu_q, const void* slots, int n, int W,
                                 hipStream_t stream) {
  if (n <= 0) return 0;
  save_last_rows_kernel<<<n, 256, 0, stream>>>(static_cast<float*>(state), static_cast<const float*>(x),
                                               static_cast<const int*>(cu_q), static_cast<const int*>(slots), W);
  return PK_CHECK_LAUNCH();
}

// y_dt: element type of y (-1: no y).  hist == nullptr: no history / average.  inv != nullptr: y is
// gathered (see NormFusion); state != nullptr: last rows are saved (token_seq, cu_q, slots given).
PK_EXPORT int pkm_sum_gain_norm(void* out, void* out_act, const void* x, const void* y, const void* rows, float alpha,
                                const void* gain, float eps, int R, int W, void* hist, long long hist_stride, int nh,
                                const void* coef, int dt, int y_dt, int nslab, const void* inv, int top, void* state,
                                const void* token_seq, const void* cu_q, const void* slots, hipStream_t stream) {
  if (R <= 0) return 0;
  if (hist && (nh < 1 || !coef)) return -1;
  if ((inv && (!y || top < 1 || rows)) || (state && (!token_seq || !cu_q || !slots || rows))) return -1;
  if (W > 16384 || nslab < 1 || (nslab > 1 && (!y || inv || rows))) return -1;
  const NormFusion f{nslab, static_cast<int64_t>(R) * W, static_cast<const int*>(inv), top, static_cast<float*>(state), static_cast<const int*>(token_seq),
                     static_cast<const int*>(cu_q), static_cast<const int*>(slots)};
  const size_t lds = static_cast<size_t>(W) * sizeof(float);
  // two coordinates per thread when the row allows: a token's chain of dependent loads (gathered
  // expert rows, the history entries) is the latency of a decode-sized launch
  const int threads = W >= 2048 ? 1024 : (W >= 1024 ? 512 : 256);
#define PKM_SGN(E, Y)                                                                                             \
  sum_gain_norm_kernel<E, Y><<<R, threads, lds, stream>>>(static_cast<float*>(out), static_cast<E*>(out_act),         \
                                                      static_cast<const float*>(x), static_cast<const Y*>(y),     \
                                                      static_cast<const int*>(rows), alpha,                       \
                                                      static_cast<const float*>(gain), eps, W,                    \
                                                      static_cast<float*>(hist), hist_stride, nh,                 \
                                                      static_cast<const float*>(coef), f)
  if (y == nullptr || y_dt == kF32) {
    PKM_DISPATCH(dt, E, PKM_SGN(E, float));
  } else if (y_dt == kBF16) {
    PKM_DISPATCH(dt, E, PKM_SGN(E, bf16_t));
  } else {
    return -2;
  }
#undef PKM_SGN
  return PK_CHECK_LAUNCH();
}
