// Latent attention over a paged cache of per-token latents (no positional part).
//
// Every token caches ONE vector c (kv_rank numbers, RMS-normed with a learned weight); head a's
// key and value are W_uk[a] c and W_uv[a] c.  The kernels work in the latent space, for prompts
// and for decoding alike: the caller folds W_uk into the query (q~ = W_uk[a]^T q, kv_rank numbers)
// and applies W_uv to the attended latent afterwards, so
//
//     score(i, j, a) = scale * q~[i, a] . c[j]        o~[i, a] = sum_j softmax_j(score) c[j]
//
// and all heads of a token read the same cached rows: the (token, head) pairs of a sequence are
// the rows of one tile problem  S = Q~ C^T, O~ = P C  against a key tile staged once in LDS.
//
//   latent_norm_cache   c = dkv / sqrt(mean(dkv^2) + eps) * w  ->  cache[slot]      (fp32 maths)
//   latent_attention    causal softmax attention of q~ over the cached latents; scores, softmax
//                       and the output accumulation in fp32; key tiles always start at key 0 of
//                       the sequence, so a row's sums do not depend on how its prompt was cut
//                       or on what else the step holds
//   gate_merge          out[t, a*V + v] = o[a][t][v] * sigmoid(g[t, a*V + v])
#include "mix_common.h"

using namespace pkm;

namespace {

template <typename T>
__global__ void __launch_bounds__(128)
latent_norm_cache_kernel(T* __restrict__ cache, const T* __restrict__ dkv, int64_t dkv_stride,
                         const float* __restrict__ w, const int* __restrict__ slot_mapping, int R, float eps) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int slot = slot_mapping[t];
  const T* src = dkv + static_cast<int64_t>(t) * dkv_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = ld<T>(src + i);
    ss += v * v;
  }
  ss = pk::block_sum(ss, red);
  if (slot < 0) return;
  const float k = 1.f / sqrtf(ss / static_cast<float>(R) + eps);
  T* dst = cache + static_cast<int64_t>(slot) * R;
  for (int i = threadIdx.x; i < R; i += blockDim.x) st<T>(dst + i, ld<T>(src + i) * k * w[i]);
}

constexpr int kBQ = 16;       // (token, head) rows per workgroup
constexpr int kThreads = 256;  // 16 rows x 16 lanes

// NR: output accumulators per thread = ceil(R / 16)
template <typename T, int NR>
__global__ void __launch_bounds__(kThreads)
latent_attention_kernel(T* __restrict__ out, int64_t out_st, int64_t out_sh, const T* __restrict__ q, int64_t q_st,
                        int64_t q_sh, const T* __restrict__ cache, const int* __restrict__ block_tables, int max_blocks,
                        const int* __restrict__ cu_q, const int* __restrict__ context_lens, int n_seqs, int H, int R,
                        int block_size, int BK, float scale) {
  extern __shared__ float smem[];
  // which sequence / row tile is this workgroup's
  int s = 0, tile = blockIdx.x;
  for (; s < n_seqs; ++s) {
    const int rows = (cu_q[s + 1] - cu_q[s]) * H;
    const int nt = (rows + kBQ - 1) / kBQ;
    if (tile < nt) break;
    tile -= nt;
  }
  if (s >= n_seqs) return;
  const int q0 = cu_q[s], qlen = cu_q[s + 1] - q0, ctx = context_lens[s];
  const int n_rows = qlen * H;
  const int row0 = tile * kBQ;
  const int RS = R + 1;  // odd row stride: conflict-free column walks
  float* qs = smem;                 // [kBQ][RS]
  float* cs = qs + kBQ * RS;        // [BK][RS]
  float* ps = cs + BK * RS;         // [kBQ][BK]
  float* m_s = ps + kBQ * BK;       // [kBQ] running max
  float* l_s = m_s + kBQ;           // [kBQ] running sum
  float* a_s = l_s + kBQ;           // [kBQ] rescale of this tile
  const int tid = threadIdx.x;
  const int qi = tid >> 4, kg = tid & 15;
  const int* bt = block_tables + static_cast<int64_t>(s) * max_blocks;

  // stage the query rows
  for (int e = tid; e < kBQ * R; e += kThreads) {
    const int r = e / R, c = e - r * R;
    const int row = row0 + r;
    float v = 0.f;
    if (row < n_rows) {
      const int tl = row / H, h = row - tl * H;
      v = ld<T>(q + static_cast<int64_t>(q0 + tl) * q_st + static_cast<int64_t>(h) * q_sh + c);
    }
    qs[r * RS + c] = v;
  }
  if (tid < kBQ) {
    m_s[tid] = -INFINITY;
    l_s[tid] = 0.f;
  }
  // position of this thread's row; rows past the sequence's end see nothing
  const int my_row = row0 + qi;
  const int my_pos = my_row < n_rows ? ctx - qlen + my_row / H : -1;
  const int last_row = min(row0 + kBQ, n_rows) - 1;
  const int max_pos = ctx - qlen + last_row / H;  // keys 0..max_pos are visible to some row
  float acc[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) acc[i] = 0.f;
  __syncthreads();

  for (int k0 = 0; k0 <= max_pos; k0 += BK) {
    const int nk = min(BK, max_pos + 1 - k0);
    // stage the key tile
    for (int e = tid; e < BK * R; e += kThreads) {
      const int j = e / R, c = e - j * R;
      float v = 0.f;
      if (j < nk) {
        const int key = k0 + j;
        const int64_t slot = static_cast<int64_t>(bt[key / block_size]) * block_size + key % block_size;
        v = ld<T>(cache + slot * R + c);
      }
      cs[j * RS + c] = v;
    }
    __syncthreads();
    // scores of row qi against keys kg, kg + 16, ...
    float tmax = -INFINITY;
    for (int j = kg; j < BK; j += 16) {
      float d = 0.f;
      const float* qr = qs + qi * RS;
      const float* cr = cs + j * RS;
      for (int c = 0; c < R; ++c) d += qr[c] * cr[c];
      d = (k0 + j <= my_pos) ? d * scale : -INFINITY;
      ps[qi * BK + j] = d;
      tmax = fmaxf(tmax, d);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
    const float m_old = m_s[qi];
    const float m_new = fmaxf(m_old, tmax);
    float tsum = 0.f;
    for (int j = kg; j < BK; j += 16) {
      const float sc = ps[qi * BK + j];
      const float p = (m_new == -INFINITY || sc == -INFINITY) ? 0.f : expf(sc - m_new);
      ps[qi * BK + j] = p;
      tsum += p;
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) tsum += __shfl_xor(tsum, o, 64);
    const float resc = (m_old == -INFINITY) ? 0.f : expf(m_old - m_new);
    __syncthreads();  // every lane of the row has read m_old and its own scores
    if (kg == 0) {
      m_s[qi] = m_new;
      l_s[qi] = l_s[qi] * resc + tsum;
    }
    // o~ += P C: this thread owns latent coordinates kg, kg + 16, ... of row qi
#pragma unroll
    for (int i = 0; i < NR; ++i) acc[i] *= resc;
    for (int j = 0; j < nk; ++j) {
      const float p = ps[qi * BK + j];
      const float* cr = cs + j * RS + kg;
#pragma unroll
      for (int i = 0; i < NR; ++i)
        if (kg + 16 * i < R) acc[i] += p * cr[16 * i];
    }
    __syncthreads();
  }
  if (my_row < n_rows) {
    const float l = l_s[qi];
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const int tl = my_row / H, h = my_row - tl * H;
    T* dst = out + static_cast<int64_t>(q0 + tl) * out_st + static_cast<int64_t>(h) * out_sh;
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (kg + 16 * i < R) st<T>(dst + kg + 16 * i, acc[i] * inv);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
gate_merge_kernel(T* __restrict__ out, const T* __restrict__ o, int64_t o_st, int64_t o_sh, const T* __restrict__ g,
                  int64_t g_stride, int H, int V) {
  const int t = blockIdx.x;
  for (int e = threadIdx.x; e < H * V; e += blockDim.x) {
    const int h = e / V, v = e - h * V;
    const float a = ld<T>(o + static_cast<int64_t>(t) * o_st + static_cast<int64_t>(h) * o_sh + v);
    const float z = ld<T>(g + static_cast<int64_t>(t) * g_stride + e);
    st<T>(out + static_cast<int64_t>(t) * H * V + e, a * sigmoidf(z));
  }
}

}  // namespace

PK_EXPORT int pkm_latent_norm_cache(void* cache, const void* dkv, long long dkv_stride, const void* w,
                                    const void* slot_mapping, int T, int R, float eps, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  PKM_DISPATCH(dt, E, latent_norm_cache_kernel<E><<<T, 128, 0, stream>>>(
                          static_cast<E*>(cache), static_cast<const E*>(dkv), dkv_stride, static_cast<const float*>(w),
                          static_cast<const int*>(slot_mapping), R, eps));
  return PK_CHECK_LAUNCH();
}

// key tile size for a latent of R numbers: the largest of 64 / 32 / 16 / 8 whose tiles fit 96 KiB of LDS
static int latent_key_tile(int R) {
  for (int bk = 64; bk >= 8; bk >>= 1) {
    const size_t bytes = (static_cast<size_t>(kBQ + bk) * (R + 1) + kBQ * bk + 3 * kBQ) * sizeof(float);
    if (bytes <= 96 * 1024) return bk;
  }
  return 0;
}

PK_EXPORT int pkm_latent_attention(void* out, long long out_st, long long out_sh, const void* q, long long q_st,
                                   long long q_sh, const void* cache, const void* block_tables, int max_blocks,
                                   const void* cu_q, const void* context_lens, int n_seqs, int T, int H, int R,
                                   int block_size, float scale, int dt, hipStream_t stream) {
  if (T <= 0 || n_seqs <= 0) return 0;
  const int BK = latent_key_tile(R);
  if (BK == 0 || R > 1024 || block_size <= 0) return -1;
  const size_t lds = (static_cast<size_t>(kBQ + BK) * (R + 1) + kBQ * BK + 3 * kBQ) * sizeof(float);
  const int64_t rows = static_cast<int64_t>(T) * H;
  const int grid = static_cast<int>((rows + kBQ - 1) / kBQ + n_seqs);
#define PKM_LA(E, NR)                                                                                            \
  {                                                                                                              \
    auto kern = latent_attention_kernel<E, NR>;                                                                  \
    if (lds > 48 * 1024) {                                                                                       \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                              \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
      if (e != hipSuccess) return static_cast<int>(e);                                                           \
    }                                                                                                            \
    kern<<<grid, kThreads, lds, stream>>>(static_cast<E*>(out), out_st, out_sh, static_cast<const E*>(q), q_st,  \
                                          q_sh, static_cast<const E*>(cache),                                    \
                                          static_cast<const int*>(block_tables), max_blocks,                     \
                                          static_cast<const int*>(cu_q), static_cast<const int*>(context_lens),  \
                                          n_seqs, H, R, block_size, BK, scale);                                  \
  }
  if (R <= 128) {
    PKM_DISPATCH(dt, E, PKM_LA(E, 8));
  } else if (R <= 512) {
    PKM_DISPATCH(dt, E, PKM_LA(E, 32));
  } else {
    PKM_DISPATCH(dt, E, PKM_LA(E, 64));
  }
#undef PKM_LA
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_gate_merge(void* out, const void* o, long long o_st, long long o_sh, const void* g,
                             long long g_stride, int T, int H, int V, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  PKM_DISPATCH(dt, E, gate_merge_kernel<E><<<T, 256, 0, stream>>>(static_cast<E*>(out), static_cast<const E*>(o), o_st,
                                                                  o_sh, static_cast<const E*>(g), g_stride, H, V));
  return PK_CHECK_LAUNCH();
}
