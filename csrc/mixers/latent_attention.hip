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

// column of key k (0..31) inside a 32-key tile of the latent-major copy: the key-slot order of the
// matrix-core kernels' second product (see latent_attention_mfma_kernel)
__host__ __device__ __forceinline__ int key_slot(int k) { return ((k & 15) >> 2) * 8 + (k & 3) + 4 * (k >> 4); }

// cache_t (optional): the latent-major copy [blocks][block_size / 32][R][32 key slots]
template <typename T>
__global__ void __launch_bounds__(128)
latent_norm_cache_kernel(T* __restrict__ cache, T* __restrict__ cache_t, int block_size, const T* __restrict__ dkv,
                         int64_t dkv_stride, const float* __restrict__ w, const int* __restrict__ slot_mapping, int R,
                         float eps) {
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
  T* dst_t = nullptr;
  if (cache_t) {
    const int kb = slot % block_size;
    dst_t = cache_t + (static_cast<int64_t>(slot / block_size) * (block_size / 32) + kb / 32) * R * 32 + key_slot(kb & 31);
  }
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = ld<T>(src + i) * k * w[i];
    st<T>(dst + i, v);
    if (dst_t) st<T>(dst_t + static_cast<int64_t>(i) * 32, v);
  }
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

// Softmax bookkeeping of the matrix-core kernels.  Scores are kept in log2 units (scale * log2 e
// folded into one multiply).  The running reference m only moves when a tile's maximum exceeds it
// by more than kLazyMax: weights are then at most 2^kLazyMax (exact in fp32, and in bf16 as the
// second product's operand), the softmax is unchanged (any reference gives the same quotient),
// and the 128-register rescale of the output tile runs on a few tiles instead of nearly all.
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLazyMax = 10.f;

// ---- bf16 on the matrix cores -------------------------------------------------------------------
// 128 (token, head) rows per workgroup, 16 per wave; 32-key tiles (the cached tile is re-read by
// every workgroup of a sequence, so rows per workgroup set the kernel's memory traffic).  Both products run transposed on
// mfma_f32_16x16x32_bf16 so that the softmax weights never leave their registers:
//
//   S^T [keys x rows] = C [keys x R] . Q~^T     A = key rows from LDS `cs`, B = the wave's Q~ (registers)
//   O~^T [R x rows]  += C^T [R x keys] . P^T    A = latent rows from the transposed LDS copy `ct`,
//                                               B = P^T straight from the S^T accumulators
//
// An accumulator lane (g, n) holds query row n and keys 4g..4g+3 of each 16-key half; the B operand
// of the second product wants 8 key slots per lane, so slot (g, e) is key 4g+e of the first half
// for e < 4 and key 16+4g+e-4 of the second, and `ct` stores its columns in that slot order.
// The tile is staged twice (key-major and latent-major) because it is both the key and the value.
// threads of the prompt kernel: 8 waves = 128 (token, head) rows per workgroup share every staged tile
constexpr int kPromptThreads = 512;

template <int R>
__global__ void __launch_bounds__(kPromptThreads)
latent_attention_mfma_kernel(bf16_t* __restrict__ out, int64_t out_st, int64_t out_sh, const bf16_t* __restrict__ q,
                             int64_t q_st, int64_t q_sh, const bf16_t* __restrict__ cache,
                             const bf16_t* __restrict__ cache_t, const int* __restrict__ block_tables, int max_blocks,
                             const int* __restrict__ cu_q, const int* __restrict__ context_lens, int n_seqs, int H,
                             int block_size, float scale) {
  constexpr int NT = kPromptThreads, BQ = NT / 4, BK = 32, NKK = R / 32, NRT = R / 16, CS = R + 8, CT = BK + 8, R8 = R / 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* cs = reinterpret_cast<bf16_t*>(smem_raw);  // [BK][CS]   key-major
  bf16_t* ct = cs + BK * CS;                          // [R][CT]    latent-major, key slots permuted
  int s = 0, tile = blockIdx.x;
  for (; s < n_seqs; ++s) {
    const int nt = ((cu_q[s + 1] - cu_q[s]) * H + BQ - 1) / BQ;
    if (tile < nt) break;
    tile -= nt;
  }
  if (s >= n_seqs) return;
  const int q0 = cu_q[s], qlen = cu_q[s + 1] - q0, ctx = context_lens[s];
  const int n_rows = qlen * H, row0 = tile * BQ;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, n = lane & 15;
  const int* bt = block_tables + static_cast<int64_t>(s) * max_blocks;
  const int my_row = row0 + 16 * wave + n;
  const bool valid = my_row < n_rows;
  const int tl = valid ? my_row / H : 0, h = valid ? my_row - tl * H : 0;
  const int my_pos = valid ? ctx - qlen + tl : -1;
  const int max_pos = ctx - qlen + (min(row0 + BQ, n_rows) - 1) / H;

  pk::bf16x8_t qf[NKK];
  {
    const bf16_t* qr = q + static_cast<int64_t>(q0 + tl) * q_st + static_cast<int64_t>(h) * q_sh + 8 * g;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      pk::u32x4 v = {0u, 0u, 0u, 0u};
      if (valid) v = *reinterpret_cast<const pk::u32x4*>(qr + kk * 32);
      qf[kk] = __builtin_bit_cast(pk::bf16x8_t, v);
    }
  }
  pk::f32x4 o[NRT];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) o[rt] = pk::f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const float scale2 = scale * kLog2e;  // scores in log2 units: a weight is one exp2

  // with the latent-major copy a tile is one contiguous run in each layout (pages hold whole 32-key
  // tiles) and every thread's loads are issued before its first store; keys past the visible ones
  // are stale cache rows: finite, and their weights are zero.  Issuing tile t+1's loads before tile
  // t's products was tried twice: at 4 waves it cost the second workgroup per CU (slower), at 8
  // waves and a 512-wide latent the extra live registers spill (the compiler's resource report).
  constexpr int NIT = (4 * R + NT - 1) / NT;
  pk::u32x4 kv[NIT], tv[NIT];
  auto fetch = [&](int k0) {
    const int64_t blk = bt[k0 / block_size];
    const bf16_t* ksrc = cache + (blk * block_size + k0 % block_size) * R;
    const bf16_t* tsrc = cache_t + (blk * (block_size / 32) + (k0 % block_size) / 32) * R * 32;
#pragma unroll
    for (int i = 0; i < NIT; ++i) {
      const int c = tid + NT * i;
      if (c < 4 * R) {
        kv[i] = *reinterpret_cast<const pk::u32x4*>(ksrc + c * 8);
        tv[i] = *reinterpret_cast<const pk::u32x4*>(tsrc + c * 8);
      }
    }
  };

  for (int k0 = 0; k0 <= max_pos; k0 += BK) {
    const int nk = min(BK, max_pos + 1 - k0);
    if (cache_t) {
      fetch(k0);
#pragma unroll
      for (int i = 0; i < NIT; ++i) {
        const int c = tid + NT * i;
        if (c < 4 * R) {
          const int key = c / R8, r8 = c - key * R8;
          *reinterpret_cast<pk::u32x4*>(cs + key * CS + r8 * 8) = kv[i];
          *reinterpret_cast<pk::u32x4*>(ct + (c >> 2) * CT + (c & 3) * 8) = tv[i];
        }
      }
    } else {  // no latent-major copy in the cache: transpose while staging
      for (int c = tid; c < BK * R8; c += NT) {
        const int key = c / R8, r8 = c - key * R8;
        pk::u32x4 v = {0u, 0u, 0u, 0u};
        if (key < nk) {
          const int kp = k0 + key;
          const int64_t slot = static_cast<int64_t>(bt[kp / block_size]) * block_size + kp % block_size;
          v = *reinterpret_cast<const pk::u32x4*>(cache + slot * R + r8 * 8);
        }
        *reinterpret_cast<pk::u32x4*>(cs + key * CS + r8 * 8) = v;
        bf16_t* dst = ct + (r8 * 8) * CT + key_slot(key);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          dst[(2 * e) * CT] = static_cast<bf16_t>(v[e] & 0xffffu);
          dst[(2 * e + 1) * CT] = static_cast<bf16_t>(v[e] >> 16);
        }
      }
    }
    __syncthreads();
    if (__any(my_pos >= k0)) {
      pk::f32x4 sa[2] = {pk::f32x4{0.f, 0.f, 0.f, 0.f}, pk::f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const bf16_t* kr = cs + (sub * 16 + n) * CS + 8 * g;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk)
          sa[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(kr + kk * 32), qf[kk], sa[sub], 0, 0, 0);
      }
      float sc[8];
      float tmax = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = k0 + (e >> 2) * 16 + 4 * g + (e & 3);
        sc[e] = key <= my_pos ? sa[e >> 2][e & 3] * scale2 : -INFINITY;
        tmax = fmaxf(tmax, sc[e]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = tmax > m_run + kLazyMax ? tmax : m_run;  // the reference moves only on a real jump
      float p[8], tsum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = sc[e] == -INFINITY ? 0.f : exp2f(sc[e] - m_new);
        tsum += p[e];
      }
      tsum += __shfl_xor(tsum, 16, 64);
      tsum += __shfl_xor(tsum, 32, 64);
      const float resc = m_run == -INFINITY ? (m_new == -INFINITY ? 1.f : 0.f) : exp2f(m_run - m_new);
      m_run = m_new;
      l_run = l_run * resc + tsum;
      pk::u32x4 pw;
#pragma unroll
      for (int e = 0; e < 4; ++e) pw[e] = pk::pack2(p[2 * e], p[2 * e + 1]);
      const pk::bf16x8_t pb = __builtin_bit_cast(pk::bf16x8_t, pw);
      if (__any(resc != 1.f)) {
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) o[rt] *= resc;
      }
      const bf16_t* vr = ct + n * CT + 8 * g;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt)
        o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(vr + rt * 16 * CT), pb, o[rt], 0, 0, 0);
    }
    __syncthreads();
  }
  if (valid) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    bf16_t* dst = out + static_cast<int64_t>(q0 + tl) * out_st + static_cast<int64_t>(h) * out_sh + 4 * g;
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      uint2 w;
      w.x = pk::pack2(o[rt][0] * inv, o[rt][1] * inv);
      w.y = pk::pack2(o[rt][2] * inv, o[rt][3] * inv);
      *reinterpret_cast<uint2*>(dst + rt * 16) = w;
    }
  }
}

// ---- the 512-wide latent: tiles staged by LDS-DMA into two buffers ------------------------------
// At R = 512 a wave's 16 rows hold 128 output accumulators and 64 registers of folded queries, so
// there is no room to keep the next tile in registers and only two waves fit a SIMD: the tile loads
// go straight to LDS instead (buffer_load ... lds, no VGPRs), tile t+1 into the other buffer while
// tile t's products run, one barrier per tile.  A wave instruction moves 1 KiB: exactly one
// key-major row (padded to 1040 B in LDS through the instruction's LDS base), or 16 rows of the
// latent-major copy, whose 16-byte parts are XOR-swizzled by the row on the GLOBAL side of the
// copy (lane l fetches part (l & 3) ^ part_swizzle(l >> 2) of row l >> 2) so that the unpadded
// 64-byte rows read conflict-free.  Needs the latent-major cache copy (pages of whole 32-key tiles).
// part_swizzle(r) = (r2, r3 ^ r1) as (low, high) bit: a fragment read takes 16 rows at one part,
// and the 16 rows' 16-byte parts then fall on 16 different 16-byte bank groups whether the LDS
// serves 8 lanes over 32 banks or 16 lanes over 64 banks per pass.
__device__ __forceinline__ int part_swizzle(int r) { return ((r >> 2) & 1) | ((((r >> 3) ^ (r >> 1)) & 1) << 1); }

__global__ void __launch_bounds__(kPromptThreads)
latent_attention_dma512_kernel(bf16_t* __restrict__ out, int64_t out_st, int64_t out_sh, const bf16_t* __restrict__ q,
                               int64_t q_st, int64_t q_sh, const bf16_t* __restrict__ cache,
                               const bf16_t* __restrict__ cache_t, const int* __restrict__ block_tables, int max_blocks,
                               const int* __restrict__ cu_q, const int* __restrict__ context_lens, int n_seqs, int H,
                               int block_size, float scale) {
  constexpr int R = 512, NT = kPromptThreads, BQ = NT / 4, BK = 32, NKK = R / 32, NRT = R / 16, CS = R + 8;
  constexpr int kCsBytes = BK * CS * 2, kCtBytes = R * BK * 2, kBuf = kCsBytes + kCtBytes;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  int s = 0, tile = blockIdx.x;
  for (; s < n_seqs; ++s) {
    const int nt = ((cu_q[s + 1] - cu_q[s]) * H + BQ - 1) / BQ;
    if (tile < nt) break;
    tile -= nt;
  }
  if (s >= n_seqs) return;
  const int q0 = cu_q[s], qlen = cu_q[s + 1] - q0, ctx = context_lens[s];
  const int n_rows = qlen * H, row0 = tile * BQ;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, n = lane & 15;
  const int wu = __builtin_amdgcn_readfirstlane(wave);
  const int* bt = block_tables + static_cast<int64_t>(s) * max_blocks;
  const int my_row = row0 + 16 * wave + n;
  const bool valid = my_row < n_rows;
  const int tl = valid ? my_row / H : 0, h = valid ? my_row - tl * H : 0;
  const int my_pos = valid ? ctx - qlen + tl : -1;
  const int max_pos = ctx - qlen + (min(row0 + BQ, n_rows) - 1) / H;

  pk::bf16x8_t qf[NKK];
  {
    const bf16_t* qr = q + static_cast<int64_t>(q0 + tl) * q_st + static_cast<int64_t>(h) * q_sh + 8 * g;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      pk::u32x4 v = {0u, 0u, 0u, 0u};
      if (valid) v = *reinterpret_cast<const pk::u32x4*>(qr + kk * 32);
      qf[kk] = __builtin_bit_cast(pk::bf16x8_t, v);
    }
  }
  pk::f32x4 o[NRT];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) o[rt] = pk::f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const float scale2 = scale * kLog2e;  // scores in log2 units: a weight is one exp2

  // lane offsets of the two copies: key-major rows are taken as they lie, latent-major parts swizzled
  const unsigned kvo = static_cast<unsigned>(lane) * 16u;
  const unsigned tvo = static_cast<unsigned>(((lane >> 2) * 4 + ((lane & 3) ^ part_swizzle(lane >> 2))) * 16);
  auto issue = [&](int k0, int buf) {  // this wave's 4 + 4 KiB of the tile at k0
    const int blk = __builtin_amdgcn_readfirstlane(bt[k0 / block_size]);
    const int kin = k0 % block_size;
    const bf16_t* ksrc = cache + (static_cast<int64_t>(blk) * block_size + kin) * R;
    const bf16_t* tsrc = cache_t + (static_cast<int64_t>(blk) * (block_size / 32) + kin / 32) * R * 32;
    const auto krs = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(ksrc), static_cast<short>(0), kCtBytes, 0x00020000);
    const auto trs = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(tsrc), static_cast<short>(0), kCtBytes, 0x00020000);
    unsigned char* base = smem_raw + buf * kBuf;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = wu * 4 + j;  // key row / 16-row block of the latent-major copy
      __builtin_amdgcn_raw_ptr_buffer_load_lds(krs, (__attribute__((address_space(3))) void*)(base + row * (CS * 2)), 16, kvo,
                                               static_cast<unsigned>(row) * 1024u, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(trs, (__attribute__((address_space(3))) void*)(base + kCsBytes + row * 1024),
                                               16, tvo, static_cast<unsigned>(row) * 1024u, 0, 0);
    }
  };
  if (max_pos >= 0) issue(0, 0);
  int buf = 0;
  for (int k0 = 0; k0 <= max_pos; k0 += BK, buf ^= 1) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // tile k0 has landed for every wave, and nobody still reads the other buffer
    if (k0 + BK <= max_pos) issue(k0 + BK, buf ^ 1);
    if (__any(my_pos >= k0)) {
      const bf16_t* cs = reinterpret_cast<const bf16_t*>(smem_raw + buf * kBuf);
      const bf16_t* ct = reinterpret_cast<const bf16_t*>(smem_raw + buf * kBuf + kCsBytes);
      pk::f32x4 sa[2] = {pk::f32x4{0.f, 0.f, 0.f, 0.f}, pk::f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const bf16_t* kr = cs + (sub * 16 + n) * CS + 8 * g;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk)
          sa[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(kr + kk * 32), qf[kk], sa[sub], 0, 0, 0);
      }
      float sc[8];
      float tmax = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = k0 + (e >> 2) * 16 + 4 * g + (e & 3);
        sc[e] = key <= my_pos ? sa[e >> 2][e & 3] * scale2 : -INFINITY;
        tmax = fmaxf(tmax, sc[e]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = tmax > m_run + kLazyMax ? tmax : m_run;  // the reference moves only on a real jump
      float p[8], tsum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = sc[e] == -INFINITY ? 0.f : exp2f(sc[e] - m_new);
        tsum += p[e];
      }
      tsum += __shfl_xor(tsum, 16, 64);
      tsum += __shfl_xor(tsum, 32, 64);
      const float resc = m_run == -INFINITY ? (m_new == -INFINITY ? 1.f : 0.f) : exp2f(m_run - m_new);
      m_run = m_new;
      l_run = l_run * resc + tsum;
      pk::u32x4 pw;
#pragma unroll
      for (int e = 0; e < 4; ++e) pw[e] = pk::pack2(p[2 * e], p[2 * e + 1]);
      const pk::bf16x8_t pb = __builtin_bit_cast(pk::bf16x8_t, pw);
      if (__any(resc != 1.f)) {
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) o[rt] *= resc;
      }
      // row rt*16 + n of the latent-major tile, part g, at its swizzled place
      const bf16_t* vr = ct + (n * 4 + (g ^ part_swizzle(n))) * 8;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt)
        o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(vr + rt * 16 * 32), pb, o[rt], 0, 0, 0);
    }
  }
  if (valid) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    bf16_t* dst = out + static_cast<int64_t>(q0 + tl) * out_st + static_cast<int64_t>(h) * out_sh + 4 * g;
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      uint2 w;
      w.x = pk::pack2(o[rt][0] * inv, o[rt][1] * inv);
      w.y = pk::pack2(o[rt][2] * inv, o[rt][3] * inv);
      *reinterpret_cast<uint2*>(dst + rt * 16) = w;
    }
  }
}

static int g_latent_dma = 1;  // 0: the 512-wide latent takes the register-staged kernel too (tests)
PK_EXPORT int pkm_set_latent_dma(int on) {
  g_latent_dma = on;
  return 0;
}

static int launch_latent_dma512(void* out, long long out_st, long long out_sh, const void* q, long long q_st,
                                long long q_sh, const void* cache, const void* cache_t, const void* block_tables,
                                int max_blocks, const void* cu_q, const void* context_lens, int n_seqs, int T, int H,
                                int block_size, float scale, hipStream_t stream) {
  constexpr int lds = 2 * (32 * 520 * 2 + 512 * 32 * 2);
  static bool attr_set = false;
  if (!attr_set) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(latent_attention_dma512_kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return static_cast<int>(e);
    attr_set = true;
  }
  constexpr int BQ = kPromptThreads / 4;
  const int grid = static_cast<int>((static_cast<int64_t>(T) * H + BQ - 1) / BQ + n_seqs);
  latent_attention_dma512_kernel<<<grid, kPromptThreads, lds, stream>>>(
      static_cast<bf16_t*>(out), out_st, out_sh, static_cast<const bf16_t*>(q), q_st, q_sh,
      static_cast<const bf16_t*>(cache), static_cast<const bf16_t*>(cache_t), static_cast<const int*>(block_tables),
      max_blocks, static_cast<const int*>(cu_q), static_cast<const int*>(context_lens), n_seqs, H, block_size, scale);
  return PK_CHECK_LAUNCH();
}

// ---- decoding on the matrix cores -----------------------------------------------------------------
// One query token per sequence: its H heads are the 16-row tiles.  Every wave owns a run of `part`
// keys (a multiple of 32) and takes both products' A operands straight from the cache -- key-major
// rows for S^T, the latent-major copy for O~^T -- so nothing is staged and no barrier is needed; it
// leaves (max, sum, unnormalised o~) per head in the workspace and latent_merge_kernel combines the
// runs.  `part` comes from the cache capacity, not from the batch: a position's sums are the same
// in every step.
template <int R>
__global__ void __launch_bounds__(256)
latent_decode_mfma_kernel(float* __restrict__ ws_o, float* __restrict__ ws_ml, const bf16_t* __restrict__ q,
                          int64_t q_st, int64_t q_sh, const bf16_t* __restrict__ cache,
                          const bf16_t* __restrict__ cache_t, const int* __restrict__ block_tables, int max_blocks,
                          const int* __restrict__ cu_q, const int* __restrict__ context_lens, int H, int block_size,
                          int part, int n_parts, float scale) {
  constexpr int NKK = R / 32, NRT = R / 16;
  const int s = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, n = lane & 15;
  const int wp = blockIdx.y * 4 + wave;
  const int ctx = context_lens[s], tok = cu_q[s];
  const int k_lo = wp * part, k_hi = min(k_lo + part, ctx);
  const int* bt = block_tables + static_cast<int64_t>(s) * max_blocks;
  for (int h0 = 0; h0 < H; h0 += 16) {
    const int h = h0 + n;
    const bool valid = h < H;
    const int64_t wrow = (static_cast<int64_t>(s) * n_parts + wp) * H + h;
    if (k_lo >= k_hi) {  // an empty run
      if (valid && g == 0) {
        ws_ml[wrow * 2] = -INFINITY;
        ws_ml[wrow * 2 + 1] = 0.f;
      }
      continue;
    }
    pk::bf16x8_t qf[NKK];
    {
      const bf16_t* qr = q + static_cast<int64_t>(tok) * q_st + static_cast<int64_t>(valid ? h : 0) * q_sh + 8 * g;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        pk::u32x4 v = {0u, 0u, 0u, 0u};
        if (valid) v = *reinterpret_cast<const pk::u32x4*>(qr + kk * 32);
        qf[kk] = __builtin_bit_cast(pk::bf16x8_t, v);
      }
    }
    pk::f32x4 o[NRT];
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) o[rt] = pk::f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
  const float scale2 = scale * kLog2e;  // scores in log2 units: a weight is one exp2
    for (int k0 = k_lo; k0 < k_hi; k0 += 32) {
      pk::f32x4 sa[2] = {pk::f32x4{0.f, 0.f, 0.f, 0.f}, pk::f32x4{0.f, 0.f, 0.f, 0.f}};
      const int blk = bt[k0 / block_size];
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const int kp = k0 + sub * 16 + n;  // this lane's key row; past the context: any cached row, masked below
        const bf16_t* kr = cache + (static_cast<int64_t>(blk) * block_size + kp % block_size) * R + 8 * g;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk)
          sa[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(kr + kk * 32), qf[kk], sa[sub], 0, 0, 0);
      }
      float sc[8], tmax = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = k0 + (e >> 2) * 16 + 4 * g + (e & 3);
        sc[e] = key < k_hi ? sa[e >> 2][e & 3] * scale2 : -INFINITY;
        tmax = fmaxf(tmax, sc[e]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = tmax > m_run + kLazyMax ? tmax : m_run;  // the reference moves only on a real jump
      float p[8], tsum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = sc[e] == -INFINITY ? 0.f : exp2f(sc[e] - m_new);
        tsum += p[e];
      }
      tsum += __shfl_xor(tsum, 16, 64);
      tsum += __shfl_xor(tsum, 32, 64);
      const float resc = m_run == -INFINITY ? 0.f : exp2f(m_run - m_new);
      m_run = m_new;
      l_run = l_run * resc + tsum;
      pk::u32x4 pw;
#pragma unroll
      for (int e = 0; e < 4; ++e) pw[e] = pk::pack2(p[2 * e], p[2 * e + 1]);
      const pk::bf16x8_t pb = __builtin_bit_cast(pk::bf16x8_t, pw);
      if (__any(resc != 1.f)) {
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) o[rt] *= resc;
      }
      const bf16_t* vr = cache_t + ((static_cast<int64_t>(blk) * (block_size / 32) + (k0 % block_size) / 32) * R + n) * 32 + 8 * g;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt)
        o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(vr + rt * 16 * 32), pb, o[rt], 0, 0, 0);
    }
    if (valid) {
      if (g == 0) {
        ws_ml[wrow * 2] = m_run;
        ws_ml[wrow * 2 + 1] = l_run;
      }
      float* dst = ws_o + wrow * R + 4 * g;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) *reinterpret_cast<pk::f32x4*>(dst + rt * 16) = o[rt];
    }
  }
}

// out[token s, head h] = sum_p e^(m_p - M) o_p / sum_p e^(m_p - M) l_p over the n_parts (<= 64) runs:
// the first wave turns the runs' (max, sum) into weights, then every thread sums its coordinates
__global__ void __launch_bounds__(128)
latent_merge_kernel(bf16_t* __restrict__ out, int64_t out_st, int64_t out_sh, const float* __restrict__ ws_o,
                    const float* __restrict__ ws_ml, const int* __restrict__ cu_q, int H, int R, int n_parts) {
  __shared__ float wgt[64];
  const int s = blockIdx.x, h = blockIdx.y;
  const int64_t base = static_cast<int64_t>(s) * n_parts * H + h;
  if (threadIdx.x < 64) {
    const int p = threadIdx.x;
    const bool in = p < n_parts;
    const float m = in ? ws_ml[(base + static_cast<int64_t>(p) * H) * 2] : -INFINITY;
    const float l = in ? ws_ml[(base + static_cast<int64_t>(p) * H) * 2 + 1] : 0.f;
    const float M = pk::wave_max(m);
    const float w = m == -INFINITY ? 0.f : exp2f(m - M);  // the runs' maxima are in log2 units
    const float L = pk::wave_sum(w * l);
    wgt[p] = L > 0.f ? w / L : 0.f;
  }
  __syncthreads();
  bf16_t* dst = out + static_cast<int64_t>(cu_q[s]) * out_st + static_cast<int64_t>(h) * out_sh;
  // four coordinates per thread; the runs' loads are independent of each other (an empty run's
  // slab was never written: its value is discarded, not multiplied)
  for (int r = 4 * threadIdx.x; r < R; r += 4 * blockDim.x) {
    pk::f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int p = 0; p < n_parts; ++p) {
      const pk::f32x4 v = *reinterpret_cast<const pk::f32x4*>(ws_o + (base + static_cast<int64_t>(p) * H) * R + r);
      const float w = wgt[p];
#pragma unroll
      for (int e = 0; e < 4; ++e) a[e] += w != 0.f ? w * v[e] : 0.f;
    }
    uint2 o2;
    o2.x = pk::pack2(a[0], a[1]);
    o2.y = pk::pack2(a[2], a[3]);
    *reinterpret_cast<uint2*>(dst + r) = o2;
  }
}

template <int R>
static int launch_latent_decode(void* out, long long out_st, long long out_sh, const void* q, long long q_st,
                                long long q_sh, const void* cache, const void* cache_t, const void* block_tables,
                                int max_blocks, const void* cu_q, const void* context_lens, int n_seqs, int H,
                                int block_size, float scale, void* ws_o, void* ws_ml, int part, int n_parts,
                                hipStream_t stream) {
  latent_decode_mfma_kernel<R><<<dim3(n_seqs, n_parts / 4), 256, 0, stream>>>(
      static_cast<float*>(ws_o), static_cast<float*>(ws_ml), static_cast<const bf16_t*>(q), q_st, q_sh,
      static_cast<const bf16_t*>(cache), static_cast<const bf16_t*>(cache_t), static_cast<const int*>(block_tables),
      max_blocks, static_cast<const int*>(cu_q), static_cast<const int*>(context_lens), H, block_size, part, n_parts,
      scale);
  latent_merge_kernel<<<dim3(n_seqs, H), 128, 0, stream>>>(static_cast<bf16_t*>(out), out_st, out_sh,
                                                           static_cast<const float*>(ws_o),
                                                           static_cast<const float*>(ws_ml),
                                                           static_cast<const int*>(cu_q), H, R, n_parts);
  return PK_CHECK_LAUNCH();
}

template <int R>
static int launch_latent_mfma(void* out, long long out_st, long long out_sh, const void* q, long long q_st,
                              long long q_sh, const void* cache, const void* cache_t, const void* block_tables,
                              int max_blocks, const void* cu_q, const void* context_lens, int n_seqs, int T, int H,
                              int block_size, float scale, hipStream_t stream) {
  constexpr size_t lds = (32 * (R + 8) + R * 40) * sizeof(bf16_t);
  auto kern = latent_attention_mfma_kernel<R>;
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  constexpr int BQ = kPromptThreads / 4;
  const int grid = static_cast<int>((static_cast<int64_t>(T) * H + BQ - 1) / BQ + n_seqs);
  kern<<<grid, kPromptThreads, lds, stream>>>(static_cast<bf16_t*>(out), out_st, out_sh, static_cast<const bf16_t*>(q), q_st, q_sh,
                                   static_cast<const bf16_t*>(cache), static_cast<const bf16_t*>(cache_t),
                                   static_cast<const int*>(block_tables), max_blocks, static_cast<const int*>(cu_q),
                                   static_cast<const int*>(context_lens), n_seqs, H, block_size, scale);
  return PK_CHECK_LAUNCH();
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

PK_EXPORT int pkm_latent_norm_cache(void* cache, void* cache_t, int block_size, const void* dkv, long long dkv_stride,
                                    const void* w, const void* slot_mapping, int T, int R, float eps, int dt,
                                    hipStream_t stream) {
  if (T <= 0) return 0;
  if (cache_t && (block_size <= 0 || block_size % 32)) return -1;
  PKM_DISPATCH(dt, E, latent_norm_cache_kernel<E><<<T, 128, 0, stream>>>(
                          static_cast<E*>(cache), static_cast<E*>(cache_t), block_size, static_cast<const E*>(dkv),
                          dkv_stride, static_cast<const float*>(w), static_cast<const int*>(slot_mapping), R, eps));
  return PK_CHECK_LAUNCH();
}

// 0: every launch takes the fp32-FMA kernel (tests compare the two)
static int g_latent_mfma = 1;
PK_EXPORT int pkm_set_latent_mfma(int on) {
  g_latent_mfma = on;
  return 0;
}

// key tile size for a latent of R numbers: the largest of 64 / 32 / 16 / 8 whose tiles fit 96 KiB of LDS
static int latent_key_tile(int R) {
  for (int bk = 64; bk >= 8; bk >>= 1) {
    const size_t bytes = (static_cast<size_t>(kBQ + bk) * (R + 1) + kBQ * bk + 3 * kBQ) * sizeof(float);
    if (bytes <= 96 * 1024) return bk;
  }
  return 0;
}

// latents the matrix-core kernels are built for
PK_EXPORT int pkm_latent_mfma_rank(int R) {
  switch (R) {
    case 32: case 64: case 96: case 128: case 160: case 192: case 256: case 320: case 384: case 512:
      return 1;
    default:
      return 0;
  }
}

// Decoding: sequences 0..n_seqs-1 with ONE query token each (token cu_q[s]); bf16, a latent of
// pkm_latent_mfma_rank, the latent-major cache copy.  ws_o [n_seqs, n_parts, H, R] and ws_ml
// [n_seqs, n_parts, H, 2] fp32; `part` keys per run (multiple of 32), n_parts a multiple of 4 with
// part * n_parts >= the longest context.
PK_EXPORT int pkm_latent_decode(void* out, long long out_st, long long out_sh, const void* q, long long q_st,
                                long long q_sh, const void* cache, const void* cache_t, const void* block_tables,
                                int max_blocks, const void* cu_q, const void* context_lens, int n_seqs, int H, int R,
                                int block_size, float scale, void* ws_o, void* ws_ml, int part, int n_parts,
                                hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (!cache_t || part <= 0 || part % 32 || n_parts <= 0 || n_parts % 4 || n_parts > 64 || block_size % 32 || q_st % 8 || q_sh % 8 ||
      reinterpret_cast<uintptr_t>(q) % 16 || reinterpret_cast<uintptr_t>(cache) % 16 ||
      reinterpret_cast<uintptr_t>(cache_t) % 16)
    return -1;
#define PKM_LD(RR)                                                                                                  \
  case RR:                                                                                                          \
    return launch_latent_decode<RR>(out, out_st, out_sh, q, q_st, q_sh, cache, cache_t, block_tables, max_blocks,   \
                                    cu_q, context_lens, n_seqs, H, block_size, scale, ws_o, ws_ml, part, n_parts,   \
                                    stream);
  switch (R) {
    PKM_LD(32) PKM_LD(64) PKM_LD(96) PKM_LD(128) PKM_LD(160) PKM_LD(192) PKM_LD(256) PKM_LD(320) PKM_LD(384) PKM_LD(512)
    default:
      return -1;
  }
#undef PKM_LD
}

PK_EXPORT int pkm_latent_attention(void* out, long long out_st, long long out_sh, const void* q, long long q_st,
                                   long long q_sh, const void* cache, const void* cache_t, const void* block_tables,
                                   int max_blocks, const void* cu_q, const void* context_lens, int n_seqs, int T, int H,
                                   int R, int block_size, float scale, int dt, hipStream_t stream) {
  if (T <= 0 || n_seqs <= 0) return 0;
  if (cache_t && block_size % 32) return -1;
  // bf16 with a latent the MFMA kernel is built for and 8-byte-aligned rows: the matrix cores
  if (dt == kBF16 && g_latent_mfma && q_st % 8 == 0 && q_sh % 8 == 0 && out_st % 4 == 0 && out_sh % 4 == 0 &&
      reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(cache) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 8 == 0) {
    if (R == 512 && cache_t && g_latent_dma)
      return launch_latent_dma512(out, out_st, out_sh, q, q_st, q_sh, cache, cache_t, block_tables, max_blocks, cu_q,
                                  context_lens, n_seqs, T, H, block_size, scale, stream);
#define PKM_LM(RR)                                                                                                 \
  case RR:                                                                                                         \
    return launch_latent_mfma<RR>(out, out_st, out_sh, q, q_st, q_sh, cache, cache_t, block_tables, max_blocks,    \
                                  cu_q, context_lens, n_seqs, T, H, block_size, scale, stream);
    switch (R) {
      PKM_LM(32) PKM_LM(64) PKM_LM(96) PKM_LM(128) PKM_LM(160) PKM_LM(192) PKM_LM(256) PKM_LM(320) PKM_LM(384) PKM_LM(512)
      default:
        break;
    }
#undef PKM_LM
  }
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
