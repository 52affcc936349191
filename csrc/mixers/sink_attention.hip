// Grouped-query attention over a paged cache with rotated unit-RMS queries / keys, position-rotated
// values, capped scores and a softmax sink.
//
//   rope_norm_cache   q, k: pairs (2i, 2i+1) of the first 2 * qk_pairs coordinates turn by the token's
//                     position (fp32 (cos, sin) table rows), then each head is divided by its RMS over D;
//                     v: every pair of its V coordinates turns by the position (its own table).
//                     q -> [T, H, D]; k -> cache [blocks, G, block_size, D]; v -> cache
//                     [blocks, G, V, block_size] (transposed per page)
//   sink_attention    score = q . k * head_scale[h], then cap * tanh(score / cap) if cap > 0;
//                     p_j = exp(score_j) / (sink + sum_j' exp(score_j')) over the keys j <= the token;
//                     o = sum_j p_j v_j, turned back by the token's position (values were cached turned
//                     by theirs).  Scores, softmax and the value sum are fp32 for both element types.
//
// The (token, head) pairs of a sequence that share a KV head are the rows of one tile problem
// against key / value tiles staged once in LDS.  Key tiles of a prompt row always start at key 0 of
// the sequence; a decoded token's keys are cut into runs whose length comes from the cache
// capacity, merged by a second kernel -- so a position's sums do not depend on how its prompt was
// cut or on what else the step holds.
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kMaxPairs = 4;  // pairs per lane of a 64-lane wave: heads of up to 512 coordinates

// IN: element type of the projection output; with nslab > 1 (IN = float) it is the decode GEMM's
// split-K slabs [nslab][T][stride], summed on the way in
template <typename T, typename IN>
__global__ void __launch_bounds__(64)
rope_norm_cache_kernel(T* __restrict__ q_out, const IN* __restrict__ qkv, int64_t stride, int nslab, int64_t slab_stride,
                       const int* __restrict__ positions,
                       const int* __restrict__ slot_mapping, const float* __restrict__ qk_table, int qk_pairs,
                       const float* __restrict__ v_table, int table_rows, T* __restrict__ k_cache,
                       T* __restrict__ v_cache, int H, int G, int D, int V, int bs, float eps) {
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  int pos = positions[t];
  pos = pos < 0 ? 0 : (pos >= table_rows ? max(table_rows - 1, 0) : pos);
  const int slot = slot_mapping[t];
  const IN* row = qkv + static_cast<int64_t>(t) * stride;
  auto get = [&](const IN* p) {
    float v = ld<IN>(p);
    for (int sl = 1; sl < nslab; ++sl) v += ld<IN>(p + sl * slab_stride);
    return v;
  };
  if (item < H + G) {
    const IN* src = row + static_cast<int64_t>(item) * D;
    const float* cs = qk_table ? qk_table + static_cast<int64_t>(pos) * qk_pairs * 2 : nullptr;
    float u[kMaxPairs], v[kMaxPairs];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxPairs; ++i) {
      const int p = lane + 64 * i;
      u[i] = v[i] = 0.f;
      if (2 * p < D) {
        float a = get(src + 2 * p);
        float b = 2 * p + 1 < D ? get(src + 2 * p + 1) : 0.f;
        if (cs && p < qk_pairs) {
          const float c = cs[2 * p], s = cs[2 * p + 1];
          const float na = a * c - b * s;
          b = b * c + a * s;
          a = na;
        }
        u[i] = a;
        v[i] = b;
        ss += a * a + b * b;
      }
    }
    ss = pk::wave_sum(ss);
    const float k = 1.f / sqrtf(ss / static_cast<float>(D) + eps);
    T* dst;
    if (item < H) {
      dst = q_out + (static_cast<int64_t>(t) * H + item) * D;
    } else {
      if (slot < 0) return;
      dst = k_cache + ((static_cast<int64_t>(slot / bs) * G + (item - H)) * bs + slot % bs) * D;
    }
#pragma unroll
    for (int i = 0; i < kMaxPairs; ++i) {
      const int p = lane + 64 * i;
      if (2 * p < D) st<T>(dst + 2 * p, u[i] * k);
      if (2 * p + 1 < D) st<T>(dst + 2 * p + 1, v[i] * k);
    }
  } else {
    if (slot < 0) return;
    const int g = item - H - G;
    const IN* src = row + static_cast<int64_t>(H + G) * D + static_cast<int64_t>(g) * V;
    const float* cs = v_table ? v_table + static_cast<int64_t>(pos) * (V / 2) * 2 : nullptr;
    T* dst = v_cache + (static_cast<int64_t>(slot / bs) * G + g) * V * bs + slot % bs;
    for (int p = lane; 2 * p < V; p += 64) {
      float a = get(src + 2 * p);
      float b = 2 * p + 1 < V ? get(src + 2 * p + 1) : 0.f;
      if (cs && 2 * p + 1 < V) {
        const float c = cs[2 * p], s = cs[2 * p + 1];
        const float na = a * c - b * s;
        b = b * c + a * s;
        a = na;
      }
      st<T>(dst + static_cast<int64_t>(2 * p) * bs, a);
      if (2 * p + 1 < V) st<T>(dst + static_cast<int64_t>(2 * p + 1) * bs, b);
    }
  }
}

constexpr int kBQ = 16;        // (token, head) rows per workgroup
constexpr int kThreads = 256;  // 16 rows x 16 lanes

struct SinkArgs {
  void* out;           // [T, H * V]
  const void* q;       // [T, H, D]
  const void* k_cache;
  const void* v_cache;
  const int* block_tables;
  int64_t bt_stride;
  const int* cu_q;
  const int* context_lens;
  const int* positions;
  const float* head_scale;
  const float* v_table;
  int table_rows;
  int n_seqs, H, G, D, V, bs, BK;
  float softcap, sink;
  // decoded tokens: keys cut into n_parts runs of `part` keys, partial sums in the workspace
  int part, n_parts;
  float* ws_o;   // [n_seqs, n_parts, H, V]
  float* ws_ml;  // [n_seqs, n_parts, H, 2]
};

// NV: output accumulators per thread = ceil(V / 16).  SPLIT: one query token per sequence, this
// workgroup covers keys [part * blockIdx.z, ...) and leaves (max, sum, unnormalised o) behind.
template <typename T, int NV, bool SPLIT>
__global__ void __launch_bounds__(kThreads) sink_attention_kernel(SinkArgs a) {
  extern __shared__ float smem[];
  const int H = a.H, G = a.G, D = a.D, V = a.V, BK = a.BK, bs = a.bs;
  const int R = H / G;  // query heads per KV head
  const int g = blockIdx.y;
  int s = 0, tile = blockIdx.x;
  if (SPLIT) {
    const int ntile = (R + kBQ - 1) / kBQ;
    s = blockIdx.x / ntile;
    tile = blockIdx.x - s * ntile;
  } else {
    for (; s < a.n_seqs; ++s) {
      const int rows = (a.cu_q[s + 1] - a.cu_q[s]) * R;
      const int nt = (rows + kBQ - 1) / kBQ;
      if (tile < nt) break;
      tile -= nt;
    }
    if (s >= a.n_seqs) return;
  }
  const int q0 = a.cu_q[s], qlen = a.cu_q[s + 1] - q0, ctx = a.context_lens[s];
  const int n_rows = qlen * R;
  const int row0 = tile * kBQ;
  const int DS = D + 1, VS = V + 1;  // odd row strides: conflict-free column walks
  float* qs = smem;                  // [kBQ][DS]
  float* ks = qs + kBQ * DS;         // [BK][DS]
  float* vs = ks + BK * DS;          // [BK][VS]
  float* ps = vs + BK * VS;          // [kBQ][BK]
  float* m_s = ps + kBQ * BK;        // [kBQ] running max
  float* l_s = m_s + kBQ;            // [kBQ] running sum
  const int tid = threadIdx.x;
  const int qi = tid >> 4, kg = tid & 15;
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_stride;
  const T* q = static_cast<const T*>(a.q);
  const T* kc = static_cast<const T*>(a.k_cache);
  const T* vc = static_cast<const T*>(a.v_cache);

  for (int e = tid; e < kBQ * D; e += kThreads) {
    const int r = e / D, c = e - r * D;
    const int row = row0 + r;
    float v = 0.f;
    if (row < n_rows) {
      const int tl = row / R, h = g * R + row - tl * R;
      v = ld<T>(q + (static_cast<int64_t>(q0 + tl) * H + h) * D + c);
    }
    qs[r * DS + c] = v;
  }
  const bool with_sink = !SPLIT && a.sink > 0.f;
  if (tid < kBQ) {
    m_s[tid] = with_sink ? 0.f : -INFINITY;  // the sink is a key of score 0 without a value
    l_s[tid] = with_sink ? a.sink : 0.f;
  }
  const int my_row = row0 + qi;
  const bool live = my_row < n_rows;
  const int my_tl = live ? my_row / R : 0;
  const int my_h = g * R + (live ? my_row - my_tl * R : 0);
  const int my_pos = live ? ctx - qlen + my_tl : -1;
  const float hs = a.head_scale[my_h];
  const int last_row = min(row0 + kBQ, n_rows) - 1;
  int k_begin = 0, k_end = ctx - qlen + last_row / R + 1;  // keys [k_begin, k_end) are visible to some row
  if (SPLIT) {
    k_begin = blockIdx.z * a.part;
    k_end = min(k_end, k_begin + a.part);
  }
  float acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = 0.f;
  __syncthreads();

  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
    const int nk = min(BK, k_end - k0);
    for (int e = tid; e < BK * D; e += kThreads) {
      const int j = e / D, c = e - j * D;
      float v = 0.f;
      if (j < nk) {
        const int key = k0 + j;
        v = ld<T>(kc + ((static_cast<int64_t>(bt[key / bs]) * G + g) * bs + key % bs) * D + c);
      }
      ks[j * DS + c] = v;
    }
    for (int e = tid; e < BK * V; e += kThreads) {
      const int c = e / BK, j = e - c * BK;
      float v = 0.f;
      if (j < nk) {
        const int key = k0 + j;
        v = ld<T>(vc + ((static_cast<int64_t>(bt[key / bs]) * G + g) * V + c) * bs + key % bs);
      }
      vs[j * VS + c] = v;
    }
    __syncthreads();
    float tmax = -INFINITY;
    for (int j = kg; j < BK; j += 16) {
      float d = 0.f;
      const float* qr = qs + qi * DS;
      const float* kr = ks + j * DS;
      for (int c = 0; c < D; ++c) d += qr[c] * kr[c];
      d *= hs;
      if (a.softcap > 0.f) d = a.softcap * tanhf(d / a.softcap);
      d = (j < nk && k0 + j <= my_pos) ? d : -INFINITY;
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
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] *= resc;
    for (int j = 0; j < nk; ++j) {
      const float p = ps[qi * BK + j];
      const float* vr = vs + j * VS + kg;
#pragma unroll
      for (int i = 0; i < NV; ++i)
        if (kg + 16 * i < V) acc[i] += p * vr[16 * i];
    }
    __syncthreads();
  }
  if (SPLIT) {
    if (live) {
      const int64_t at = (static_cast<int64_t>(s) * a.n_parts + blockIdx.z) * H + my_h;
#pragma unroll
      for (int i = 0; i < NV; ++i)
        if (kg + 16 * i < V) a.ws_o[at * V + kg + 16 * i] = acc[i];
      if (kg == 0) {
        a.ws_ml[at * 2] = m_s[qi];
        a.ws_ml[at * 2 + 1] = l_s[qi];
      }
    }
    return;
  }
  const float l = l_s[qi];
  const float inv = l > 0.f ? 1.f / l : 0.f;
  int pos = a.positions[q0 + my_tl];
  pos = pos < 0 ? 0 : (pos >= a.table_rows ? max(a.table_rows - 1, 0) : pos);
  const float* cs = a.v_table ? a.v_table + static_cast<int64_t>(pos) * (V / 2) * 2 : nullptr;
  T* dst = static_cast<T*>(a.out) + (static_cast<int64_t>(q0 + my_tl) * H + my_h) * V;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = kg + 16 * i;
    float o = acc[i] * inv;
    const float other = __shfl_xor(o, 1, 64);  // the pair's second coordinate lives in the next lane
    if (cs && c < V) {
      const float co = cs[(c >> 1) * 2], si = cs[(c >> 1) * 2 + 1];
      o = (c & 1) ? o * co - other * si : o * co + other * si;  // turned back: angle -position
    }
    if (live && c < V) st<T>(dst + c, o);
  }
}

// out[token of sequence s, head h] from the runs' (max, sum, o): one workgroup per (sequence, head).
// The first wave turns the (at most 64) runs' maxima and sums into one weight per run, then every
// thread sums its coordinate pair over the runs and turns it back by the token's position.
template <typename T>
__global__ void __launch_bounds__(128)
sink_merge_kernel(T* __restrict__ out, const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                  const int* __restrict__ cu_q, const int* __restrict__ positions, const float* __restrict__ v_table,
                  int table_rows, int n_parts, int H, int V, float sink) {
  __shared__ float wgt[64];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tok = cu_q[s];
  if (threadIdx.x < 64) {
    const int p = threadIdx.x;
    const int64_t at = (static_cast<int64_t>(s) * n_parts + p) * H + h;
    const float m = p < n_parts ? ws_ml[at * 2] : -INFINITY;
    const float l = p < n_parts ? ws_ml[at * 2 + 1] : 0.f;
    float M = fmaxf(m, sink > 0.f ? 0.f : -INFINITY);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
    const float w = m == -INFINITY ? 0.f : expf(m - M);
    float L = w * l;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) L += __shfl_xor(L, o, 64);
    if (sink > 0.f) L += sink * expf(-M);
    wgt[p] = L > 0.f ? w / L : 0.f;
  }
  __syncthreads();
  int pos = positions[tok];
  pos = pos < 0 ? 0 : (pos >= table_rows ? max(table_rows - 1, 0) : pos);
  const float* cs = v_table ? v_table + static_cast<int64_t>(pos) * (V / 2) * 2 : nullptr;
  T* dst = out + (static_cast<int64_t>(tok) * H + h) * V;
  const float* base = ws_o + (static_cast<int64_t>(s) * n_parts * H + h) * V;
  for (int pr = threadIdx.x; 2 * pr < V; pr += blockDim.x) {
    float u = 0.f, v = 0.f;
    const bool two = 2 * pr + 1 < V;
    for (int p = 0; p < n_parts; ++p) {
      const float w = wgt[p];
      const float* row = base + static_cast<int64_t>(p) * H * V + 2 * pr;
      u += w * row[0];
      if (two) v += w * row[1];
    }
    if (cs && two) {
      const float co = cs[2 * pr], si = cs[2 * pr + 1];
      const float nu = u * co + v * si;
      v = v * co - u * si;
      u = nu;
    }
    st<T>(dst + 2 * pr, u);
    if (two) st<T>(dst + 2 * pr + 1, v);
  }
}

// ---- bf16 on the matrix cores -------------------------------------------------------------------
// Prompt portions: 128 (token, head) rows of one KV head per workgroup, 16 per wave, against 32-key
// tiles (two staged per barrier pair); a tile is one contiguous run of the key cache and one of the transposed value cache (pages
// hold whole 32-key tiles).  Both products run transposed on mfma_f32_16x16x32_bf16 so that the
// softmax weights never leave their registers:
//
//   S^T [keys x rows] = K [keys x D] . Q^T      A = key rows from LDS, B = the wave's Q (registers)
//   O^T [V x rows]   += V^T [V x keys] . P^T    A = value rows from LDS, B = P^T from the S^T accumulators
//
// An accumulator lane (g4, n) holds query row n and keys 4 g4 .. 4 g4 + 3 of each 16-key half; the B
// operand of the second product wants 8 key slots per lane, so slot (g4, e) is key 4 g4 + e of the
// first half for e < 4 and key 16 + 4 g4 + e - 4 of the second: the value tile is written to LDS in
// that slot order.  Scores are kept in log2 units; the running reference starts at 0 with the sink's
// weight in the sum and moves only when a tile's maximum exceeds it by 2^10 (any reference gives the
// same quotient).  The output lane holds coordinate pairs (4 g4, 4 g4 + 1), (4 g4 + 2, 4 g4 + 3) of
// each 16-wide block, so the turn back by the token's position is lane-local.
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLazyMax = 10.f;
constexpr int kPromptThreads = 512;

__host__ __device__ __forceinline__ int key_slot(int k) { return ((k & 15) >> 2) * 8 + (k & 3) + 4 * (k >> 4); }

// the capped score in log2 units: cap * tanh(raw * hs / cap) * log2(e).  `small` (uniform over the
// wave: every argument of this tile is below 0.06) takes tanh's series x - x^3/3 + 2x^5/15, whose
// first dropped term is below fp32 rounding there; otherwise tanh(x) = 1 - 2 / (2^(2 x log2 e) + 1)
// on the hardware's exp2 and reciprocal (two transcendental instructions per score).
__device__ __forceinline__ float capped(float raw, float hs, float cap, float inv_cap, bool small) {
  const float s = raw * hs;
  if (cap <= 0.f) return s * kLog2e;
  const float x = s * inv_cap;
  if (small) {
    const float x2 = x * x;
    return (cap * kLog2e) * (x + x * x2 * (-1.f / 3.f + x2 * (2.f / 15.f)));
  }
  const float e = exp2f(x * (2.f * kLog2e));
  return (cap * kLog2e) * (1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f));
}

// whether every lane's largest |raw * hs / cap| of a tile stays below the series' range
__device__ __forceinline__ bool small_args(const pk::f32x4* sa, float hs, float inv_cap) {
  float m = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) m = fmaxf(m, fabsf(sa[e >> 2][e & 3]));
  return __all(m * fabsf(hs) * inv_cap < 0.06f);
}

template <int D, int V>
__global__ void __launch_bounds__(kPromptThreads) sink_attention_mfma_kernel(SinkArgs a) {
  constexpr int NT = kPromptThreads, BQ = NT / 4, BK = 32, NSUB = 2, NKK = D / 32, NRT = V / 16, CS = D + 8, CT = BK + 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* ks = reinterpret_cast<bf16_t*>(smem_raw);  // [NSUB * BK][CS]  key-major
  bf16_t* vt = ks + NSUB * BK * CS;                   // [NSUB][V][CT]    value-major, key slots permuted
  const int H = a.H, G = a.G, bs = a.bs, R = H / G;
  const int gh = blockIdx.y;
  int s = 0, tile = blockIdx.x;
  for (; s < a.n_seqs; ++s) {
    const int nt = ((a.cu_q[s + 1] - a.cu_q[s]) * R + BQ - 1) / BQ;
    if (tile < nt) break;
    tile -= nt;
  }
  if (s >= a.n_seqs) return;
  const int q0 = a.cu_q[s], qlen = a.cu_q[s + 1] - q0, ctx = a.context_lens[s];
  const int n_rows = qlen * R, row0 = tile * BQ;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, n = lane & 15;
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_stride;
  const int my_row = row0 + 16 * wave + n;
  const bool valid = my_row < n_rows;
  const int tl = valid ? my_row / R : 0, h = gh * R + (valid ? my_row - tl * R : 0);
  const int my_pos = valid ? ctx - qlen + tl : -1;
  const int max_pos = ctx - qlen + (min(row0 + BQ, n_rows) - 1) / R;
  const bf16_t* q = static_cast<const bf16_t*>(a.q);
  const bf16_t* kc = static_cast<const bf16_t*>(a.k_cache);
  const bf16_t* vc = static_cast<const bf16_t*>(a.v_cache);
  const float hs = a.head_scale[h], cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;

  pk::bf16x8_t qf[NKK];
  {
    const bf16_t* qr = q + (static_cast<int64_t>(q0 + tl) * H + h) * D + 8 * g;
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
  const bool with_sink = a.sink > 0.f;
  float m_run = with_sink ? 0.f : -INFINITY, l_run = with_sink ? a.sink : 0.f;

  constexpr int KCH = BK * D / 8, VCH = V * BK / 8;  // 16-byte chunks of a 32-key key tile / value tile
  constexpr int KIT = (KCH + NT - 1) / NT, VIT = (VCH + NT - 1) / NT;
  // Two 32-key tiles are staged per barrier pair; the next pair's loads are issued before this
  // pair's products and land in LDS after them.
  pk::u32x4 kv[NSUB][KIT], vv[NSUB][VIT];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int st = 0; st < NSUB; ++st) {
      const int kk0 = k0 + BK * st;
      if (kk0 > max_pos) break;
      const int64_t blk = bt[kk0 / bs];
      const bf16_t* ksrc = kc + ((blk * G + gh) * bs + kk0 % bs) * D;
      const bf16_t* vsrc = vc + (blk * G + gh) * V * bs + kk0 % bs;
#pragma unroll
      for (int i = 0; i < KIT; ++i) {
        const int c = tid + NT * i;
        if (c < KCH) kv[st][i] = *reinterpret_cast<const pk::u32x4*>(ksrc + c * 8);
      }
#pragma unroll
      for (int i = 0; i < VIT; ++i) {
        const int c = tid + NT * i;
        if (c < VCH) vv[st][i] = *reinterpret_cast<const pk::u32x4*>(vsrc + static_cast<int64_t>(c >> 2) * bs + (c & 3) * 8);
      }
    }
  };
  if (max_pos >= 0) fetch(0);
  for (int k0 = 0; k0 <= max_pos; k0 += NSUB * BK) {
#pragma unroll
    for (int st = 0; st < NSUB; ++st) {
      if (k0 + BK * st > max_pos) break;
#pragma unroll
      for (int i = 0; i < KIT; ++i) {
        const int c = tid + NT * i;
        if (c < KCH) {
          const int key = c / (D / 8), d8 = c - key * (D / 8);
          *reinterpret_cast<pk::u32x4*>(ks + (st * BK + key) * CS + d8 * 8) = kv[st][i];
        }
      }
#pragma unroll
      for (int i = 0; i < VIT; ++i) {
        const int c = tid + NT * i;
        if (c < VCH) {
          const int row = c >> 2, k8 = (c & 3) * 8;  // keys k8 .. k8 + 7 of value row `row`
          uint2 lo, hi;
          lo.x = vv[st][i][0];
          lo.y = vv[st][i][1];
          hi.x = vv[st][i][2];
          hi.y = vv[st][i][3];
          *reinterpret_cast<uint2*>(vt + (st * V + row) * CT + key_slot(k8)) = lo;
          *reinterpret_cast<uint2*>(vt + (st * V + row) * CT + key_slot(k8 + 4)) = hi;
        }
      }
    }
    __syncthreads();
    if (k0 + NSUB * BK <= max_pos) fetch(k0 + NSUB * BK);
#pragma unroll
    for (int st = 0; st < NSUB; ++st) {
      const int kk0 = k0 + BK * st;
      if (kk0 > max_pos || !__any(my_pos >= kk0)) break;
      pk::f32x4 sa[2] = {pk::f32x4{0.f, 0.f, 0.f, 0.f}, pk::f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const bf16_t* kr = ks + (st * BK + sub * 16 + n) * CS + 8 * g;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk)
          sa[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(kr + kk * 32), qf[kk], sa[sub], 0, 0, 0);
      }
      float sc[8];
      float tmax = -INFINITY;
      const bool small = small_args(sa, hs, inv_cap);
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[e] = capped(sa[e >> 2][e & 3], hs, cap, inv_cap, small);
      if (__any(my_pos < kk0 + BK - 1)) {  // a tile that reaches past some row's own key: mask
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int key = kk0 + (e >> 2) * 16 + 4 * g + (e & 3);
          sc[e] = key <= my_pos ? sc[e] : -INFINITY;
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) tmax = fmaxf(tmax, sc[e]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = tmax > m_run + kLazyMax ? tmax : m_run;  // the reference moves only on a real jump
      float p[8], tsum = 0.f;
      if (__any(m_new == -INFINITY)) {  // a row without any key yet (no sink): keep its weights at zero
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = sc[e] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sc[e] - m_new);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = __builtin_amdgcn_exp2f(sc[e] - m_new);  // 2^-inf = 0
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) tsum += p[e];
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
      const bf16_t* vr = vt + (st * V + n) * CT + 8 * g;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt)
        o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(vr + rt * 16 * CT), pb, o[rt], 0, 0, 0);
    }
    __syncthreads();
  }
  if (valid) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    int pos = a.positions[q0 + tl];
    pos = pos < 0 ? 0 : (pos >= a.table_rows ? max(a.table_rows - 1, 0) : pos);
    const float* cs = a.v_table ? a.v_table + static_cast<int64_t>(pos) * V : nullptr;  // V / 2 pairs of (cos, sin)
    bf16_t* dst = static_cast<bf16_t*>(a.out) + (static_cast<int64_t>(q0 + tl) * H + h) * V + 4 * g;
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      float w0 = o[rt][0] * inv, w1 = o[rt][1] * inv, w2 = o[rt][2] * inv, w3 = o[rt][3] * inv;
      if (cs) {  // turned back: angle -position
        const float4 t = *reinterpret_cast<const float4*>(cs + (rt * 16 + 4 * g));  // (cos, sin) of two pairs
        const float n0 = w0 * t.x + w1 * t.y, n1 = w1 * t.x - w0 * t.y;
        const float n2 = w2 * t.z + w3 * t.w, n3 = w3 * t.z - w2 * t.w;
        w0 = n0, w1 = n1, w2 = n2, w3 = n3;
      }
      uint2 w;
      w.x = pk::pack2(w0, w1);
      w.y = pk::pack2(w2, w3);
      *reinterpret_cast<uint2*>(dst + rt * 16) = w;
    }
  }
}

// A decoded token on the matrix cores: one wave per (sequence, KV head, run of `part` keys), the
// KV head's query heads are the rows of its 16-row tile; both products take their A operands
// straight from the caches (key rows; value rows at the lane's 8 key slots), so nothing is staged
// and no barrier is needed.  It leaves (max, sum, unnormalised o) per head for sink_merge_kernel
// (natural-log units, like the FMA kernel's runs).
template <int D, int V>
__global__ void __launch_bounds__(64) sink_decode_mfma_kernel(SinkArgs a) {
  constexpr int NKK = D / 32, NRT = V / 16;
  const int H = a.H, G = a.G, bs = a.bs, R = H / G;
  const int ntile = (R + 15) / 16;
  const int s = blockIdx.x / ntile, tile = blockIdx.x - s * ntile, gh = blockIdx.y, part = blockIdx.z;
  const int lane = threadIdx.x, g = lane >> 4, n = lane & 15;
  const int tok = a.cu_q[s], ctx = a.context_lens[s];
  const int hr = tile * 16 + n;
  const bool valid = hr < R;
  const int h = gh * R + (valid ? hr : 0);
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_stride;
  const bf16_t* q = static_cast<const bf16_t*>(a.q);
  const bf16_t* kc = static_cast<const bf16_t*>(a.k_cache);
  const bf16_t* vc = static_cast<const bf16_t*>(a.v_cache);
  const float hs = a.head_scale[h], cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  const int k_begin = part * a.part, k_end = min(ctx, k_begin + a.part);
  pk::bf16x8_t qf[NKK];
  {
    const bf16_t* qr = q + (static_cast<int64_t>(tok) * H + h) * D + 8 * g;
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
  for (int k0 = k_begin; k0 < k_end; k0 += 32) {
    const int64_t blk = bt[k0 / bs];
    const bf16_t* ksrc = kc + ((blk * G + gh) * bs + k0 % bs) * D;
    const bf16_t* vsrc = vc + (blk * G + gh) * V * bs + k0 % bs;
    pk::f32x4 sa[2] = {pk::f32x4{0.f, 0.f, 0.f, 0.f}, pk::f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const bf16_t* kr = ksrc + (sub * 16 + n) * D + 8 * g;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk)
        sa[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(kr + kk * 32), qf[kk], sa[sub], 0, 0, 0);
    }
    // value rows at this lane's key slots: keys 4 g .. 4 g + 3 and 16 + 4 g .. 16 + 4 g + 3
    pk::u32x4 vfr[NRT];
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      const bf16_t* vr = vsrc + static_cast<int64_t>(rt * 16 + n) * bs + 4 * g;
      const uint2 lo = *reinterpret_cast<const uint2*>(vr), hi = *reinterpret_cast<const uint2*>(vr + 16);
      vfr[rt] = pk::u32x4{lo.x, lo.y, hi.x, hi.y};
    }
    float sc[8];
    float tmax = -INFINITY;
    const bool small = small_args(sa, hs, inv_cap);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = k0 + (e >> 2) * 16 + 4 * g + (e & 3);
      sc[e] = (valid && key < k_end) ? capped(sa[e >> 2][e & 3], hs, cap, inv_cap, small) : -INFINITY;
      tmax = fmaxf(tmax, sc[e]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = (m_run == -INFINITY || tmax > m_run + kLazyMax) ? tmax : m_run;
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
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      o[rt] *= resc;
      o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pk::bf16x8_t, vfr[rt]), pb, o[rt], 0, 0, 0);
    }
  }
  if (valid) {
    const int64_t at = (static_cast<int64_t>(s) * a.n_parts + part) * H + h;
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt)
      *reinterpret_cast<float4*>(a.ws_o + at * V + rt * 16 + 4 * g) = float4{o[rt][0], o[rt][1], o[rt][2], o[rt][3]};
    if (g == 0) {
      a.ws_ml[at * 2] = m_run == -INFINITY ? -INFINITY : m_run / kLog2e;  // the merge works in natural-log units
      a.ws_ml[at * 2 + 1] = l_run;
    }
  }
}

// head sizes the matrix-core kernels are built for (bf16, pages of whole 32-key tiles)
bool mfma_sizes(int D, int V) { return (D == 64 || D == 128) && (V == 64 || V == 128); }

template <bool DECODE>
int launch_mfma(const SinkArgs& a, dim3 grid, hipStream_t stream) {
#define PKM_SM(DD, VV)                                                                                  \
  if (a.D == DD && a.V == VV) {                                                                         \
    if (DECODE) {                                                                                       \
      sink_decode_mfma_kernel<DD, VV><<<grid, 64, 0, stream>>>(a);                                      \
    } else {                                                                                            \
      const size_t lds = 2 * (32 * (DD + 8) + VV * 40) * sizeof(bf16_t);                                    \
      sink_attention_mfma_kernel<DD, VV><<<grid, kPromptThreads, lds, stream>>>(a);                     \
    }                                                                                                   \
    return PK_CHECK_LAUNCH();                                                                           \
  }
  PKM_SM(64, 64)
  PKM_SM(64, 128)
  PKM_SM(128, 64)
  PKM_SM(128, 128)
#undef PKM_SM
  return -1;
}

int g_sink_mfma = 1;  // 0: every launch takes the FMA kernels (tests compare the two)

// key tile: the largest of 64 / 32 / 16 / 8 whose tiles fit 60 KiB of LDS; 0: the heads are too wide
int key_tile(int D, int V) {
  for (int bk = 64; bk >= 8; bk >>= 1) {
    const size_t b = (static_cast<size_t>(kBQ) * (D + 1) + static_cast<size_t>(bk) * (D + V + 2) + kBQ * bk + 2 * kBQ) * 4;
    if (b <= 60 * 1024) return bk;
  }
  return 0;
}

size_t lds_bytes(int D, int V, int bk) {
  return (static_cast<size_t>(kBQ) * (D + 1) + static_cast<size_t>(bk) * (D + V + 2) + kBQ * bk + 2 * kBQ) * 4;
}

template <typename T, bool SPLIT>
int launch_sink(const SinkArgs& a, dim3 grid, hipStream_t stream) {
  const size_t lds = lds_bytes(a.D, a.V, a.BK);
  const int nv = (a.V + 15) / 16;
#define PKM_SINK(NV) sink_attention_kernel<T, NV, SPLIT><<<grid, kThreads, lds, stream>>>(a)
  if (nv <= 1) {
    PKM_SINK(1);
  } else if (nv <= 2) {
    PKM_SINK(2);
  } else if (nv <= 4) {
    PKM_SINK(4);
  } else if (nv <= 8) {
    PKM_SINK(8);
  } else if (nv <= 16) {
    PKM_SINK(16);
  } else {
    PKM_SINK(32);
  }
#undef PKM_SINK
  return PK_CHECK_LAUNCH();
}

}  // namespace

// nslab > 1: qkv is fp32 split-K slabs [nslab][T][stride] (dt is then the type of q_out and the caches)
PK_EXPORT int pkm_rope_norm_cache(void* q_out, const void* qkv, long long stride, int nslab, const void* positions,
                                  const void* slot_mapping, const void* qk_table, int qk_pairs, const void* v_table,
                                  int table_rows, void* k_cache, void* v_cache, int T, int H, int G, int D, int V,
                                  int bs, float eps, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (D < 1 || D > 128 * kMaxPairs || V < 1 || 2 * qk_pairs > D || ((qk_table || v_table) && table_rows < 1)) return -1;
  if (v_table && (V & 1)) return -1;
  const dim3 grid(T, H + 2 * G);
  if (nslab > 1) {
    PKM_DISPATCH(dt, E, rope_norm_cache_kernel<E, float><<<grid, 64, 0, stream>>>(
                            static_cast<E*>(q_out), static_cast<const float*>(qkv), stride, nslab,
                            static_cast<int64_t>(T) * stride, static_cast<const int*>(positions),
                            static_cast<const int*>(slot_mapping), static_cast<const float*>(qk_table), qk_pairs,
                            static_cast<const float*>(v_table), table_rows, static_cast<E*>(k_cache),
                            static_cast<E*>(v_cache), H, G, D, V, bs, eps));
    return PK_CHECK_LAUNCH();
  }
  PKM_DISPATCH(dt, E, rope_norm_cache_kernel<E, E><<<grid, 64, 0, stream>>>(
                          static_cast<E*>(q_out), static_cast<const E*>(qkv), stride, 1, 0, static_cast<const int*>(positions),
                          static_cast<const int*>(slot_mapping), static_cast<const float*>(qk_table), qk_pairs,
                          static_cast<const float*>(v_table), table_rows, static_cast<E*>(k_cache),
                          static_cast<E*>(v_cache), H, G, D, V, bs, eps));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_set_sink_mfma(int on) {
  g_sink_mfma = on;
  return 0;
}

// keys per run and runs of a decoded token for caches of up to `capacity` tokens per sequence
PK_EXPORT int pkm_sink_decode_part(int capacity, int D, int V, int bs, int dt) {
  if (g_sink_mfma && dt == kBF16 && bs % 32 == 0 && mfma_sizes(D, V)) {
    const int part = ((capacity + 31) / 32 + 31) / 32 * 32;  // at most 32 runs of whole 32-key tiles
    return part < 64 ? 64 : part;
  }
  const int bk = key_tile(D, V);
  if (bk == 0) return -1;
  int part = (capacity + 31) / 32;             // at most 32 runs
  part = (part + bk - 1) / bk * bk;
  return part < 4 * bk ? 4 * bk : part;
}

// The first num_decode sequences hold one token each and take the split kernel + merge when the
// workspace (ws_o [num_decode, n_parts, H, V], ws_ml [num_decode, n_parts, H, 2] fp32) is given.
PK_EXPORT int pkm_sink_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                 const void* block_tables, long long bt_stride, const void* cu_q,
                                 const void* context_lens, const void* positions, const void* head_scale,
                                 const void* v_table, int table_rows, int n_seqs, int T, int H, int G, int D, int V,
                                 int bs, float softcap, float sink, int num_decode, void* ws_o, void* ws_ml, int part,
                                 int n_parts, int dt, hipStream_t stream) {
  if (n_seqs <= 0 || T <= 0) return 0;
  if (G < 1 || H % G || V > 512 || n_parts > 64 || (v_table && ((V & 1) || table_rows < 1))) return -1;
  const int bk = key_tile(D, V);
  if (bk == 0) return -1;
  SinkArgs a{out, q, k_cache, v_cache, static_cast<const int*>(block_tables), bt_stride, static_cast<const int*>(cu_q),
             static_cast<const int*>(context_lens), static_cast<const int*>(positions),
             static_cast<const float*>(head_scale), static_cast<const float*>(v_table), table_rows, n_seqs, H, G, D, V,
             bs, bk, softcap, sink, part, n_parts, static_cast<float*>(ws_o), static_cast<float*>(ws_ml)};
  const int R = H / G;
  const bool mfma = g_sink_mfma && dt == kBF16 && bs % 32 == 0 && mfma_sizes(D, V);
  int nd = (ws_o && ws_ml && n_parts > 1) ? (num_decode < n_seqs ? num_decode : n_seqs) : 0;
  if (nd > 0) {
    SinkArgs d = a;
    d.n_seqs = nd;
    int rc;
    if (mfma) {
      if (part < 32 || part % 32) return -1;
      rc = launch_mfma<true>(d, dim3(nd * ((R + 15) / 16), G, n_parts), stream);
    } else {
      if (part < bk || part % bk) return -1;
      const dim3 grid(nd * ((R + kBQ - 1) / kBQ), G, n_parts);
      PKM_DISPATCH(dt, E, rc = launch_sink<E, true>(d, grid, stream));
    }
    if (rc) return rc;
    const dim3 mg(nd, H);
    PKM_DISPATCH(dt, E, sink_merge_kernel<E><<<mg, 128, 0, stream>>>(
                            static_cast<E*>(out), d.ws_o, d.ws_ml, d.cu_q, d.positions, d.v_table, table_rows, n_parts,
                            H, V, sink));
    rc = PK_CHECK_LAUNCH();
    if (rc) return rc;
  }
  if (n_seqs > nd) {
    SinkArgs p = a;
    p.n_seqs = n_seqs - nd;
    p.block_tables += static_cast<int64_t>(nd) * bt_stride;
    p.cu_q += nd;
    p.context_lens += nd;
    // row tiles: every sequence adds at most one partly filled tile
    int rc;
    if (mfma) {
      rc = launch_mfma<false>(p, dim3(((T - nd) * R + 127) / 128 + p.n_seqs, G), stream);
    } else {
      const int tiles = ((T - nd) * R + kBQ - 1) / kBQ + p.n_seqs;
      PKM_DISPATCH(dt, E, rc = launch_sink<E, false>(p, dim3(tiles, G), stream));
    }
    if (rc) return rc;
  }
  return 0;
}
