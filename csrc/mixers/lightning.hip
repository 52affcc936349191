// Lightning attention: linear attention with one constant decay per head.
//
//     S_t = decay_h * S_{t-1} + k_t v_t^T        o_t = S_t^T q_t        q, k, v = silu(projections)
//
// The state S [D, V] of a (sequence, head) is fp32 and lives in the sequence's state slot between
// steps.  One workgroup owns 16 value columns of one (sequence, head): thread (dg, vc) keeps rows
// dg, dg + 16, ... of column vc in registers and walks the portion's tokens in order; q, k, v of up to
// 32 tokens at a time are staged in LDS with the SiLU applied.  A token's sums run in the same order
// whether it arrives in a long prompt portion or alone, so results do not depend on the cut.
// The first token of a portion reads the slot unless it is position 0 (a new sequence starts from
// zeros whatever an earlier owner left); the state after the portion's last token is written back.
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kMaxChunk = 32;  // tokens staged per group (fewer when a head is wide)
constexpr int kCols = 16;   // value columns per workgroup

__device__ __forceinline__ float siluf(float z) { return z / (1.f + expf(-z)); }

template <typename T, int ND>
__global__ void __launch_bounds__(256)
lightning_kernel(float* __restrict__ out, const T* __restrict__ qkv, int64_t stride, float* __restrict__ state,
                 const float* __restrict__ decay, const int* __restrict__ cu_q, const int* __restrict__ positions,
                 const int* __restrict__ slots, int H, int D, int V, int kChunk) {
  extern __shared__ float smem[];
  float* qs = smem;                 // [kChunk][D]
  float* ks = qs + kChunk * D;      // [kChunk][D]
  float* vs = ks + kChunk * D;      // [kChunk][kCols]
  const int s = blockIdx.x / H, h = blockIdx.x - s * H;
  const int v0 = blockIdx.y * kCols;
  const int a = cu_q[s], b = cu_q[s + 1];
  if (b <= a) return;
  const int tid = threadIdx.x, dg = tid & 15, vc = tid >> 4;
  const int col = v0 + vc;
  const int slot = slots[s];
  const float dec = decay[h];
  float S[ND];
  float* sp = slot >= 0 ? state + ((static_cast<int64_t>(slot) * H + h) * D) * V : nullptr;
  const bool carry = sp != nullptr && positions[a] > 0;
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = dg + 16 * i;
    S[i] = (carry && d < D && col < V) ? sp[static_cast<int64_t>(d) * V + col] : 0.f;
  }
  const int64_t qo = static_cast<int64_t>(h) * D, ko = static_cast<int64_t>(H) * D + qo;
  const int64_t vo = 2 * static_cast<int64_t>(H) * D + static_cast<int64_t>(h) * V + v0;
  for (int t0 = a; t0 < b; t0 += kChunk) {
    const int nt = min(kChunk, b - t0);
    __syncthreads();
    for (int e = tid; e < nt * D; e += 256) {
      const int t = e / D, d = e - t * D;
      const T* row = qkv + static_cast<int64_t>(t0 + t) * stride;
      qs[e] = siluf(ld<T>(row + qo + d));
      ks[e] = siluf(ld<T>(row + ko + d));
    }
    for (int e = tid; e < nt * kCols; e += 256) {
      const int t = e / kCols, c = e - t * kCols;
      vs[e] = v0 + c < V ? siluf(ld<T>(qkv + static_cast<int64_t>(t0 + t) * stride + vo + c)) : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float vv = vs[t * kCols + vc];
      const float* kr = ks + t * D;
      const float* qr = qs + t * D;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < ND; ++i) {
        const int d = dg + 16 * i;
        if (d < D) {
          S[i] = dec * S[i] + kr[d] * vv;
          o += S[i] * qr[d];
        }
      }
      o += __shfl_xor(o, 8, 64);
      o += __shfl_xor(o, 4, 64);
      o += __shfl_xor(o, 2, 64);
      o += __shfl_xor(o, 1, 64);
      if (dg == 0 && col < V) out[(static_cast<int64_t>(t0 + t) * H + h) * V + col] = o;
    }
  }
  if (sp != nullptr && col < V) {
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int d = dg + 16 * i;
      if (d < D) sp[static_cast<int64_t>(d) * V + col] = S[i];
    }
  }
}

// The wider form for heads of up to 256 key coordinates: a workgroup owns 64 value columns of one
// (sequence, head), lane = column; wave w of NW keeps key rows w * NR .. w * NR + NR - 1 of its
// columns in registers, so a token costs each wave NR broadcast reads of k and q for 2 * NR * 64
// multiply-adds and no cross-lane traffic; the waves' partial outputs of a 16-token group are
// summed in wave order through LDS (coalesced stores).  The next group's q, k, v are fetched into
// registers before the current group is computed.  Same order of sums for any cut of the prompt.
constexpr int kWideChunk = 16;
constexpr int kWideCols = 64;

template <typename T, int NR, int NW>
__global__ void __launch_bounds__(64 * NW)
lightning_wide_kernel(float* __restrict__ out, const T* __restrict__ qkv, int64_t stride, float* __restrict__ state,
                      const float* __restrict__ decay, const int* __restrict__ cu_q, const int* __restrict__ positions,
                      const int* __restrict__ slots, int H, int D, int V) {
  constexpr int DP = NW * NR;  // padded key width: rows past D hold zeros
  constexpr int NT = 64 * NW;
  constexpr int QK_IT = (kWideChunk * DP + NT - 1) / NT, V_IT = (kWideChunk * kWideCols + NT - 1) / NT;
  __shared__ __attribute__((aligned(16))) float qs[kWideChunk][DP];
  __shared__ __attribute__((aligned(16))) float ks[kWideChunk][DP];
  __shared__ float vs[kWideChunk][kWideCols];
  __shared__ float po[NW][kWideChunk][kWideCols];
  const int s = blockIdx.x / H, h = blockIdx.x - s * H;
  const int v0 = blockIdx.y * kWideCols;
  const int a = cu_q[s], b = cu_q[s + 1];
  if (b <= a) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int col = v0 + lane;
  const int slot = slots[s];
  const float dec = decay[h];
  float* sp = slot >= 0 ? state + ((static_cast<int64_t>(slot) * H + h) * D) * V : nullptr;
  const bool carry = sp != nullptr && positions[a] > 0;
  float S[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = w * NR + i;
    S[i] = (carry && d < D && col < V) ? sp[static_cast<int64_t>(d) * V + col] : 0.f;
  }
  const int64_t qo = static_cast<int64_t>(h) * D, ko = static_cast<int64_t>(H) * D + qo;
  const int64_t vo = 2 * static_cast<int64_t>(H) * D + static_cast<int64_t>(h) * V + v0;
  float rq[QK_IT], rk[QK_IT], rv[V_IT];
  auto fetch = [&](int t0) {  // raw projections of the group starting at token t0 (zeros outside)
    const int nt = min(kWideChunk, b - t0);
#pragma unroll
    for (int i = 0; i < QK_IT; ++i) {
      const int e = tid + NT * i, t = e / DP, d = e - t * DP;
      const bool ok = t < nt && d < D;
      const T* row = qkv + static_cast<int64_t>(t0 + (ok ? t : 0)) * stride;
      rq[i] = ok ? ld<T>(row + qo + d) : -INFINITY;
      rk[i] = ok ? ld<T>(row + ko + d) : -INFINITY;
    }
#pragma unroll
    for (int i = 0; i < V_IT; ++i) {
      const int e = tid + NT * i, t = e / kWideCols, c = e - t * kWideCols;
      const bool ok = t < nt && v0 + c < V;
      rv[i] = ok ? ld<T>(qkv + static_cast<int64_t>(t0 + (ok ? t : 0)) * stride + vo + c) : -INFINITY;
    }
  };
  fetch(a);
  for (int t0 = a; t0 < b; t0 += kWideChunk) {
    const int nt = min(kWideChunk, b - t0);
#pragma unroll
    for (int i = 0; i < QK_IT; ++i) {
      const int e = tid + NT * i;
      if (e < kWideChunk * DP) {
        (&qs[0][0])[e] = rq[i] == -INFINITY ? 0.f : siluf(rq[i]);
        (&ks[0][0])[e] = rk[i] == -INFINITY ? 0.f : siluf(rk[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < V_IT; ++i) {
      const int e = tid + NT * i;
      if (e < kWideChunk * kWideCols) (&vs[0][0])[e] = rv[i] == -INFINITY ? 0.f : siluf(rv[i]);
    }
    __syncthreads();
    if (t0 + kWideChunk < b) fetch(t0 + kWideChunk);  // in flight while this group is computed
#pragma unroll 4
    for (int t = 0; t < nt; ++t) {
      const float vv = vs[t][lane];
      const float* kr = &ks[t][w * NR];
      const float* qr = &qs[t][w * NR];
      float o0 = 0.f, o1 = 0.f;
      if (NR % 4 == 0) {
#pragma unroll
        for (int i = 0; i < NR; i += 4) {
          const float4 k4 = *reinterpret_cast<const float4*>(kr + i), q4 = *reinterpret_cast<const float4*>(qr + i);
          S[i] = dec * S[i] + k4.x * vv;
          o0 += S[i] * q4.x;
          S[i + 1] = dec * S[i + 1] + k4.y * vv;
          o1 += S[i + 1] * q4.y;
          S[i + 2] = dec * S[i + 2] + k4.z * vv;
          o0 += S[i + 2] * q4.z;
          S[i + 3] = dec * S[i + 3] + k4.w * vv;
          o1 += S[i + 3] * q4.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          S[i] = dec * S[i] + kr[i] * vv;
          if (i & 1) {
            o1 += S[i] * qr[i];
          } else {
            o0 += S[i] * qr[i];
          }
        }
      }
      po[w][t][lane] = o0 + o1;
    }
    __syncthreads();
    for (int e = tid; e < nt * kWideCols; e += NT) {
      const int t = e / kWideCols, c = e - t * kWideCols;
      if (v0 + c < V) {
        float o = po[0][t][c];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) o += po[ww][t][c];
        out[(static_cast<int64_t>(t0 + t) * H + h) * V + v0 + c] = o;
      }
    }
    // the next group's staging writes qs / ks / vs only; po is rewritten after its barrier
  }
  if (sp != nullptr && col < V) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = w * NR + i;
      if (d < D) sp[static_cast<int64_t>(d) * V + col] = S[i];
    }
  }
}

}  // namespace

// out [T, H, V] fp32; qkv [T, H*D | H*D | H*V] pre-activation (row stride `stride` elements);
// state [slots, H, D, V] fp32; sequences 0..n_seqs-1 own tokens cu_q[s]..cu_q[s+1]-1.
PK_EXPORT int pkm_lightning_attention(void* out, const void* qkv, long long stride, void* state, const void* decay,
                                      const void* cu_q, const void* positions, const void* slots, int n_seqs, int T,
                                      int H, int D, int V, int num_decode, int dt, hipStream_t stream) {
  if (n_seqs <= 0 || T <= 0) return 0;
  if (D < 1 || D > 512 || V < 1) return -1;
  if (D <= 256) {
    const dim3 wgrid(n_seqs * H, (V + kWideCols - 1) / kWideCols);
    const int nw = D > 64 ? 8 : 4;
    const int nr = (D + nw - 1) / nw;
#define PKM_LIGHTW(NR, NW)                                                                                          \
  PKM_DISPATCH(dt, E, lightning_wide_kernel<E, NR, NW><<<wgrid, 64 * NW, 0, stream>>>(                               \
                          static_cast<float*>(out), static_cast<const E*>(qkv), stride, static_cast<float*>(state), \
                          static_cast<const float*>(decay), static_cast<const int*>(cu_q),                          \
                          static_cast<const int*>(positions), static_cast<const int*>(slots), H, D, V))
    if (nw == 4) {
      if (nr <= 2) {
        PKM_LIGHTW(2, 4);
      } else if (nr <= 4) {
        PKM_LIGHTW(4, 4);
      } else if (nr <= 8) {
        PKM_LIGHTW(8, 4);
      } else {
        PKM_LIGHTW(16, 4);
      }
    } else if (nr <= 12) {
      PKM_LIGHTW(12, 8);
    } else if (nr <= 16) {
      PKM_LIGHTW(16, 8);
    } else if (nr <= 24) {
      PKM_LIGHTW(24, 8);
    } else {
      PKM_LIGHTW(32, 8);
    }
#undef PKM_LIGHTW
    return PK_CHECK_LAUNCH();
  }
  const dim3 grid(n_seqs * H, (V + kCols - 1) / kCols);
  const int chunk = max(1, min(kMaxChunk, 15360 / (2 * D + kCols)));  // at most 60 KiB of LDS
  const size_t lds = static_cast<size_t>(chunk) * (2 * D + kCols) * sizeof(float);
  const int nd = (D + 15) / 16;
#define PKM_LIGHT(ND)                                                                                              \
  PKM_DISPATCH(dt, E, lightning_kernel<E, ND><<<grid, 256, lds, stream>>>(                                          \
                          static_cast<float*>(out), static_cast<const E*>(qkv), stride, static_cast<float*>(state), \
                          static_cast<const float*>(decay), static_cast<const int*>(cu_q),                          \
                          static_cast<const int*>(positions), static_cast<const int*>(slots), H, D, V, chunk))
  if (nd <= 1) {
    PKM_LIGHT(1);
  } else if (nd <= 2) {
    PKM_LIGHT(2);
  } else if (nd <= 4) {
    PKM_LIGHT(4);
  } else if (nd <= 8) {
    PKM_LIGHT(8);
  } else if (nd <= 16) {
    PKM_LIGHT(16);
  } else {
    PKM_LIGHT(32);
  }
#undef PKM_LIGHT
  return PK_CHECK_LAUNCH();
}
