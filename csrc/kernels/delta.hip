// Gated delta rule (gfx950, wave64).
//
// Per head, with unit vectors q (times dim^-1/2) and k, a decay g in (0, 1) and a write strength
// beta in (0, 1) per token:
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// Every value column j of S is an independent recurrence over its own [dim] vector:
//     a = S_j . k,  b = S_j . q   (both on the state before the token)
//     u_j = beta (v_j - g a);   o_j = g b + u_j (k . q);   S_j <- g S_j + k u_j
// so the kernel gives a column to 16 lanes (a DPP row: the two dot products are row rotations), a
// workgroup 16 columns of one (sequence, head), and walks the tokens in order.  Tokens are staged in
// groups of 16: raw q / k rows in LDS, unit norms and k . q by one DPP row per token, beta and the decay
// (sigmoid, softplus, two exponentials) by one lane per token, so the serial part of a token is two
// multiply-add sweeps over the lane's state registers and the row sums.  A group's inputs are fetched
// into registers while the previous group's recurrence runs.  All of it is f32; the
// state [slots, heads, vdim, dim] keeps a column contiguous.  delta_finish norms each head's output
// (unit RMS times a weight shared by the heads) and applies the SiLU gate.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));  // row_ror:8
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));  // row_ror:4
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));  // row_ror:2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));  // row_ror:1
  return v;
}

constexpr int DR_TT = 16;   // tokens per staged group
constexpr int DR_COLS = 16; // value columns per workgroup

// NS: state entries per lane; lane `sub` of a column owns dims sub * NS .. sub * NS + NS - 1, kept in
// LDS at [r * 16 + sub] so that the 16 lanes of a row read consecutive words.
// VL (bf16, rows of whole 16-byte vectors): q / k rows are fetched as 16-byte vectors, 8 dims a thread,
// instead of NS scattered 2-byte loads a thread.
template <typename T, int NS, bool VL>
__global__ void __launch_bounds__(256) delta_rule_kernel(const T* __restrict__ qkv, long ldq, const T* __restrict__ gba,
                                                         long ldg, int H, int G, int d, int dv,
                                                         const float* __restrict__ neg_a,
                                                         const float* __restrict__ dt_bias, float* __restrict__ state,
                                                         const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                         const int* __restrict__ ctx, const int* __restrict__ rows,
                                                         float* __restrict__ raw) {
  constexpr int DP = 16 * NS;
  __shared__ float qs[DR_TT * DP], ks[DR_TT * DP], vs[DR_TT * DR_COLS], bg[DR_TT * 4];
  const int h = blockIdx.y, s = blockIdx.z;
  const int n = qlen[s];
  if (n <= 0) return;   // the whole workgroup
  const int tid = threadIdx.x, sub = tid & 15, col = tid >> 4;
  const int j0 = blockIdx.x * DR_COLS, j = j0 + col;
  const bool live = j < dv;
  const int kvh = h / (H / G);
  const int q0 = qstart[s], p0 = ctx[s] - n;
  float* sp = state + (((long)rows[s] * H + h) * dv + (live ? j : dv - 1)) * d;
  float S[NS];
#pragma unroll
  for (int r = 0; r < NS; ++r) {
    const int i = sub * NS + r;
    S[r] = (p0 > 0 && live && i < d) ? sp[i] : 0.f;
  }
  const long oq = (long)kvh * d, ok = (long)G * d + (long)kvh * d, ov = 2L * G * d + (long)h * dv;
  const long ob = (long)H * dv + h, oa = (long)H * dv + H + h;
  const float na = neg_a[h], dtb = dt_bias[h], qscale = 1.f / sqrtf((float)d);
  // a group's inputs are fetched into registers one group ahead, so their latency hides under the
  // previous group's recurrence: NS entries of q and of k, one of v, and (lanes < 16) the two logits
  constexpr int NFV = (NS + 7) / 8;          // 16-byte chunks of q (and of k) a thread moves per group: 16 rows of d / 8
  float pq[VL ? 1 : NS], pk[VL ? 1 : NS], pv = 0.f, pb = 0.f, pa = 0.f;
  uint4 vq[VL ? NFV : 1], vk[VL ? NFV : 1];
  const int dch = d >> 3;                    // chunks per row (VL: d % 8 == 0)
  auto fetch = [&](int t0) {
    const int nt = min(DR_TT, n - t0);
    if constexpr (VL) {
#pragma unroll
      for (int f = 0; f < NFV; ++f) {
        const int e = tid + 256 * f;
        const int tt = e / dch, ch = e - tt * dch;
        vq[f] = make_uint4(0u, 0u, 0u, 0u);
        vk[f] = make_uint4(0u, 0u, 0u, 0u);
        if (tt < nt) {
          const u16* row = reinterpret_cast<const u16*>(qkv) + (long)(q0 + t0 + tt) * ldq + 8 * ch;
          vq[f] = *reinterpret_cast<const uint4*>(row + oq);
          vk[f] = *reinterpret_cast<const uint4*>(row + ok);
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < NS; ++r) {
        const int e = tid + 256 * r;
        const int tt = e / DP, c = e % DP;       // c = r' * 16 + sub'  ->  dim sub' * NS + r'
        const int i = (c & 15) * NS + (c >> 4);
        const bool okx = tt < nt && i < d;
        const T* row = qkv + (long)(q0 + t0 + (okx ? tt : 0)) * ldq;
        pq[r] = okx ? ldf(row + oq + i) : 0.f;
        pk[r] = okx ? ldf(row + ok + i) : 0.f;
      }
    }
    {
      const int tt = tid / DR_COLS, c = tid % DR_COLS;
      pv = (tt < nt && j0 + c < dv) ? ldf(qkv + (long)(q0 + t0 + tt) * ldq + ov + j0 + c) : 0.f;
    }
    if (tid < nt) {
      const T* row = gba + (long)(q0 + t0 + tid) * ldg;
      pb = ldf(row + ob);
      pa = ldf(row + oa);
    }
  };
  if constexpr (VL) {   // dims past d (the lanes' padding) are never written again: zero them once
    for (int e = tid; e < DR_TT * DP; e += 256) { qs[e] = 0.f; ks[e] = 0.f; }
  }
  fetch(0);
  for (int t0 = 0; t0 < n; t0 += DR_TT) {
    const int nt = min(DR_TT, n - t0);
    __syncthreads();   // the previous group is consumed
    if constexpr (VL) {
#pragma unroll
      for (int f = 0; f < NFV; ++f) {
        const int e = tid + 256 * f;
        const int tt = e / dch, ch = e - tt * dch;
        if (tt < DR_TT) {
          float q8[8], k8[8];
          unpack8(vq[f], q8);
          unpack8(vk[f], k8);
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            const int i = 8 * ch + x;          // dim i = sub * NS + r lies at [r * 16 + sub]
            const int pos = tt * DP + (i % NS) * 16 + i / NS;
            qs[pos] = q8[x];
            ks[pos] = k8[x];
          }
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < NS; ++r) {
        qs[tid + 256 * r] = pq[r];
        ks[tid + 256 * r] = pk[r];
      }
    }
    vs[tid] = pv;
    if (tid < nt) {
      const float z = pa + dtb;
      const float sp_ = z > 20.f ? z : log1pf(expf(z));
      bg[tid * 4] = 1.f / (1.f + expf(-pb));
      bg[tid * 4 + 1] = expf(na * sp_);
    }
    __syncthreads();
    if (t0 + DR_TT < n) fetch(t0 + DR_TT);
    {   // unit q (times dim^-1/2) and k, and k . q: the 16 lanes of a DPP row take one token
      const int tt = tid >> 4;
      float qv[NS], kv[NS], sq = 0.f, sk = 0.f;
#pragma unroll
      for (int r = 0; r < NS; ++r) {
        qv[r] = qs[tt * DP + r * 16 + sub];
        kv[r] = ks[tt * DP + r * 16 + sub];
        sq += qv[r] * qv[r];
        sk += kv[r] * kv[r];
      }
      sq = row16_sum(sq);
      sk = row16_sum(sk);
      const float rq = qscale / sqrtf(sq + 1e-6f), rk = 1.f / sqrtf(sk + 1e-6f);
      float kq = 0.f;
#pragma unroll
      for (int r = 0; r < NS; ++r) {
        qv[r] *= rq;
        kv[r] *= rk;
        qs[tt * DP + r * 16 + sub] = qv[r];
        ks[tt * DP + r * 16 + sub] = kv[r];
        kq += qv[r] * kv[r];
      }
      kq = row16_sum(kq);
      if (sub == 0) bg[tt * 4 + 2] = kq;
    }
    __syncthreads();
    float o_m = 0.f;
#pragma unroll 4
    for (int u = 0; u < nt; ++u) {   // unrolled: the LDS reads of the next tokens do not depend on the state
      const float beta = bg[u * 4], g = bg[u * 4 + 1], kq = bg[u * 4 + 2], v = vs[u * DR_COLS + col];
      float kk[NS];
      float a2[2] = {0.f, 0.f}, b2[2] = {0.f, 0.f};
#pragma unroll
      for (int r = 0; r < NS; ++r) {
        kk[r] = ks[u * DP + r * 16 + sub];
        a2[r & 1] += S[r] * kk[r];
        b2[r & 1] += S[r] * qs[u * DP + r * 16 + sub];
      }
      const float a = row16_sum(a2[0] + a2[1]);
      const float b = row16_sum(b2[0] + b2[1]);
      const float uu = beta * (v - g * a);
#pragma unroll
      for (int r = 0; r < NS; ++r) S[r] = g * S[r] + kk[r] * uu;
      if (sub == u) o_m = g * b + uu * kq;
    }
    if (live && sub < nt) raw[((long)(q0 + t0 + sub) * H + h) * dv + j] = o_m;
  }
  if (!live) return;
#pragma unroll
  for (int r = 0; r < NS; ++r) {
    const int i = sub * NS + r;
    if (i < d) sp[i] = S[r];
  }
}

// out = raw / rms(raw over dv) * w * silu(gate): one wave per (token, head)
template <typename T>
__global__ void __launch_bounds__(256) delta_finish_kernel(const float* __restrict__ raw, const T* __restrict__ gba, long ldg,
                                                           int H, int dv, const float* __restrict__ w, float eps,
                                                           const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                           int S, T* __restrict__ out, long rows_total) {
  const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows_total) return;
  const int lane = threadIdx.x & 63;
  const long tok = r / H;
  const int h = (int)(r % H);
  bool live = false;   // tokens of no sequence (graph padding) become zeros
  for (int s = 0; s < S; ++s) live |= tok >= qstart[s] && tok < qstart[s] + qlen[s];
  if (!live) {
    for (int j = lane; j < dv; j += 64) stf(out + tok * ((long)H * dv) + (long)h * dv + j, 0.f);
    return;
  }
  const float* o = raw + r * dv;
  float ss = 0.f;
  for (int j = lane; j < dv; j += 64) ss += o[j] * o[j];
  ss = wave_sum(ss);
  const float rs = 1.f / sqrtf(ss / (float)dv + eps);
  for (int j = lane; j < dv; j += 64) {
    const float z = ldf(gba + tok * ldg + (long)h * dv + j);
    stf(out + tok * ((long)H * dv) + (long)h * dv + j, o[j] * rs * w[j] * (z / (1.f + expf(-z))));
  }
}

template <typename T, bool VL>
int launch_delta(int ns, dim3 g, hipStream_t st, const T* qkv, long ldq, const T* gba, long ldg, int H, int G, int d, int dv,
                 const float* neg_a, const float* dt_bias, float* state, const int* qstart, const int* qlen, const int* ctx,
                 const int* rows, float* raw) {
#define DELTA(NS) hipLaunchKernelGGL((delta_rule_kernel<T, NS, VL>), g, dim3(256), 0, st, qkv, ldq, gba, ldg, H, G, d, dv, neg_a, dt_bias, state, qstart, qlen, ctx, rows, raw)
  if (ns <= 1) DELTA(1); else if (ns <= 2) DELTA(2); else if (ns <= 4) DELTA(4); else if (ns <= 8) DELTA(8); else DELTA(16);
#undef DELTA
  return (int)hipGetLastError();
}

}  // namespace

// qkv [T, 2 G d + H dv] (q | k | v after convolution and SiLU), gba [T, H dv + 2 H] (gate | beta |
// decay logits), state [slots, H, dv, d] f32, raw [T, H, dv] f32 scratch, out [T, H dv].
extern "C" int dllm_delta_rule(const void* qkv, long ldq, const void* gba, long ldg, int f32, int H, int G, int d, int dv,
                               const float* neg_a, const float* dt_bias, const float* norm_w, float eps, float* state,
                               const int* qstart, const int* qlen, const int* ctx, const int* rows, float* raw, void* out,
                               int S, long T, hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  if (d < 1 || d > 256 || G < 1 || H % G) return -1;
  const int ns = (d + 15) / 16;
  const dim3 g((dv + DR_COLS - 1) / DR_COLS, H, S);
  const long rows_total = T * H;
  const dim3 gf((unsigned)((rows_total + 3) / 4));
  int rc;
  if (f32) {
    rc = launch_delta<float, false>(ns, g, st, (const float*)qkv, ldq, (const float*)gba, ldg, H, G, d, dv, neg_a, dt_bias,
                                    state, qstart, qlen, ctx, rows, raw);
    hipLaunchKernelGGL(delta_finish_kernel<float>, gf, dim3(256), 0, st, raw, (const float*)gba, ldg, H, dv, norm_w, eps,
                       qstart, qlen, S, (float*)out, rows_total);
  } else {
    // 16-byte row vectors: every q / k head starts on a 16-byte boundary of a 16-byte aligned row
    const bool vl = d % 8 == 0 && ldq % 8 == 0 && ((uintptr_t)qkv & 15) == 0;
    if (vl)
      rc = launch_delta<u16, true>(ns, g, st, (const u16*)qkv, ldq, (const u16*)gba, ldg, H, G, d, dv, neg_a, dt_bias, state,
                                   qstart, qlen, ctx, rows, raw);
    else
      rc = launch_delta<u16, false>(ns, g, st, (const u16*)qkv, ldq, (const u16*)gba, ldg, H, G, d, dv, neg_a, dt_bias, state,
                                    qstart, qlen, ctx, rows, raw);
    hipLaunchKernelGGL(delta_finish_kernel<u16>, gf, dim3(256), 0, st, raw, (const u16*)gba, ldg, H, dv, norm_w, eps, qstart,
                       qlen, S, (u16*)out, rows_total);
  }
  return rc ? rc : (int)hipGetLastError();
}
