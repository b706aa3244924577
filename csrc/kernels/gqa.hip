// Grouped-query softmax attention over paged keys / values with any head widths (gfx950, wave64).
//
//   attn_prep   one workgroup per token: rotate-half positions on the first `rot` dims of every q / k
//               head, each head to unit RMS (f32), q times a per-head scale; k and v go to their
//               page slots, q to a dense [T, H, d] buffer.
//   paged_gqa   one workgroup per (tile of new tokens, key/value head, group of <= 16 query heads):
//               its rows are tokens x query heads of the group (<= 16).  Keys are walked in tiles
//               staged in LDS as f32; a lane owns a key for the scores (one K read feeds the wave's
//               four rows), f32 online softmax per row, then a lane owns value dims for the weighted
//               sum (one V read feeds four rows).  The output is multiplied by sigmoid(gate).
//
// Cache layout: K [blocks, block, G, d], V [blocks, block, G, dv] (bf16 or f32 like the activations);
// every score, weight and sum is f32.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

template <typename T>
__global__ void __launch_bounds__(256) attn_prep_kernel(const T* __restrict__ proj, long ld, int H, int G, int d, int dv,
                                                        const float* __restrict__ cos_sin, int tab_w, int rot, float eps,
                                                        const float* __restrict__ qscale, const int* __restrict__ pos,
                                                        const int* __restrict__ slots, T* __restrict__ kc,
                                                        T* __restrict__ vc, T* __restrict__ q) {
  const long tok = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* r = proj + tok * ld;
  const int slot = slots[tok];
  const int half = rot >> 1;
  const float* cs = cos_sin + (long)pos[tok] * tab_w;
  for (int hh = wave; hh < H + G; hh += 4) {
    const bool is_q = hh < H;
    if (!is_q && slot < 0) continue;
    const T* x = r + (long)hh * d;    // q heads, then k heads, are consecutive in the projection
    float ss = 0.f;
    for (int i = lane; i < d; i += 64) {
      float v = ldf(x + i);
      if (i < rot) {
        const int f = i < half ? i : i - half;
        const float c = cs[f], sn = cs[half + f];
        const float p = ldf(x + (i < half ? i + half : i - half));
        v = i < half ? v * c - p * sn : v * c + p * sn;
      }
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float sc = (is_q ? qscale[hh] : 1.f) / sqrtf(ss / (float)d + eps);
    T* dst = is_q ? q + (tok * H + hh) * d : kc + ((long)slot * G + (hh - H)) * d;
    for (int i = lane; i < d; i += 64) {
      float v = ldf(x + i);
      if (i < rot) {
        const int f = i < half ? i : i - half;
        const float c = cs[f], sn = cs[half + f];
        const float p = ldf(x + (i < half ? i + half : i - half));
        v = i < half ? v * c - p * sn : v * c + p * sn;
      }
      stf(dst + i, v * sc);
    }
  }
  if (slot >= 0) {
    const T* v = r + (long)(H + G) * d;
    for (int i = threadIdx.x; i < G * dv; i += 256) vc[(long)slot * G * dv + i] = v[i];
  }
}

constexpr int GA_ROWS = 16;   // rows per workgroup: 4 per wave

// KT keys per tile (64, or 32 when the tile would not fit the LDS), NJ = ceil(dv / 64)
template <typename T, int NJ>
__global__ void __launch_bounds__(256) paged_gqa_kernel(const T* __restrict__ q, const T* __restrict__ kc,
                                                        const T* __restrict__ vc, const int* __restrict__ bt, int bt_ld,
                                                        int BSZ, const int* __restrict__ qstart,
                                                        const int* __restrict__ qlen, const int* __restrict__ ctx,
                                                        const int* __restrict__ tile_seq, const int* __restrict__ tile_tok0,
                                                        const T* __restrict__ gate, long ldg, T* __restrict__ out, int H,
                                                        int G, int d, int dv, int TQ, int KT) {
  extern __shared__ float sm[];
  const int s = tile_seq[blockIdx.x];
  const int n = qlen[s];
  const int tok0 = tile_tok0[blockIdx.x];
  if (n <= 0 || tok0 >= n) return;   // the whole workgroup (padding tiles)
  const int g = blockIdx.y, R = H / G;
  const int r0 = blockIdx.z * GA_ROWS, Rh = min(GA_ROWS, R - r0);
  const int nq = min(TQ, n - tok0), nrows = nq * Rh;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  const int dp = d | 1;
  float* Qs = sm;                      // [16][d]
  float* Ks = Qs + GA_ROWS * d;        // [KT][d | 1]
  float* Vs = Ks + KT * dp;            // [KT][dv]
  float* Ps = Vs + KT * dv;            // [16][64]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // row rr -> (token tok0 + rr / Rh, query head g R + r0 + rr % Rh); rows past nrows are idle
  for (int e = tid; e < GA_ROWS * d; e += 256) {
    const int rr = e / d, i = e % d;
    float v = 0.f;
    if (rr < nrows) v = ldf(q + ((long)(q0 + tok0 + rr / Rh) * H + g * R + r0 + rr % Rh) * d + i);
    Qs[e] = v;
  }
  float m[4], l[4], O[4][NJ];
  int rpos[4];
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int rr = wave + 4 * x;
    m[x] = -INFINITY;
    l[x] = 0.f;
    rpos[x] = rr < nrows ? p0 + tok0 + rr / Rh : -1;   // -1: sees no key
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj) O[x][jj] = 0.f;
  }
  const int last = p0 + tok0 + nq - 1;   // the newest key any row sees
  const int* btr = bt + (long)s * bt_ld;
  for (int k0 = 0; k0 <= last; k0 += KT) {
    const int nk = min(KT, last + 1 - k0);
    __syncthreads();   // the previous tile is consumed (and Qs is written)
    for (int e = tid; e < KT * d; e += 256) {
      const int kk = e / d, i = e % d;
      float v = 0.f;
      if (kk < nk) {
        const int pk = k0 + kk;
        v = ldf(kc + (((long)btr[pk / BSZ] * BSZ + pk % BSZ) * G + g) * d + i);
      }
      Ks[kk * dp + i] = v;
    }
    for (int e = tid; e < KT * dv; e += 256) {
      const int kk = e / dv, jx = e % dv;
      float v = 0.f;
      if (kk < nk) {
        const int pk = k0 + kk;
        v = ldf(vc + (((long)btr[pk / BSZ] * BSZ + pk % BSZ) * G + g) * dv + jx);
      }
      Vs[e] = v;
    }
    __syncthreads();
    // scores: lane = key; the wave's rows are wave, wave + 4, wave + 8, wave + 12
    float sc[4] = {0.f, 0.f, 0.f, 0.f};
    if (lane < KT) {
      const float* kr = Ks + lane * dp;
#pragma unroll 4
      for (int i = 0; i < d; ++i) {
        const float kv = kr[i];
#pragma unroll
        for (int x = 0; x < 4; ++x) sc[x] += Qs[(wave + 4 * x) * d + i] * kv;
      }
    }
    const int pk = k0 + lane;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const bool vis = lane < nk && pk <= rpos[x];
      const float sv = vis ? sc[x] : -INFINITY;
      const float mn = fmaxf(m[x], wave_max(sv));
      float p = 0.f, f = 1.f;
      if (mn > -INFINITY) {
        p = vis ? expf(sv - mn) : 0.f;
        f = expf(m[x] - mn);    // m = -inf before the first visible key: f = 0, and O and l are 0
      }
      l[x] = l[x] * f + wave_sum(p);
      m[x] = mn;
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) O[x][jj] *= f;
      Ps[(wave + 4 * x) * 64 + lane] = p;
    }
    __syncthreads();
    // weighted sum: lane owns value dims lane, lane + 64, ...
    for (int kk = 0; kk < nk; ++kk) {
      float vv[NJ];
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) vv[jj] = lane + 64 * jj < dv ? Vs[kk * dv + lane + 64 * jj] : 0.f;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const float p = Ps[(wave + 4 * x) * 64 + kk];
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) O[x][jj] += p * vv[jj];
      }
    }
  }
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int rr = wave + 4 * x;
    if (rr >= nrows) continue;
    const long tok = q0 + tok0 + rr / Rh;
    const int h = g * R + r0 + rr % Rh;
    const float inv = 1.f / l[x];
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj) {
      const int jx = lane + 64 * jj;
      if (jx >= dv) continue;
      float o = O[x][jj] * inv;
      if (gate) o *= 1.f / (1.f + expf(-ldf(gate + tok * ldg + (long)h * dv + jx)));
      stf(out + tok * ((long)H * dv) + (long)h * dv + jx, o);
    }
  }
}

long gqa_lds(int d, int dv, int KT) { return 4L * (GA_ROWS * d + (long)KT * (d | 1) + (long)KT * dv + GA_ROWS * 64); }

#define ENSURE_LDS(kernel, bytes)                                                                          \
  do {                                                                                                     \
    static long have_ = 48 * 1024;                                                                         \
    if ((bytes) > have_) {                                                                                 \
      hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)); \
      have_ = (bytes);                                                                                     \
    }                                                                                                      \
  } while (0)

template <typename T, int NJ>
int launch_gqa(dim3 grid, long lds, hipStream_t st, const T* q, const T* kc, const T* vc, const int* bt, int bt_ld, int BSZ,
               const int* qstart, const int* qlen, const int* ctx, const int* tile_seq, const int* tile_tok0, const T* gate,
               long ldg, T* out, int H, int G, int d, int dv, int TQ, int KT) {
  ENSURE_LDS((paged_gqa_kernel<T, NJ>), lds);
  hipLaunchKernelGGL((paged_gqa_kernel<T, NJ>), grid, dim3(256), lds, st, q, kc, vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq,
                     tile_tok0, gate, ldg, out, H, G, d, dv, TQ, KT);
  return (int)hipGetLastError();
}

template <typename T>
int launch_gqa_t(int nj, dim3 grid, long lds, hipStream_t st, const void* q, const void* kc, const void* vc, const int* bt,
                 int bt_ld, int BSZ, const int* qstart, const int* qlen, const int* ctx, const int* tile_seq,
                 const int* tile_tok0, const void* gate, long ldg, void* out, int H, int G, int d, int dv, int TQ, int KT) {
#define GQA(NJ) return launch_gqa<T, NJ>(grid, lds, st, (const T*)q, (const T*)kc, (const T*)vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq, tile_tok0, (const T*)gate, ldg, (T*)out, H, G, d, dv, TQ, KT)
  if (nj <= 1) GQA(1);
  if (nj <= 2) GQA(2);
  GQA(4);
#undef GQA
}

}  // namespace

extern "C" int dllm_attn_prep(const void* proj, long ld, int f32, int H, int G, int d, int dv, const float* cos_sin,
                              int tab_w, int rot, float eps, const float* qscale, const int* pos, const int* slots, void* kc,
                              void* vc, void* q, long T, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > d || (rot & 1) || rot > tab_w) return -1;
  if (f32)
    hipLaunchKernelGGL(attn_prep_kernel<float>, dim3((unsigned)T), dim3(256), 0, st, (const float*)proj, ld, H, G, d, dv, cos_sin,
                       tab_w, rot, eps, qscale, pos, slots, (float*)kc, (float*)vc, (float*)q);
  else
    hipLaunchKernelGGL(attn_prep_kernel<u16>, dim3((unsigned)T), dim3(256), 0, st, (const u16*)proj, ld, H, G, d, dv, cos_sin,
                       tab_w, rot, eps, qscale, pos, slots, (u16*)kc, (u16*)vc, (u16*)q);
  return (int)hipGetLastError();
}

// tokens one workgroup covers for H / G query heads per key/value head
extern "C" int dllm_gqa_tile_tokens(int H, int G) {
  const int R = H / G;
  return R >= GA_ROWS ? 1 : GA_ROWS / R;
}

extern "C" int dllm_paged_gqa(const void* q, const void* kc, const void* vc, int f32, const int* bt, int bt_ld, int BSZ,
                              const int* qstart, const int* qlen, const int* ctx, const int* tile_seq, const int* tile_tok0,
                              int n_tiles, const void* gate, long ldg, void* out, int H, int G, int d, int dv,
                              hipStream_t st) {
  if (n_tiles <= 0) return 0;
  if (G < 1 || H % G || dv > 256 || d < 1) return -1;
  int KT = 64;
  if (gqa_lds(d, dv, KT) > 150 * 1024) KT = 32;
  const long lds = gqa_lds(d, dv, KT);
  if (lds > 150 * 1024) return -2;
  const int R = H / G;
  const dim3 grid(n_tiles, G, (R + GA_ROWS - 1) / GA_ROWS);
  const int nj = (dv + 63) / 64;
  const int TQ = dllm_gqa_tile_tokens(H, G);
  if (f32)
    return launch_gqa_t<float>(nj, grid, lds, st, q, kc, vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq, tile_tok0, gate, ldg,
                               out, H, G, d, dv, TQ, KT);
  return launch_gqa_t<u16>(nj, grid, lds, st, q, kc, vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq, tile_tok0, gate, ldg, out,
                           H, G, d, dv, TQ, KT);
}
