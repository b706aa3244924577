// Latent attention: softmax attention whose keys and values are one shared compressed vector per
// token (a normed latent of `rank` dims plus a rotated key part of `rot` dims that every head
// shares).  The per-head key up-projection is absorbed into the query on the host side, so a row
// (token, head) scores key j as  q_lat . c_j + q_rot . kr_j  and returns  sum_j p_j c_j  (the value
// up-projection follows as a per-head batched GEMM).  Only [c_j | kr_j] is cached, paged in
// 16-token blocks.
//
//   latent_kv_write   one wave per token: RMS-norm the latent (f32), rotate the shared key part
//                     (interleaved pairs), write both into the token's cache slot
//   latent_attention  one workgroup per 16 rows (token-major (token, head) rows of one sequence):
//                     the rows' queries staged once in LDS as f32 (rotation and the score scale
//                     applied while staging); keys walk in tiles staged in LDS as f32;
//                     phase 1: a lane owns a key and sums q . k over the dims (q read as LDS
//                     broadcasts, k with an odd row stride: no bank conflicts) -> f32 scores, causal
//                     mask, online softmax per row (wave reductions);
//                     phase 2: a lane owns latent dims lane, lane + 64, ... and accumulates p . c.
//                     Each wave owns 4 of the 16 rows through both phases.  Small grids (decode) split
//                     a row's keys over several workgroups; latent_combine merges their partials.
// Activations and the cache are bf16 or f32 (template); scores, softmax and sums are f32.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

template <typename T>
__global__ void __launch_bounds__(64) latent_kv_write_kernel(const T* __restrict__ ckv, long ld, int rank, int rot,
                                                             const float* __restrict__ w, float eps,
                                                             const int* __restrict__ pos,
                                                             const float* __restrict__ cos_sin, int tab_w,
                                                             const int* __restrict__ slots, T* __restrict__ cache) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const int slot = slots[t];
  if (slot < 0) return;
  const T* r = ckv + (long)t * ld;
  float s = 0.f;
  for (int i = lane; i < rank; i += 64) { const float v = ldf(r + i); s += v * v; }
  s = wave_sum(s);
  const float rs = 1.f / sqrtf(s / (float)rank + eps);
  T* dst = cache + (long)slot * (rank + rot);
  for (int i = lane; i < rank; i += 64) stf(dst + i, ldf(r + i) * rs * w[i]);
  const float* cs = cos_sin + (long)pos[t] * tab_w;
  const int half = rot >> 1;
  for (int i = lane; i < half; i += 64) {
    const float u = ldf(r + rank + 2 * i), v = ldf(r + rank + 2 * i + 1);
    const float c = cs[i], sn = cs[half + i];
    stf(dst + rank + 2 * i, u * c - v * sn);
    stf(dst + rank + 2 * i + 1, v * c + u * sn);
  }
}

constexpr int LROWS = 16;

// one cache row -> f32 in LDS, lanes along the row (bf16 rows of even length move 4 bytes per lane)
__device__ __forceinline__ void stage_row(const float* src, float* dst, int Dp, int lane) {
  for (int c = lane; c < Dp; c += 64) dst[c] = src[c];
}
__device__ __forceinline__ void stage_row(const u16* src, float* dst, int Dp, int lane) {
  if ((Dp & 1) == 0) {
    const uint32_t* s2 = reinterpret_cast<const uint32_t*>(src);
    for (int c = lane; c < (Dp >> 1); c += 64) {
      const uint32_t w = s2[c];
      dst[2 * c] = __uint_as_float(w << 16);
      dst[2 * c + 1] = __uint_as_float(w & 0xffff0000u);
    }
  } else {
    for (int c = lane; c < Dp; c += 64) dst[c] = bf2f(src[c]);
  }
}

// RI: latent dims per lane in phase 2 (rank <= 64 RI)
template <typename T, int RI>
__global__ void __launch_bounds__(256) latent_attention_kernel(
    const T* __restrict__ qa, const T* __restrict__ q, long ldq, int H, int dim, int rot, int rank, long Ttot,
    const float* __restrict__ cos_sin, int tab_w, const T* __restrict__ cache, const int* __restrict__ bt, int bt_w,
    const int* __restrict__ qstart, const int* __restrict__ qlen, const int* __restrict__ ctx,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_tok0, float scale, T* __restrict__ out, int KT,
    int tpe, int kstride, int vec, int splits, float* __restrict__ part_o, float* __restrict__ part_ml) {
  extern __shared__ float sm[];
  const int entry = blockIdx.y;
  const int s = tile_seq[entry];
  const int n = qlen[s];
  if (n <= 0) return;
  const int tok0 = tile_tok0[entry];
  if (tok0 >= n) return;
  const int ntok = min(tpe, n - tok0);
  const int nrows = ntok * H;                  // rows of this entry, token-major
  const int row0 = blockIdx.x * LROWS;
  if (row0 >= nrows) return;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  const int Dp = rank + rot;
  float* qsh = sm;                              // [16][Dp]
  float* ksh = qsh + LROWS * Dp;                // [KT][kstride]
  float* psh = ksh + KT * kstride;              // [16][64]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = rot >> 1;
  // stage the rows' queries (f32, scaled): latent part from qa [H, T, rank], rotated part from q
  for (int e = tid; e < LROWS * Dp; e += 256) {
    const int rr = e / Dp, c = e % Dp, row = row0 + rr;
    float v = 0.f;
    if (row < nrows) {
      const int tl = tok0 + row / H, h = row % H;
      const long tok = q0 + tl;
      if (c < rank) {
        v = ldf(qa + ((long)h * Ttot + tok) * rank + c);
      } else {
        const int i = (c - rank) >> 1;
        const T* qr = q + tok * ldq + (long)h * (dim + rot) + dim + 2 * i;
        const float u = ldf(qr), w = ldf(qr + 1);
        const float* cs = cos_sin + (long)(p0 + tl) * tab_w;
        v = ((c - rank) & 1) ? w * cs[i] + u * cs[half + i] : u * cs[i] - w * cs[half + i];
      }
      v *= scale;
    }
    qsh[e] = v;
  }
  // causal horizon of the block: the last row's position
  const int last_row = min(row0 + LROWS, nrows) - 1;
  const int kmax = p0 + tok0 + last_row / H + 1;
  int rpos[4];
  bool rok[4];
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int row = row0 + wave * 4 + a;
    rok[a] = row < nrows;
    rpos[a] = p0 + tok0 + (rok[a] ? row / H : 0);
  }
  float m[4], l[4], acc[4][RI];
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    m[a] = -INFINITY;
    l[a] = 0.f;
#pragma unroll
    for (int i = 0; i < RI; ++i) acc[a][i] = 0.f;
  }
  const int* btr = bt + (long)s * bt_w;
  // split over keys (small grids): split z of `splits` walks its share of the key tiles and leaves
  // unnormalised partials; latent_combine merges them
  const int ntiles = (kmax + KT - 1) / KT;
  const int kbeg = (int)((long)ntiles * blockIdx.z / splits) * KT;
  const int kend = min(kmax, (int)((long)ntiles * (blockIdx.z + 1) / splits) * KT);
  for (int k0 = kbeg; k0 < kend; k0 += KT) {
    const int nk = min(KT, kend - k0);
    __syncthreads();   // the previous tile is consumed (and the queries are staged)
    // the tile's pages: read once, so the row loads below do not each wait for a block-table entry
    const int pg0 = k0 >> 4, npg = ((k0 + nk - 1) >> 4) - pg0 + 1;
    const int pg = lane < npg ? btr[pg0 + lane] : 0;
#pragma unroll 4
    for (int kk = wave; kk < nk; kk += 4) {          // a wave per key row, lanes along the row
      const int kidx = k0 + kk;
      const long page = __shfl(pg, (kidx >> 4) - pg0);
      stage_row(cache + (page * 16 + (kidx & 15)) * Dp, ksh + kk * kstride, Dp, lane);
    }
    __syncthreads();
    // phase 1: lane = key
    float sc[4] = {0.f, 0.f, 0.f, 0.f};
    if (lane < nk) {
      const float* kr = ksh + lane * kstride;
      const float* qr = qsh + (wave * 4) * Dp;
      if (vec) {          // 16-byte LDS reads: rows are 16-byte aligned, kstride / 4 is odd (no bank conflicts)
#pragma unroll 8
        for (int c = 0; c < Dp; c += 4) {
          const float4 kv = *reinterpret_cast<const float4*>(kr + c);
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            const float4 qv = *reinterpret_cast<const float4*>(qr + a * Dp + c);
            sc[a] += qv.x * kv.x + qv.y * kv.y + qv.z * kv.z + qv.w * kv.w;
          }
        }
      } else {
        for (int c = 0; c < Dp; ++c) {
          const float kv = kr[c];
#pragma unroll
          for (int a = 0; a < 4; ++a) sc[a] += qr[a * Dp + c] * kv;
        }
      }
    }
    float alpha[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const bool vis = lane < nk && rok[a] && (k0 + lane) <= rpos[a];
      const float sv = vis ? sc[a] : -INFINITY;
      const float mn = fmaxf(m[a], wave_max(sv));
      float p = 0.f;
      alpha[a] = 1.f;
      if (mn != -INFINITY) {
        p = vis ? expf(sv - mn) : 0.f;
        alpha[a] = expf(m[a] - mn);     // m = -inf -> 0
        m[a] = mn;
      }
      l[a] = l[a] * alpha[a] + wave_sum(p);
      psh[(wave * 4 + a) * 64 + lane] = p;
    }
    __syncthreads();
    // phase 2: lane = latent dim
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int i = 0; i < RI; ++i) acc[a][i] *= alpha[a];
#pragma unroll 4
    for (int kk = 0; kk < nk; ++kk) {
      float kv[RI];
#pragma unroll
      for (int i = 0; i < RI; ++i) {
        const int c = lane + 64 * i;
        kv[i] = c < rank ? ksh[kk * kstride + c] : 0.f;
      }
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const float p = psh[(wave * 4 + a) * 64 + kk];
#pragma unroll
        for (int i = 0; i < RI; ++i) acc[a][i] += p * kv[i];
      }
    }
  }
  if (splits > 1) {
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const long pr = (((long)entry * gridDim.x + blockIdx.x) * LROWS + wave * 4 + a) * splits + blockIdx.z;
      if (lane == 0) { part_ml[2 * pr] = m[a]; part_ml[2 * pr + 1] = l[a]; }
#pragma unroll
      for (int i = 0; i < RI; ++i) {
        const int c = lane + 64 * i;
        if (c < rank) part_o[pr * rank + c] = acc[a][i];
      }
    }
    return;
  }
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int row = row0 + wave * 4 + a;
    if (row >= nrows) continue;
    const long tok = q0 + tok0 + row / H;
    const int h = row % H;
    const float inv = l[a] > 0.f ? 1.f / l[a] : 0.f;
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      const int c = lane + 64 * i;
      if (c < rank) stf(out + ((long)h * Ttot + tok) * rank + c, acc[a][i] * inv);
    }
  }
}

// ---------------------------------------------------------------- bf16 models: matrix-core form
// Same row blocks, key tiles, causal mask, online softmax and key splits as above, with both products
// on v_mfma_f32_16x16x32_bf16 (operands bf16 from the cache, f32 accumulation):
//   scores   S[16 rows x 16 keys] per wave (wave w: keys 16w..16w+15 of the tile): A = query rows
//            (LDS, bf16, the rotation applied while staging, the score scale applied to the f32 sums),
//            B = key rows (LDS, row-major copy of the tile);
//   softmax  in the accumulator layout (a lane holds rows 4g..4g+3 of one key): row maxima by DPP
//            over the 16 lanes of a row group, then across the waves through LDS; a lane keeps a
//            partial row sum of its own keys until the end;
//   weights  written to LDS as bf16 hi + lo parts (p = hi + lo to 2^-17), so the second product sees
//            f32 weights to 16 bits of mantissa through two MFMAs;
//   output   O[16 rows x rank]: wave w owns latent column blocks w, w + 4, ...; A = weights (hi, lo),
//            B = a TRANSPOSED copy of the tile's latent part in LDS ([dim][key], made from the
//            row-major tile by a second pass), because the product contracts over keys and an operand
//            holds 8 consecutive contraction indices per lane.
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false)));
  return v;
}
__device__ __forceinline__ float row16_add(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));
  return v;
}

struct MfmaLds { int Dpad, qstr, ktstr, pstr, RB; long bytes; };
static inline MfmaLds mfma_lds(int rank, int rot, int KT, int rows = LROWS) {
  MfmaLds L;
  L.Dpad = (rank + rot + 31) & ~31;
  L.qstr = L.Dpad + 8;
  L.ktstr = KT + 8;
  L.pstr = KT + 8;
  L.RB = (rank + 15) / 16;
  L.bytes = 2L * (rows * L.qstr + (long)KT * L.qstr + (long)L.RB * 16 * L.ktstr + 2L * rows * L.pstr) + 4L * 4 * rows;
  return L;
}

// A key tile's rows into registers: wave w takes rows w, w + 4, ..., a lane 16 bytes of a row (two per
// row cover up to 1024 entries); rows past `kend` and lanes past the row's end get zeros.
template <int KT>
__device__ __forceinline__ void fetch_tile(uint4 (&pf)[KT / 4][2], const u16* __restrict__ cache,
                                           const int* __restrict__ btr, int k0, int kend, int Dp, int lane, int wave) {
  const int nk = min(KT, kend - k0);
  const int pg0 = k0 >> 4, npg = ((k0 + nk - 1) >> 4) - pg0 + 1;
  const int pg = lane < npg ? btr[pg0 + lane] : 0;
#pragma unroll
  for (int r = 0; r < KT / 4; ++r) {
    const int kk = wave + 4 * r, kidx = k0 + kk;
    const bool live = kk < nk;
    const long page = __shfl(pg, live ? (kidx >> 4) - pg0 : 0);
    const uint4* src = reinterpret_cast<const uint4*>(cache + (page * 16 + (kidx & 15)) * Dp);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c8 = lane + 64 * j;
      pf[r][j] = (live && c8 < (Dp >> 3)) ? src[c8] : make_uint4(0u, 0u, 0u, 0u);
    }
  }
}

// LR: 16-row blocks per workgroup (1: decode steps and short portions; 2: prompt portions, where the
// tile's staging, transposition and barriers then serve 32 rows and every wave has a score task at
// 32-key tiles).  Score tasks (row block, 16 keys) are dealt to the waves round-robin.
template <int CB, int KT, int LR>
__global__ void __launch_bounds__(256) latent_attention_mfma_kernel(
    const u16* __restrict__ qa, const u16* __restrict__ q, long ldq, int H, int dim, int rot, int rank, long Ttot,
    const float* __restrict__ cos_sin, int tab_w, const u16* __restrict__ cache, const int* __restrict__ bt, int bt_w,
    const int* __restrict__ qstart, const int* __restrict__ qlen, const int* __restrict__ ctx,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_tok0, float scale, u16* __restrict__ out,
    int tpe, int splits, float* __restrict__ part_o, float* __restrict__ part_ml, int Dpad, int qstr, int ktstr,
    int pstr, int RB) {
  constexpr int RPB = 16 * LR;                      // rows per workgroup
  constexpr int NKB = KT >> 4;                      // 16-key blocks per tile
  constexpr int NT = (LR * NKB + 3) / 4;            // score tasks per wave
  extern __shared__ __attribute__((aligned(16))) unsigned char smraw[];
  const int entry = blockIdx.y;
  const int s = tile_seq[entry];
  const int n = qlen[s];
  if (n <= 0) return;
  const int tok0 = tile_tok0[entry];
  if (tok0 >= n) return;
  const int ntok = min(tpe, n - tok0);
  const int nrows = ntok * H;
  const int row0 = blockIdx.x * RPB;
  if (row0 >= nrows) return;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  const int Dp = rank + rot;
  u16* qsh = reinterpret_cast<u16*>(smraw);             // [RPB][qstr]
  u16* ksh = qsh + RPB * qstr;                          // [KT][qstr]
  u16* ktr = ksh + KT * qstr;                           // [RB * 16][ktstr]: latent part transposed
  u16* phi = ktr + RB * 16 * ktstr;                     // [RPB][pstr]
  u16* plo = phi + RPB * pstr;
  float* wred = reinterpret_cast<float*>(plo + RPB * pstr);   // [4][RPB]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, g = lane >> 4;
  const int half = rot >> 1;
  for (int e = tid; e < RPB * Dpad; e += 256) {
    const int rr = e / Dpad, c = e - rr * Dpad, row = row0 + rr;
    float v = 0.f;
    if (row < nrows && c < Dp) {
      const int tl = tok0 + row / H, h = row % H;
      const long tok = q0 + tl;
      if (c < rank) {
        v = bf2f(qa[((long)h * Ttot + tok) * rank + c]);
      } else {
        const int i = (c - rank) >> 1;
        const u16* qr = q + tok * ldq + (long)h * (dim + rot) + dim + 2 * i;
        const float u = bf2f(qr[0]), w = bf2f(qr[1]);
        const float* cs = cos_sin + (long)(p0 + tl) * tab_w;
        v = ((c - rank) & 1) ? w * cs[i] + u * cs[half + i] : u * cs[i] - w * cs[half + i];
      }
    }
    qsh[rr * qstr + c] = f2bf(v);
  }
  // zero what no staging pass writes: the key rows' padded dims
  for (int e = tid; e < KT * qstr; e += 256) ksh[e] = 0;
  const int last_row = min(row0 + RPB, nrows) - 1;
  const int kmax = p0 + tok0 + last_row / H + 1;
  int rpos[LR][4];
  bool rok[LR][4];
  float m[LR][4], l[LR][4];
  f32x4 acc[CB][LR];
#pragma unroll
  for (int b = 0; b < LR; ++b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = row0 + 16 * b + 4 * g + i;
      rok[b][i] = row < nrows;
      rpos[b][i] = p0 + tok0 + (rok[b][i] ? row / H : 0);
      m[b][i] = -INFINITY;
      l[b][i] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < CB; ++j) acc[j][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int* btr = bt + (long)s * bt_w;
  const int ntiles = (kmax + KT - 1) / KT;
  const int kbeg = (int)((long)ntiles * blockIdx.z / splits) * KT;
  const int kend = min(kmax, (int)((long)ntiles * (blockIdx.z + 1) / splits) * KT);
  // rows of a multiple of 8 entries (and at most 1024) move as 16-byte vectors, one tile ahead
  const bool pre = (Dp & 7) == 0 && Dp <= 1024;
  uint4 pf[KT / 4][2];
  if (pre && kbeg < kend) fetch_tile<KT>(pf, cache, btr, kbeg, kend, Dp, lane, wave);
  for (int k0 = kbeg; k0 < kend; k0 += KT) {
    const int nk = min(KT, kend - k0);
    __syncthreads();
    if (pre) {
      // this tile's rows were fetched into registers while the previous tile was computed; put them
      // in LDS and start the next tile's fetch, which the products below then hide
#pragma unroll
      for (int r = 0; r < KT / 4; ++r) {
        const int kk = wave + 4 * r;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int c8 = lane + 64 * j;
          if (c8 < (Dp >> 3)) *reinterpret_cast<uint4*>(ksh + kk * qstr + 8 * c8) = pf[r][j];
        }
      }
      if (k0 + KT < kend) fetch_tile<KT>(pf, cache, btr, k0 + KT, kend, Dp, lane, wave);
    } else {
      const int pg0 = k0 >> 4, npg = ((k0 + nk - 1) >> 4) - pg0 + 1;
      const int pg = lane < npg ? btr[pg0 + lane] : 0;
#pragma unroll
      for (int r = 0; r < KT / 4; ++r) {        // a wave per key row; rows past the tile's end are zeros
        const int kk = wave + 4 * r, kidx = k0 + kk;
        const bool live = kk < nk;
        const long page = __shfl(pg, live ? (kidx >> 4) - pg0 : 0);
        const uint32_t* src = reinterpret_cast<const uint32_t*>(cache + (page * 16 + (kidx & 15)) * Dp);
        for (int c2 = lane; c2 < (Dp >> 1); c2 += 64) {
          const uint32_t w = live ? src[c2] : 0u;
          *reinterpret_cast<uint32_t*>(ksh + kk * qstr + 2 * c2) = w;
        }
      }
    }
    __syncthreads();
    // the latent part once more, transposed ([dim][key]): threads along the dims read 8 keys' entries
    // (2-byte reads of consecutive halfwords) and write them as one 16-byte vector
    {
      const int ndim = RB * 16;
      for (int e = tid; e < ndim * (KT / 8); e += 256) {
        const int kg = e / ndim, c = e - kg * ndim;
        uint32_t w4[4] = {0u, 0u, 0u, 0u};
        if (c < rank) {
          const u16* col = ksh + (8 * kg) * qstr + c;
#pragma unroll
          for (int x = 0; x < 4; ++x)
            w4[x] = (uint32_t)col[(2 * x) * qstr] | ((uint32_t)col[(2 * x + 1) * qstr] << 16);
        }
        *reinterpret_cast<uint4*>(ktr + c * ktstr + 8 * kg) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
      }
    }
    __syncthreads();
    // scores: task t of this wave is (row block, key block) number wave + 4 t
    float sv[NT][4];
    bool vis[NT][4];
    float wm[LR][4];
#pragma unroll
    for (int b = 0; b < LR; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) wm[b][i] = -INFINITY;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int task = wave + 4 * t;
      const bool on = task < LR * NKB;
      const int rb = on ? task / NKB : 0, kb = on ? task % NKB : 0;
      f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
      if (on) {
        const u16* ap = qsh + (16 * rb + lr) * qstr + 8 * g;
        const u16* bp = ksh + (16 * kb + lr) * qstr + 8 * g;
        for (int st = 0; st < Dpad; st += 32) {
          const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(ap + st));
          const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(bp + st));
          sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, sacc, 0, 0, 0);
        }
      }
      const int kidx = k0 + 16 * kb + lr;
#pragma unroll
      for (int b = 0; b < LR; ++b) {          // (static indexing of the per-row-block registers)
        if (b == rb) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            vis[t][i] = on && kidx < kend && rok[b][i] && kidx <= rpos[b][i];
            sv[t][i] = vis[t][i] ? sacc[i] * scale : -INFINITY;
            wm[b][i] = fmaxf(wm[b][i], row16_max(sv[t][i]));
          }
        }
      }
    }
    if (lr == 0) {
#pragma unroll
      for (int b = 0; b < LR; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) wred[wave * RPB + 16 * b + 4 * g + i] = wm[b][i];
    }
    __syncthreads();
    float alpha[LR][4];
#pragma unroll
    for (int b = 0; b < LR; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * b + 4 * g + i;
        const float tm = fmaxf(fmaxf(wred[r], wred[RPB + r]), fmaxf(wred[2 * RPB + r], wred[3 * RPB + r]));
        const float mn = fmaxf(m[b][i], tm);
        alpha[b][i] = mn != -INFINITY ? expf(m[b][i] - mn) : 1.f;
        m[b][i] = mn;
        l[b][i] *= alpha[b][i];
      }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int task = wave + 4 * t;
      if (task < LR * NKB) {
        const int rb = task / NKB, kb = task % NKB;
#pragma unroll
        for (int b = 0; b < LR; ++b) {
          if (b == rb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float p = (vis[t][i] && m[b][i] != -INFINITY) ? expf(sv[t][i] - m[b][i]) : 0.f;
              l[b][i] += p;
              const u16 hi = f2bf(p);
              const int r = 16 * b + 4 * g + i;
              phi[r * pstr + 16 * kb + lr] = hi;
              plo[r * pstr + 16 * kb + lr] = f2bf(p - bf2f(hi));
            }
          }
        }
      }
    }
    __syncthreads();
    // weighted latents of this wave's column blocks
#pragma unroll
    for (int j = 0; j < CB; ++j) {
      const int cb = wave + 4 * j;
      if (cb < RB) {
#pragma unroll
        for (int b = 0; b < LR; ++b)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[j][b][i] *= alpha[b][i];
        const u16* bp = ktr + (cb * 16 + lr) * ktstr + 8 * g;
        for (int ks = 0; ks < KT; ks += 32) {
          const bf16x8 bv = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(bp + ks));
#pragma unroll
          for (int b = 0; b < LR; ++b) {
            const int ro = (16 * b + lr) * pstr + ks + 8 * g;
            const bf16x8 ah = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(phi + ro));
            const bf16x8 al = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(plo + ro));
            acc[j][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, bv, acc[j][b], 0, 0, 0);
            acc[j][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, bv, acc[j][b], 0, 0, 0);
          }
        }
      }
    }
  }
  // row sums: over the 16 lanes of a row group, then over the waves
  __syncthreads();
#pragma unroll
  for (int b = 0; b < LR; ++b)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float t = row16_add(l[b][i]);
      if (lr == 0) wred[wave * RPB + 16 * b + 4 * g + i] = t;
    }
  __syncthreads();
#pragma unroll
  for (int b = 0; b < LR; ++b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * b + 4 * g + i;
      const float lt = wred[r] + wred[RPB + r] + wred[2 * RPB + r] + wred[3 * RPB + r];
      if (splits > 1) {
        const long pr = (((long)entry * gridDim.x + blockIdx.x) * RPB + r) * splits + blockIdx.z;
        if (wave == 0 && lr == 0) { part_ml[2 * pr] = m[b][i]; part_ml[2 * pr + 1] = lt; }
#pragma unroll
        for (int j = 0; j < CB; ++j) {
          const int c = (wave + 4 * j) * 16 + lr;
          if (wave + 4 * j < RB && c < rank) part_o[pr * rank + c] = acc[j][b][i];
        }
      } else {
        const int row = row0 + r;
        if (row < nrows) {
          const long tok = q0 + tok0 + row / H;
          const int h = row % H;
          const float inv = lt > 0.f ? 1.f / lt : 0.f;
#pragma unroll
          for (int j = 0; j < CB; ++j) {
            const int c = (wave + 4 * j) * 16 + lr;
            if (wave + 4 * j < RB && c < rank) out[((long)h * Ttot + tok) * rank + c] = f2bf(acc[j][b][i] * inv);
          }
        }
      }
    }
  }
}

// one wave per (entry, row): merge the splits' (max, sum, weighted latent) partials
template <typename T>
__global__ void __launch_bounds__(256) latent_combine_kernel(const float* __restrict__ part_o,
                                                             const float* __restrict__ part_ml, int splits, int gx,
                                                             int H, int rank, long Ttot, const int* __restrict__ qstart,
                                                             const int* __restrict__ qlen, const int* __restrict__ tile_seq,
                                                             const int* __restrict__ tile_tok0, int tpe, long n_rows,
                                                             T* __restrict__ out, int rpb) {
  const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  const int lane = threadIdx.x & 63;
  const int rl = (int)(r % rpb);
  const long eb = r / rpb;
  const int bx = (int)(eb % gx), entry = (int)(eb / gx);
  const int s = tile_seq[entry];
  const int n = qlen[s], tok0 = tile_tok0[entry];
  if (n <= 0 || tok0 >= n) return;
  const int row = bx * rpb + rl;
  if (row >= min(tpe, n - tok0) * H) return;
  const float* ml = part_ml + 2 * r * splits;
  float M = -INFINITY;
  for (int z = 0; z < splits; ++z) M = fmaxf(M, ml[2 * z]);
  float L = 0.f;
  for (int z = 0; z < splits; ++z) L += ml[2 * z] == -INFINITY ? 0.f : ml[2 * z + 1] * expf(ml[2 * z] - M);
  const float inv = L > 0.f ? 1.f / L : 0.f;
  const long tok = qstart[s] + tok0 + row / H;
  const int h = row % H;
  for (int c = lane; c < rank; c += 64) {
    float o = 0.f;
    for (int z = 0; z < splits; ++z)
      if (ml[2 * z] != -INFINITY) o += part_o[(r * splits + z) * rank + c] * expf(ml[2 * z] - M);
    stf(out + ((long)h * Ttot + tok) * rank + c, o * inv);
  }
}

}  // namespace

extern "C" int dllm_latent_kv_write(const void* ckv, long ld, int f32, int rank, int rot, const float* w, float eps,
                                    const int* pos, const float* cos_sin, int tab_w, const int* slots, void* cache,
                                    int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || (rot & 1) || rot > tab_w || rank < 1) return -1;
  if (f32)
    hipLaunchKernelGGL(latent_kv_write_kernel<float>, dim3(T), dim3(64), 0, st, (const float*)ckv, ld, rank, rot, w, eps, pos,
                       cos_sin, tab_w, slots, (float*)cache);
  else
    hipLaunchKernelGGL(latent_kv_write_kernel<u16>, dim3(T), dim3(64), 0, st, (const u16*)ckv, ld, rank, rot, w, eps, pos,
                       cos_sin, tab_w, slots, (u16*)cache);
  return (int)hipGetLastError();
}

namespace {
template <typename T>
int launch_latent(int ri, dim3 g, long lds, hipStream_t st, const T* qa, const T* q, long ldq, int H, int dim, int rot,
                  int rank, long Ttot, const float* cos_sin, int tab_w, const T* cache, const int* bt, int bt_w,
                  const int* qstart, const int* qlen, const int* ctx, const int* tile_seq, const int* tile_tok0,
                  float scale, T* out, int KT, int tpe, int kstride, int vec, int splits, float* part_o, float* part_ml) {
#define LAT(RI)                                                                                                        \
  do {                                                                                                                 \
    static long have_ = 48 * 1024; /* raised once per size: no attribute call inside a later stream capture */        \
    if (lds > have_) {                                                                                                 \
      hipFuncSetAttribute((const void*)latent_attention_kernel<T, RI>, hipFuncAttributeMaxDynamicSharedMemorySize,    \
                          (int)lds);                                                                                   \
      have_ = lds;                                                                                                     \
    }                                                                                                                  \
    hipLaunchKernelGGL((latent_attention_kernel<T, RI>), g, dim3(256), lds, st, qa, q, ldq, H, dim, rot, rank, Ttot,   \
                       cos_sin, tab_w, cache, bt, bt_w, qstart, qlen, ctx, tile_seq, tile_tok0, scale, out, KT, tpe,   \
                       kstride, vec, splits, part_o, part_ml);                                                         \
  } while (0)
  if (ri <= 1) LAT(1); else if (ri <= 2) LAT(2); else if (ri <= 4) LAT(4); else LAT(8);
#undef LAT
  if (splits > 1) {
    const long n_rows = (long)g.y * g.x * LROWS;
    hipLaunchKernelGGL(latent_combine_kernel<T>, dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, st, part_o, part_ml, splits,
                       (int)g.x, H, rank, Ttot, qstart, qlen, tile_seq, tile_tok0, tpe, n_rows, out, LROWS);
  }
  return (int)hipGetLastError();
}
}  // namespace

namespace {
int launch_latent_mfma(dim3 g, hipStream_t st, const u16* qa, const u16* q, long ldq, int H, int dim, int rot, int rank,
                       long Ttot, const float* cos_sin, int tab_w, const u16* cache, const int* bt, int bt_w,
                       const int* qstart, const int* qlen, const int* ctx, const int* tile_seq, const int* tile_tok0,
                       float scale, u16* out, int KT, int tpe, int splits, float* part_o, float* part_ml, int rows) {
  const MfmaLds L = mfma_lds(rank, rot, KT, rows);
  const int cbs = (L.RB + 3) / 4;
#define LATM3(CB, KTC, LRC)                                                                                                 \
  do {                                                                                                                 \
    static long have_ = 48 * 1024;                                                                                     \
    if (L.bytes > have_) {                                                                                             \
      hipFuncSetAttribute((const void*)latent_attention_mfma_kernel<CB, KTC, LRC>,                                     \
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.bytes);                                   \
      have_ = L.bytes;                                                                                                 \
    }                                                                                                                  \
    hipLaunchKernelGGL((latent_attention_mfma_kernel<CB, KTC, LRC>), g, dim3(256), L.bytes, st, qa, q, ldq, H, dim, rot, \
                       rank, Ttot, cos_sin, tab_w, cache, bt, bt_w, qstart, qlen, ctx, tile_seq, tile_tok0, scale, out, \
                       tpe, splits, part_o, part_ml, L.Dpad, L.qstr, L.ktstr, L.pstr, L.RB);                           \
  } while (0)
#define LATM2(CB, KTC)                                                                                                 \
  do {                                                                                                                 \
    if (rows == 32) LATM3(CB, KTC, 2); else LATM3(CB, KTC, 1);                                                         \
  } while (0)
#define LATM(CB)                                                                                                       \
  do {                                                                                                                 \
    if (KT == 64) LATM2(CB, 64); else LATM2(CB, 32);                                                                   \
  } while (0)
  if (cbs <= 1) LATM(1); else if (cbs <= 2) LATM(2); else if (cbs <= 4) LATM(4); else LATM(8);
#undef LATM
#undef LATM2
#undef LATM3
  if (splits > 1) {
    const long n_rows = (long)g.y * g.x * rows;
    hipLaunchKernelGGL(latent_combine_kernel<u16>, dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, st, part_o, part_ml,
                       splits, (int)g.x, H, rank, Ttot, qstart, qlen, tile_seq, tile_tok0, tpe, n_rows, out, rows);
  }
  return (int)hipGetLastError();
}
}  // namespace

// 1 when the matrix-core kernel takes this shape with `rows` (16 or 32) rows per workgroup (bf16, even
// widths, a 32-key tile fits the LDS)
extern "C" int dllm_latent_mfma_ok(int rank, int rot, int rows) {
  if ((rank & 1) || (rot & 1) || rank < 2 || rank > 512 || (rows != 16 && rows != 32)) return 0;
  return mfma_lds(rank, rot, 32, rows).bytes <= 150 * 1024;
}

extern "C" int dllm_latent_attention(const void* qa, const void* q, long ldq, int f32, int H, int dim, int rot, int rank,
                                     long Ttot, const float* cos_sin, int tab_w, const void* cache, const int* bt,
                                     int bt_w, const int* qstart, const int* qlen, const int* ctx, const int* tile_seq,
                                     const int* tile_tok0, int n_entries, float scale, void* out, int splits,
                                     float* part_o, float* part_ml, int mfma, int rows, hipStream_t st) {
  if (n_entries <= 0 || Ttot <= 0) return 0;
  if (rank < 1 || rank > 512 || rot < 0 || (rot & 1) || rot > tab_w || H < 1) return -1;
  if (splits < 1 || (splits > 1 && (!part_o || !part_ml))) return -3;
  if (mfma && !f32 && dllm_latent_mfma_ok(rank, rot, rows)) {
    const int KTm = mfma_lds(rank, rot, 64, rows).bytes <= 150 * 1024 ? 64 : 32;
    const int tpe_m = H >= rows ? 1 : rows / H;
    const dim3 gm((tpe_m * H + rows - 1) / rows, n_entries, splits);
    return launch_latent_mfma(gm, st, (const u16*)qa, (const u16*)q, ldq, H, dim, rot, rank, Ttot, cos_sin, tab_w,
                              (const u16*)cache, bt, bt_w, qstart, qlen, ctx, tile_seq, tile_tok0, scale, (u16*)out, KTm,
                              tpe_m, splits, part_o, part_ml, rows);
  }
  if (rows != LROWS) return -4;   // only the matrix-core kernel has the 32-row form
  // key rows in LDS: an odd stride for 4-byte reads; when the row length is a multiple of 4 a stride
  // that is 4 x odd, so a lane's 16-byte reads are aligned and spread over all banks
  const int Dp = rank + rot, vec = (Dp & 3) == 0;
  const int kstride = vec ? (((Dp >> 2) & 1) ? Dp : Dp + 4) : (Dp | 1);
  int KT = 64;
  while (KT > 8 && 4L * (LROWS * Dp + (long)KT * kstride + LROWS * 64) > 140 * 1024) KT >>= 1;
  const long lds = 4L * (LROWS * Dp + (long)KT * kstride + LROWS * 64);
  if (lds > 150 * 1024) return -2;
  const int tpe = H >= 16 ? 1 : 16 / H;
  if (splits < 1 || (splits > 1 && (!part_o || !part_ml))) return -3;
  const dim3 g((tpe * H + LROWS - 1) / LROWS, n_entries, splits);
  const int ri = (rank + 63) / 64;
  if (f32)
    return launch_latent<float>(ri, g, lds, st, (const float*)qa, (const float*)q, ldq, H, dim, rot, rank, Ttot, cos_sin,
                                tab_w, (const float*)cache, bt, bt_w, qstart, qlen, ctx, tile_seq, tile_tok0, scale,
                                (float*)out, KT, tpe, kstride, vec, splits, part_o, part_ml);
  return launch_latent<u16>(ri, g, lds, st, (const u16*)qa, (const u16*)q, ldq, H, dim, rot, rank, Ttot, cos_sin, tab_w,
                            (const u16*)cache, bt, bt_w, qstart, qlen, ctx, tile_seq, tile_tok0, scale, (u16*)out, KT, tpe, kstride, vec, splits, part_o, part_ml);
}
