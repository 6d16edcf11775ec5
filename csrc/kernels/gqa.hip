// Grouped-query softmax attention over paged keys / values with any head widths (gfx950, wave64).
//
//   attn_prep   one workgroup per token: rotate-half positions on the first `rot` dims of every q / k
//               head, each head to unit RMS (f32), q times a per-head scale; k and v go to their
//               page slots, q to a dense [T, H, d] buffer.
//   qk_norm_prep  attention inputs with biases, a weighted RMS norm of every q / k vector before its
//               rotation, and `maps` score maps per head (differential attention: 2): query rows of
//               one key/value head leave ordered (map, head in group), so the grouped-query kernels
//               below pair them with key head (kv head, map); diff_combine merges the two maps.
//   proj_norm_prep  attention inputs whose q / k RMS norm runs over the whole projection (all heads
//               together, weights of that length) before the rotation; rotary pairs (2i, 2i + 1) or
//               (i, i + rot / 2); a per-head q scale; optionally every value head to unit RMS.
//   paged_gqa   one workgroup per (tile of new tokens, key/value head, group of <= 16 query heads):
//               its rows are tokens x query heads of the group (<= 16).  Keys are walked in tiles
//               staged in LDS as f32; a lane owns a key for the scores (one K read feeds the wave's
//               four rows), f32 online softmax per row, then a lane owns value dims for the weighted
//               sum (one V read feeds four rows).  The output is multiplied by sigmoid(gate).
//
//   paged_gqa_mfma  the bf16 form on the matrix cores: 64 rows per workgroup, 16 per wave, so a row's
//               softmax never leaves its wave.  Q stays in registers as MFMA operands; a 64-key tile is
//               staged once for the four waves (K row-major, V already transposed in its page);
//               scores on v_mfma_f32_16x16x32_bf16 with f32 sums; online softmax in the accumulator
//               layout (row maxima over the 16 lanes of a DPP row); the weights go through the wave's
//               own LDS patch as bf16 hi + lo parts, so the weighted sum sees them to 16 bits of
//               mantissa through two MFMAs.  Key blocks above a wave's newest row are skipped.
//
// Both attention kernels take a window (a row at position p sees keys p - win < j <= p), kept first
// keys (j < keep stays visible at any distance; the tiles between the kept keys and the window are
// not read) and a sink (one more term exp(0) times `sink` in the denominator, with no value).
//
// Cache layout: K [blocks, G, block, d], V [blocks, G, dv, block] (bf16 or f32 like the activations;
// V is kept transposed inside its page because the weighted sum runs over keys); every score,
// weight and sum is f32.
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
                                                        T* __restrict__ vc, T* __restrict__ q, int BSZ) {
  const long tok = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* r = proj + tok * ld;
  const int slot = slots[tok];
  const long blk = slot >= 0 ? slot / BSZ : 0;
  const int off = slot >= 0 ? slot % BSZ : 0;
  const int half = rot >> 1;
  const float* cs = cos_sin + (long)pos[tok] * tab_w;
  const int hh = blockIdx.y * 4 + wave;     // q heads, then k heads, are consecutive in the projection
  if (hh < H + G && (hh < H || slot >= 0)) {
    const bool is_q = hh < H;
    const T* x = r + (long)hh * d;
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
    T* dst = is_q ? q + (tok * H + hh) * d : kc + ((blk * G + (hh - H)) * BSZ + off) * d;
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
  if (slot >= 0) {   // values: this workgroup's share of the G * dv entries
    const T* v = r + (long)(H + G) * d;
    for (int i = blockIdx.y * 256 + threadIdx.x; i < G * dv; i += gridDim.y * 256)
      vc[((blk * G + i / dv) * dv + i % dv) * BSZ + off] = v[i];
  }
}

// One wave per q / k vector (head, map): bias, weighted RMS norm over d, rotate-half positions on the
// first `rot` dims, q times `qscale`.  Query unit (h, m) of key/value head g = h / R leaves as row
// g M R + m R + h % R of q [T, H M, d]; key unit (g, m) goes to key head g M + m of the page.
template <typename T>
__global__ void __launch_bounds__(256) qk_norm_prep_kernel(const T* __restrict__ proj, long ld, const float* __restrict__ bias,
                                                           int H, int G, int M, int d, int dv,
                                                           const float* __restrict__ qw, const float* __restrict__ kw,
                                                           const float* __restrict__ cos_sin, int tab_w, int rot, float eps,
                                                           float qscale, const int* __restrict__ pos,
                                                           const int* __restrict__ slots, T* __restrict__ kc,
                                                           T* __restrict__ vc, T* __restrict__ q, int BSZ) {
  const long tok = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* r = proj + tok * ld;
  const int slot = kc ? slots[tok] : -1;
  const long blk = slot >= 0 ? slot / BSZ : 0;
  const int off = slot >= 0 ? slot % BSZ : 0;
  const int half = rot >> 1;
  const float* cs = cos_sin + (long)pos[tok] * tab_w;
  const int nq = H * M, nk = kc ? G * M : 0;
  const int u = blockIdx.y * 4 + wave;     // q units, then k units, are consecutive in the projection
  if (u < nq + nk && (u < nq || slot >= 0)) {
    const bool is_q = u < nq;
    const T* x = r + (long)u * d;
    const float* b = bias ? bias + (long)u * d : nullptr;
    const float* w = is_q ? qw : kw;
    float ss = 0.f;
    for (int i = lane; i < d; i += 64) {
      const float v = ldf(x + i) + (b ? b[i] : 0.f);
      ss += v * v;
    }
    const float sc = 1.f / sqrtf(wave_sum(ss) / (float)d + eps);
    T* dst;
    if (is_q) {
      const int h = u / M, m = u % M, R = H / G;
      dst = q + (tok * nq + (long)(h / R) * M * R + m * R + h % R) * d;
    } else {
      dst = kc + ((blk * nk + (u - nq)) * BSZ + off) * d;
    }
    const float os = is_q ? qscale : 1.f;
    for (int i = lane; i < d; i += 64) {
      float v = (ldf(x + i) + (b ? b[i] : 0.f)) * sc * w[i];
      if (i < rot) {
        const int f = i < half ? i : i - half;
        const int j = i < half ? i + half : i - half;
        const float c = cs[f], sn = cs[half + f];
        const float p = (ldf(x + j) + (b ? b[j] : 0.f)) * sc * w[j];
        v = i < half ? v * c - p * sn : v * c + p * sn;
      }
      stf(dst + i, v * os);
    }
  }
  if (slot >= 0) {   // values: this workgroup's share of the G * dv entries
    const long vo = (long)(nq + nk) * d;
    for (int i = blockIdx.y * 256 + threadIdx.x; i < G * dv; i += gridDim.y * 256)
      stf(vc + ((blk * G + i / dv) * dv + i % dv) * BSZ + off, ldf(r + vo + i) + (bias ? bias[vo + i] : 0.f));
  }
}

// One workgroup per token.  q (H d entries) and k (G d entries) are each normed over their whole
// length with weights qw / kw, then rotated on the first `rot` dims of every head: pairs (2i, 2i + 1)
// when `inter`, else (i, i + rot / 2), angle index i; q times qscale[head].  vnorm: every value head
// divided by its root mean square.  kc null: proj holds q alone.
template <typename T>
__global__ void __launch_bounds__(256) proj_norm_prep_kernel(const T* __restrict__ proj, long ld, int H, int G, int d, int dv,
                                                             const float* __restrict__ qw, const float* __restrict__ kw,
                                                             const float* __restrict__ cos_sin, int tab_w, int rot,
                                                             int inter, float eps, const float* __restrict__ qscale,
                                                             int vnorm, const int* __restrict__ pos,
                                                             const int* __restrict__ slots, T* __restrict__ kc,
                                                             T* __restrict__ vc, T* __restrict__ q, int BSZ,
                                                             T* __restrict__ zrow, int zn) {
  // zrow: a [T, zn] buffer whose row of this token is cleared (the attention output of a step with
  // padding rows, which no attention tile writes)
  __shared__ float red[16];
  const long tok = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (zrow)
    for (int e = tid; e < zn; e += 256) stf(zrow + tok * zn + e, 0.f);
  const T* r = proj + tok * ld;
  const int slot = kc ? slots[tok] : -1;
  const long blk = slot >= 0 ? slot / BSZ : 0;
  const int off = slot >= 0 ? slot % BSZ : 0;
  const int half = rot >> 1;
  const float* cs = cos_sin + (long)pos[tok] * tab_w;
  const int nq = H * d, nk = slot >= 0 ? G * d : 0;
  float sq = 0.f, sk = 0.f;
  for (int e = tid; e < nq; e += 256) { const float v = ldf(r + e); sq += v * v; }
  for (int e = tid; e < nk; e += 256) { const float v = ldf(r + nq + e); sk += v * v; }
  const float rq = 1.f / sqrtf(block_sum(sq, red) / (float)nq + eps);
  const float rk = nk ? 1.f / sqrtf(block_sum(sk, red) / (float)nk + eps) : 0.f;   // slot is uniform in the workgroup
  // a wave per q / k head, a lane per dim: no index arithmetic beyond adds
  const int units = H + (nk ? G : 0);
  for (int un = wave; un < units; un += 4) {
    const bool is_q = un < H;
    const int hh = is_q ? un : un - H;
    const T* x = r + (is_q ? 0 : nq) + hh * d;              // this head's columns
    const float* w = (is_q ? qw : kw) + hh * d;
    const float sc = is_q ? rq : rk;
    const float os = is_q ? qscale[hh] : 1.f;
    T* dst = is_q ? q + (tok * H + hh) * d : kc + ((blk * G + hh) * BSZ + off) * d;
    for (int i = lane; i < d; i += 64) {
      float v = ldf(x + i) * sc * w[i];
      if (i < rot) {
        int j, f;
        bool first;
        if (inter) { j = i ^ 1; f = i >> 1; first = !(i & 1); }
        else { first = i < half; j = first ? i + half : i - half; f = first ? i : i - half; }
        const float cc = cs[f], sn = cs[half + f];
        const float pv = ldf(x + j) * sc * w[j];
        v = first ? v * cc - pv * sn : v * cc + pv * sn;
      }
      stf(dst + i, v * os);
    }
  }
  if (slot >= 0) {   // values: a wave per value head
    const T* vv = r + nq + nk;
    for (int g = wave; g < G; g += 4) {
      float sv = 1.f;
      if (vnorm) {
        float ss = 0.f;
        for (int i = lane; i < dv; i += 64) { const float v = ldf(vv + g * dv + i); ss += v * v; }
        sv = 1.f / sqrtf(wave_sum(ss) / (float)dv + eps);
      }
      for (int i = lane; i < dv; i += 64) stf(vc + ((blk * G + g) * dv + i) * BSZ + off, ldf(vv + g * dv + i) * sv);
    }
  }
}

// a [T, G, 2, R, dv] f32 (the two maps' outputs) -> out [T, G R, dv] = unit-RMS(a1 - lam a2) * scale:
// one wave per (token, head)
template <typename T>
__global__ void __launch_bounds__(256) diff_combine_kernel(const float* __restrict__ a, T* __restrict__ out, long units, int H,
                                                           int G, int dv, float lam, float eps, float scale) {
  const long u = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (u >= units) return;
  const long tok = u / H;
  const int h = (int)(u % H), R = H / G;
  const float* a1 = a + ((tok * G + h / R) * 2 * R + h % R) * dv;
  const float* a2 = a1 + (long)R * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += 64) {
    const float o = a1[i] - lam * a2[i];
    ss += o * o;
  }
  const float sc = scale / sqrtf(wave_sum(ss) / (float)dv + eps);
  for (int i = lane; i < dv; i += 64) stf(out + u * dv + i, (a1[i] - lam * a2[i]) * sc);
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
                                                        int G, int d, int dv, int TQ, int KT, int win, int GV,
                                                        float* __restrict__ out32, int keep, float sink) {
  // win > 0: a row at position p sees keys p - win < j <= p, and keys j < keep.  GV value heads: key
  // head g reads value head g / (G / GV).  out32: the output stays f32.  sink: one more term of score 0
  // and that weight in the denominator.
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
  const int gv = g / (G / GV);
  const int first = win > 0 ? max(0, p0 + tok0 - win + 1) : 0;   // the oldest key any row sees
  for (int k0 = (keep > 0 ? 0 : first / KT * KT); k0 <= last; k0 += KT) {
    if (k0 >= keep && k0 + KT <= first) continue;   // between the kept keys and the window (uniform in the workgroup)
    const int nk = min(KT, last + 1 - k0);
    __syncthreads();   // the previous tile is consumed (and Qs is written)
    for (int e = tid; e < KT * d; e += 256) {
      const int kk = e / d, i = e % d;
      float v = 0.f;
      if (kk < nk) {
        const int pk = k0 + kk;
        v = ldf(kc + (((long)btr[pk / BSZ] * G + g) * BSZ + pk % BSZ) * d + i);
      }
      Ks[kk * dp + i] = v;
    }
    for (int e = tid; e < KT * dv; e += 256) {
      const int kk = e / dv, jx = e % dv;
      float v = 0.f;
      if (kk < nk) {
        const int pk = k0 + kk;
        v = ldf(vc + (((long)btr[pk / BSZ] * GV + gv) * dv + jx) * BSZ + pk % BSZ);
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
      const bool vis = lane < nk && pk <= rpos[x] && (win <= 0 || pk > rpos[x] - win || pk < keep);
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
    const float inv = 1.f / (l[x] + (sink > 0.f ? sink * expf(-m[x]) : 0.f));
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj) {
      const int jx = lane + 64 * jj;
      if (jx >= dv) continue;
      float o = O[x][jj] * inv;
      if (gate) o *= 1.f / (1.f + expf(-ldf(gate + tok * ldg + (long)h * dv + jx)));
      if (out32) out32[tok * ((long)H * dv) + (long)h * dv + jx] = o;
      else stf(out + tok * ((long)H * dv) + (long)h * dv + jx, o);
    }
  }
}

// ---------------------------------------------------------------- bf16 on the matrix cores
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

constexpr int GM_ROWS = 64, GM_KT = 64, GM_BS = 16;   // rows per workgroup, keys per tile, keys per page
typedef float f32x2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));

// SZ >= max(d, dv) in {64, 128, 256}: d is walked in SZ / 32 MFMA steps, dv in SZ / 16 column blocks
// (steps and blocks past the real widths are skipped).  d % 8 == 0 (16-byte key rows).
// MFMA operand layout (16x16x32): with lr = lane & 15, g4 = lane >> 4, A holds row lr, contraction
// indices 8 g4 .. 8 g4 + 7; B holds column lr, the same indices; the accumulator holds rows
// 4 g4 .. 4 g4 + 3 of column lr.
template <int SZ>
__global__ void __launch_bounds__(256) paged_gqa_mfma_kernel(const u16* __restrict__ q, const u16* __restrict__ kc,
                                                             const u16* __restrict__ vc, const int* __restrict__ bt,
                                                             int bt_ld, const int* __restrict__ qstart,
                                                             const int* __restrict__ qlen, const int* __restrict__ ctx,
                                                             const int* __restrict__ tile_seq,
                                                             const int* __restrict__ tile_tok0, const u16* __restrict__ gate,
                                                             long ldg, u16* __restrict__ out, int H, int G, int d, int dv,
                                                             int TQ, int splits, float* __restrict__ part, int win, int GV,
                                                             float* __restrict__ out32, int keep, float sink) {
  constexpr int DS = SZ / 32, VB = SZ / 16, NKB = GM_KT / 16;
  constexpr int KSTR = SZ + 8, VSTR = GM_KT + 8, PSTR = GM_KT + 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smraw[];
  const int s = tile_seq[blockIdx.x];
  const int n = qlen[s];
  const int tok0 = tile_tok0[blockIdx.x];
  if (n <= 0 || tok0 >= n) return;   // the whole workgroup (padding tiles)
  const int g = blockIdx.y, R = H / G;
  const int nq = min(TQ, n - tok0), nrows = nq * R;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  u16* ksh = reinterpret_cast<u16*>(smraw);          // [KT][KSTR]
  u16* vtr = ksh + GM_KT * KSTR;                      // [SZ][VSTR]: values transposed, [dim][key]
  u16* pw = vtr + SZ * VSTR;                          // [4 waves][hi | lo][16][PSTR]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, g4 = lane >> 4;
  u16* phi = pw + wave * (2 * 16 * PSTR);
  u16* plo = phi + 16 * PSTR;
  // row rr -> (token tok0 + rr / R, query head g R + rr % R)
  bf16x8 qa[DS];
  {
    const int row = 16 * wave + lr;
    const bool rk = row < nrows;
    const u16* qp = q + ((long)(q0 + tok0 + (rk ? row / R : 0)) * H + g * R + (rk ? row % R : 0)) * d;
#pragma unroll
    for (int st = 0; st < DS; ++st) {
      const int c = st * 32 + 8 * g4;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (rk && c < d) v = *reinterpret_cast<const uint4*>(qp + c);
      qa[st] = __builtin_bit_cast(bf16x8, v);
    }
  }
  int rpos[4];
  float m[4], l[4];
  f32x4 acc[VB];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 16 * wave + 4 * g4 + i;
    rpos[i] = row < nrows ? p0 + tok0 + row / R : -1;     // -1: sees no key
    m[i] = -INFINITY;
    l[i] = 0.f;
  }
#pragma unroll
  for (int cb = 0; cb < VB; ++cb) acc[cb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int wave_last = 16 * wave < nrows ? p0 + tok0 + (min(16 * wave + 15, nrows - 1)) / R : -1;
  // the oldest row of the wave; idle rows (past nrows) are masked, so a wave that has any never skips the mask
  const int wave_first = 16 * wave + 15 < nrows ? p0 + tok0 + (16 * wave) / R : -1;
  // with a window: the wave's oldest live row (tiles wholly before its window are skipped)
  const int wave_old = 16 * wave < nrows ? p0 + tok0 + (16 * wave) / R : 0x3fffffff;
  const int last = p0 + tok0 + nq - 1;   // the newest key any row sees
  const int* btr = bt + (long)s * bt_ld;
  constexpr int KCH = SZ / 8;            // 16-byte chunks of a staged key row
  constexpr int NF = SZ / 32;            // chunks of K, and of V, a thread moves per tile
  // Score block kb, column lr stands for key 4 lr + kb of the tile (K rows are staged in that order),
  // so a lane's four blocks are four neighbouring keys and its weights leave as 8-byte vectors.
  uint4 pk_[NF], pv_[NF];
  // A thread moves the same (key, chunk) and (dim, page, half) of every tile (tiles start at multiples
  // of 64 keys), so only the page ids change from tile to tile: offsets inside a page are kept.
  long koff[NF], voff[NF];
  int kkey[NF], vpg[NF];
  bool kon[NF], von[NF];
  const long kpage = (long)G * GM_BS * d, vpage = (long)GV * dv * GM_BS;
  const int gv = g / (G / GV);
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int e = tid + 256 * f;
    const int kk = e / KCH, c = (e % KCH) * 8;
    kkey[f] = kk;
    kon[f] = c < d;
    koff[f] = ((long)g * GM_BS + (kk & 15)) * d + c;
    const int j = e / (GM_KT / 8), cc = e % (GM_KT / 8);
    vpg[f] = cc >> 1;
    von[f] = j < dv;
    voff[f] = ((long)gv * dv + j) * GM_BS + 8 * (cc & 1);
  }
  auto fetch = [&](int k0) {
    const int nk = min(GM_KT, last + 1 - k0);
    const int* pg = btr + (k0 >> 4);
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      pk_[f] = make_uint4(0u, 0u, 0u, 0u);
      if (kon[f] && kkey[f] < nk) pk_[f] = *reinterpret_cast<const uint4*>(kc + pg[kkey[f] >> 4] * kpage + koff[f]);
      pv_[f] = make_uint4(0u, 0u, 0u, 0u);
      if (von[f] && 16 * vpg[f] < nk) pv_[f] = *reinterpret_cast<const uint4*>(vc + pg[vpg[f]] * vpage + voff[f]);
    }
  };
  // small grids (decode steps) split a row's key tiles over `splits` workgroups; each leaves its
  // running maximum, sum and unnormalised output in `part`, gqa_combine merges them
  const int tfirst = win > 0 ? max(0, p0 + tok0 - win + 1) / GM_KT : 0;   // the oldest tile of the window any row sees
  // kept first keys: their tiles come before the window's in the walk; tile number v of the walk is
  // tile v of the sequence for v < nkeep, else tile tfirst + v - nkeep
  const int nkeep = win > 0 ? min(tfirst, (keep + GM_KT - 1) / GM_KT) : 0;
  const int ntiles = last / GM_KT + 1 - tfirst + nkeep;
  const int vbeg = (int)((long)ntiles * blockIdx.z / splits);
  const int vend = (int)((long)ntiles * (blockIdx.z + 1) / splits);   // exclusive
  auto tile_k0 = [&](int v) { return (v < nkeep ? v : tfirst + v - nkeep) * GM_KT; };
  if (vbeg < vend) fetch(tile_k0(vbeg));
  for (int vt = vbeg; vt < vend; ++vt) {
    const int k0 = tile_k0(vt);
    __syncthreads();   // the previous tile is consumed
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const int e = tid + 256 * f;
      const int kk = e / KCH, c = (e % KCH) * 8;
      *reinterpret_cast<uint4*>(ksh + (16 * (kk & 3) + (kk >> 2)) * KSTR + c) = pk_[f];
      const int j = e / (GM_KT / 8), cc = e % (GM_KT / 8);
      *reinterpret_cast<uint4*>(vtr + j * VSTR + 8 * cc) = pv_[f];
    }
    if (vt + 1 < vend) fetch(tile_k0(vt + 1));   // the next tile's loads fly under this tile's products
    __syncthreads();
    if (k0 > wave_last) continue;   // this wave's rows see nothing of the tile (the barriers above are uniform)
    if (win > 0 && k0 >= keep && k0 + GM_KT - 1 <= wave_old - win) continue;   // ... or the tile lies before every row's window
    f32x4 sacc[NKB];
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      sacc[kb] = f32x4{0.f, 0.f, 0.f, 0.f};
      const u16* bp = ksh + (16 * kb + lr) * KSTR + 8 * g4;
#pragma unroll
      for (int st = 0; st < DS; ++st) {
        if (st * 32 < d) {
          const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(bp + st * 32));
          sacc[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[st], b, sacc[kb], 0, 0, 0);
        }
      }
    }
    float alpha[4];
    const int key0 = k0 + 4 * lr;
    // a tile below the wave's oldest row needs no mask (wave-uniform)
    const bool full = k0 + GM_KT - 1 <= wave_first && (win <= 0 || k0 > wave_last - win);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float sv[NKB];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
        sv[kb] = (full || (key0 + kb <= rpos[i] && (win <= 0 || key0 + kb > rpos[i] - win || key0 + kb < keep)))
                     ? sacc[kb][i] : -INFINITY;
      float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
      mx = row16_max(mx);
      const float mn = fmaxf(m[i], mx);
      const bool any = mn > -INFINITY;
      alpha[i] = any ? __expf(m[i] - mn) : 1.f;   // m = -inf before the first visible key: 0, and acc, l are 0
      m[i] = mn;
      l[i] *= alpha[i];
      float p[NKB];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        p[kb] = any ? __expf(sv[kb] - mn) : 0.f;   // exp(-inf) = 0 for masked keys
        l[i] += p[kb];
      }
      // p = hi + lo with both parts bf16 (the packed conversions round to nearest even)
      const uint32_t h01 = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2v{p[0], p[1]}, bf16x2v));
      const uint32_t h23 = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2v{p[2], p[3]}, bf16x2v));
      const f32x2v r01 = {p[0] - __uint_as_float(h01 << 16), p[1] - __uint_as_float(h01 & 0xffff0000u)};
      const f32x2v r23 = {p[2] - __uint_as_float(h23 << 16), p[3] - __uint_as_float(h23 & 0xffff0000u)};
      const uint32_t l01 = __builtin_bit_cast(uint32_t, __builtin_convertvector(r01, bf16x2v));
      const uint32_t l23 = __builtin_bit_cast(uint32_t, __builtin_convertvector(r23, bf16x2v));
      *reinterpret_cast<uint2*>(phi + (4 * g4 + i) * PSTR + 4 * lr) = make_uint2(h01, h23);
      *reinterpret_cast<uint2*>(plo + (4 * g4 + i) * PSTR + 4 * lr) = make_uint2(l01, l23);
    }
    __builtin_amdgcn_wave_barrier();   // the patch is this wave's own: its LDS writes are in order before the reads
    // once the running maxima have settled no row of the wave rescales: skip the sweep over the sums
    const bool rescale = __any(alpha[0] != 1.f || alpha[1] != 1.f || alpha[2] != 1.f || alpha[3] != 1.f);
#pragma unroll
    for (int cb = 0; cb < VB; ++cb) {
      if (cb * 16 >= dv) continue;
      if (rescale) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[cb][i] *= alpha[i];
      }
      const u16* bp = vtr + (16 * cb + lr) * VSTR + 8 * g4;
#pragma unroll
      for (int ks = 0; ks < GM_KT; ks += 32) {
        if (k0 + ks > wave_last) continue;
        const bf16x8 bv = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(bp + ks));
        const bf16x8 ah = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(phi + lr * PSTR + ks + 8 * g4));
        const bf16x8 al = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(plo + lr * PSTR + ks + 8 * g4));
        acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, bv, acc[cb], 0, 0, 0);
        acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, bv, acc[cb], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lt = row16_add(l[i]);
    const int row = 16 * wave + 4 * g4 + i;
    if (row >= nrows) continue;
    if (part) {
      float* pr = part + ((((long)blockIdx.x * G + g) * splits + blockIdx.z) * GM_ROWS + row) * (dv + 2);
      if (lr == 0) { pr[0] = m[i]; pr[1] = lt; }
#pragma unroll
      for (int cb = 0; cb < VB; ++cb)
        if (16 * cb + lr < dv) pr[2 + 16 * cb + lr] = acc[cb][i];
      continue;
    }
    const long tok = q0 + tok0 + row / R;
    const int h = g * R + row % R;
    const float inv = 1.f / (lt + (sink > 0.f ? sink * __expf(-m[i]) : 0.f));
#pragma unroll
    for (int cb = 0; cb < VB; ++cb) {
      const int jx = 16 * cb + lr;
      if (jx >= dv) continue;
      float o = acc[cb][i] * inv;
      if (gate) o *= 1.f / (1.f + expf(-bf2f(gate[tok * ldg + (long)h * dv + jx])));
      if (out32) out32[tok * ((long)H * dv) + (long)h * dv + jx] = o;
      else out[tok * ((long)H * dv) + (long)h * dv + jx] = f2bf(o);
    }
  }
}

// merge the key splits of paged_gqa_mfma: one wave per (tile, kv head, row)
__global__ void __launch_bounds__(256) gqa_combine_kernel(const float* __restrict__ part, int splits,
                                                          const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                          const int* __restrict__ tile_seq,
                                                          const int* __restrict__ tile_tok0, const u16* __restrict__ gate,
                                                          long ldg, u16* __restrict__ out, int H, int G, int dv, int TQ,
                                                          float* __restrict__ out32, float sink) {
  const int s = tile_seq[blockIdx.x];
  const int n = qlen[s], tok0 = tile_tok0[blockIdx.x];
  if (n <= 0 || tok0 >= n) return;
  const int g = blockIdx.y, R = H / G;
  const int nrows = min(TQ, n - tok0) * R;
  const int lane = threadIdx.x & 63;
  for (int row = blockIdx.z * 4 + (threadIdx.x >> 6); row < nrows; row += 4 * gridDim.z) {
    const float* pr = part + (((long)blockIdx.x * G + g) * splits * GM_ROWS + row) * (dv + 2);
    const long zs = (long)GM_ROWS * (dv + 2);
    // lane z holds split z's maximum and sum (splits <= 64); weights travel by shuffles
    const float mz = lane < splits ? pr[lane * zs] : -INFINITY;
    const float lz = lane < splits ? pr[lane * zs + 1] : 0.f;
    const float M = wave_max(mz);
    const float wz = mz > -INFINITY ? expf(mz - M) : 0.f;
    const float L = wave_sum(lz * wz) + (sink > 0.f ? sink * expf(-M) : 0.f);
    const long tok = qstart[s] + tok0 + row / R;
    const int h = g * R + row % R;
    for (int j0 = 0; j0 < dv; j0 += 64) {     // every lane stays in the loop: the shuffles read all lanes
      const int jx = j0 + lane;
      const bool on = jx < dv;
      float o = 0.f;
#pragma unroll 4
      for (int z = 0; z < splits; ++z) {
        const float w = __shfl(wz, z, 64);
        if (on) o += pr[z * zs + 2 + jx] * w;
      }
      if (!on) continue;
      o /= L;
      if (gate) o *= 1.f / (1.f + expf(-bf2f(gate[tok * ldg + (long)h * dv + jx])));
      if (out32) out32[tok * ((long)H * dv) + (long)h * dv + jx] = o;
      else out[tok * ((long)H * dv) + (long)h * dv + jx] = f2bf(o);
    }
  }
}

long gqa_mfma_lds(int SZ) { return 2L * (GM_KT * (SZ + 8) + (long)SZ * (GM_KT + 8) + 4L * 2 * 16 * (GM_KT + 8)); }

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
               long ldg, T* out, int H, int G, int d, int dv, int TQ, int KT, int win, int GV, float* out32, int keep,
               float sink) {
  ENSURE_LDS((paged_gqa_kernel<T, NJ>), lds);
  hipLaunchKernelGGL((paged_gqa_kernel<T, NJ>), grid, dim3(256), lds, st, q, kc, vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq,
                     tile_tok0, gate, ldg, out, H, G, d, dv, TQ, KT, win, GV, out32, keep, sink);
  return (int)hipGetLastError();
}

template <typename T>
int launch_gqa_t(int nj, dim3 grid, long lds, hipStream_t st, const void* q, const void* kc, const void* vc, const int* bt,
                 int bt_ld, int BSZ, const int* qstart, const int* qlen, const int* ctx, const int* tile_seq,
                 const int* tile_tok0, const void* gate, long ldg, void* out, int H, int G, int d, int dv, int TQ, int KT,
                 int win, int GV, float* out32, int keep, float sink) {
#define GQA(NJ) return launch_gqa<T, NJ>(grid, lds, st, (const T*)q, (const T*)kc, (const T*)vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq, tile_tok0, (const T*)gate, ldg, (T*)out, H, G, d, dv, TQ, KT, win, GV, out32, keep, sink)
  if (nj <= 1) GQA(1);
  if (nj <= 2) GQA(2);
  GQA(4);
#undef GQA
}

}  // namespace

extern "C" int dllm_attn_prep(const void* proj, long ld, int f32, int H, int G, int d, int dv, const float* cos_sin,
                              int tab_w, int rot, float eps, const float* qscale, const int* pos, const int* slots, void* kc,
                              void* vc, void* q, long T, int BSZ, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > d || (rot & 1) || rot > tab_w) return -1;
  const dim3 grid((unsigned)T, (H + G + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(attn_prep_kernel<float>, grid, dim3(256), 0, st, (const float*)proj, ld, H, G, d, dv, cos_sin, tab_w, rot,
                       eps, qscale, pos, slots, (float*)kc, (float*)vc, (float*)q, BSZ);
  else
    hipLaunchKernelGGL(attn_prep_kernel<u16>, grid, dim3(256), 0, st, (const u16*)proj, ld, H, G, d, dv, cos_sin, tab_w, rot, eps,
                       qscale, pos, slots, (u16*)kc, (u16*)vc, (u16*)q, BSZ);
  return (int)hipGetLastError();
}

// The matrix-core form takes bf16, 16-key pages, key rows of whole 16-byte vectors, widths <= 256 and
// at most 64 query heads per key/value head.
extern "C" int dllm_gqa_mfma_ok(int f32, int H, int G, int d, int dv, int BSZ) {
  return !f32 && BSZ == GM_BS && G >= 1 && H % G == 0 && H / G <= GM_ROWS && d % 8 == 0 && d <= 256 && dv <= 256 && d >= 8;
}

// tokens one workgroup covers for H / G query heads per key/value head
extern "C" int dllm_gqa_tile_tokens(int H, int G, int mfma) {
  const int R = H / G, rows = mfma ? GM_ROWS : GA_ROWS;
  return R >= rows ? 1 : rows / R;
}

extern "C" int dllm_paged_gqa(const void* q, const void* kc, const void* vc, int f32, const int* bt, int bt_ld, int BSZ,
                              const int* qstart, const int* qlen, const int* ctx, const int* tile_seq, const int* tile_tok0,
                              int n_tiles, const void* gate, long ldg, void* out, int H, int G, int d, int dv, int mfma,
                              int splits, float* part, int win, int GV, int out_f32, int keep, float sink, hipStream_t st) {
  if (n_tiles <= 0) return 0;
  if (G < 1 || H % G || dv > 256 || d < 1 || GV < 1 || G % GV || win < 0 || keep < 0 || sink < 0.f) return -1;
  if (win <= 0) keep = 0;     // without a window every key is seen anyway
  float* out32 = out_f32 ? (float*)out : nullptr;
  if (mfma) {
    if (!dllm_gqa_mfma_ok(f32, H, G, d, dv, BSZ)) return -1;
    const int sz = d > dv ? d : dv;
    if (splits < 1 || (splits > 1 && !part)) return -1;
    const dim3 grid(n_tiles, G, splits);
    const int TQ = dllm_gqa_tile_tokens(H, G, 1);
    float* pp = splits > 1 ? part : nullptr;
#define GQM(SZ)                                                                                                          \
  do {                                                                                                                   \
    const long lds = gqa_mfma_lds(SZ);                                                                                   \
    ENSURE_LDS(paged_gqa_mfma_kernel<SZ>, lds);                                                                          \
    hipLaunchKernelGGL(paged_gqa_mfma_kernel<SZ>, grid, dim3(256), lds, st, (const u16*)q, (const u16*)kc, (const u16*)vc, bt, \
                       bt_ld, qstart, qlen, ctx, tile_seq, tile_tok0, (const u16*)gate, ldg, (u16*)out, H, G, d, dv, TQ, \
                       splits, pp, win, GV, out32, keep, sink);                                                          \
  } while (0)
    if (sz <= 64) GQM(64); else if (sz <= 128) GQM(128); else GQM(256);
#undef GQM
    if (pp) {
      const int rows = (TQ * (H / G) < GM_ROWS ? TQ * (H / G) : GM_ROWS);
      hipLaunchKernelGGL(gqa_combine_kernel, dim3(n_tiles, G, (rows + 3) / 4), dim3(256), 0, st, pp, splits, qstart, qlen,
                         tile_seq, tile_tok0, (const u16*)gate, ldg, (u16*)out, H, G, dv, TQ, out32, sink);
    }
    return (int)hipGetLastError();
  }
  int KT = 64;
  if (gqa_lds(d, dv, KT) > 150 * 1024) KT = 32;
  const long lds = gqa_lds(d, dv, KT);
  if (lds > 150 * 1024) return -2;
  const int R = H / G;
  const dim3 grid(n_tiles, G, (R + GA_ROWS - 1) / GA_ROWS);
  const int nj = (dv + 63) / 64;
  const int TQ = dllm_gqa_tile_tokens(H, G, 0);
  if (f32)
    return launch_gqa_t<float>(nj, grid, lds, st, q, kc, vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq, tile_tok0, gate, ldg,
                               out, H, G, d, dv, TQ, KT, win, GV, out32, keep, sink);
  return launch_gqa_t<u16>(nj, grid, lds, st, q, kc, vc, bt, bt_ld, BSZ, qstart, qlen, ctx, tile_seq, tile_tok0, gate, ldg, out,
                           H, G, d, dv, TQ, KT, win, GV, out32, keep, sink);
}

extern "C" int dllm_qk_norm_prep(const void* proj, long ld, int f32, const float* bias, int H, int G, int M, int d, int dv,
                                 const float* qw, const float* kw, const float* cos_sin, int tab_w, int rot, float eps,
                                 float qscale, const int* pos, const int* slots, void* kc, void* vc, void* q, long T, int BSZ,
                                 hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > d || (rot & 1) || rot > tab_w || H < 1 || G < 1 || H % G || M < 1) return -1;
  const int units = H * M + (kc ? G * M : 0);
  const dim3 grid((unsigned)T, (units + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(qk_norm_prep_kernel<float>, grid, dim3(256), 0, st, (const float*)proj, ld, bias, H, G, M, d, dv, qw, kw,
                       cos_sin, tab_w, rot, eps, qscale, pos, slots, (float*)kc, (float*)vc, (float*)q, BSZ);
  else
    hipLaunchKernelGGL(qk_norm_prep_kernel<u16>, grid, dim3(256), 0, st, (const u16*)proj, ld, bias, H, G, M, d, dv, qw, kw,
                       cos_sin, tab_w, rot, eps, qscale, pos, slots, (u16*)kc, (u16*)vc, (u16*)q, BSZ);
  return (int)hipGetLastError();
}

extern "C" int dllm_diff_combine(const float* a, void* out, int f32, long T, int H, int G, int dv, float lam, float eps,
                                 float scale, hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || H % G) return -1;
  const long units = T * H;
  const dim3 grid((unsigned)((units + 3) / 4));
  if (f32)
    hipLaunchKernelGGL(diff_combine_kernel<float>, grid, dim3(256), 0, st, a, (float*)out, units, H, G, dv, lam, eps, scale);
  else
    hipLaunchKernelGGL(diff_combine_kernel<u16>, grid, dim3(256), 0, st, a, (u16*)out, units, H, G, dv, lam, eps, scale);
  return (int)hipGetLastError();
}

extern "C" int dllm_proj_norm_prep(const void* proj, long ld, int f32, int H, int G, int d, int dv, const float* qw,
                                   const float* kw, const float* cos_sin, int tab_w, int rot, int inter, float eps,
                                   const float* qscale, int vnorm, const int* pos, const int* slots, void* kc, void* vc, void* q,
                                   long T, int BSZ, void* zrow, int zn, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > d || (rot & 1) || rot > tab_w || H < 1 || G < 1 || H % G) return -1;
  const dim3 grid((unsigned)T);
  if (f32)
    hipLaunchKernelGGL(proj_norm_prep_kernel<float>, grid, dim3(256), 0, st, (const float*)proj, ld, H, G, d, dv, qw, kw, cos_sin,
                       tab_w, rot, inter, eps, qscale, vnorm, pos, slots, (float*)kc, (float*)vc, (float*)q, BSZ, (float*)zrow, zn);
  else
    hipLaunchKernelGGL(proj_norm_prep_kernel<u16>, grid, dim3(256), 0, st, (const u16*)proj, ld, H, G, d, dv, qw, kw, cos_sin,
                       tab_w, rot, inter, eps, qscale, vnorm, pos, slots, (u16*)kc, (u16*)vc, (u16*)q, BSZ, (u16*)zrow, zn);
  return (int)hipGetLastError();
}
