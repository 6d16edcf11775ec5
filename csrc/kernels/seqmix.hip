// Sequence mixers beside softmax attention, and the f32 residual stream (gfx950, wave64).
//
//   rms_rows         y = x / sqrt(mean(x^2) + eps) (* w): one wave per row, any row length, strided rows
//   norm_resadd      x (f32) += rmsnorm(y) * w, plus the stream rounded to the model dtype: one
//                    workgroup per token
//   conv_silu        short causal convolution per channel + SiLU over a packed batch: token-parallel;
//                    the inputs before a sequence's first new token come from its state slot
//   scan             Mamba-1 selective scan: 16 lanes per channel share its states, tokens in order;
//                    softplus, decay, state and the output gate in f32; refills the convolution state
//   retention        decayed linear attention: one workgroup per (sequence, head), the [dim x vdim]
//                    state in LDS, rotate-half positions applied while q / k are staged, unit-RMS
//                    heads and the SiLU gate in the same launch
//   retention_chunk  the same recurrence for prompt portions in its chunked form (32 tokens at a time:
//                    scores inside the chunk + the carried state), one workgroup per (head, 32 value
//                    columns, sequence); retention_finish norms and gates
//   resadd_norm      x (f32) += rmsnorm(y) * w with y one branch or the normed average of two, plus the
//                    next sublayer's normed input; depth_mix: a weighted sum over the f32 stack of
//                    layer results, plus the normed input of the next layer; gelu_erf; conv_refill
//   relu2_scale      relu(x)^2 (* a per-(token, expert) gate): squared-ReLU experts, dense form
//   dense_gate       top-k (id, weight) pairs -> [T, E] gate matrix
//   polynorm         a N(z) + b N(z^2) + c N(z^3) + e per row (N: to unit RMS), one workgroup per row
//   group_router     sigmoid scores, group-limited top-k, weights = scores: one wave per token
//   swiglu_scale     silu(gate) * up * a per-(token, expert) weight: SwiGLU experts, dense form
//   softcap          cap * tanh(x / cap) in f32;  gated_group_norm: rmsnorm in parts of y silu(z)
//   ls_resadd_ln     x (f32) += ls * (y + bias + sigmoid(g) y2 + hw h), then the layer norm (mean and
//                    variance, weight and bias) of the next sublayer's input: one workgroup per token
//   glu_act          gated activations of a fused gate | up projection: SiLU gate, or clamped with
//                    g sigmoid(alpha g) (u + 1)
//   route_topk       group-limited top-k routing with sigmoid or softmax scores, a correction on the
//                    choice and identity experts (group_router is its sigmoid / two-best form)
//
// Activations are bf16 or f32 (template T = u16 / float); every sum, state, norm and gate is f32.
// Sequence metadata: qstart / qlen / ctx / rows per sequence (int32); a sequence with qlen 0 is
// skipped, one whose first new position (ctx - qlen) is 0 starts from a zero state.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }

// ---------------------------------------------------------------- rms_rows
template <typename TI, typename TO>
__global__ void __launch_bounds__(256) rms_rows_kernel(const TI* __restrict__ x, long ldx, const float* __restrict__ w,
                                                       TO* __restrict__ y, long ldy, int rows, int n, float eps,
                                                       int groups) {
  // a wave per (row, part): `groups` equal consecutive parts of a row, each by its own root mean square
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (unit >= rows * groups) return;
  const int row = unit / groups, c0 = (unit % groups) * n;
  const TI* xr = x + (long)row * ldx + c0;
  float s = 0.f;
  for (int i = lane; i < n; i += 64) { const float v = ldf(xr + i); s += v * v; }
  s = wave_sum(s);
  const float r = 1.f / sqrtf(s / (float)n + eps);
  TO* yr = y + (long)row * ldy + c0;
  for (int i = lane; i < n; i += 64) stf(yr + i, ldf(xr + i) * r * (w ? w[c0 + i] : 1.f));
}

// ---------------------------------------------------------------- norm_resadd
template <typename T>
__global__ void __launch_bounds__(256) norm_resadd_kernel(const T* __restrict__ y, long ldy, const float* __restrict__ w,
                                                          float* __restrict__ x, T* __restrict__ xl, int H, float eps,
                                                          int groups, const float* __restrict__ bias) {
  __shared__ float red[16];
  const long row = blockIdx.x;
  const T* yr = y + row * ldy;
  float* xr = x + row * (long)H;
  if (groups > 1) {   // a wave per part of the row: no workgroup barrier
    const int n = H / groups, lane = threadIdx.x & 63;
    for (int g = threadIdx.x >> 6; g < groups; g += 4) {
      const int c0 = g * n;
      float s = 0.f;
      for (int i = lane; i < n; i += 64) { const float v = ldf(yr + c0 + i) + (bias ? bias[c0 + i] : 0.f); s += v * v; }
      const float r = 1.f / sqrtf(wave_sum(s) / (float)n + eps);
      for (int i = lane; i < n; i += 64) {
        const float v = xr[c0 + i] + (ldf(yr + c0 + i) + (bias ? bias[c0 + i] : 0.f)) * r * w[c0 + i];
        xr[c0 + i] = v;
        if (xl) stf(xl + row * (long)H + c0 + i, v);
      }
    }
    return;
  }
  float s = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) { const float v = ldf(yr + i) + (bias ? bias[i] : 0.f); s += v * v; }
  const float r = 1.f / sqrtf(block_sum(s, red) / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256) {
    const float v = xr[i] + (ldf(yr + i) + (bias ? bias[i] : 0.f)) * r * w[i];
    xr[i] = v;
    if (xl) stf(xl + row * (long)H + i, v);
  }
}

// ---------------------------------------------------------------- resadd_norm, depth_mix, gelu
// The tail of a sublayer whose output is normed before the add, and the norm ahead of the next
// sublayer, for one token per workgroup:
//   y = a                                        (one branch)
//   y = (rmsnorm(a) wa + rmsnorm(b) wb) / 2      (two mixers side by side)
//   x += rmsnorm(y) w_post;  xn = rmsnorm(x) w_next  (xn = x rounded when w_next is null)
template <typename T>
__global__ void __launch_bounds__(256) resadd_norm_kernel(const T* __restrict__ a, long lda, const T* __restrict__ b,
                                                          long ldb, const float* __restrict__ wa,
                                                          const float* __restrict__ wb, const float* __restrict__ w_post,
                                                          float* __restrict__ x, const float* __restrict__ w_next,
                                                          T* __restrict__ xn, int H, float eps,
                                                          const float* __restrict__ dw, int dn, long TH) {
  __shared__ float red[16];
  extern __shared__ float yb[];   // [H]; entry i is touched by thread i % 256 only
  const long row = blockIdx.x;
  const T* ar = a + row * lda;
  const T* br = b ? b + row * ldb : nullptr;
  float ra = 1.f, rb = 1.f;
  if (br) {
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
      const float va = ldf(ar + i), vb = ldf(br + i);
      sa += va * va;
      sb += vb * vb;
    }
    ra = 1.f / sqrtf(block_sum(sa, red) / (float)H + eps);
    rb = 1.f / sqrtf(block_sum(sb, red) / (float)H + eps);
  }
  float sy = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float y = ldf(ar + i);
    if (br) y = 0.5f * (y * ra * wa[i] + ldf(br + i) * rb * wb[i]);
    yb[i] = y;
    sy += y * y;
  }
  const float ry = 1.f / sqrtf(block_sum(sy, red) / (float)H + eps);
  float* xr = x + row * (long)H;
  float sx = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float v = xr[i] + yb[i] * ry * w_post[i];
    xr[i] = v;
    if (dw) {
      // the layer ends here: x is slot dn - 1 of the f32 stack (slot 0 lies dn - 1 slots before it);
      // the weighted sum over slots 0 .. dn - 1 goes to slot dn and on to the next norm
      const float* p0 = xr + i - (long)(dn - 1) * TH;
      float acc = 0.f;
      for (int j = 0; j + 1 < dn; ++j) acc += dw[j] * p0[j * TH];
      acc += dw[dn - 1] * v;
      xr[i + TH] = acc;
      v = acc;
    }
    yb[i] = v;
    sx += v * v;
  }
  if (!xn) return;
  float rx = 1.f;
  if (w_next) rx = 1.f / sqrtf(block_sum(sx, red) / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256) stf(xn + row * (long)H + i, w_next ? yb[i] * rx * w_next[i] : yb[i]);
}

// X[n] = sum_{j<n} w[j] X[j] for one token per workgroup (X [slots][T][H] f32), xn = rmsnorm(X[n]) w_next
template <typename T>
__global__ void __launch_bounds__(256) depth_mix_kernel(float* __restrict__ X, const float* __restrict__ w, int n, long TH,
                                                        const float* __restrict__ w_next, T* __restrict__ xn, int H,
                                                        float eps) {
  __shared__ float red[16];
  extern __shared__ float yb[];
  const long row = blockIdx.x;
  float sx = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    const float* p = X + row * (long)H + i;
    float acc = 0.f;
    for (int j = 0; j < n; ++j) acc += w[j] * p[j * TH];
    X[n * TH + row * (long)H + i] = acc;
    yb[i] = acc;
    sx += acc * acc;
  }
  if (!xn) return;
  float rx = 1.f;
  if (w_next) rx = 1.f / sqrtf(block_sum(sx, red) / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256) stf(xn + row * (long)H + i, w_next ? yb[i] * rx * w_next[i] : yb[i]);
}

template <typename T>
__global__ void __launch_bounds__(256) gelu_erf_kernel(const T* __restrict__ x, T* __restrict__ y, long n) {
  for (long e = (long)blockIdx.x * 256 + threadIdx.x; e < n; e += (long)gridDim.x * 256) {
    const float v = ldf(x + e);
    stf(y + e, 0.5f * v * (1.f + erff(v * 0.70710678118654752f)));
  }
}

// the last K - 1 inputs of every sequence go to its slot (read before they are overwritten)
template <typename T>
__global__ void __launch_bounds__(256) conv_refill_kernel(const T* __restrict__ x, long ldx, T* __restrict__ conv, int Km1,
                                                          int C, const int* __restrict__ qstart,
                                                          const int* __restrict__ qlen, const int* __restrict__ ctx,
                                                          const int* __restrict__ rows) {
  const int s = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  const int n = qlen[s];
  if (n <= 0 || c >= C) return;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  T* cs = conv + (long)rows[s] * Km1 * C + c;
  float u[8];
  for (int k = 0; k < Km1; ++k) {
    const int i = n - Km1 + k;
    u[k] = i >= 0 ? ldf(x + (long)(q0 + i) * ldx + c) : (p0 > 0 ? ldf(cs + (long)(Km1 + i) * C) : 0.f);
  }
  for (int k = 0; k < Km1; ++k) stf(cs + (long)k * C, u[k]);
}

// ---------------------------------------------------------------- causal conv + SiLU
// x and y may be the same buffer in a step of single tokens (every output element is written by the
// thread that alone has read its input), so neither is declared restrict.
template <typename T>
__global__ void __launch_bounds__(256) conv_silu_kernel(const T* x, long ldx, const float* __restrict__ w,
                                                        const float* __restrict__ b, const T* state,
                                                        const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                        const int* __restrict__ ctx, const int* __restrict__ rows,
                                                        T* y, int C, int K, T* refill, int act) {
  // act 0: y = silu(b + conv);  act 1: y = x + b + conv (an input convolution ahead of a mixer)
  const int s = blockIdx.y;
  const int n = qlen[s];
  if (n <= 0) return;
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  if (c >= C) return;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  const T* st = state + (long)rows[s] * (K - 1) * C;
  const int step = 4 * gridDim.z;
  const float bias = b[c];
  float x0 = 0.f;     // the first token's own input (read before its output is stored)
  for (int j = blockIdx.z * 4 + (threadIdx.x >> 6); j < n; j += step) {
    float acc = bias;
    for (int k = 0; k + 1 < K; ++k) {
      const int i = j - (K - 1) + k;
      float u = 0.f;
      if (i >= 0) u = ldf(x + (long)(q0 + i) * ldx + c);
      else if (p0 > 0) u = ldf(st + (long)(K - 1 + i) * C + c);
      acc += w[c * K + k] * u;
    }
    const float xj = ldf(x + (long)(q0 + j) * ldx + c);
    if (j == 0) x0 = xj;
    acc += w[c * K + K - 1] * xj;
    stf(y + (long)(q0 + j) * C + c, act ? acc + xj : silu_f(acc));
  }
  // decode steps (`refill` set; every sequence brings one token, which this thread alone has read
  // the slot for): shift the slot's inputs by one and append the token's, in the same launch
  if (refill && n == 1 && K > 1 && blockIdx.z == 0 && (threadIdx.x >> 6) == 0) {
    T* sw = refill + (long)rows[s] * (K - 1) * C + c;
    for (int k = 0; k + 1 < K - 1; ++k) stf(sw + (long)k * C, p0 > 0 ? ldf(sw + (long)(k + 1) * C) : 0.f);
    stf(sw + (long)(K - 2) * C, x0);
  }
}

// The same convolution for prompt portions of bf16 rows of whole 16-byte vectors: a lane owns 8
// neighbouring channels (one vector), a wave walks a run of CV_RUN consecutive tokens with the last
// K - 1 input rows in registers, so every input row is loaded once per run (plus K - 1 rows of history
// at its start) and every output row leaves as one vector store.
constexpr int CV_RUN = 8;
template <int K>
__global__ void __launch_bounds__(256) conv_vec_kernel(const u16* __restrict__ x, long ldx, const float* __restrict__ w,
                                                       const float* __restrict__ b, const u16* __restrict__ state,
                                                       const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                       const int* __restrict__ ctx, const int* __restrict__ rows,
                                                       u16* __restrict__ y, int C, int act) {
  const int s = blockIdx.y;
  const int n = qlen[s];
  if (n <= 0) return;
  const int c = (blockIdx.x * 64 + (threadIdx.x & 63)) * 8;
  if (c >= C) return;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  const u16* st = state + (long)rows[s] * (K - 1) * C;
  float wk[K][8], bias[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    bias[e] = b[c + e];
#pragma unroll
    for (int k = 0; k < K; ++k) wk[k][e] = w[(c + e) * K + k];
  }
  const int stride = 4 * gridDim.z * CV_RUN;
  for (int j0 = (blockIdx.z * 4 + (threadIdx.x >> 6)) * CV_RUN; j0 < n; j0 += stride) {
    float hist[K > 1 ? K - 1 : 1][8];
#pragma unroll
    for (int k = 0; k + 1 < K; ++k) {
      const int i = j0 - (K - 1) + k;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (i >= 0) v = ld16(x + (long)(q0 + i) * ldx + c);
      else if (p0 > 0) v = ld16(st + (long)(K - 1 + i) * C + c);
      unpack8(v, hist[k]);
    }
    const int jn = min(CV_RUN, n - j0);
    for (int jj = 0; jj < jn; ++jj) {
      float cur[8], o[8];
      unpack8(ld16(x + (long)(q0 + j0 + jj) * ldx + c), cur);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float acc = bias[e];
#pragma unroll
        for (int k = 0; k + 1 < K; ++k) acc += wk[k][e] * hist[k][e];
        acc += wk[K - 1][e] * cur[e];
        o[e] = act ? acc + cur[e] : silu_f(acc);
      }
      st16(y + (long)(q0 + j0 + jj) * C + c, pack8(o));
#pragma unroll
      for (int k = 0; k + 2 < K; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) hist[k][e] = hist[k + 1][e];
      if (K > 1) {
#pragma unroll
        for (int e = 0; e < 8; ++e) hist[K - 2][e] = cur[e];
      }
    }
  }
}

// ---------------------------------------------------------------- selective scan
// 16 lanes per channel; lane `sub` owns states sub, sub + 16, ... (NS of them).  Tokens run in
// groups of 16: the group's B / C rows are staged once per workgroup in LDS (every channel reads the
// same rows), and lane `sub` of a channel prepares token `sub` of the group (softplus step, input,
// gate) and finishes it (skip term, SiLU gate, store), so the serial part of a token is only the
// state update itself: NS exponentials and multiply-adds, a 16-lane sum, two broadcasts.
// sum over the 16 lanes of a DPP row (rotations inside the row): every lane ends with the total
__device__ __forceinline__ float row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));  // row_ror:8
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));  // row_ror:4
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));  // row_ror:2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));  // row_ror:1
  return v;
}

template <typename T> struct fastexp;
template <> struct fastexp<u16> { static __device__ __forceinline__ float f(float x) { return __expf(x); } };
template <> struct fastexp<float> { static __device__ __forceinline__ float f(float x) { return expf(x); } };

template <typename T, int NS>
__global__ void __launch_bounds__(256) scan_kernel(const T* __restrict__ xc, const T* __restrict__ dt_raw,
                                                   const float* __restrict__ dt_bias, const float* __restrict__ A,
                                                   const T* __restrict__ dbc, long ldd, int dt_rank,
                                                   const float* __restrict__ Dv, const T* __restrict__ xz, long ldz,
                                                   float* __restrict__ ssm, T* __restrict__ conv, int Km1,
                                                   const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                   const int* __restrict__ ctx, const int* __restrict__ rows,
                                                   T* __restrict__ out, int C, int N) {
  __shared__ float bcs[16 * 256];       // [16 tokens][2N], N <= 128
  __shared__ float dts[256], xs[256];   // [16 channels][16 tokens]: step size and input of the group's tokens
  const int s = blockIdx.y;
  const int n = qlen[s];
  if (n <= 0) return;                   // the whole workgroup
  const int tid = threadIdx.x, sub = tid & 15;
  const int c0 = blockIdx.x * 16 + (tid >> 4);
  const bool live = c0 < C;
  const int c = live ? c0 : C - 1;      // idle channels shadow the last one and store nothing
  const int q0 = qstart[s], p0 = ctx[s] - n, row = rows[s];
  const int N2 = 2 * N;
  float a[NS], S[NS];
  float* sp = ssm + ((long)row * C + c) * N;
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int nn = sub + 16 * i;
    a[i] = nn < N ? A[(long)c * N + nn] : 0.f;
    S[i] = (nn < N && p0 > 0) ? sp[nn] : 0.f;
  }
  const float dtb = dt_bias[c], dd = Dv[c];
  for (int t0 = 0; t0 < n; t0 += 16) {
    const int nt = min(16, n - t0);
    __syncthreads();                    // the previous group's rows are consumed
    for (int e = tid; e < nt * N2; e += 256) {
      const int tt = e / N2, k = e - tt * N2;
      bcs[e] = ldf(dbc + (long)(q0 + t0 + tt) * ldd + dt_rank + k);
    }
    const long tok = q0 + t0 + min(sub, nt - 1);
    const float raw = ldf(dt_raw + tok * C + c) + dtb;
    const float dt_m = raw > 20.f ? raw : log1pf(expf(raw));
    const float x_m = ldf(xc + tok * C + c);
    const float z_m = ldf(xz + tok * ldz + C + c);
    dts[tid] = dt_m;
    xs[tid] = x_m;
    __syncthreads();
    float y_m = 0.f;
    const int g0 = tid & ~15;
#pragma unroll 4
    for (int u = 0; u < nt; ++u) {
      const float dt = dts[g0 + u], xv = xs[g0 + u];   // independent of the state: read ahead
      const float* bc = bcs + u * N2;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int nn = sub + 16 * i;
        if (nn < N) {
          S[i] = fastexp<T>::f(dt * a[i]) * S[i] + dt * xv * bc[nn];
          acc += S[i] * bc[N + nn];
        }
      }
      acc = row16_sum(acc);
      if (sub == u) y_m = acc;
    }
    if (live && sub < nt) stf(out + tok * C + c, (y_m + dd * x_m) * silu_f(z_m));
  }
  if (!live) return;
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int nn = sub + 16 * i;
    if (nn < N) sp[nn] = S[i];
  }
  if (sub == 0 && Km1 > 0) {
    // the last K-1 inputs of the sequence: new tokens where there are enough, else the slot's older ones
    T* cs = conv + (long)row * Km1 * C + c;
    float u[8];
    for (int k = 0; k < Km1; ++k) {
      const int i = n - Km1 + k;
      u[k] = i >= 0 ? ldf(xz + (long)(q0 + i) * ldz + c) : (p0 > 0 ? ldf(cs + (long)(Km1 + i) * C) : 0.f);
    }
    for (int k = 0; k < Km1; ++k) stf(cs + (long)k * C, u[k]);
  }
}

// ---------------------------------------------------------------- retention
// One workgroup per (head, sequence).  LDS: state [d][dv], staged q / k (rotated, k scaled) and v of
// TT tokens, partial sums of the row groups (double-buffered), the TT outputs.
constexpr int RT_TT = 8;

template <typename T>
__global__ void __launch_bounds__(256) retention_kernel(const T* __restrict__ qkvg, long ld, int H, int d, int dv,
                                                        const float* __restrict__ cos_sin, int tab_w, int rot,
                                                        const float* __restrict__ decay, float* __restrict__ state,
                                                        float eps, const int* __restrict__ qstart,
                                                        const int* __restrict__ qlen, const int* __restrict__ ctx,
                                                        const int* __restrict__ rows, T* __restrict__ out, int LJ,
                                                        int act, float kscale, float* __restrict__ raw) {
  extern __shared__ float sm[];
  const int h = blockIdx.x, s = blockIdx.y;
  const int n = qlen[s];
  if (n <= 0) return;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  const int G = 256 / LJ;
  float* S = sm;                       // [d][dv]
  float* qs = S + d * dv;              // [TT][d]
  float* ks = qs + RT_TT * d;          // [TT][d]
  float* vs = ks + RT_TT * d;          // [TT][dv]
  float* os = vs + RT_TT * dv;         // [TT][dv]
  float* part = os + RT_TT * dv;       // [2][G][dv]
  const int tid = threadIdx.x, j0 = tid % LJ, g = tid / LJ;
  float* sg = state + ((long)rows[s] * H + h) * d * dv;
  for (int e = tid; e < d * dv; e += 256) S[e] = p0 > 0 ? sg[e] : 0.f;
  const float dec = decay[h];
  const int half = rot >> 1;
  const long oq = (long)h * d, ok = (long)H * d + (long)h * d, ov = 2L * H * d + (long)h * dv,
             og = 2L * H * d + (long)H * dv + (long)h * dv;
  int buf = 0;
  for (int t0 = 0; t0 < n; t0 += RT_TT) {
    const int nt = min(RT_TT, n - t0);
    __syncthreads();   // the previous tile's outputs are consumed, the state is loaded
    for (int e = tid; e < nt * d; e += 256) {
      const int tt = e / d, i = e % d;
      const T* r = qkvg + (long)(q0 + t0 + tt) * ld;
      float qv = ldf(r + oq + i), kv = ldf(r + ok + i);
      if (i < rot) {
        const int f = i < half ? i : i - half;
        const float* cs = cos_sin + (long)(p0 + t0 + tt) * tab_w;
        const float c = cs[f], sn = cs[half + f];
        const int pi = i < half ? i + half : i - half;
        const float qp = ldf(r + oq + pi), kp = ldf(r + ok + pi);
        // pair (u, v) = (x[f], x[f + half]) -> (u c - v s, v c + u s)
        qv = i < half ? qv * c - qp * sn : qv * c + qp * sn;
        kv = i < half ? kv * c - kp * sn : kv * c + kp * sn;
      }
      if (act) { qv = silu_f(qv); kv = silu_f(kv); }
      qs[e] = qv;
      ks[e] = kv * kscale;
    }
    for (int e = tid; e < nt * dv; e += 256) {
      const int tt = e / dv, j = e % dv;
      const float vv = ldf(qkvg + (long)(q0 + t0 + tt) * ld + ov + j);
      vs[e] = act ? silu_f(vv) : vv;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float* q = qs + tt * d;
      const float* k = ks + tt * d;
      for (int j = j0; j < dv; j += LJ) {
        const float v = vs[tt * dv + j];
        float acc = 0.f;
        for (int i = g; i < d; i += G) {
          const float sv = dec * S[i * dv + j] + k[i] * v;
          S[i * dv + j] = sv;
          acc += sv * q[i];
        }
        part[(buf * G + g) * dv + j] = acc;
      }
      __syncthreads();
      for (int j = tid; j < dv; j += 256) {
        float o = 0.f;
        for (int gg = 0; gg < G; ++gg) o += part[(buf * G + gg) * dv + j];
        os[tt * dv + j] = o;
      }
      buf ^= 1;
    }
    __syncthreads();
    if (raw) {   // the caller norms and gates (heads normed together)
      for (int e = tid; e < nt * dv; e += 256) {
        const int tt = e / dv, j = e % dv;
        raw[((long)(q0 + t0 + tt) * H + h) * dv + j] = os[e];
      }
      continue;
    }
    // unit-RMS head, SiLU gate, store: one wave per token
    for (int tt = tid >> 6; tt < nt; tt += 4) {
      const int lane = tid & 63;
      float ss = 0.f;
      for (int j = lane; j < dv; j += 64) ss += os[tt * dv + j] * os[tt * dv + j];
      ss = wave_sum(ss);
      const float r = 1.f / sqrtf(ss / (float)dv + eps);
      const long tok = q0 + t0 + tt;
      for (int j = lane; j < dv; j += 64) {
        const float gz = ldf(qkvg + tok * ld + og + j);
        stf(out + tok * ((long)H * dv) + (long)h * dv + j, os[tt * dv + j] * r * silu_f(gz));
      }
    }
  }
  __syncthreads();
  for (int e = tid; e < d * dv; e += 256) sg[e] = S[e];
}

// ---------------------------------------------------------------- retention, chunked (prompt portions)
// One workgroup per (head, 32-column slice of the value dim, sequence); tokens in chunks of 32.
// With the chunk's rotated q / k (k scaled) and v slice in LDS and g = decay:
//   A[t][s] = g^(t-s) q_t . k_s  (s <= t)            scores inside the chunk, f32
//   o_t     = g^(t+1) q_t^T S + sum_s A[t][s] v_s     S: the state slice before the chunk
//   S      <- g^n S + sum_s g^(n-1-s) k_s v_s^T       n tokens in the chunk
// The raw outputs go to an f32 buffer; retention_finish norms each head and applies the gate.
constexpr int RC_T = 32, RC_V = 32;

template <typename T>
__global__ void __launch_bounds__(256) retention_chunk_kernel(const T* __restrict__ qkvg, long ld, int H, int d, int dv,
                                                              const float* __restrict__ cos_sin, int tab_w, int rot,
                                                              const float* __restrict__ decay, float* __restrict__ state,
                                                              const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                              const int* __restrict__ ctx, const int* __restrict__ rows,
                                                              float* __restrict__ raw, int act, float kscale) {
  extern __shared__ float sm[];
  const int h = blockIdx.x, v0 = blockIdx.y * RC_V, s = blockIdx.z;
  const int n = qlen[s];
  if (n <= 0) return;
  const int q0 = qstart[s], p0 = ctx[s] - n;
  const int nv = min(RC_V, dv - v0), dp = d + 1;
  float* Qs = sm;                       // [RC_T][d + 1]
  float* Ks = Qs + RC_T * dp;           // [RC_T][d + 1]
  float* Vs = Ks + RC_T * dp;           // [RC_T][RC_V]
  float* As = Vs + RC_T * RC_V;         // [RC_T][RC_T + 1]
  float* S = As + RC_T * (RC_T + 1);    // [d][RC_V]
  float* gp = S + d * RC_V;             // [RC_T + 1] powers of the decay
  const int tid = threadIdx.x;
  float* sg = state + ((long)rows[s] * H + h) * d * dv;
  for (int e = tid; e < d * RC_V; e += 256) {
    const int i = e / RC_V, j = e % RC_V;
    S[e] = (p0 > 0 && j < nv) ? sg[(long)i * dv + v0 + j] : 0.f;
  }
  const float dec = decay[h];
  if (tid <= RC_T) gp[tid] = powf(dec, (float)tid);
  const int half = rot >> 1;
  const long oq = (long)h * d, ok = (long)H * d + (long)h * d, ov = 2L * H * d + (long)h * dv + v0;
  for (int t0 = 0; t0 < n; t0 += RC_T) {
    const int nt = min(RC_T, n - t0);
    __syncthreads();   // state loaded / previous chunk's state update done
    for (int e = tid; e < RC_T * d; e += 256) {
      const int tt = e / d, i = e % d;
      float qv = 0.f, kv = 0.f;
      if (tt < nt) {
        const T* r = qkvg + (long)(q0 + t0 + tt) * ld;
        qv = ldf(r + oq + i);
        kv = ldf(r + ok + i);
        if (i < rot) {
          const int f = i < half ? i : i - half;
          const float* cs = cos_sin + (long)(p0 + t0 + tt) * tab_w;
          const float c = cs[f], sn = cs[half + f];
          const int pi = i < half ? i + half : i - half;
          const float qp = ldf(r + oq + pi), kp = ldf(r + ok + pi);
          qv = i < half ? qv * c - qp * sn : qv * c + qp * sn;
          kv = i < half ? kv * c - kp * sn : kv * c + kp * sn;
        }
        if (act) { qv = silu_f(qv); kv = silu_f(kv); }
      }
      Qs[tt * dp + i] = qv;
      Ks[tt * dp + i] = kv * kscale;
    }
    for (int e = tid; e < RC_T * RC_V; e += 256) {
      const int tt = e / RC_V, j = e % RC_V;
      float vv = (tt < nt && j < nv) ? ldf(qkvg + (long)(q0 + t0 + tt) * ld + ov + j) : 0.f;
      Vs[e] = act ? silu_f(vv) : vv;
    }
    __syncthreads();
    // scores inside the chunk: thread (t, 4 keys u0..u0+3); one q read serves four sums
    {
      const int t = tid >> 3, u0 = (tid & 7) * 4;
      float a4[4] = {0.f, 0.f, 0.f, 0.f};
      if (u0 <= t) {
        const float* q = Qs + t * dp;
        const float* k = Ks + u0 * dp;
#pragma unroll 8
        for (int i = 0; i < d; ++i) {
          const float qv = q[i];
#pragma unroll
          for (int x = 0; x < 4; ++x) a4[x] += qv * k[x * dp + i];
        }
      }
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int u = u0 + x;
        As[t * (RC_T + 1) + u] = (u <= t && t < nt) ? a4[x] * gp[t - u] : 0.f;
      }
    }
    __syncthreads();
    // outputs: thread (t, 4 value columns j0..j0+3)
    {
      const int t = tid >> 3, j0 = (tid & 7) * 4;
      const float* q = Qs + t * dp;
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
      for (int i = 0; i < d; ++i) {
        const float qv = q[i];
        const float4 sv = *reinterpret_cast<const float4*>(S + i * RC_V + j0);
        o4[0] += qv * sv.x; o4[1] += qv * sv.y; o4[2] += qv * sv.z; o4[3] += qv * sv.w;
      }
      const float g1 = gp[t + 1];
#pragma unroll
      for (int x = 0; x < 4; ++x) o4[x] *= g1;
      const float* a = As + t * (RC_T + 1);
      for (int u = 0; u <= t; ++u) {
        const float av = a[u];
        const float4 vv = *reinterpret_cast<const float4*>(Vs + u * RC_V + j0);
        o4[0] += av * vv.x; o4[1] += av * vv.y; o4[2] += av * vv.z; o4[3] += av * vv.w;
      }
      if (t < nt) {
#pragma unroll
        for (int x = 0; x < 4; ++x)
          if (j0 + x < nv) raw[((long)(q0 + t0 + t) * H + h) * dv + v0 + j0 + x] = o4[x];
      }
    }
    __syncthreads();
    // state: thread (row i, 16 value columns); rows in passes of 128
    {
      const int jb = (tid & 1) * 16;
      const float gn = gp[nt];
      for (int i = tid >> 1; i < d; i += 128) {
        float acc[16];
#pragma unroll
        for (int x = 0; x < 16; ++x) acc[x] = gn * S[i * RC_V + jb + x];
#pragma unroll 4
        for (int u = 0; u < nt; ++u) {
          const float kv = gp[nt - 1 - u] * Ks[u * dp + i];
          const float* v = Vs + u * RC_V + jb;
#pragma unroll
          for (int x = 0; x < 16; x += 4) {
            const float4 vv = *reinterpret_cast<const float4*>(v + x);
            acc[x] += kv * vv.x; acc[x + 1] += kv * vv.y; acc[x + 2] += kv * vv.z; acc[x + 3] += kv * vv.w;
          }
        }
#pragma unroll
        for (int x = 0; x < 16; ++x) S[i * RC_V + jb + x] = acc[x];
      }
    }
  }
  __syncthreads();
  for (int e = tid; e < d * RC_V; e += 256) {
    const int i = e / RC_V, j = e % RC_V;
    if (j < nv) sg[(long)i * dv + v0 + j] = S[e];
  }
}

// unit-RMS heads and the SiLU gate over the raw outputs: one wave per (token, head)
template <typename T>
__global__ void __launch_bounds__(256) retention_finish_kernel(const float* __restrict__ raw, const T* __restrict__ qkvg,
                                                               long ld, int H, int d, int dv, float eps,
                                                               const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                               int S, T* __restrict__ out, long rows_total) {
  const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows_total) return;
  const int lane = threadIdx.x & 63;
  const long tok = r / H;
  const int h = (int)(r % H);
  // tokens of no sequence (graph padding) keep their zeros
  bool live = false;
  for (int s = 0; s < S; ++s) live |= tok >= qstart[s] && tok < qstart[s] + qlen[s];
  if (!live) return;
  const float* o = raw + r * dv;
  float ss = 0.f;
  for (int j = lane; j < dv; j += 64) ss += o[j] * o[j];
  ss = wave_sum(ss);
  const float rs = 1.f / sqrtf(ss / (float)dv + eps);
  const long og = 2L * H * d + (long)H * dv + (long)h * dv;
  for (int j = lane; j < dv; j += 64)
    stf(out + tok * ((long)H * dv) + (long)h * dv + j, o[j] * rs * silu_f(ldf(qkvg + tok * ld + og + j)));
}

// the heads of a token normed together (weight w over heads x dv), times sigmoid(gate): one
// workgroup per token
template <typename T>
__global__ void __launch_bounds__(256) heads_norm_gate_kernel(const float* __restrict__ raw, const T* __restrict__ qkvg,
                                                              long ld, long og, int n, const float* __restrict__ w,
                                                              float eps, const int* __restrict__ qstart,
                                                              const int* __restrict__ qlen, int S, T* __restrict__ out) {
  __shared__ float red[16];
  const long tok = blockIdx.x;
  bool live = false;
  for (int s = 0; s < S; ++s) live |= tok >= qstart[s] && tok < qstart[s] + qlen[s];
  if (!live) {           // the whole workgroup: rows of no sequence (graph padding) become zeros
    for (int j = threadIdx.x; j < n; j += 256) stf(out + tok * n + j, 0.f);
    return;
  }
  const float* o = raw + tok * n;
  float ss = 0.f;
  for (int j = threadIdx.x; j < n; j += 256) ss += o[j] * o[j];
  const float rs = 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
  for (int j = threadIdx.x; j < n; j += 256) {
    const float gz = ldf(qkvg + tok * ld + og + j);
    stf(out + tok * n + j, o[j] * rs * w[j] / (1.f + expf(-gz)));
  }
}

// ---------------------------------------------------------------- squared ReLU, dense gate
template <typename T>
__global__ void __launch_bounds__(256) relu2_kernel(const T* __restrict__ x, const float* __restrict__ gate, int E,
                                                    int ff, T* __restrict__ y, long rows, int n) {
  const long total = rows * (long)n;
  for (long e = (long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long)gridDim.x * 256) {
    const float v = fmaxf(ldf(x + e), 0.f);
    float r = v * v;
    if (gate) r *= gate[(e / n) * E + (int)(e % n) / ff];
    stf(y + e, r);
  }
}

__global__ void __launch_bounds__(256) dense_gate_kernel(const int* __restrict__ ids, const float* __restrict__ wts,
                                                         float* __restrict__ g, long P, int k, int E) {
  const long p = (long)blockIdx.x * 256 + threadIdx.x;
  if (p >= P) return;
  const int e = ids[p];
  if (e >= 0 && e < E) g[(p / k) * E + e] = wts[p];   // a token's k experts are distinct
}


// ---------------------------------------------------------------- PolyNorm, grouped sigmoid router, SwiGLU dense form, softcap
// y = a N(z) + b N(z^2) + c N(z^3) + e per row, N(u) = u / sqrt(mean(u^2) + eps): one workgroup per row
template <typename T>
__global__ void __launch_bounds__(256) polynorm_kernel(const T* __restrict__ z, long ldz, const float* __restrict__ coef,
                                                       T* __restrict__ y, int n, float eps) {
  __shared__ float red[16];
  const long row = blockIdx.x;
  const T* zr = z + row * ldz;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = ldf(zr + i), v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  const float inv = 1.f / (float)n;
  const float r1 = coef[0] / sqrtf(block_sum(s1, red) * inv + eps);
  const float r2 = coef[1] / sqrtf(block_sum(s2, red) * inv + eps);
  const float r3 = coef[2] / sqrtf(block_sum(s3, red) * inv + eps);
  const float e = coef[3];
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = ldf(zr + i);
    stf(y + row * (long)n + i, v * (r1 + v * (r2 + v * r3)) + e);
  }
}

// (value, index) maximum over the wave; equal values: the lower index
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, 64);
    const int oi = __shfl_xor(idx, o, 64);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
}

constexpr int ROUTER_MAX_E = 1024;

// One wave per token over the first E columns of its logits row.  Scores s: sigmoid (smode 0) or
// softmax (1); choice scores c = s + corr.  `count` groups of neighbours; a group's score is the sum
// of its two best choice scores (gmode 0) or its best (1); the `top` best c inside the `keep` best
// groups are chosen (ties: the lower index); weights are the scores s.  Outputs >= real are identity
// experts: their weights leave summed in idw[t], and as 0 in wts.
__global__ void __launch_bounds__(256) route_topk_kernel(const float* __restrict__ logits, long ld, int T, int E, int top,
                                                         int count, int keep, int smode, int gmode,
                                                         const float* __restrict__ corr, int real, int* __restrict__ ids,
                                                         float* __restrict__ wts, float* __restrict__ idw) {
  // per wave: scores [E], choice scores [E] (-inf: taken), group scores [E], kept-group flags [E bytes]
  extern __shared__ float rsm[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  const int per_wave = 3 * E + (E + 3) / 4;
  float* sc = rsm + wave * per_wave;
  float* ch = sc + E;
  float* gs = ch + E;
  unsigned char* ok = reinterpret_cast<unsigned char*>(gs + E);
  const float* z = logits + (long)t * ld;
  if (smode == 0) {
    for (int e = lane; e < E; e += 64) sc[e] = 1.f / (1.f + expf(-z[e]));
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) { const float v = expf(z[e] - mx); sc[e] = v; sum += v; }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) sc[e] = sc[e] / sum;
  }
  for (int e = lane; e < E; e += 64) ch[e] = sc[e] + (corr ? corr[e] : 0.f);
  const int per = E / count;
  const bool limited = count > 1 && keep < count;
  if (limited) {
    __builtin_amdgcn_wave_barrier();
    for (int g = lane; g < count; g += 64) {
      float a = -INFINITY, b = -INFINITY;     // the two best
      for (int j = 0; j < per; ++j) {
        const float v = ch[g * per + j];
        if (v > a) { b = a; a = v; } else if (v > b) b = v;
      }
      gs[g] = (gmode == 0 && per > 1) ? a + b : a;
      ok[g] = 0;
    }
    __builtin_amdgcn_wave_barrier();
    for (int kk = 0; kk < keep; ++kk) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < count; g += 64) {
        const float v = gs[g];
        if (!ok[g] && (v > bv || bi == 0x7fffffff)) { bv = v; bi = g; }
      }
      wave_argmax(bv, bi);
      if (bi == 0x7fffffff) bi = 0;
      if (lane == 0) ok[bi] = 1;
      __builtin_amdgcn_wave_barrier();
    }
  }
  float isum = 0.f;
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = ch[e];
      if (v > bv && (!limited || ok[e / per])) { bv = v; bi = e; }
    }
    wave_argmax(bv, bi);
    if (bi == 0x7fffffff) bi = 0;     // a row of NaNs (stale padding) compares false everywhere: stay inside the arrays
    if (lane == 0) {
      const float w = sc[bi];
      ids[(long)t * top + j] = bi;
      wts[(long)t * top + j] = bi < real ? w : 0.f;
      if (bi >= real) isum += w;
      ch[bi] = -INFINITY;     // taken
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0 && idw) idw[t] = isum;
}

// gu [rows, E 2 ff] (per expert: gate columns, then up columns) -> y [rows, E ff] = silu(gate) up gate[row, expert]
template <typename T>
__global__ void __launch_bounds__(256) swiglu_scale_kernel(const T* __restrict__ gu, const float* __restrict__ gate, int E,
                                                           int ff, T* __restrict__ y, long total) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const long n = (long)E * ff, row = i / n;
  const int c = (int)(i % n), e = c / ff, j = c % ff;
  const float w = gate[row * E + e];
  float v = 0.f;
  if (w != 0.f) {
    const T* p = gu + row * 2 * n + (long)e * 2 * ff + j;
    v = silu_f(ldf(p)) * ldf(p + ff) * w;
  }
  stf(y + i, v);
}

template <typename T>
__global__ void __launch_bounds__(256) softcap_kernel(const T* __restrict__ x, float cap, float* __restrict__ y, long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) y[i] = cap * tanhf(ldf(x + i) / cap);
}

// out = rmsnorm over each of `groups` parts of (y silu(z)), times w: a wave per (row, part)
template <typename T>
__global__ void __launch_bounds__(256) gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z, long ldz,
                                                               const float* __restrict__ w, T* __restrict__ out, int rows,
                                                               int n, int groups, float eps) {
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (unit >= rows * groups) return;
  const int row = unit / groups, c0 = (unit % groups) * n;
  const float* yr = y + (long)row * n * groups + c0;
  const T* zr = z + (long)row * ldz + c0;
  float s = 0.f;
  for (int i = lane; i < n; i += 64) { const float v = yr[i] * silu_f(ldf(zr + i)); s += v * v; }
  const float r = 1.f / sqrtf(wave_sum(s) / (float)n + eps);
  T* o = out + (long)row * n * groups + c0;
  for (int i = lane; i < n; i += 64) stf(o + i, yr[i] * silu_f(ldf(zr + i)) * r * w[c0 + i]);
}

}  // namespace

// ---------------------------------------------------------------- layer-norm layers with layer scale
// One workgroup per token.  With y: x += ls * (y + bias + sigmoid(g2) y2 + hw h) (every term after y
// optional; g2 and hw hold one number per token).  Then out = (x - mean) / sqrt(var + eps) * w + b with
// the variance taken around the mean in a second pass over the row kept in LDS.
template <typename T>
__global__ void __launch_bounds__(256) ls_resadd_ln_kernel(const T* __restrict__ y, long ldy, const float* __restrict__ ls,
                                                           const float* __restrict__ bias, const T* __restrict__ y2,
                                                           long ldy2, const float* __restrict__ g2, long ldg2,
                                                           const T* __restrict__ h, long ldh, const float* __restrict__ hw,
                                                           float* __restrict__ x, const float* __restrict__ w,
                                                           const float* __restrict__ b, T* __restrict__ out, int H,
                                                           float eps) {
  __shared__ float red[16];
  extern __shared__ float yb[];   // [H]; entry i is touched by thread i % 256 only
  const long row = blockIdx.x;
  float* xr = x + row * (long)H;
  const float s2 = (y && y2) ? (g2 ? 1.f / (1.f + expf(-g2[row * ldg2])) : 1.f) : 0.f;
  const float sh = (y && h) ? hw[row] : 0.f;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float v = xr[i];
    if (y) {
      float t = ldf(y + row * ldy + i);
      if (bias) t += bias[i];
      if (y2) t += s2 * ldf(y2 + row * ldy2 + i);
      if (h) t += sh * ldf(h + row * ldh + i);
      v += ls ? ls[i] * t : t;
      xr[i] = v;
    }
    yb[i] = v;
    sum += v;
  }
  const float mean = block_sum(sum, red) / (float)H;
  float sq = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) { const float dv = yb[i] - mean; sq += dv * dv; }
  const float r = 1.f / sqrtf(block_sum(sq, red) / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256) stf(out + row * (long)H + i, (yb[i] - mean) * r * w[i] + b[i]);
}

// gu [rows, 2 ff] (gate columns, then up columns) + bias -> y [rows, ff].  mode 0: silu(g) u;
// mode 1: g <- min(g, limit), u <- clamp(u, -limit, limit), y = g sigmoid(alpha g) (u + 1)
template <typename T>
__global__ void __launch_bounds__(256) glu_act_kernel(const T* __restrict__ gu, long ld, const float* __restrict__ bias,
                                                      int ff, int mode, float limit, float alpha, T* __restrict__ y,
                                                      long rows) {
  // grid: x over the ff columns, y over the rows (strided when there are more rows than the grid is
  // tall), so that no thread divides
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= ff) return;
  const float bg = bias ? bias[c] : 0.f, bu = bias ? bias[ff + c] : 0.f;
  for (long r = blockIdx.y; r < rows; r += gridDim.y) {
    float g = ldf(gu + r * ld + c) + bg, u = ldf(gu + r * ld + ff + c) + bu;
    float a = 1.f;
    if (mode != 0) {
      g = fminf(g, limit);
      u = fminf(fmaxf(u, -limit), limit) + 1.f;
      a = alpha;
    }
    // the result is rounded to bf16 in bf16 models: the hardware exponential and reciprocal are exact enough there
    const float den = 1.f + fastexp<T>::f(-a * g);
    const float sg = sizeof(T) == 2 ? g * __builtin_amdgcn_rcpf(den) : g / den;
    stf(y + r * (long)ff + c, sg * u);
  }
}

// Raise a kernel's dynamic-LDS limit when a launch needs more than it has been given so far (once per
// size: a later launch inside a stream capture then makes no attribute call).
#define ENSURE_LDS(kernel, bytes)                                                                          \
  do {                                                                                                     \
    static long have_ = 48 * 1024;                                                                         \
    if ((bytes) > have_) {                                                                                 \
      hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)); \
      have_ = (bytes);                                                                                     \
    }                                                                                                      \
  } while (0)

#define BY_T(f32, call_u16, call_f32) \
  if (f32) { call_f32; } else { call_u16; }

extern "C" int dllm_rms_rows(const void* x, long ldx, int x_f32, const float* w, void* y, long ldy, int y_f32, int rows,
                             int n, float eps, int groups, hipStream_t st) {
  if (rows <= 0 || n <= 0) return rows == 0 ? 0 : -1;
  if (groups < 1 || n % groups) return -1;
  n /= groups;     // the kernel's rows are the parts
  const dim3 g((rows * groups + 3) / 4), b(256);
  if (x_f32 && y_f32)
    hipLaunchKernelGGL((rms_rows_kernel<float, float>), g, b, 0, st, (const float*)x, ldx, w, (float*)y, ldy, rows, n, eps, groups);
  else if (x_f32)
    hipLaunchKernelGGL((rms_rows_kernel<float, u16>), g, b, 0, st, (const float*)x, ldx, w, (u16*)y, ldy, rows, n, eps, groups);
  else if (y_f32)
    hipLaunchKernelGGL((rms_rows_kernel<u16, float>), g, b, 0, st, (const u16*)x, ldx, w, (float*)y, ldy, rows, n, eps, groups);
  else
    hipLaunchKernelGGL((rms_rows_kernel<u16, u16>), g, b, 0, st, (const u16*)x, ldx, w, (u16*)y, ldy, rows, n, eps, groups);
  return (int)hipGetLastError();
}

extern "C" int dllm_norm_resadd(const void* y, long ldy, int f32, const float* w, float* x, void* xl, int rows, int H,
                                float eps, int groups, const float* bias, hipStream_t st) {
  if (rows <= 0) return rows == 0 ? 0 : -1;
  if (groups < 1 || H % groups) return -1;
  BY_T(f32,
       hipLaunchKernelGGL(norm_resadd_kernel<u16>, dim3(rows), dim3(256), 0, st, (const u16*)y, ldy, w, x, (u16*)xl, H, eps, groups, bias),
       hipLaunchKernelGGL(norm_resadd_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)y, ldy, w, x, (float*)xl, H, eps, groups, bias))
  return (int)hipGetLastError();
}

// dw != null: x is slot dn - 1 of an f32 stack [slots][rows][H]; the launch also writes slot dn, the
// sum over j < dn of dw[j] * slot j, and norms that for xn
extern "C" int dllm_resadd_norm(const void* a, long lda, const void* b, long ldb, int f32, const float* wa, const float* wb,
                                const float* w_post, float* x, const float* w_next, void* xn, int rows, int H, float eps,
                                const float* dw, int dn, hipStream_t st) {
  if (rows <= 0) return rows == 0 ? 0 : -1;
  const long lds = 4L * H;
  if (lds > 150 * 1024) return -2;
  if (f32) {
    ENSURE_LDS(resadd_norm_kernel<float>, lds);
    hipLaunchKernelGGL(resadd_norm_kernel<float>, dim3(rows), dim3(256), lds, st, (const float*)a, lda, (const float*)b, ldb, wa,
                       wb, w_post, x, w_next, (float*)xn, H, eps, dw, dn, (long)rows * H);
  } else {
    ENSURE_LDS(resadd_norm_kernel<u16>, lds);
    hipLaunchKernelGGL(resadd_norm_kernel<u16>, dim3(rows), dim3(256), lds, st, (const u16*)a, lda, (const u16*)b, ldb, wa, wb,
                       w_post, x, w_next, (u16*)xn, H, eps, dw, dn, (long)rows * H);
  }
  return (int)hipGetLastError();
}

extern "C" int dllm_depth_mix(float* X, const float* w, int n, long T, int H, const float* w_next, void* xn, int f32,
                              float eps, hipStream_t st) {
  if (T <= 0) return T == 0 ? 0 : -1;
  const long lds = 4L * H;
  if (lds > 150 * 1024) return -2;
  if (f32) {
    ENSURE_LDS(depth_mix_kernel<float>, lds);
    hipLaunchKernelGGL(depth_mix_kernel<float>, dim3((unsigned)T), dim3(256), lds, st, X, w, n, T * H, w_next, (float*)xn, H, eps);
  } else {
    ENSURE_LDS(depth_mix_kernel<u16>, lds);
    hipLaunchKernelGGL(depth_mix_kernel<u16>, dim3((unsigned)T), dim3(256), lds, st, X, w, n, T * H, w_next, (u16*)xn, H, eps);
  }
  return (int)hipGetLastError();
}

extern "C" int dllm_gelu_erf(const void* x, void* y, int f32, long n, hipStream_t st) {
  if (n <= 0) return 0;
  long gr = (n + 255) / 256;
  if (gr > 8192) gr = 8192;
  BY_T(f32,
       hipLaunchKernelGGL(gelu_erf_kernel<u16>, dim3((int)gr), dim3(256), 0, st, (const u16*)x, (u16*)y, n),
       hipLaunchKernelGGL(gelu_erf_kernel<float>, dim3((int)gr), dim3(256), 0, st, (const float*)x, (float*)y, n))
  return (int)hipGetLastError();
}

extern "C" int dllm_conv_refill(const void* x, long ldx, int f32, void* conv, int Km1, int C, const int* qstart,
                                const int* qlen, const int* ctx, const int* rows, int S, hipStream_t st) {
  if (S <= 0 || Km1 <= 0) return 0;
  if (Km1 > 8) return -1;
  const dim3 g((C + 255) / 256, S);
  BY_T(f32,
       hipLaunchKernelGGL(conv_refill_kernel<u16>, g, dim3(256), 0, st, (const u16*)x, ldx, (u16*)conv, Km1, C, qstart, qlen, ctx, rows),
       hipLaunchKernelGGL(conv_refill_kernel<float>, g, dim3(256), 0, st, (const float*)x, ldx, (float*)conv, Km1, C, qstart, qlen, ctx, rows))
  return (int)hipGetLastError();
}

// refill != 0: a step of single tokens; the kernel also moves each token's input into its slot
extern "C" int dllm_conv_silu(const void* x, long ldx, int f32, const float* w, const float* b, void* state,
                              const int* qstart, const int* qlen, const int* ctx, const int* rows, void* y, int T,
                              int S, int C, int K, int refill, int act, hipStream_t st) {
  if (T <= 0 || S <= 0) return 0;
  if (K < 1 || K > 9) return -1;
  // prompt portions of bf16 rows made of whole, aligned 16-byte vectors: the vector kernel
  if (!f32 && !refill && K <= 5 && T >= 4 * S && C % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
      ((uintptr_t)y % 16) == 0 && ((uintptr_t)state % 16) == 0) {
    int gzv = (T + 4 * CV_RUN - 1) / (4 * CV_RUN);
    if (gzv > 256) gzv = 256;
    const dim3 gv((C / 8 + 63) / 64, S, gzv);
#define CONV_VEC(KK)                                                                                                       \
  hipLaunchKernelGGL(conv_vec_kernel<KK>, gv, dim3(256), 0, st, (const u16*)x, ldx, w, b, (const u16*)state, qstart, qlen, ctx, \
                     rows, (u16*)y, C, act)
    switch (K) {
      case 1: CONV_VEC(1); break;
      case 2: CONV_VEC(2); break;
      case 3: CONV_VEC(3); break;
      case 4: CONV_VEC(4); break;
      default: CONV_VEC(5); break;
    }
#undef CONV_VEC
    return (int)hipGetLastError();
  }
  int gz = (T + 31) / 32;
  if (gz > 128) gz = 128;
  const dim3 g((C + 63) / 64, S, gz), blk(256);
  BY_T(f32,
       hipLaunchKernelGGL(conv_silu_kernel<u16>, g, blk, 0, st, (const u16*)x, ldx, w, b, (const u16*)state, qstart, qlen, ctx, rows, (u16*)y, C, K, refill ? (u16*)state : nullptr, act),
       hipLaunchKernelGGL(conv_silu_kernel<float>, g, blk, 0, st, (const float*)x, ldx, w, b, (const float*)state, qstart, qlen, ctx, rows, (float*)y, C, K, refill ? (float*)state : nullptr, act))
  return (int)hipGetLastError();
}

namespace {
template <typename T>
int launch_scan(int ns, dim3 g, hipStream_t st, const T* xc, const T* dt_raw, const float* dt_bias, const float* A,
                const T* dbc, long ldd, int dt_rank, const float* D, const T* xz, long ldz, float* ssm, T* conv, int Km1,
                const int* qstart, const int* qlen, const int* ctx, const int* rows, T* out, int C, int N) {
#define SCAN(NS) hipLaunchKernelGGL((scan_kernel<T, NS>), g, dim3(256), 0, st, xc, dt_raw, dt_bias, A, dbc, ldd, dt_rank, D, xz, ldz, ssm, conv, Km1, qstart, qlen, ctx, rows, out, C, N)
  if (ns <= 1) SCAN(1); else if (ns <= 2) SCAN(2); else if (ns <= 4) SCAN(4); else SCAN(8);
#undef SCAN
  return (int)hipGetLastError();
}
}  // namespace

extern "C" int dllm_selective_scan(const void* xc, const void* dt_raw, int f32, const float* dt_bias, const float* A,
                                   const void* dbc, long ldd, int dt_rank, const float* D, const void* xz, long ldz,
                                   float* ssm, void* conv, int Km1, const int* qstart, const int* qlen, const int* ctx,
                                   const int* rows, void* out, int S, int C, int N, hipStream_t st) {
  if (S <= 0) return 0;
  if (N < 1 || N > 128 || Km1 < 0 || Km1 > 8) return -1;
  const int ns = (N + 15) / 16;
  const dim3 g((C + 15) / 16, S);
  if (f32)
    return launch_scan<float>(ns, g, st, (const float*)xc, (const float*)dt_raw, dt_bias, A, (const float*)dbc, ldd, dt_rank,
                              D, (const float*)xz, ldz, ssm, (float*)conv, Km1, qstart, qlen, ctx, rows, (float*)out, C, N);
  return launch_scan<u16>(ns, g, st, (const u16*)xc, (const u16*)dt_raw, dt_bias, A, (const u16*)dbc, ldd, dt_rank, D,
                          (const u16*)xz, ldz, ssm, (u16*)conv, Km1, qstart, qlen, ctx, rows, (u16*)out, C, N);
}

extern "C" long dllm_retention_lds(int d, int dv) {
  int lj = 1;
  while (lj < dv && lj < 64) lj <<= 1;
  const int G = 256 / lj;
  return 4L * ((long)d * dv + RT_TT * (2L * d + 2L * dv) + 2L * G * dv);
}

extern "C" int dllm_retention(const void* qkvg, long ld, int f32, int H, int d, int dv, const float* cos_sin, int tab_w,
                              int rot, const float* decay, float* state, float eps, const int* qstart, const int* qlen,
                              const int* ctx, const int* rows, void* out, int S, int act, float kscale, float* raw,
                              hipStream_t st) {
  if (S <= 0) return 0;
  if (rot < 0 || rot > d || (rot & 1) || rot > tab_w) return -1;
  const long lds = dllm_retention_lds(d, dv);
  if (lds > 150 * 1024) return -2;
  int lj = 1;
  while (lj < dv && lj < 64) lj <<= 1;
  const dim3 g(H, S);
  if (f32) {
    ENSURE_LDS(retention_kernel<float>, lds);
    hipLaunchKernelGGL(retention_kernel<float>, g, dim3(256), lds, st, (const float*)qkvg, ld, H, d, dv, cos_sin, tab_w, rot,
                       decay, state, eps, qstart, qlen, ctx, rows, (float*)out, lj, act, kscale, raw);
  } else {
    ENSURE_LDS(retention_kernel<u16>, lds);
    hipLaunchKernelGGL(retention_kernel<u16>, g, dim3(256), lds, st, (const u16*)qkvg, ld, H, d, dv, cos_sin, tab_w, rot,
                       decay, state, eps, qstart, qlen, ctx, rows, (u16*)out, lj, act, kscale, raw);
  }
  return (int)hipGetLastError();
}

extern "C" long dllm_retention_chunk_lds(int d) {
  return 4L * (2L * RC_T * (d + 1) + RC_T * RC_V + RC_T * (RC_T + 1) + (long)d * RC_V + RC_T + 1);
}

// Chunked form for prompt portions: `raw` is an f32 scratch [T, H, dv].
extern "C" int dllm_retention_chunked(const void* qkvg, long ld, int f32, int H, int d, int dv, const float* cos_sin,
                                      int tab_w, int rot, const float* decay, float* state, float eps, const int* qstart,
                                      const int* qlen, const int* ctx, const int* rows, float* raw, void* out, int S,
                                      long T, int act, float kscale, int finish, hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  if (rot < 0 || rot > d || (rot & 1) || rot > tab_w) return -1;
  const long lds = dllm_retention_chunk_lds(d);
  if (lds > 150 * 1024) return -2;
  const dim3 g(H, (dv + RC_V - 1) / RC_V, S);
  const long rows_total = T * H;
  const dim3 gf((unsigned)((rows_total + 3) / 4));
  if (f32) {
    ENSURE_LDS(retention_chunk_kernel<float>, lds);
    hipLaunchKernelGGL(retention_chunk_kernel<float>, g, dim3(256), lds, st, (const float*)qkvg, ld, H, d, dv, cos_sin, tab_w,
                       rot, decay, state, qstart, qlen, ctx, rows, raw, act, kscale);
    if (finish) hipLaunchKernelGGL(retention_finish_kernel<float>, gf, dim3(256), 0, st, raw, (const float*)qkvg, ld, H, d, dv, eps, qstart,
                       qlen, S, (float*)out, rows_total);
  } else {
    ENSURE_LDS(retention_chunk_kernel<u16>, lds);
    hipLaunchKernelGGL(retention_chunk_kernel<u16>, g, dim3(256), lds, st, (const u16*)qkvg, ld, H, d, dv, cos_sin, tab_w, rot,
                       decay, state, qstart, qlen, ctx, rows, raw, act, kscale);
    if (finish) hipLaunchKernelGGL(retention_finish_kernel<u16>, gf, dim3(256), 0, st, raw, (const u16*)qkvg, ld, H, d, dv, eps, qstart, qlen,
                       S, (u16*)out, rows_total);
  }
  return (int)hipGetLastError();
}

// raw [T, n] f32 (n = heads x dv) -> out = rmsnorm over n * w * sigmoid(gate); the gate is column
// `og` onwards of qkvg
extern "C" int dllm_heads_norm_gate(const float* raw, const void* qkvg, long ld, int f32, long og, int n, const float* w,
                                    float eps, const int* qstart, const int* qlen, int S, void* out, long T,
                                    hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  BY_T(f32,
       hipLaunchKernelGGL(heads_norm_gate_kernel<u16>, dim3((unsigned)T), dim3(256), 0, st, raw, (const u16*)qkvg, ld, og, n, w, eps, qstart, qlen, S, (u16*)out),
       hipLaunchKernelGGL(heads_norm_gate_kernel<float>, dim3((unsigned)T), dim3(256), 0, st, raw, (const float*)qkvg, ld, og, n, w, eps, qstart, qlen, S, (float*)out))
  return (int)hipGetLastError();
}

extern "C" int dllm_relu2_scale(const void* x, int f32, const float* gate, int E, int ff, void* y, long rows, int n,
                                hipStream_t st) {
  const long total = rows * (long)n;
  if (total <= 0) return 0;
  long gr = (total + 255) / 256;
  if (gr > 8192) gr = 8192;
  BY_T(f32,
       hipLaunchKernelGGL(relu2_kernel<u16>, dim3((int)gr), dim3(256), 0, st, (const u16*)x, gate, E, ff, (u16*)y, rows, n),
       hipLaunchKernelGGL(relu2_kernel<float>, dim3((int)gr), dim3(256), 0, st, (const float*)x, gate, E, ff, (float*)y, rows, n))
  return (int)hipGetLastError();
}

extern "C" int dllm_dense_gate(const int* ids, const float* wts, float* g, long T, int k, int E, hipStream_t st) {
  const long P = T * k;
  if (P <= 0) return 0;
  hipLaunchKernelGGL(dense_gate_kernel, dim3((int)((P + 255) / 256)), dim3(256), 0, st, ids, wts, g, P, k, E);
  return (int)hipGetLastError();
}

extern "C" int dllm_polynorm(const void* z, long ldz, int f32, const float* coef, void* y, long rows, int n, float eps,
                             hipStream_t st) {
  if (rows <= 0 || n <= 0) return rows == 0 ? 0 : -1;
  BY_T(f32,
       hipLaunchKernelGGL(polynorm_kernel<u16>, dim3((unsigned)rows), dim3(256), 0, st, (const u16*)z, ldz, coef, (u16*)y, n, eps),
       hipLaunchKernelGGL(polynorm_kernel<float>, dim3((unsigned)rows), dim3(256), 0, st, (const float*)z, ldz, coef, (float*)y, n, eps))
  return (int)hipGetLastError();
}

extern "C" int dllm_route_topk(const float* logits, long ld, int T, int E, int top, int count, int keep, int smode, int gmode,
                               const float* corr, int real, int* ids, float* wts, float* idw, hipStream_t st) {
  if (T <= 0) return 0;
  if (E < 1 || E > ROUTER_MAX_E || ld < E || count < 1 || E % count || keep < 1 || keep > count || top < 1 ||
      top > keep * (E / count) || real < 0)
    return -1;
  const long lds = 4L * 4 * (3 * E + (E + 3) / 4);     // sized by the outputs: small routers keep every CU full
  ENSURE_LDS(route_topk_kernel, lds);
  hipLaunchKernelGGL(route_topk_kernel, dim3((T + 3) / 4), dim3(256), lds, st, logits, ld, T, E, top, count, keep, smode, gmode,
                     corr, real, ids, wts, idw);
  return (int)hipGetLastError();
}

extern "C" int dllm_group_router(const float* logits, int T, int E, int top, int count, int keep, int* ids, float* wts,
                                 hipStream_t st) {
  return dllm_route_topk(logits, E, T, E, top, count, keep, 0, 0, nullptr, E, ids, wts, nullptr, st);
}

extern "C" int dllm_swiglu_scale(const void* gu, int f32, const float* gate, int E, int ff, void* y, long rows,
                                 hipStream_t st) {
  const long total = rows * E * ff;
  if (total <= 0) return 0;
  const dim3 g((unsigned)((total + 255) / 256));
  BY_T(f32,
       hipLaunchKernelGGL(swiglu_scale_kernel<u16>, g, dim3(256), 0, st, (const u16*)gu, gate, E, ff, (u16*)y, total),
       hipLaunchKernelGGL(swiglu_scale_kernel<float>, g, dim3(256), 0, st, (const float*)gu, gate, E, ff, (float*)y, total))
  return (int)hipGetLastError();
}

extern "C" int dllm_softcap(const void* x, int f32, float cap, float* y, long n, hipStream_t st) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return -1;
  const dim3 g((unsigned)((n + 255) / 256));
  BY_T(f32,
       hipLaunchKernelGGL(softcap_kernel<u16>, g, dim3(256), 0, st, (const u16*)x, cap, y, n),
       hipLaunchKernelGGL(softcap_kernel<float>, g, dim3(256), 0, st, (const float*)x, cap, y, n))
  return (int)hipGetLastError();
}

extern "C" int dllm_gated_group_norm(const float* y, const void* z, long ldz, int f32, const float* w, void* out, int rows,
                                     int n, int groups, float eps, hipStream_t st) {
  if (rows <= 0) return 0;
  if (groups < 1 || n % groups) return -1;
  const dim3 g((rows * groups + 3) / 4);
  BY_T(f32,
       hipLaunchKernelGGL(gated_group_norm_kernel<u16>, g, dim3(256), 0, st, y, (const u16*)z, ldz, w, (u16*)out, rows, n / groups, groups, eps),
       hipLaunchKernelGGL(gated_group_norm_kernel<float>, g, dim3(256), 0, st, y, (const float*)z, ldz, w, (float*)out, rows, n / groups, groups, eps))
  return (int)hipGetLastError();
}

extern "C" int dllm_ls_resadd_ln(const void* y, long ldy, int f32, const float* ls, const float* bias, const void* y2, long ldy2,
                                 const float* g2, long ldg2, const void* h, long ldh, const float* hw, float* x,
                                 const float* w, const float* b, void* out, long rows, int H, float eps, hipStream_t st) {
  if (rows <= 0) return 0;
  const long lds = 4L * H;
  if (lds > 150 * 1024) return -1;
  if (f32) {
    ENSURE_LDS(ls_resadd_ln_kernel<float>, lds);
    hipLaunchKernelGGL(ls_resadd_ln_kernel<float>, dim3((unsigned)rows), dim3(256), lds, st, (const float*)y, ldy, ls, bias,
                       (const float*)y2, ldy2, g2, ldg2, (const float*)h, ldh, hw, x, w, b, (float*)out, H, eps);
  } else {
    ENSURE_LDS(ls_resadd_ln_kernel<u16>, lds);
    hipLaunchKernelGGL(ls_resadd_ln_kernel<u16>, dim3((unsigned)rows), dim3(256), lds, st, (const u16*)y, ldy, ls, bias,
                       (const u16*)y2, ldy2, g2, ldg2, (const u16*)h, ldh, hw, x, w, b, (u16*)out, H, eps);
  }
  return (int)hipGetLastError();
}

extern "C" int dllm_glu_act(const void* gu, long ld, int f32, const float* bias, int ff, int mode, float limit, float alpha,
                            void* y, long rows, hipStream_t st) {
  const long total = rows * ff;
  if (total <= 0) return 0;
  if (mode < 0 || mode > 1) return -1;
  const dim3 grid((unsigned)((ff + 255) / 256), (unsigned)(rows < 2048 ? rows : 2048));
  BY_T(f32,
       hipLaunchKernelGGL(glu_act_kernel<u16>, grid, dim3(256), 0, st, (const u16*)gu, ld, bias, ff, mode, limit, alpha, (u16*)y, rows),
       hipLaunchKernelGGL(glu_act_kernel<float>, grid, dim3(256), 0, st, (const float*)gu, ld, bias, ff, mode, limit, alpha, (float*)y, rows))
  return (int)hipGetLastError();
}
