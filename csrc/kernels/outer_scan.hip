// Gated outer-product recurrences with a scalar decay per head and token (gfx950, wave64):
//
//     S_t = a_t S_(t-1) + b_t k_t v_t^T          (S: [N x vdim] f32 per sequence and head)
//     y_t = S_t^T q_t
//
//   ssd_scan   Mamba-2: k = B, q = C (shared by a group of heads), v = x;  dt = softplus(logit + bias),
//              a = exp(neg_a dt), b = dt;  y += D x.  Output f32 (the gated norm follows).
//   mlstm      matrix-memory LSTM: capped input gate i, log-sigmoid forget gate f, running maximum m
//              (0 at the start): m' = max(f + m, i), a = exp(f + m - m'), b = exp(i - m');  a
//              normaliser n_t = a n + b k rides along as one more value column (v = 1), and
//              y = S^T q / (max(|n . q|, exp(-m')) + 1e-6).  mlstm_finish: heads to unit RMS, weight,
//              sigmoid gate.
//
// One workgroup per (16 value columns, head, sequence); thread = (column, strip of state rows): a
// thread keeps rows strip, strip + strips, ... of its column in registers.  Tokens run in groups of
// 16: the group's k / q rows, values and gate numbers are staged once in LDS, every thread then walks
// the 16 tokens on its registers and leaves per-strip partial sums in LDS, and after one barrier
// the sums over strips are formed and stored for all 16 tokens at once.  Sequence metadata as in
// the other mixers (qstart / qlen / ctx / rows; a sequence whose first new position is 0 starts from
// zero state whatever its slot holds).
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

constexpr int OS_COLS = 16;   // value columns per workgroup
constexpr int OS_TG = 16;     // tokens per group

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float logsigmoid_f(float x) { return x < 0.f ? x - log1pf(expf(x)) : -log1pf(expf(-x)); }

// MLSTM = false: ssd_scan; true: mlstm.  NPT >= ceil(N / strips); the staged k / q rows are padded with
// zeros to NPT * strips entries, so the walk over a thread's state rows has no bounds test (rows past
// N stay zero) and its LDS reads (k and q of a row side by side, 8 bytes) can be issued together.
template <typename T, bool MLSTM, int NPT>
__global__ void __launch_bounds__(256) outer_scan_kernel(const T* __restrict__ kq, long ld_kq, int k_off, int q_off, int kq_heads_div,
                                                         const T* __restrict__ vsrc, long ld_v, int v_off,
                                                         const T* __restrict__ gsrc, long ld_g, int g_off, int g_off2,
                                                         const float* __restrict__ p0v, const float* __restrict__ p1v,
                                                         const float* __restrict__ p2v, float cap, float qscale,
                                                         float* __restrict__ state, float* __restrict__ nm, int NCB,
                                                         const int* __restrict__ qstart, const int* __restrict__ qlen,
                                                         const int* __restrict__ ctx, const int* __restrict__ rows,
                                                         float* __restrict__ out, int H, int N, int dv) {
  constexpr int CW = OS_COLS + (MLSTM ? 1 : 0);
  constexpr int STRIPS = 256 / CW;
  extern __shared__ float sm[];
  const int s = blockIdx.z, h = blockIdx.y, cb = blockIdx.x;
  const int n_new = qlen[s];
  if (n_new <= 0) return;
  const int q0 = qstart[s], p0 = ctx[s] - n_new;
  const int slot = rows[s];
  const int tid = threadIdx.x;
  const int c = tid % CW, strip = tid / CW;
  const bool live = strip < STRIPS;
  const int v0 = cb * OS_COLS;
  const bool is_norm = MLSTM && c == OS_COLS;
  const bool col_ok = live && (is_norm || v0 + c < dv);
  constexpr int NP = NPT * STRIPS;
  float2* KQ = reinterpret_cast<float2*>(sm);   // [TG][NP] (k, q)
  float* Vs = sm + 2 * OS_TG * NP;      // [TG][CW]
  float* Ga = Vs + OS_TG * CW;          // [TG]  SSD: a_t;  mLSTM: i_t
  float* Gb = Ga + OS_TG;               // [TG]  SSD: b_t;  mLSTM: f_t
  float* Ms = Gb + OS_TG;               // [TG]  mLSTM: m_t
  float* Ps = Ms + OS_TG;               // [TG][STRIPS][CW] partial sums
  const int kh = h / kq_heads_div;      // SSD: the head's group; mLSTM: the head
  float S[NPT];
  float* sp = state + (((long)slot * H + h) * N) * dv + v0 + c;
  float* np = MLSTM ? nm + (((long)slot * H + h) * NCB + cb) * (N + 1) : nullptr;
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int n = strip + k * STRIPS;
    float v = 0.f;
    if (col_ok && n < N && p0 > 0) v = is_norm ? np[n] : sp[(long)n * dv];
    S[k] = v;
  }
  float m = 0.f;
  if (MLSTM && p0 > 0) m = np[N];
  const float hp0 = p0v ? p0v[h] : 0.f, hp1 = p1v ? p1v[h] : 0.f, hp2 = p2v ? p2v[h] : 0.f;
  for (int t0 = 0; t0 < n_new; t0 += OS_TG) {
    const int nt = min(OS_TG, n_new - t0);
    __syncthreads();     // the previous group's sums are stored
    for (int e = tid; e < nt * NP; e += 256) {
      const int t = e / NP, n = e % NP;
      float2 v = make_float2(0.f, 0.f);
      if (n < N) {
        const T* r = kq + (long)(q0 + t0 + t) * ld_kq + (long)kh * N + n;
        v = make_float2(ldf(r + k_off), ldf(r + q_off) * qscale);
      }
      KQ[e] = v;
    }
    for (int e = tid; e < nt * CW; e += 256) {
      const int t = e / CW, cc = e % CW;
      float v = 0.f;
      if (MLSTM && cc == OS_COLS) v = 1.f;
      else if (v0 + cc < dv) v = ldf(vsrc + (long)(q0 + t0 + t) * ld_v + v_off + (long)h * dv + v0 + cc);
      Vs[e] = v;
    }
    if (tid < nt) {
      const T* g = gsrc + (long)(q0 + t0 + tid) * ld_g;
      if (MLSTM) {
        // hp0 / hp1: the input and forget gates' biases
        Ga[tid] = cap * tanhf((ldf(g + g_off + h) + hp0) / cap);
        Gb[tid] = logsigmoid_f(cap * tanhf((ldf(g + g_off2 + h) + hp1) / cap));
      } else {
        // hp0: step bias, hp1: -exp(A_log)
        const float dt = softplus_f(ldf(g + g_off + h) + hp0);
        Ga[tid] = expf(hp1 * dt);
        Gb[tid] = dt;
      }
    }
    __syncthreads();
    if (live) {
      for (int t = 0; t < nt; ++t) {
        float a, b;
        if (MLSTM) {
          const float ig = Ga[t], fg = Gb[t];
          const float m2 = fmaxf(fg + m, ig);
          a = expf(fg + m - m2);
          b = expf(ig - m2);
          m = m2;
          if (tid == 0) Ms[t] = m2;
        } else {
          a = Ga[t];
          b = Gb[t];
        }
        const float bv = b * Vs[t * CW + c];
        const float2* kqr = KQ + t * NP + strip;
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < NPT; ++k) {
          const float2 kq2 = kqr[k * STRIPS];
          S[k] = a * S[k] + kq2.x * bv;
          acc += S[k] * kq2.y;
        }
        Ps[(t * STRIPS + strip) * CW + c] = acc;
      }
    }
    __syncthreads();
    for (int e = tid; e < nt * OS_COLS; e += 256) {
      const int t = e / OS_COLS, cc = e % OS_COLS;
      if (v0 + cc >= dv) continue;
      float y = 0.f;
#pragma unroll
      for (int z = 0; z < STRIPS; ++z) y += Ps[(t * STRIPS + z) * CW + cc];
      if (MLSTM) {
        float nq = 0.f;
#pragma unroll
        for (int z = 0; z < STRIPS; ++z) nq += Ps[(t * STRIPS + z) * CW + OS_COLS];
        y /= fmaxf(fabsf(nq), expf(-Ms[t])) + 1e-6f;
      } else {
        y += hp2 * Vs[t * CW + cc];      // hp2: the skip weight D
      }
      out[(long)(q0 + t0 + t) * ((long)H * dv) + (long)h * dv + v0 + cc] = y;
    }
  }
  if (col_ok) {
#pragma unroll
    for (int k = 0; k < NPT; ++k) {
      const int n = strip + k * STRIPS;
      if (n < N) {
        if (is_norm) np[n] = S[k]; else sp[(long)n * dv] = S[k];
      }
    }
    if (is_norm && strip == 0) np[N] = m;
  }
}

// each head's row of `raw` to unit RMS, times w[head, :], times sigmoid(gate): one wave per (token, head)
template <typename T>
__global__ void __launch_bounds__(256) head_norm_gate_kernel(const float* __restrict__ raw, const T* __restrict__ gate, long ldg,
                                                             const float* __restrict__ w, T* __restrict__ out, long units,
                                                             int H, int dv, float eps) {
  const long u = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (u >= units) return;
  const long tok = u / H;
  const int h = (int)(u % H);
  const float* r = raw + u * dv;
  float s = 0.f;
  for (int i = lane; i < dv; i += 64) s += r[i] * r[i];
  const float sc = 1.f / sqrtf(wave_sum(s) / (float)dv + eps);
  for (int i = lane; i < dv; i += 64) {
    const float g = ldf(gate + tok * ldg + (long)h * dv + i);
    stf(out + u * dv + i, r[i] * sc * w[h * dv + i] / (1.f + expf(-g)));
  }
}

constexpr int OS_NPT[] = {1, 2, 3, 4, 5, 6, 8, 9, 10, 12, 16, 20, 24, 32};   // instantiated rows per thread

template <bool MLSTM> int outer_npt(int N) {
  constexpr int STRIPS = 256 / (OS_COLS + (MLSTM ? 1 : 0));
  const int need = (N + STRIPS - 1) / STRIPS;
  for (int v : OS_NPT)
    if (v >= need) return v;
  return -1;
}

template <bool MLSTM> long outer_lds(int N) {
  constexpr int CW = OS_COLS + (MLSTM ? 1 : 0);
  constexpr int STRIPS = 256 / CW;
  const int npt = outer_npt<MLSTM>(N);
  if (npt < 0) return 1L << 40;
  return 4L * (2L * OS_TG * npt * STRIPS + OS_TG * CW + 3 * OS_TG + (long)OS_TG * STRIPS * CW);
}

#define ENSURE_LDS(kernel, bytes)                                                                                \
  do {                                                                                                           \
    static long have_ = 48 * 1024;                                                                               \
    if ((bytes) > have_) {                                                                                       \
      (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)); \
      have_ = (bytes);                                                                                           \
    }                                                                                                            \
  } while (0)

template <typename T, bool MLSTM, int NPT>
int launch_outer(dim3 grid, long lds, hipStream_t st, const void* kq, long ld_kq, int k_off, int q_off, int kdiv, const void* v,
                 long ld_v, int v_off, const void* g, long ld_g, int g_off, int g_off2, const float* p0, const float* p1,
                 const float* p2, float cap, float qscale, float* state, float* nm, int NCB, const int* qstart,
                 const int* qlen, const int* ctx, const int* rows, float* out, int H, int N, int dv) {
  ENSURE_LDS((outer_scan_kernel<T, MLSTM, NPT>), lds);
  hipLaunchKernelGGL((outer_scan_kernel<T, MLSTM, NPT>), grid, dim3(256), lds, st, (const T*)kq, ld_kq, k_off, q_off, kdiv,
                     (const T*)v, ld_v, v_off, (const T*)g, ld_g, g_off, g_off2, p0, p1, p2, cap, qscale, state, nm, NCB,
                     qstart, qlen, ctx, rows, out, H, N, dv);
  return (int)hipGetLastError();
}

template <typename T, bool MLSTM, typename... A>
int launch_outer_npt(int N, A... a) {
  switch (outer_npt<MLSTM>(N)) {
#define OS_CASE(V) case V: return launch_outer<T, MLSTM, V>(a...);
    OS_CASE(1) OS_CASE(2) OS_CASE(3) OS_CASE(4) OS_CASE(5) OS_CASE(6) OS_CASE(8) OS_CASE(9) OS_CASE(10) OS_CASE(12)
    OS_CASE(16) OS_CASE(20) OS_CASE(24) OS_CASE(32)
#undef OS_CASE
    default: return -2;
  }
}

}  // namespace

extern "C" int dllm_outer_scan_cols() { return OS_COLS; }

// xbc [T, ld] = x | B | C (convolved, activated), step logits at gates[:, dt_col + head]
extern "C" int dllm_ssd_scan(const void* xbc, long ld, const void* gates, long ld_g, int dt_col, int f32, int H, int dv, int N,
                             int G, const float* dt_bias, const float* neg_a, const float* D, float* state,
                             const int* qstart, const int* qlen, const int* ctx, const int* rows, int S, float* out,
                             hipStream_t st) {
  if (S <= 0) return 0;
  if (H < 1 || G < 1 || H % G || N < 1 || dv < 1) return -1;
  const long lds = outer_lds<false>(N);
  if (lds > 150 * 1024) return -2;
  const dim3 grid((dv + OS_COLS - 1) / OS_COLS, H, S);
  const int inner = H * dv;
  if (f32)
    return launch_outer_npt<float, false>(N, grid, lds, st, xbc, ld, inner, inner + G * N, H / G, xbc, ld, 0, gates, ld_g, dt_col,
                                          0, dt_bias, neg_a, D, 0.f, 1.f, state, (float*)nullptr, 0, qstart, qlen, ctx, rows,
                                          out, H, N, dv);
  return launch_outer_npt<u16, false>(N, grid, lds, st, xbc, ld, inner, inner + G * N, H / G, xbc, ld, 0, gates, ld_g, dt_col, 0,
                                      dt_bias, neg_a, D, 0.f, 1.f, state, (float*)nullptr, 0, qstart, qlen, ctx, rows, out, H,
                                      N, dv);
}

// proj [T, ld] = q | k | v | output gate | input-gate logits | forget-gate logits; gate_b = both gates' biases
extern "C" int dllm_mlstm(const void* proj, long ld, int f32, int H, int d, int dv, const float* gate_b, float cap,
                          float* state, float* nm, int NCB, float eps, const float* norm_w, const int* qstart,
                          const int* qlen, const int* ctx, const int* rows, int S, long T, float* raw, void* out,
                          hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || d < 1 || dv < 1 || !(cap > 0.f) || NCB != (dv + OS_COLS - 1) / OS_COLS) return -1;
  const long lds = outer_lds<true>(d);
  if (lds > 150 * 1024) return -2;
  const dim3 grid(NCB, H, S);
  const int kc = H * d, vc = 2 * H * d, gc = 2 * H * d + H * dv, ic = gc + H * dv, fc = ic + H;
  const float qs = 1.f / sqrtf((float)d);
  int rc = 0;
  if (S > 0) {
    if (f32)
      rc = launch_outer_npt<float, true>(d, grid, lds, st, proj, ld, kc, 0, 1, proj, ld, vc, proj, ld, ic, fc, gate_b, gate_b + H,
                                         (const float*)nullptr, cap, qs, state, nm, NCB, qstart, qlen, ctx, rows, raw, H, d, dv);
    else
      rc = launch_outer_npt<u16, true>(d, grid, lds, st, proj, ld, kc, 0, 1, proj, ld, vc, proj, ld, ic, fc, gate_b, gate_b + H,
                                       (const float*)nullptr, cap, qs, state, nm, NCB, qstart, qlen, ctx, rows, raw, H, d, dv);
    if (rc) return rc;
  }
  const long units = T * H;
  const dim3 g2((unsigned)((units + 3) / 4));
  if (f32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, g2, dim3(256), 0, st, raw, (const float*)proj + gc, ld, norm_w, (float*)out,
                       units, H, dv, eps);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<u16>, g2, dim3(256), 0, st, raw, (const u16*)proj + gc, ld, norm_w, (u16*)out, units,
                       H, dv, eps);
  return (int)hipGetLastError();
}
