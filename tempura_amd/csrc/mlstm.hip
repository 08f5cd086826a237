// The matrix-memory recurrence of an mLSTM mixer, and what turns its read-out into the rows of the output product.
//
// Per head, with a memory S [dim, vdim], a normaliser n [dim] and a running maximum m (all zero at a request's start),
// a token with log gates i and f, key k, value v and query q does
//     m' = max(f + m, i)      S' = e^(f + m - m') S + e^(i - m') k v^T      n' = e^(f + m - m') n + e^(i - m') k
//     o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)
// The normaliser is one more value column whose value is always 1 (its read-out is n' . q), so the scan works on
// vdim + 1 independent columns and needs nothing from its neighbours: a block owns a request, a head and 256 / KS
// columns; a lane keeps PER key channels of one column in registers, the KS lanes of a column add their partial
// read-outs by row permutes.  Every column carries a copy of m in the state (no column reads what another writes).
// The division, which needs the normaliser's column, is left to the kernel behind the scan.
//
// Gates: i = cap tanh((x_i + b_i) / cap), f = logsigmoid(cap tanh((x_f + b_f) / cap)).  A kernel in front of the scan (a
// wave per request and head, 64 tokens a turn) forms them, the running maximum and, per token, the decay
// keep = e^(f + m - m') and the input weight put = e^(i - m'): inside the scan they would stand in every chunk's way
// (a chain of lane exchanges and transcendental functions between two barriers while the other waves wait).  m over
// 64 tokens comes from two prefix scans over the lanes (F_t = sum_(s<=t) f_s, m_t = F_t + max(m_0, max_(s<=t) (i_s - F_s))):
// the read-out does not depend on which m is used as long as the decay, the input weight and the floor e^(-m') use
// the same one, so the order of these sums changes rounding only.
//
// State of a request from state_off on: [heads][vdim + 1][dim] (a head's memory column by column, the normaliser
// last), then [heads][vdim + 1] copies of m.  Everything is float32.
#include <math.h>

#include "column_sum.h"
#include "common.h"

struct MlstmArgs {
  const float* proj;       // [n, stride] float32 sums of the input product
  int stride, q_col, k_col, v_col, i_col, f_col;
  const float* i_bias;     // [heads]
  const float* f_bias;     // [heads]
  float* keep;             // [n, heads] e^(f + m - m')
  float* put;              // [n, heads] e^(i - m')
  float cap, q_scale;
  float* state;
  size_t state_stride, state_off;
  const int* cu_seqlens;
  const int* state_slots;
  float* num;              // [n, heads * vdim] S'^T q
  float* nq;               // [n, heads] n' . q
  float* mrun;             // [n, heads] m'
  int heads, dim, vdim;
};

__device__ inline float m_logsigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// grid: (requests, heads); block: one wave.
__global__ __launch_bounds__(64) void mlstm_gates_kernel(MlstmArgs a) {
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int start = a.cu_seqlens[r], len = a.cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  const int cols = a.vdim + 1;
  const float* m_mem = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off + (size_t)a.heads * cols * a.dim + (size_t)h * cols;
  float m = m_mem[0];      // (every column's copy is the same number)
  const float bi = a.i_bias[h], bf = a.f_bias[h];
  for (int t0 = 0; t0 < len; t0 += TP_WAVE) {
    const bool mine = t0 + lane < len;
    float gi = -INFINITY, gf = 0.f;      // (lanes past the run's end pass the sums along unchanged)
    if (mine) {
      const size_t row = (size_t)(start + t0 + lane) * a.stride;
      gi = a.cap * tanhf((a.proj[row + a.i_col + h] + bi) / a.cap);
      gf = m_logsigmoid(a.cap * tanhf((a.proj[row + a.f_col + h] + bf) / a.cap));
    }
    float F = gf;
#pragma unroll
    for (int d = 1; d < TP_WAVE; d *= 2) {
      const float o = __shfl_up(F, d, TP_WAVE);
      if (lane >= d) F += o;
    }
    float G = mine ? gi - F : -INFINITY;
#pragma unroll
    for (int d = 1; d < TP_WAVE; d *= 2) {
      const float o = __shfl_up(G, d, TP_WAVE);
      if (lane >= d) G = fmaxf(G, o);
    }
    const float m_new = F + fmaxf(m, G);
    float m_prev = __shfl_up(m_new, 1, TP_WAVE);
    if (lane == 0) m_prev = m;
    if (mine) {
      const size_t p = (size_t)(start + t0 + lane) * a.heads + h;
      a.keep[p] = expf(gf + m_prev - m_new);
      a.put[p] = expf(gi - m_new);
      a.mrun[p] = m_new;
    }
    m = __shfl(m_new, TP_WAVE - 1, TP_WAVE);
  }
}

template <int PER, int KS>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(MlstmArgs a) {
  constexpr int DP = PER * KS, CW = TP_WAVE / KS, CB = 4 * CW;
  constexpr int TC = DP <= 256 ? 16 : 4096 / DP;
  constexpr int NI = (TC * DP + 255) / 256, NV = (TC * CB + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs[TC * DP];
  __shared__ __attribute__((aligned(16))) float kk[TC * DP];
  __shared__ float vs[TC * CB];
  __shared__ float keep_s[TC], put_s[TC];
  const int r = blockIdx.x, h = blockIdx.y;
  const int start = a.cu_seqlens[r], len = a.cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  const int tid = threadIdx.x, wave = tid / TP_WAVE, lane = tid % TP_WAVE;
  const int ks = lane % KS, jl = wave * CW + lane / KS;
  const int cols = a.vdim + 1;
  const int j = blockIdx.z * CB + jl;
  const bool col_ok = j < cols, is_n = j == a.vdim;

  float* base = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off;
  float* S_mem = base + ((size_t)h * cols + (col_ok ? j : 0)) * a.dim;
  float* m_mem = base + (size_t)a.heads * cols * a.dim + (size_t)h * cols;   // (read by the kernel in front, written here)
  const bool vec = a.dim % 4 == 0 && ((uintptr_t)S_mem % 16) == 0;
  float S[PER];
#pragma unroll
  for (int e4 = 0; e4 < PER / 4; ++e4) {
    const int i = ks * PER + e4 * 4;
    if (vec && col_ok && i < a.dim) {
      const float4 v = *(const float4*)(S_mem + i);
      S[e4 * 4 + 0] = v.x; S[e4 * 4 + 1] = v.y; S[e4 * 4 + 2] = v.z; S[e4 * 4 + 3] = v.w;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) S[e4 * 4 + c] = (col_ok && i + c < a.dim) ? S_mem[i + c] : 0.f;
    }
  }
  const int q_col = a.q_col + h * a.dim, k_col = a.k_col + h * a.dim, v_col = a.v_col + h * a.vdim;
  float rq[NI], rk[NI], rv[NV], ri = 0.f, rf = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / DP, i = idx % DP;
      const bool in = idx < TC * DP && t0 + t < len && i < a.dim;
      const size_t row = (size_t)(start + t0 + t) * a.stride;
      rq[it] = in ? a.proj[row + q_col + i] * a.q_scale : 0.f;
      rk[it] = in ? a.proj[row + k_col + i] : 0.f;
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / CB, c = idx % CB;
      const int col = blockIdx.z * CB + c;
      float v = 0.f;
      if (idx < TC * CB && t0 + t < len) {
        if (col < a.vdim) v = a.proj[(size_t)(start + t0 + t) * a.stride + v_col + col];
        else if (col == a.vdim) v = 1.f;      // the normaliser's column
      }
      rv[it] = v;
    }
    if (tid < TC && t0 + tid < len) {
      const size_t p = (size_t)(start + t0 + tid) * a.heads + h;
      ri = a.put[p];
      rf = a.keep[p];
    }
  };
  struct Tok {
    float4 q[PER / 4], k[PER / 4];
    float keep, put_v;
  };
  auto take = [&](Tok& x, int t) {
    const float4* q4 = (const float4*)(qs + t * DP + ks * PER);
    const float4* k4 = (const float4*)(kk + t * DP + ks * PER);
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      x.q[e4] = q4[e4];
      x.k[e4] = k4[e4];
    }
    x.keep = keep_s[t];
    x.put_v = put_s[t] * vs[t * CB + jl];
  };
  const int out_width = a.heads * a.vdim;
  auto step = [&](const Tok& x, int t_run, int t) {
    float part[PER / 4];
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      const float qa[4] = {x.q[e4].x, x.q[e4].y, x.q[e4].z, x.q[e4].w}, ka[4] = {x.k[e4].x, x.k[e4].y, x.k[e4].z, x.k[e4].w};
      float p = 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = e4 * 4 + c;
        S[e] = fmaf(x.keep, S[e], ka[c] * x.put_v);
        p = fmaf(S[e], qa[c], p);
      }
      part[e4] = p;
    }
    float rs = part[0];
#pragma unroll
    for (int e4 = 1; e4 < PER / 4; ++e4) rs += part[e4];   // (a fixed order: the same sums wherever the token stands)
    rs = column_sum<KS>(rs);
    if (ks == 0 && col_ok) {
      const size_t row = (size_t)(start + t_run);
      if (is_n) {
        a.nq[row * a.heads + h] = rs;
      } else {
        a.num[row * out_width + (size_t)h * a.vdim + j] = rs;
      }
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < len; t0 += TC) {
    const int tc = min(TC, len - t0);
    __syncthreads();   // the chunk before has been consumed
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * 256 + tid;
      if (idx < TC * DP) {
        qs[idx] = rq[it];
        kk[idx] = rk[it];
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      if (idx < TC * CB) vs[idx] = rv[it];
    }
    if (tid < TC) {
      keep_s[tid] = rf;
      put_s[tid] = ri;
    }
    __syncthreads();
    if (t0 + TC < len) fetch(t0 + TC);   // on its way while this chunk runs
    Tok A, B;
    take(A, 0);
    for (int t = 0; t < tc; t += 2) {
      if (t + 1 < tc) take(B, t + 1);
      step(A, t0 + t, t);
      if (t + 1 < tc) {
        if (t + 2 < tc) take(A, t + 2);
        step(B, t0 + t + 1, t + 1);
      }
    }
  }
#pragma unroll
  for (int e4 = 0; e4 < PER / 4; ++e4) {
    const int i = ks * PER + e4 * 4;
    if (vec && col_ok && i < a.dim) {
      *(float4*)(S_mem + i) = make_float4(S[e4 * 4 + 0], S[e4 * 4 + 1], S[e4 * 4 + 2], S[e4 * 4 + 3]);
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (col_ok && i + c < a.dim) S_mem[i + c] = S[e4 * 4 + c];
    }
  }
  if (ks == 0 && col_ok) m_mem[j] = a.mrun[(size_t)(start + len - 1) * a.heads + h];
}

// out[t, out_col0 + h * vdim + d] = unit_rms(num[t, h, :] / (max(|nq|, e^(-m)) + 1e-6))[d] * w[h * vdim + d]
//                                   * sigmoid(proj[t, gate_col + h * vdim + d]) * scale.     One wave per (token, head).
template <typename TO>
__global__ __launch_bounds__(256) void mlstm_out_kernel(const float* __restrict__ num, const float* __restrict__ nq,
                                                        const float* __restrict__ mrun, const float* __restrict__ w,
                                                        const float* __restrict__ proj, int stride, int gate_col, float eps,
                                                        float scale, TO* __restrict__ out, int out_stride, int out_col0,
                                                        long pairs, int heads, int vdim) {
  const long p = (long)blockIdx.x * 4 + threadIdx.x / TP_WAVE;
  const int lane = threadIdx.x % TP_WAVE;
  if (p >= pairs) return;
  const long t = p / heads;
  const int h = (int)(p % heads);
  const float inv = 1.0f / (fmaxf(fabsf(nq[p]), expf(-mrun[p])) + 1e-6f);
  const float* row = num + (size_t)p * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += TP_WAVE) {
    const float o = row[d] * inv;
    ss = fmaf(o, o, ss);
  }
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)vdim + eps);
  TO* dst = out + (size_t)t * out_stride + out_col0 + (size_t)h * vdim;
  const float* gr = proj + (size_t)t * stride + gate_col + (size_t)h * vdim;
  for (int d = lane; d < vdim; d += TP_WAVE) {
    const float g = 1.0f / (1.0f + expf(-gr[d]));
    from_float(dst + d, row[d] * inv * rstd * w[(size_t)h * vdim + d] * g * scale);
  }
}

// proj columns from col0 on: [q (heads * dim) | k (heads * dim) | v (heads * vdim) | gate (heads * vdim) | i (heads) | f (heads)].
// scratch: float32 [n * heads * (vdim + 4)].
extern "C" int tp_mlstm_scan(const float* proj, int stride, int col0, const float* i_bias, const float* f_bias, float cap,
                             float q_scale, float* state, size_t state_stride, size_t state_off, const int* cu_seqlens,
                             const int* state_slots, float* scratch, const float* norm_w, float eps, float scale, void* out,
                             int out_dt, int out_stride, int out_col0, int n, int n_req, int heads, int dim, int vdim,
                             hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_req >= 0 && heads > 0 && dim > 0 && vdim > 0 && col0 >= 0, "mlstm_scan: bad sizes");
  TP_REQUIRE(dim <= 1024, "mlstm_scan: key size %d exceeds 1024", dim);
  TP_REQUIRE(cap > 0.f, "mlstm_scan: the gates' cap must be positive");
  const int width = 2 * heads * dim + 2 * heads * vdim + 2 * heads;
  TP_REQUIRE(stride >= col0 + width, "mlstm_scan: rows too short");
  TP_REQUIRE(state_stride >= state_off + (size_t)heads * (vdim + 1) * (dim + 1), "mlstm_scan: state rows too short");
  TP_REQUIRE(heads <= 65535, "mlstm_scan: too many heads");
  TP_REQUIRE(out_stride >= out_col0 + heads * vdim, "mlstm_scan: output rows too short");
  if (n == 0 || n_req == 0) return 0;
  MlstmArgs a;
  a.proj = proj;
  a.stride = stride;
  a.q_col = col0;
  a.k_col = col0 + heads * dim;
  a.v_col = col0 + 2 * heads * dim;
  const int gate_col = a.v_col + heads * vdim;
  a.i_col = gate_col + heads * vdim;
  a.f_col = a.i_col + heads;
  a.i_bias = i_bias;
  a.f_bias = f_bias;
  a.cap = cap;
  a.q_scale = q_scale;
  a.state = state;
  a.state_stride = state_stride;
  a.state_off = state_off;
  a.cu_seqlens = cu_seqlens;
  a.state_slots = state_slots;
  a.num = scratch;
  a.nq = scratch + (size_t)n * heads * vdim;
  a.mrun = a.nq + (size_t)n * heads;
  a.keep = a.mrun + (size_t)n * heads;
  a.put = a.keep + (size_t)n * heads;
  a.heads = heads;
  a.dim = dim;
  a.vdim = vdim;
  const long pairs = (long)n * heads;
  TP_REQUIRE((pairs + 3) / 4 < 0x7fffffffL, "mlstm_scan: too many rows");
  TP_REQUIRE(n_req <= 0x7fffffff / 1, "mlstm_scan: too many requests");
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3(n_req, heads), dim3(64), 0, s, a);
  // PER key channels a lane (8 up to a key size of 128, then 16, then 32), KS lanes a column (a power of two)
  const int per = dim <= 128 ? 8 : (dim <= 256 ? 16 : 32);
  int ks = 1;
  while (ks * per < dim) ks *= 2;
  const int cb = 4 * (TP_WAVE / ks);
  const dim3 grid(n_req, heads, (vdim + 1 + cb - 1) / cb);
  TP_REQUIRE(grid.z <= 65535, "mlstm_scan: too many value columns");
#define SCAN(P, K) hipLaunchKernelGGL((mlstm_scan_kernel<P, K>), grid, dim3(256), 0, s, a)
  if (per == 8) {
    if (ks == 1) SCAN(8, 1);
    else if (ks == 2) SCAN(8, 2);
    else if (ks == 4) SCAN(8, 4);
    else if (ks == 8) SCAN(8, 8);
    else SCAN(8, 16);
  } else if (per == 16) {
    SCAN(16, 16);
  } else {
    if (ks <= 16) SCAN(32, 16);
    else SCAN(32, 32);
  }
#undef SCAN
  TP_CHECK_LAUNCH("mlstm_scan");
  const dim3 og((unsigned)((pairs + 3) / 4));
  if (out_dt == TP_F32)
    hipLaunchKernelGGL(mlstm_out_kernel<float>, og, dim3(256), 0, s, a.num, a.nq, a.mrun, norm_w, proj, stride, gate_col, eps, scale,
                       (float*)out, out_stride, out_col0, pairs, heads, vdim);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(mlstm_out_kernel<bf16_t>, og, dim3(256), 0, s, a.num, a.nq, a.mrun, norm_w, proj, stride, gate_col, eps, scale,
                       (bf16_t*)out, out_stride, out_col0, pairs, heads, vdim);
  else
    TP_REQUIRE(false, "mlstm_scan: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("mlstm_out");
  return 0;
}
