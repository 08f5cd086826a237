// A gated delta-rule mixer over a batch of requests that each bring a run of tokens: the recurrence over a
// per-request state, the small second product of a low-rank projection with the recurrence's decay or a sigmoid in
// its epilogue, and the per-head norm with its gate behind the recurrence.  All arithmetic is float32; the state
// [heads, value_dim, key_dim] lives in float32 rows of a per-request state tensor (row = request slot).
//
// A request r of the batch owns tokens cu_seqlens[r] .. cu_seqlens[r + 1] - 1 and the state row state_slots[r];
// everything is read from device memory, so the same launches serve prompt portions, single decoded tokens and
// captured steps.  A token's result does not depend on how its run was cut: every token is one step of the same
// chain, in the same order of operations.
#include <math.h>

#include "common.h"
#include "column_sum.h"

__device__ inline float d_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
// ln(1 + e^v) without overflow: max(v, 0) + ln(1 + e^-|v|)
__device__ inline float d_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// ---- the recurrence ---------------------------------------------------------------------------
// Per head h (its q and k are those of key head h / (heads / kv_heads)), with q and k made unit vectors
// (x / sqrt(sum x^2 + unit_eps); q also times q_scale), beta = sigmoid(beta_raw) and a decay g per key channel:
//   S <- g * S (rows are key channels);  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
// With P = (g * S_old)^T k and R = (g * S_old)^T q the read-out is o = R + u (k . q), so one pass over a thread's
// state entries forms both sums, one reduction over the lanes that share a column adds them, and a second pass
// writes k u^T.
//
// qkv [n, row_stride] float32 holds, per token, q [kv_heads * dim] | k [kv_heads * dim] | v [heads * vdim] (after the
// convolution and its activation); decay [n, heads * dim]; beta_raw is column beta_col0 + h of `proj`.
//
// Two kernels.  delta_prep (a wave per token and key head, all tokens side by side) makes q and k unit vectors in
// place and leaves k . q per token and key head.  delta_scan is the chain: a block owns one request, one head and
// CB = 256 / KS value columns; a thread holds PER consecutive key channels of one column in registers, and the KS
// neighbouring lanes that share a column split the key channels among them (their sums meet by row permutes, no
// trip through LDS up to 16 lanes).  A wave has one instruction stream, so the time of a token is the number of
// instructions a wave issues for it: few state entries a lane (8 up to a key size of 128) keep that near 60.
// Tokens are taken TC at a time through LDS (rows padded to KS * PER channels with q = k = 0 and decay 1, so the
// run itself needs no bounds); the next chunk's values travel from memory into registers while this chunk runs.
struct DeltaArgs {
  float* qkv;
  int row_stride;
  const float* decay;
  const float* proj;
  int proj_stride, beta_col0;
  float* state;
  size_t state_stride, state_off;
  const int* cu_seqlens;
  const int* state_slots;
  float* y;
  float* kq;   // [n, kv_heads]
  int heads, kv_heads, dim, vdim;
  float q_scale, unit_eps;
};

__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaArgs a, long pairs) {
  const long p = (long)blockIdx.x * 4 + threadIdx.x / TP_WAVE;
  const int lane = threadIdx.x % TP_WAVE;
  if (p >= pairs) return;
  const long t = p / a.kv_heads;
  const int g = (int)(p % a.kv_heads);
  float* q = a.qkv + (size_t)t * a.row_stride + (size_t)g * a.dim;
  float* k = q + (size_t)a.kv_heads * a.dim;
  float sq = 0.f, sk = 0.f;
  for (int i = lane; i < a.dim; i += TP_WAVE) {
    sq = fmaf(q[i], q[i], sq);
    sk = fmaf(k[i], k[i], sk);
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  const float rq = a.q_scale / sqrtf(sq + a.unit_eps), rk = 1.0f / sqrtf(sk + a.unit_eps);
  float dot = 0.f;
  for (int i = lane; i < a.dim; i += TP_WAVE) {
    const float qv = q[i] * rq, kv = k[i] * rk;
    q[i] = qv;
    k[i] = kv;
    dot = fmaf(qv, kv, dot);
  }
  dot = wave_sum(dot);
  if (lane == 0) a.kq[p] = dot;
}

template <int PER, int KS>
__global__ __launch_bounds__(256) void delta_scan_kernel(DeltaArgs a) {
  constexpr int DP = PER * KS, CW = TP_WAVE / KS, CB = 4 * CW;
  constexpr int TC = DP <= 256 ? 16 : 4096 / DP;
  constexpr int NI = (TC * DP + 255) / 256, NV = (TC * CB + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs[TC * DP];
  __shared__ __attribute__((aligned(16))) float kk[TC * DP];
  __shared__ __attribute__((aligned(16))) float gs[TC * DP];
  __shared__ float vs[TC * CB];
  __shared__ float bs[TC];
  __shared__ float kqs[TC];
  const int r = blockIdx.x, h = blockIdx.y;
  const int start = a.cu_seqlens[r], len = a.cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  const int tid = threadIdx.x, wave = tid / TP_WAVE, lane = tid % TP_WAVE;
  const int ks = lane % KS, jl = wave * CW + lane / KS;
  const int j = blockIdx.z * CB + jl;
  const bool col_ok = j < a.vdim;
  const int kvh = h / (a.heads / a.kv_heads);

  // a head's state lies in memory column by column, [vdim][dim]: the key channels of one value column are
  // neighbours, so a lane's entries are one or two 16-byte pieces and a wave's columns one contiguous run
  float* S_mem = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off + ((size_t)h * a.vdim + (col_ok ? j : 0)) * a.dim;
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
  const int q_col = kvh * a.dim, k_col = (a.kv_heads + kvh) * a.dim, v_col = 2 * a.kv_heads * a.dim + h * a.vdim;
  const int out_width = a.heads * a.vdim;
  const size_t decay_stride = (size_t)a.heads * a.dim;

  float rq[NI], rk[NI], rg[NI], rv[NV], rb = 0.f, rkq = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / DP, i = idx % DP;
      const bool in = idx < TC * DP && t0 + t < len && i < a.dim;
      const size_t row = (size_t)(start + t0 + t);
      rq[it] = in ? a.qkv[row * a.row_stride + q_col + i] : 0.f;
      rk[it] = in ? a.qkv[row * a.row_stride + k_col + i] : 0.f;
      rg[it] = in ? a.decay[row * decay_stride + (size_t)h * a.dim + i] : 1.f;
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / CB, c = idx % CB;
      const int col = blockIdx.z * CB + c;
      rv[it] = (idx < TC * CB && t0 + t < len && col < a.vdim) ? a.qkv[(size_t)(start + t0 + t) * a.row_stride + v_col + col] : 0.f;
    }
    if (tid < TC && t0 + tid < len) {
      const size_t row = (size_t)(start + t0 + tid);
      rb = d_sigmoid(a.proj[row * a.proj_stride + a.beta_col0 + h]);
      rkq = a.kq[row * a.kv_heads + kvh];
    }
  };
  struct Tok {
    float4 q[PER / 4], k[PER / 4], g[PER / 4];
    float b, v, kq;
  };
  auto take = [&](Tok& x, int t) {
    const float4* q4 = (const float4*)(qs + t * DP + ks * PER);
    const float4* k4 = (const float4*)(kk + t * DP + ks * PER);
    const float4* g4 = (const float4*)(gs + t * DP + ks * PER);
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      x.q[e4] = q4[e4];
      x.k[e4] = k4[e4];
      x.g[e4] = g4[e4];
    }
    x.b = bs[t];
    x.v = vs[t * CB + jl];
    x.kq = kqs[t];
  };
  auto step = [&](const Tok& x, int t_run) {
    float pred[PER / 4], read[PER / 4];
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      const float qa[4] = {x.q[e4].x, x.q[e4].y, x.q[e4].z, x.q[e4].w}, ka[4] = {x.k[e4].x, x.k[e4].y, x.k[e4].z, x.k[e4].w},
                  ga[4] = {x.g[e4].x, x.g[e4].y, x.g[e4].z, x.g[e4].w};
      float p = 0.f, rd = 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = e4 * 4 + c;
        S[e] *= ga[c];
        p = fmaf(S[e], ka[c], p);
        rd = fmaf(S[e], qa[c], rd);
      }
      pred[e4] = p;
      read[e4] = rd;
    }
    float ps = pred[0], rs = read[0];
#pragma unroll
    for (int e4 = 1; e4 < PER / 4; ++e4) {   // (a fixed order: the same sums wherever the token stands)
      ps += pred[e4];
      rs += read[e4];
    }
    ps = column_sum<KS>(ps);
    rs = column_sum<KS>(rs);
    const float u = x.b * (x.v - ps);
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      S[e4 * 4 + 0] = fmaf(x.k[e4].x, u, S[e4 * 4 + 0]);
      S[e4 * 4 + 1] = fmaf(x.k[e4].y, u, S[e4 * 4 + 1]);
      S[e4 * 4 + 2] = fmaf(x.k[e4].z, u, S[e4 * 4 + 2]);
      S[e4 * 4 + 3] = fmaf(x.k[e4].w, u, S[e4 * 4 + 3]);
    }
    if (ks == 0 && col_ok) a.y[(size_t)(start + t_run) * out_width + (size_t)h * a.vdim + j] = fmaf(u, x.kq, rs);
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
        gs[idx] = rg[it];
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      if (idx < TC * CB) vs[idx] = rv[it];
    }
    if (tid < TC) {
      bs[tid] = rb;
      kqs[tid] = rkq;
    }
    __syncthreads();
    if (t0 + TC < len) fetch(t0 + TC);   // on its way while this chunk runs
    // two tokens a turn, each token's LDS reads issued before the token ahead of it is worked on: a wave issues in
    // order, and reads that start only when the chain reaches them would add their whole latency to every token
    Tok A, B;
    take(A, 0);
    for (int t = 0; t < tc; t += 2) {
      if (t + 1 < tc) take(B, t + 1);
      step(A, t0 + t);
      if (t + 1 < tc) {
        if (t + 2 < tc) take(A, t + 2);
        step(B, t0 + t + 1);
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
}

extern "C" int tp_delta_scan(float* qkv, int row_stride, const float* decay, const float* proj, int proj_stride,
                             int beta_col0, float* state, size_t state_stride, size_t state_off, const int* cu_seqlens,
                             const int* state_slots, float* y, float* kq, int n, int n_req, int heads, int kv_heads, int dim,
                             int vdim, float q_scale, float unit_eps, hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_req >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "delta_scan: bad sizes");
  TP_REQUIRE(heads % kv_heads == 0, "delta_scan: %d heads is not a multiple of %d key heads", heads, kv_heads);
  TP_REQUIRE(dim <= 1024, "delta_scan: key size %d exceeds 1024", dim);
  TP_REQUIRE(row_stride >= 2 * kv_heads * dim + heads * vdim, "delta_scan: rows too short");
  TP_REQUIRE(state_stride >= state_off + (size_t)heads * dim * vdim, "delta_scan: state rows too short");
  TP_REQUIRE(heads <= 65535, "delta_scan: too many heads");
  if (n == 0 || n_req == 0) return 0;
  DeltaArgs a{qkv, row_stride, decay, proj, proj_stride, beta_col0, state, state_stride, state_off, cu_seqlens, state_slots, y, kq,
              heads, kv_heads, dim, vdim, q_scale, unit_eps};
  const long pairs = (long)n * kv_heads;
  TP_REQUIRE((pairs + 3) / 4 < 0x7fffffffL, "delta_scan: too many rows");
  hipLaunchKernelGGL(delta_prep_kernel, dim3((unsigned)((pairs + 3) / 4)), dim3(256), 0, s, a, pairs);
  // PER key channels a lane (8 up to a key size of 128, then 16, then 32), KS lanes a column (a power of two)
  const int per = dim <= 128 ? 8 : (dim <= 256 ? 16 : 32);
  int ks = 1;
  while (ks * per < dim) ks *= 2;
  const int cb = 4 * (TP_WAVE / ks);
  const dim3 grid(n_req, heads, (vdim + cb - 1) / cb);
  TP_REQUIRE(grid.z <= 65535, "delta_scan: too many value columns");
#define SCAN(P, K) hipLaunchKernelGGL((delta_scan_kernel<P, K>), grid, dim3(256), 0, s, a)
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
  TP_CHECK_LAUNCH("delta_scan");
  return 0;
}

// ---- the second product of a low-rank projection ----------------------------------------------
// out[t, c] = f(sum_i x[t, col0 + i] * wt[i, c]) for a small inner size `rank`; x are float32 rows (the first
// product's sums), wt float32 [rank, n_out] (the weight transposed, so that neighbouring lanes read neighbouring
// values).  f: 0 the sum itself; 1 its sigmoid; 2 a decay, exp(-exp(a_log[c / per_head]) * softplus(sum + bias[c]));
// 3 a decay between exp(-rate) and 1, exp(-rate * sigmoid(sum + bias[c])).  in_act 1: tanh of every x first.
// A block takes eight rows and 256 columns; a row's sum has the same order of additions wherever the row stands.
#define LR_ROWS 8

__global__ __launch_bounds__(256) void lowrank_up_kernel(const float* __restrict__ x, int x_stride, int col0, int rank,
                                                         const float* __restrict__ wt, float* __restrict__ out, int n,
                                                         int n_out, int mode, const float* __restrict__ a_log,
                                                         const float* __restrict__ bias, int per_head, int in_act,
                                                         float rate_const) {
  // (blocks of 64 or 256 threads: a thread owns one column)
  extern __shared__ __attribute__((aligned(16))) float xs[];   // [LR_ROWS][rank4]: rows padded with zeros to four
  const int rank4 = (rank + 3) & ~3;
  const int t0 = blockIdx.x * LR_ROWS, c = blockIdx.y * blockDim.x + threadIdx.x;
  for (int idx = threadIdx.x; idx < LR_ROWS * rank4; idx += blockDim.x) {
    const int t = idx / rank4, i = idx % rank4;
    const float v = (t0 + t < n && i < rank) ? x[(size_t)(t0 + t) * x_stride + col0 + i] : 0.f;
    xs[idx] = in_act == 1 ? tanhf(v) : v;
  }
  __syncthreads();
  if (c >= n_out) return;
  float acc[LR_ROWS];
#pragma unroll
  for (int t = 0; t < LR_ROWS; ++t) acc[t] = 0.f;
#pragma unroll 4
  for (int i = 0; i < rank4; i += 4) {   // (ascending i for every row: the same sums wherever the row stands)
    float w[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) w[d] = i + d < rank ? wt[(size_t)(i + d) * n_out + c] : 0.f;
#pragma unroll
    for (int t = 0; t < LR_ROWS; ++t) {
      const float4 v = *(const float4*)(xs + t * rank4 + i);
      acc[t] = fmaf(v.x, w[0], acc[t]);
      acc[t] = fmaf(v.y, w[1], acc[t]);
      acc[t] = fmaf(v.z, w[2], acc[t]);
      acc[t] = fmaf(v.w, w[3], acc[t]);
    }
  }
  float rate = 0.f, b = 0.f;
  if (mode == 2) {
    rate = expf(a_log[c / per_head]);
    b = bias[c];
  }
  if (mode == 3) {
    rate = rate_const;
    b = bias[c];
  }
#pragma unroll
  for (int t = 0; t < LR_ROWS; ++t) {
    if (t0 + t >= n) break;
    float v = acc[t];
    if (mode == 1) v = d_sigmoid(v);
    if (mode == 2) v = expf(-rate * d_softplus(v + b));
    if (mode == 3) v = expf(-rate * d_sigmoid(v + b));
    out[(size_t)(t0 + t) * n_out + c] = v;
  }
}

extern "C" int tp_lowrank_up(const float* x, int x_stride, int col0, int rank, const float* wt, float* out, int n, int n_out,
                             int mode, const float* a_log, const float* bias, int per_head, int in_act, float rate, hipStream_t s) {
  TP_REQUIRE(n >= 0 && rank > 0 && n_out > 0 && col0 >= 0 && x_stride >= col0 + rank, "lowrank_up: bad sizes");
  TP_REQUIRE(rank <= 1024, "lowrank_up: inner size %d exceeds 1024", rank);
  TP_REQUIRE(mode >= 0 && mode <= 3 && (in_act == 0 || in_act == 1), "lowrank_up: unknown epilogue %d or input function %d", mode, in_act);
  TP_REQUIRE(mode != 3 || bias, "lowrank_up: the decay needs its biases");
  TP_REQUIRE(mode != 2 || (a_log && bias && per_head > 0), "lowrank_up: the decay needs its rates and biases");
  if (n == 0) return 0;
  // (a few rows: blocks of one wave, so that the columns are spread over many CUs)
  const int threads = n <= 64 ? 64 : 256;
  const dim3 grid((n + LR_ROWS - 1) / LR_ROWS, (n_out + threads - 1) / threads);
  TP_REQUIRE(grid.y <= 65535, "lowrank_up: too many columns");
  hipLaunchKernelGGL(lowrank_up_kernel, grid, dim3(threads), sizeof(float) * LR_ROWS * ((rank + 3) & ~3), s, x, x_stride, col0, rank, wt, out, n,
                     n_out, mode, a_log, bias, per_head, in_act, rate);
  TP_CHECK_LAUNCH("lowrank_up");
  return 0;
}

// ---- norm per head with a gate ----------------------------------------------------------------
// out[t, out_col0 + h * vdim + d] = o[t, h, d] / sqrt(mean_d o^2 + eps) * w[d] * gate[t, h * vdim + d] * scale;
// gate (float32, already between 0 and 1) may be missing.  w_stride vdim: every head has its own weight [heads, vdim]
// (0: one weight [vdim] for all).  gate_raw: the gate is sigmoid(gate[t * gate_stride + h * vdim + d]) of raw rows.
// One wave per (token, head).
template <typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const float* __restrict__ gate, float eps, float scale,
                                                             TO* __restrict__ out, int out_stride, int out_col0, long pairs,
                                                             int heads, int vdim, int w_stride, size_t gate_stride, int gate_raw) {
  const long p = (long)blockIdx.x * 4 + threadIdx.x / TP_WAVE;
  const int lane = threadIdx.x % TP_WAVE;
  if (p >= pairs) return;
  const long t = p / heads;
  const int h = (int)(p % heads);
  const float* row = o + (size_t)p * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += TP_WAVE) ss = fmaf(row[d], row[d], ss);
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)vdim + eps);
  TO* dst = out + (size_t)t * out_stride + out_col0 + (size_t)h * vdim;
  const float* wh = w + (size_t)h * w_stride;
  const float* gr = gate != nullptr ? gate + (size_t)t * gate_stride + (size_t)h * vdim : nullptr;
  for (int d = lane; d < vdim; d += TP_WAVE) {
    float v = row[d] * rstd * wh[d];
    if (gr != nullptr) v *= gate_raw ? d_sigmoid(gr[d]) : gr[d];
    from_float(dst + d, v * scale);
  }
}

extern "C" int tp_head_norm_gate(const float* o, const float* w, const float* gate, float eps, float scale, void* out, int out_dt,
                                 int out_stride, int out_col0, int n, int heads, int vdim, int w_per_head, size_t gate_stride,
                                 int gate_raw, hipStream_t s) {
  TP_REQUIRE(n >= 0 && heads > 0 && vdim > 0 && out_col0 >= 0 && out_stride >= out_col0 + heads * vdim, "head_norm_gate: bad sizes");
  if (n == 0) return 0;
  const long pairs = (long)n * heads;
  const long blocks = (pairs + 3) / 4;
  TP_REQUIRE(blocks < 0x7fffffffL, "head_norm_gate: too many rows");
  if (out_dt == TP_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, o, w, gate, eps, scale, (float*)out,
                       out_stride, out_col0, pairs, heads, vdim, w_per_head ? vdim : 0, gate_stride, gate_raw);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, s, o, w, gate, eps, scale, (bf16_t*)out,
                       out_stride, out_col0, pairs, heads, vdim, w_per_head ? vdim : 0, gate_stride, gate_raw);
  else
    TP_REQUIRE(false, "head_norm_gate: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("head_norm_gate");
  return 0;
}
