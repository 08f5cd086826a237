// A generalized delta-rule recurrence over a batch of requests that each bring a run of tokens.  Per head, with a
// state S [key, value] (both of size dim), a decay w and a removal rate a per key channel, and the unit key
// u = k / sqrt(sum k^2 + unit_eps):
//   S <- diag(w) S - (a u) (u^T S) + k v^T     (both terms read the old S);     o = S^T r.
// All arithmetic is float32; the state [heads, value, key] lives in float32 rows of a per-request state tensor (row =
// request slot), a head's matrix column by column as for the gated delta rule.
//
// For one value column j with the column s of the old state:  P = u . s,  R = sum_i w_i s_i r_i,
//   s_i <- w_i s_i - (a u)_i P + k_i v_j,       o_j = R - ((a u) . r) P + (k . r) v_j,
// so one pass over a thread's entries forms both sums, one reduction over the lanes that share the column adds them,
// and a second pass writes the column.  The two dot products that do not depend on the state come from a kernel
// that runs over all tokens side by side.
//
// A request r of the batch owns tokens cu_seqlens[r] .. cu_seqlens[r + 1] - 1 and the state row state_slots[r].  A
// token's result does not depend on how its run was cut: every token is one step of the same chain, in the same
// order of operations.
#include <math.h>

#include "common.h"
#include "column_sum.h"

__device__ inline float g_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

struct GDeltaArgs {
  const float* proj;   // rows [n, proj_stride]: r | k | v | a_raw from column col0 on, each heads * dim wide
  int proj_stride, col0;
  const float* decay;  // [n, heads * dim]
  const float* a_bias; // [heads * dim]
  float* ua;           // [n, 2, heads * dim]: the unit key, then the removal rate times the unit key
  float* dots;         // [n, heads, 2]: (a u) . r and k . r
  float* state;
  size_t state_stride, state_off;
  const int* cu_seqlens;
  const int* state_slots;
  float* y;            // [n, heads * dim]
  int heads, dim;
  float unit_eps;
};

// a wave per token and head, all tokens side by side
__global__ __launch_bounds__(256) void gdelta_prep_kernel(GDeltaArgs a, long pairs) {
  const long p = (long)blockIdx.x * 4 + threadIdx.x / TP_WAVE;
  const int lane = threadIdx.x % TP_WAVE;
  if (p >= pairs) return;
  const long t = p / a.heads;
  const int h = (int)(p % a.heads);
  const int hd = a.heads * a.dim;
  const float* r = a.proj + (size_t)t * a.proj_stride + a.col0 + (size_t)h * a.dim;
  const float* k = r + hd;
  const float* ar = r + 3 * (size_t)hd;
  const float* ab = a.a_bias + (size_t)h * a.dim;
  float* u_out = a.ua + (size_t)t * 2 * hd + (size_t)h * a.dim;
  float* au_out = u_out + hd;
  float sk = 0.f;
  for (int i = lane; i < a.dim; i += TP_WAVE) sk = fmaf(k[i], k[i], sk);
  sk = wave_sum(sk);
  const float rk = 1.0f / sqrtf(sk + a.unit_eps);
  float d1 = 0.f, d2 = 0.f;
  for (int i = lane; i < a.dim; i += TP_WAVE) {
    const float u = k[i] * rk;
    const float au = g_sigmoid(ar[i] + ab[i]) * u;
    u_out[i] = u;
    au_out[i] = au;
    d1 = fmaf(au, r[i], d1);
    d2 = fmaf(k[i], r[i], d2);
  }
  d1 = wave_sum(d1);
  d2 = wave_sum(d2);
  if (lane == 0) {
    a.dots[p * 2] = d1;
    a.dots[p * 2 + 1] = d2;
  }
}

// The chain: a block owns one request, one head and CB = 256 / KS value columns; a thread holds PER consecutive key
// channels of one column in registers, and the KS neighbouring lanes that share a column split the key channels
// among them.  Tokens are taken TC at a time through LDS (rows padded to KS * PER channels with r = k = u = 0 and
// decay 1, so the run itself needs no bounds); the next chunk's values travel from memory into registers while
// this chunk runs.
template <int PER, int KS>
__global__ __launch_bounds__(256) void gdelta_scan_kernel(GDeltaArgs a) {
  constexpr int DP = PER * KS, CW = TP_WAVE / KS, CB = 4 * CW;
  constexpr int TC = DP <= 128 ? 16 : 2048 / DP;
  constexpr int NI = (TC * DP + 255) / 256, NV = (TC * CB + 255) / 256;
  __shared__ __attribute__((aligned(16))) float rs[TC * DP];
  __shared__ __attribute__((aligned(16))) float ws[TC * DP];
  __shared__ __attribute__((aligned(16))) float us[TC * DP];
  __shared__ __attribute__((aligned(16))) float as[TC * DP];
  __shared__ __attribute__((aligned(16))) float kk[TC * DP];
  __shared__ float vs[TC * CB];
  __shared__ float d1s[TC];
  __shared__ float d2s[TC];
  const int r = blockIdx.x, h = blockIdx.y;
  const int start = a.cu_seqlens[r], len = a.cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  const int tid = threadIdx.x, wave = tid / TP_WAVE, lane = tid % TP_WAVE;
  const int ks = lane % KS, jl = wave * CW + lane / KS;
  const int j = blockIdx.z * CB + jl;
  const bool col_ok = j < a.dim;
  const int hd = a.heads * a.dim;

  float* S_mem = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off + ((size_t)h * a.dim + (col_ok ? j : 0)) * a.dim;
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
  const int r_col = a.col0 + h * a.dim, k_col = r_col + hd, v_col = r_col + 2 * hd;

  float fr[NI], fw[NI], fu[NI], fa[NI], fk[NI], fv[NV], f1 = 0.f, f2 = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / DP, i = idx % DP;
      const bool in = idx < TC * DP && t0 + t < len && i < a.dim;
      const size_t row = (size_t)(start + t0 + t);
      fr[it] = in ? a.proj[row * a.proj_stride + r_col + i] : 0.f;
      fk[it] = in ? a.proj[row * a.proj_stride + k_col + i] : 0.f;
      fw[it] = in ? a.decay[row * hd + (size_t)h * a.dim + i] : 1.f;
      fu[it] = in ? a.ua[row * 2 * hd + (size_t)h * a.dim + i] : 0.f;
      fa[it] = in ? a.ua[row * 2 * hd + hd + (size_t)h * a.dim + i] : 0.f;
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / CB, c = idx % CB;
      const int col = blockIdx.z * CB + c;
      fv[it] = (idx < TC * CB && t0 + t < len && col < a.dim) ? a.proj[(size_t)(start + t0 + t) * a.proj_stride + v_col + col] : 0.f;
    }
    if (tid < TC && t0 + tid < len) {
      const size_t pair = (size_t)(start + t0 + tid) * a.heads + h;
      f1 = a.dots[pair * 2];
      f2 = a.dots[pair * 2 + 1];
    }
  };
  struct Tok {
    float4 r[PER / 4], w[PER / 4], u[PER / 4], a[PER / 4], k[PER / 4];
    float v, d1, d2;
  };
  auto take = [&](Tok& x, int t) {
    const int off = t * DP + ks * PER;
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      x.r[e4] = ((const float4*)(rs + off))[e4];
      x.w[e4] = ((const float4*)(ws + off))[e4];
      x.u[e4] = ((const float4*)(us + off))[e4];
      x.a[e4] = ((const float4*)(as + off))[e4];
      x.k[e4] = ((const float4*)(kk + off))[e4];
    }
    x.v = vs[t * CB + jl];
    x.d1 = d1s[t];
    x.d2 = d2s[t];
  };
  auto step = [&](const Tok& x, int t_run) {
    float seen = 0.f, read = 0.f;
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      const float ra[4] = {x.r[e4].x, x.r[e4].y, x.r[e4].z, x.r[e4].w}, wa[4] = {x.w[e4].x, x.w[e4].y, x.w[e4].z, x.w[e4].w},
                  ua[4] = {x.u[e4].x, x.u[e4].y, x.u[e4].z, x.u[e4].w};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = e4 * 4 + c;
        seen = fmaf(S[e], ua[c], seen);   // (the old state)
        S[e] *= wa[c];
        read = fmaf(S[e], ra[c], read);
      }
    }
    seen = column_sum<KS>(seen);
    read = column_sum<KS>(read);
#pragma unroll
    for (int e4 = 0; e4 < PER / 4; ++e4) {
      const float aa[4] = {x.a[e4].x, x.a[e4].y, x.a[e4].z, x.a[e4].w}, ka[4] = {x.k[e4].x, x.k[e4].y, x.k[e4].z, x.k[e4].w};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = e4 * 4 + c;
        S[e] = fmaf(ka[c], x.v, fmaf(-aa[c], seen, S[e]));
      }
    }
    if (ks == 0 && col_ok) a.y[(size_t)(start + t_run) * hd + (size_t)h * a.dim + j] = fmaf(x.d2, x.v, fmaf(-x.d1, seen, read));
  };
  fetch(0);
  for (int t0 = 0; t0 < len; t0 += TC) {
    const int tc = min(TC, len - t0);
    __syncthreads();   // the chunk before has been consumed
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * 256 + tid;
      if (idx < TC * DP) {
        rs[idx] = fr[it];
        ws[idx] = fw[it];
        us[idx] = fu[it];
        as[idx] = fa[it];
        kk[idx] = fk[it];
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      if (idx < TC * CB) vs[idx] = fv[it];
    }
    if (tid < TC) {
      d1s[tid] = f1;
      d2s[tid] = f2;
    }
    __syncthreads();
    if (t0 + TC < len) fetch(t0 + TC);   // on its way while this chunk runs
    // two tokens a turn, each token's LDS reads issued before the token ahead of it is worked on
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

extern "C" size_t tp_gdelta_scan_scratch(int n, int heads, int dim) {
  // floats: ua [n, 2, heads * dim] and dots [n, heads, 2]
  return (size_t)n * 2 * heads * dim + (size_t)n * heads * 2;
}

extern "C" int tp_gdelta_scan(const float* proj, int proj_stride, int col0, const float* decay, const float* a_bias, float* state,
                              size_t state_stride, size_t state_off, const int* cu_seqlens, const int* state_slots, float* y,
                              float* scratch, int n, int n_req, int heads, int dim, float unit_eps, hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_req >= 0 && heads > 0 && dim > 0 && col0 >= 0, "general_delta_scan: bad sizes");
  TP_REQUIRE(dim <= 1024, "general_delta_scan: head size %d exceeds 1024", dim);
  TP_REQUIRE((long)proj_stride >= (long)col0 + 4L * heads * dim, "general_delta_scan: rows too short");
  TP_REQUIRE(state_stride >= state_off + (size_t)heads * dim * dim, "general_delta_scan: state rows too short");
  TP_REQUIRE(heads <= 65535, "general_delta_scan: too many heads");
  if (n == 0 || n_req == 0) return 0;
  TP_REQUIRE(scratch != nullptr, "general_delta_scan: no scratch");
  GDeltaArgs a{proj, proj_stride, col0, decay, a_bias, scratch, scratch + (size_t)n * 2 * heads * dim, state, state_stride, state_off,
               cu_seqlens, state_slots, y, heads, dim, unit_eps};
  const long pairs = (long)n * heads;
  TP_REQUIRE((pairs + 3) / 4 < 0x7fffffffL, "general_delta_scan: too many rows");
  hipLaunchKernelGGL(gdelta_prep_kernel, dim3((unsigned)((pairs + 3) / 4)), dim3(256), 0, s, a, pairs);
  // PER key channels a lane (8 up to a head size of 128, then 16, then 32), KS lanes a column (a power of two)
  const int per = dim <= 128 ? 8 : (dim <= 256 ? 16 : 32);
  int ks = 1;
  while (ks * per < dim) ks *= 2;
  const int cb = 4 * (TP_WAVE / ks);
  const dim3 grid(n_req, heads, (dim + cb - 1) / cb);
  TP_REQUIRE(grid.z <= 65535, "general_delta_scan: too many value columns");
#define SCAN(P, K) hipLaunchKernelGGL((gdelta_scan_kernel<P, K>), grid, dim3(256), 0, s, a)
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
  TP_CHECK_LAUNCH("general_delta_scan");
  return 0;
}
