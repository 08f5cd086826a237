// Small kernels around the products of a layer: an embedding with a hashed bigram table, the gate on an attention's
// output, the norm behind a sublayer added into the residual stream, a plain activation, and the router of a
// mixture of experts and what moves rows into the order of the experts and back.  Float32 arithmetic throughout; a row's result
// never depends on other rows.
#include <math.h>

#include "common.h"

__device__ inline float l_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

// ---- embedding plus a row of a hashed bigram table --------------------------------------------
// out[t] = table[token] * scale + bigram[row] (+ pos_table[position], a learned row per position), row = (previous * mul_prev + token * mul_cur) mod buckets, and row `buckets`
// (the table's last) for the token at position 0.  The previous token is the one before it in the step's run, or,
// for a run's first token, what the request's state row holds; a second kernel leaves each run's last token there.
template <typename T>
__global__ void embed_bigram_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                                    const int* __restrict__ token_req, const int* __restrict__ cu_seqlens,
                                    const int* __restrict__ state_slots, const int* __restrict__ prev_state,
                                    const T* __restrict__ table, const T* __restrict__ bigram, float* __restrict__ out,
                                    int hidden, long long mul_prev, long long mul_cur, long long buckets, float scale,
                                    const T* __restrict__ pos_table) {
  const int t = blockIdx.x;
  const int tok = tokens[t];
  long long row = buckets;
  if (bigram != nullptr && positions[t] != 0) {
    const int r = token_req[t];
    const int prev = t > cu_seqlens[r] ? tokens[t - 1] : prev_state[state_slots[r]];
    row = ((long long)prev * mul_prev + (long long)tok * mul_cur) % buckets;
  }
  const T* a = table + (size_t)tok * hidden;
  const T* b = bigram != nullptr ? bigram + (size_t)row * hidden : nullptr;
  // (scale 1 and no position table: the sum of the two rows as it always was)
  const T* p = pos_table != nullptr ? pos_table + (size_t)positions[t] * hidden : nullptr;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float v = to_float(a[c]) * scale;
    if (b != nullptr) v += to_float(b[c]);
    if (p != nullptr) v += to_float(p[c]);
    out[(size_t)t * hidden + c] = v;
  }
}

__global__ void last_token_kernel(const int* __restrict__ tokens, const int* __restrict__ cu_seqlens,
                                  const int* __restrict__ state_slots, int* __restrict__ prev_state, int n_req) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n_req) return;
  const int end = cu_seqlens[r + 1];
  if (end > cu_seqlens[r]) prev_state[state_slots[r]] = tokens[end - 1];
}

extern "C" int tp_embed_bigram(const int* tokens, const int* positions, const int* token_req, const int* cu_seqlens,
                               const int* state_slots, int* prev_state, const void* table, const void* bigram, int dt,
                               float* out, int n, int n_req, int hidden, long long mul_prev, long long mul_cur,
                               long long buckets, float scale, const void* pos_table, hipStream_t s) {
  // (bigram may be missing: the token's row times scale, plus the position's row)
  TP_REQUIRE(n >= 0 && n_req >= 0 && hidden > 0 && (bigram == nullptr || buckets > 0) && mul_prev >= 0 && mul_cur >= 0, "embed_bigram: bad sizes");
  if (n == 0) return 0;
  const int threads = hidden >= 256 ? 256 : 64;
  if (dt == TP_F32)
    hipLaunchKernelGGL(embed_bigram_kernel<float>, dim3(n), dim3(threads), 0, s, tokens, positions, token_req, cu_seqlens,
                       state_slots, prev_state, (const float*)table, (const float*)bigram, out, hidden, mul_prev, mul_cur, buckets, scale,
                       (const float*)pos_table);
  else if (dt == TP_BF16)
    hipLaunchKernelGGL(embed_bigram_kernel<bf16_t>, dim3(n), dim3(threads), 0, s, tokens, positions, token_req, cu_seqlens,
                       state_slots, prev_state, (const bf16_t*)table, (const bf16_t*)bigram, out, hidden, mul_prev, mul_cur, buckets, scale,
                       (const bf16_t*)pos_table);
  else
    TP_REQUIRE(false, "embed_bigram: unknown dtype %d", dt);
  if (n_req > 0 && bigram != nullptr)
    hipLaunchKernelGGL(last_token_kernel, dim3((n_req + 63) / 64), dim3(64), 0, s, tokens, cu_seqlens, state_slots, prev_state, n_req);
  TP_CHECK_LAUNCH("embed_bigram");
  return 0;
}

// ---- gate on a mixer's output -----------------------------------------------------------------
// out[t, out_col0 + c] = a[t, c] * sigmoid(proj[t, gate_col0 + c]) * scale (no gate: a * scale); the product is
// formed in float32 and rounded once.
template <typename T>
__global__ void sigmoid_gate_kernel(const T* __restrict__ a, const float* __restrict__ proj, int proj_stride, int gate_col0,
                                    float scale, T* __restrict__ out, int out_stride, int out_col0, int width, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / width;
  const int c = (int)(i % width);
  float v = to_float(a[i]);
  if (proj != nullptr) v *= l_sigmoid(proj[t * proj_stride + gate_col0 + c]);
  from_float(out + t * out_stride + out_col0 + c, v * scale);
}

// the same, four neighbouring columns a thread (every width, stride and first column a multiple of four)
template <typename T>
__global__ void sigmoid_gate4_kernel(const T* __restrict__ a, const float* __restrict__ proj, int proj_stride, int gate_col0,
                                     float scale, T* __restrict__ out, int out_stride, int out_col0, int width, size_t total4) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const int w4 = width / 4;
  const size_t t = i / w4;
  const int c = (int)(i % w4) * 4;
  float v[4];
  if constexpr (sizeof(T) == 2) {
    const uint2 raw = *(const uint2*)(a + t * width + c);
    bf16_t h0{(uint16_t)(raw.x & 0xffff)}, h1{(uint16_t)(raw.x >> 16)}, h2{(uint16_t)(raw.y & 0xffff)}, h3{(uint16_t)(raw.y >> 16)};
    v[0] = bf16_to_float(h0); v[1] = bf16_to_float(h1); v[2] = bf16_to_float(h2); v[3] = bf16_to_float(h3);
  } else {
    const float4 raw = *(const float4*)(a + t * width + c);
    v[0] = raw.x; v[1] = raw.y; v[2] = raw.z; v[3] = raw.w;
  }
  if (proj != nullptr) {
    const float4 g = *(const float4*)(proj + t * proj_stride + gate_col0 + c);
    v[0] *= l_sigmoid(g.x); v[1] *= l_sigmoid(g.y); v[2] *= l_sigmoid(g.z); v[3] *= l_sigmoid(g.w);
  }
  from_float4(out + t * out_stride + out_col0 + c, v[0] * scale, v[1] * scale, v[2] * scale, v[3] * scale);
}

extern "C" int tp_sigmoid_gate(const void* a, int dt, const float* proj, int proj_stride, int gate_col0, float scale, void* out,
                               int out_stride, int out_col0, int n, int width, hipStream_t s) {
  TP_REQUIRE(n >= 0 && width > 0 && out_col0 >= 0 && out_stride >= out_col0 + width, "sigmoid_gate: bad sizes");
  TP_REQUIRE(proj == nullptr || (gate_col0 >= 0 && proj_stride >= gate_col0 + width), "sigmoid_gate: gate rows too short");
  TP_REQUIRE(dt == TP_F32 || dt == TP_BF16, "sigmoid_gate: unknown dtype %d", dt);
  if (n == 0) return 0;
  const size_t esz = dt == TP_F32 ? 4 : 2;
  const bool four = width % 4 == 0 && out_stride % 4 == 0 && out_col0 % 4 == 0 && (proj == nullptr || (proj_stride % 4 == 0 && gate_col0 % 4 == 0)) &&
                    (uintptr_t)a % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)proj % 16 == 0 && esz * 4 <= 16;
  if (four) {
    const size_t total4 = (size_t)n * (width / 4);
    const dim3 grid((unsigned)((total4 + 255) / 256));
    if (dt == TP_F32)
      hipLaunchKernelGGL(sigmoid_gate4_kernel<float>, grid, dim3(256), 0, s, (const float*)a, proj, proj_stride, gate_col0, scale,
                         (float*)out, out_stride, out_col0, width, total4);
    else
      hipLaunchKernelGGL(sigmoid_gate4_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)a, proj, proj_stride, gate_col0, scale,
                         (bf16_t*)out, out_stride, out_col0, width, total4);
  } else {
    const size_t total = (size_t)n * width;
    const dim3 grid((unsigned)((total + 255) / 256));
    if (dt == TP_F32)
      hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, dim3(256), 0, s, (const float*)a, proj, proj_stride, gate_col0, scale,
                         (float*)out, out_stride, out_col0, width, total);
    else
      hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)a, proj, proj_stride, gate_col0, scale,
                         (bf16_t*)out, out_stride, out_col0, width, total);
  }
  TP_CHECK_LAUNCH("sigmoid_gate");
  return 0;
}

// ---- a sublayer's output, normed, into the residual stream ------------------------------------
// h[t] += y[t] / sqrt(mean(y[t]^2) + eps) * w; then, with w_next, the next sublayer's input
// x[t] = h[t] / sqrt(mean(h[t]^2) + eps_next) * w_next as TO.  One block per row.
template <typename TO>
__global__ __launch_bounds__(256) void norm_add_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                       const float* __restrict__ w, float eps,
                                                       const float* __restrict__ w_next, float eps_next,
                                                       TO* __restrict__ x, int width) {
  __shared__ float scratch[32];
  const size_t base = (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) ss = fmaf(y[base + c], y[base + c], ss);
  ss = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(ss / (float)width + eps);
  float ss2 = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = h[base + c] + y[base + c] * rstd * w[c];
    h[base + c] = v;
    ss2 = fmaf(v, v, ss2);
  }
  if (w_next == nullptr) return;
  ss2 = block_sum(ss2, scratch);
  const float rstd2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
  // (each thread reads back what it wrote itself)
  for (int c = threadIdx.x; c < width; c += blockDim.x) from_float(x + base + c, h[base + c] * rstd2 * w_next[c]);
}

// The same with the row in registers: every value is read once, sixteen bytes a load, all loads of a pass in flight
// together (width a multiple of four, at most 256 * 4 * NV).  The sums are formed in the generic kernel's order of
// a thread's own elements only where the widths agree; a row's result never depends on other rows either way.
template <typename TO, int NV>
__global__ __launch_bounds__(256) void norm_add_reg_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                           const float* __restrict__ w, float eps,
                                                           const float* __restrict__ w_next, float eps_next,
                                                           TO* __restrict__ x, int width) {
  __shared__ float scratch[32];
  const size_t base = (size_t)blockIdx.x * width;
  const int w4 = width / 4;
  float4 yv[NV], hv[NV], wv[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int c = k * 256 + threadIdx.x;
    if (c < w4) {
      yv[k] = *(const float4*)(y + base + 4 * c);
      hv[k] = *(const float4*)(h + base + 4 * c);
      wv[k] = *(const float4*)(w + 4 * c);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k)
    if (k * 256 + threadIdx.x < w4) {
      ss = fmaf(yv[k].x, yv[k].x, ss);
      ss = fmaf(yv[k].y, yv[k].y, ss);
      ss = fmaf(yv[k].z, yv[k].z, ss);
      ss = fmaf(yv[k].w, yv[k].w, ss);
    }
  ss = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(ss / (float)width + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int c = k * 256 + threadIdx.x;
    if (c < w4) {
      hv[k].x += yv[k].x * rstd * wv[k].x;
      hv[k].y += yv[k].y * rstd * wv[k].y;
      hv[k].z += yv[k].z * rstd * wv[k].z;
      hv[k].w += yv[k].w * rstd * wv[k].w;
      *(float4*)(h + base + 4 * c) = hv[k];
      ss2 = fmaf(hv[k].x, hv[k].x, ss2);
      ss2 = fmaf(hv[k].y, hv[k].y, ss2);
      ss2 = fmaf(hv[k].z, hv[k].z, ss2);
      ss2 = fmaf(hv[k].w, hv[k].w, ss2);
    }
  }
  if (w_next == nullptr) return;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int c = k * 256 + threadIdx.x;
    if (c < w4) wv[k] = *(const float4*)(w_next + 4 * c);
  }
  ss2 = block_sum(ss2, scratch);
  const float rstd2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int c = k * 256 + threadIdx.x;
    if (c < w4) from_float4(x + base + 4 * c, hv[k].x * rstd2 * wv[k].x, hv[k].y * rstd2 * wv[k].y, hv[k].z * rstd2 * wv[k].z, hv[k].w * rstd2 * wv[k].w);
  }
}

extern "C" int tp_norm_add(float* h, const float* y, const float* w, float eps, const float* w_next, float eps_next, void* x,
                           int x_dt, int n, int width, hipStream_t s) {
  TP_REQUIRE(n >= 0 && width > 0, "norm_add: bad sizes");
  TP_REQUIRE(w_next == nullptr || x != nullptr, "norm_add: no place for the next rows");
  if (n == 0) return 0;
  TP_REQUIRE(w_next == nullptr || x_dt == TP_F32 || x_dt == TP_BF16, "norm_add: unknown dtype %d", x_dt);
  const bool aligned = ((uintptr_t)h % 16) == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)w_next % 16) == 0 &&
                       ((uintptr_t)x % 16) == 0;
  if (width % 4 == 0 && width >= 1024 && width <= 256 * 4 * 8 && aligned) {
    const bool bf = w_next != nullptr && x_dt == TP_BF16;
#define NA(NV)                                                                                                                   \
  do {                                                                                                                           \
    if (bf)                                                                                                                      \
      hipLaunchKernelGGL((norm_add_reg_kernel<bf16_t, NV>), dim3(n), dim3(256), 0, s, h, y, w, eps, w_next, eps_next, (bf16_t*)x, width); \
    else                                                                                                                         \
      hipLaunchKernelGGL((norm_add_reg_kernel<float, NV>), dim3(n), dim3(256), 0, s, h, y, w, eps, w_next, eps_next, (float*)x, width);   \
  } while (0)
    if (width <= 2048) NA(2);
    else if (width <= 4096) NA(4);
    else NA(8);
#undef NA
    TP_CHECK_LAUNCH("norm_add");
    return 0;
  }
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  if (w_next == nullptr || x_dt == TP_F32)
    hipLaunchKernelGGL(norm_add_kernel<float>, dim3(n), dim3(threads), 0, s, h, y, w, eps, w_next, eps_next, (float*)x, width);
  else if (x_dt == TP_BF16)
    hipLaunchKernelGGL(norm_add_kernel<bf16_t>, dim3(n), dim3(threads), 0, s, h, y, w, eps, w_next, eps_next, (bf16_t*)x, width);
  else
    TP_REQUIRE(false, "norm_add: unknown dtype %d", x_dt);
  TP_CHECK_LAUNCH("norm_add");
  return 0;
}

// ---- a plain activation -----------------------------------------------------------------------
// kind 0: the tanh form of GELU, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))); kind 1: SiLU; kind 2: the exact
// GELU, 0.5 z (1 + erf(z / sqrt(2))).
__device__ inline float act_f(float z, int kind) {
  if (kind == 0) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  if (kind == 2) return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
  return z * l_sigmoid(z);
}

// Rows of a wider float32 tensor: out[t, c] = act(in[t, col0 + c]) for c < width, times sigmoid(in[t, gate_col]) when
// gate_col >= 0 (one gate a row: what a product behind it would be multiplied by, folded into its input).
template <typename TO>
__global__ void activation_rows_kernel(const float* __restrict__ in, size_t in_stride, int col0, int width, int gate_col,
                                       TO* __restrict__ out, size_t total, int kind) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / width;
  const int c = (int)(i % width);
  const float* row = in + t * in_stride;
  float v = act_f(row[col0 + c], kind);
  if (gate_col >= 0) v *= l_sigmoid(row[gate_col]);
  from_float(out + i, v);
}

extern "C" int tp_activation_rows(const float* in, size_t in_stride, int col0, int width, int gate_col, void* out, int out_dt, int n,
                                  int kind, hipStream_t s) {
  TP_REQUIRE(kind >= 0 && kind <= 2, "activation: unknown kind %d", kind);
  TP_REQUIRE(n >= 0 && width > 0 && col0 >= 0 && (size_t)(col0 + width) <= in_stride && gate_col < (long)in_stride, "activation: bad rows");
  const size_t total = (size_t)n * width;
  if (total == 0) return 0;
  const dim3 grid((unsigned)((total + 255) / 256));
  if (out_dt == TP_F32)
    hipLaunchKernelGGL(activation_rows_kernel<float>, grid, dim3(256), 0, s, in, in_stride, col0, width, gate_col, (float*)out, total, kind);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(activation_rows_kernel<bf16_t>, grid, dim3(256), 0, s, in, in_stride, col0, width, gate_col, (bf16_t*)out, total, kind);
  else
    TP_REQUIRE(false, "activation: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("activation_rows");
  return 0;
}

template <typename TI, typename TO>
__global__ void activation_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t total, int kind) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  from_float(out + i, act_f(to_float(in[i]), kind));
}

// float32 in, four neighbouring elements a thread
template <typename TO>
__global__ void activation4_kernel(const float* __restrict__ in, TO* __restrict__ out, size_t total4, int kind) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const float4 z = *(const float4*)(in + 4 * i);
  from_float4(out + 4 * i, act_f(z.x, kind), act_f(z.y, kind), act_f(z.z, kind), act_f(z.w, kind));
}

extern "C" int tp_activation(const void* in, int in_dt, void* out, int out_dt, size_t total, int kind, hipStream_t s) {
  TP_REQUIRE(kind >= 0 && kind <= 2, "activation: unknown kind %d", kind);
  if (total == 0) return 0;
  if (in_dt == TP_F32 && total % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0 && (out_dt == TP_F32 || out_dt == TP_BF16)) {
    const size_t total4 = total / 4;
    const dim3 grid4((unsigned)((total4 + 255) / 256));
    if (out_dt == TP_F32)
      hipLaunchKernelGGL(activation4_kernel<float>, grid4, dim3(256), 0, s, (const float*)in, (float*)out, total4, kind);
    else
      hipLaunchKernelGGL(activation4_kernel<bf16_t>, grid4, dim3(256), 0, s, (const float*)in, (bf16_t*)out, total4, kind);
    TP_CHECK_LAUNCH("activation");
    return 0;
  }
  const dim3 grid((unsigned)((total + 255) / 256));
#define ACT(TI, TO) hipLaunchKernelGGL((activation_kernel<TI, TO>), grid, dim3(256), 0, s, (const TI*)in, (TO*)out, total, kind)
  if (in_dt == TP_F32 && out_dt == TP_F32)
    ACT(float, float);
  else if (in_dt == TP_F32 && out_dt == TP_BF16)
    ACT(float, bf16_t);
  else if (in_dt == TP_BF16 && out_dt == TP_BF16)
    ACT(bf16_t, bf16_t);
  else
    TP_REQUIRE(false, "activation: unsupported dtypes %d -> %d", in_dt, out_dt);
#undef ACT
  TP_CHECK_LAUNCH("activation");
  return 0;
}

// ---- router of a mixture of experts -----------------------------------------------------------
// logits [n, logit_stride] float32 (the first `experts` columns count).  s = softmax over the experts; the choice
// score of expert e is s[e] + correction[e]; experts form `groups` equal groups of neighbours, a group's score is
// its largest choice score, and only experts of the `keep` best groups can be chosen (groups <= 1: all); the `top`
// allowed experts with the largest choice scores are chosen (ties: the lower index), and a chosen expert's weight
// is s[e].  dense [n, experts] gets the weight of every chosen expert and 0 elsewhere; ids and weights [n, top]
// list the chosen experts in the order of choice.  One wave per token; lane l holds experts l, l + 64, ...
#define ROUTE_PER_LANE 8   // experts <= 64 * ROUTE_PER_LANE

__device__ inline void wave_arg_best(float& v, int& i) {
#pragma unroll
  for (int o = TP_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, TP_WAVE);
    const int oi = __shfl_xor(i, o, TP_WAVE);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// score_kind 0: s = softmax over the experts; 1: s = sigmoid of each logit by itself.  The choice score is s plus the
// correction (none: s).  A group is ranked by the sum of its `group_best` largest choice scores.  The weights are the
// chosen experts' s, with `normalize` divided by their sum plus sum_eps (added in the order of choice), times `scale`.
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int logit_stride,
                                                        const float* __restrict__ correction, int experts, int top,
                                                        int groups, int keep, float* __restrict__ dense,
                                                        int* __restrict__ ids, float* __restrict__ weights, int n,
                                                        int score_kind, int group_best, int normalize, float sum_eps,
                                                        float scale, const float* __restrict__ logit_bias) {
  extern __shared__ float lds[];   // per wave: choice scores [experts], then group scores [groups]
  const int wave = threadIdx.x / TP_WAVE, lane = threadIdx.x % TP_WAVE;
  // (a wave past the last token works on the last token again and stores nothing: every wave reaches every barrier)
  const bool live = blockIdx.x * 4 + wave < n;
  const int t = live ? blockIdx.x * 4 + wave : n - 1;
  float* choice_l = lds + (size_t)wave * (experts + max(groups, 1));
  float* group_l = choice_l + experts;
  float z[ROUTE_PER_LANE], sc[ROUTE_PER_LANE], ch[ROUTE_PER_LANE];
  int won[ROUTE_PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = lane + k * TP_WAVE;
    z[k] = e < experts ? logits[(size_t)t * logit_stride + e] + (logit_bias != nullptr ? logit_bias[e] : 0.f) : -INFINITY;
    mx = fmaxf(mx, z[k]);
    won[k] = -1;
  }
  if (score_kind == 1) {
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k) sc[k] = lane + k * TP_WAVE < experts ? l_sigmoid(z[k]) : 0.f;
  } else {
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k) {
      sc[k] = lane + k * TP_WAVE < experts ? expf(z[k] - mx) : 0.f;
      sum += sc[k];
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k) sc[k] *= inv;
  }
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = lane + k * TP_WAVE;
    ch[k] = e < experts ? (correction != nullptr ? sc[k] + correction[e] : sc[k]) : -INFINITY;
    if (e < experts) {
      choice_l[e] = ch[k];
      if (live) dense[(size_t)t * experts + e] = 0.f;
    }
  }
  if (groups > 1) {
    const int per = experts / groups;
    __syncthreads();
    for (int g = lane; g < groups; g += TP_WAVE) {
      // the group's largest scores one after the other (equal scores: the lower index first), added in that order
      float total = 0.f, pv = INFINITY;
      int pi = -1;
      for (int b = 0; b < group_best; ++b) {
        float best = -INFINITY;
        int bi = -1;
        for (int i = 0; i < per; ++i) {
          const float v = choice_l[g * per + i];
          if ((v < pv || (v == pv && i > pi)) && (bi < 0 || v > best)) {
            best = v;
            bi = i;
          }
        }
        if (bi < 0) break;
        total = b == 0 ? best : total + best;
        pv = best;
        pi = bi;
      }
      group_l[g] = total;
    }
    __syncthreads();
    // the `keep` best groups, one after the other; a kept group's score becomes +inf as its mark
    for (int it = 0; it < keep; ++it) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < groups; g += TP_WAVE) {
        const float v = group_l[g];
        if (v != INFINITY && (v > bv || (v == bv && g < bi))) {
          bv = v;
          bi = g;
        }
      }
      wave_arg_best(bv, bi);
      __syncthreads();
      if (lane == 0 && bi != 0x7fffffff) group_l[bi] = INFINITY;
      __syncthreads();
    }
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k) {
      const int e = lane + k * TP_WAVE;
      if (e < experts && group_l[e / per] != INFINITY) ch[k] = -INFINITY;
    }
  }
  float chosen_sum = 0.f;
  for (int it = 0; it < top; ++it) {
    float bv = -INFINITY, bs = 0.f;
    int bi = 0x7fffffff, bk = -1;
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k) {
      const int e = lane + k * TP_WAVE;
      if (e < experts && ch[k] > bv) {   // (ascending e within a lane: the lower index wins a tie)
        bv = ch[k];
        bi = e;
        bk = k;
        bs = sc[k];
      }
    }
    float v = bv;
    int i = bi;
    wave_arg_best(v, i);
    if (i == 0x7fffffff) break;   // fewer allowed experts than `top` (uniform over the wave)
    chosen_sum += __shfl(bs, i % TP_WAVE, TP_WAVE);   // (the winner's lane holds its score; every lane adds alike)
    if (i == bi && bk >= 0) {
      // this lane owns the winner
#pragma unroll
      for (int k = 0; k < ROUTE_PER_LANE; ++k)
        if (k == bk) {
          ch[k] = -INFINITY;
          won[k] = it;
        }
    }
  }
  const float factor = normalize ? scale / (chosen_sum + sum_eps) : scale;
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    if (won[k] >= 0 && live) {
      const int e = lane + k * TP_WAVE;
      const float w = (normalize || scale != 1.0f) ? sc[k] * factor : sc[k];
      dense[(size_t)t * experts + e] = w;
      ids[(size_t)t * top + won[k]] = e;
      weights[(size_t)t * top + won[k]] = w;
    }
  }
}

extern "C" int tp_moe_route(const float* logits, int logit_stride, const float* correction, int experts, int top, int groups,
                            int keep, float* dense, int* ids, float* weights, int n, int score_kind, int group_best,
                            int normalize, float sum_eps, float scale, const float* logit_bias, hipStream_t s) {
  TP_REQUIRE(n >= 0 && experts > 0 && top > 0 && top <= experts && logit_stride >= experts, "moe_route: bad sizes");
  TP_REQUIRE(experts <= TP_WAVE * ROUTE_PER_LANE, "moe_route: %d experts exceed %d", experts, TP_WAVE * ROUTE_PER_LANE);
  TP_REQUIRE(groups <= 1 || (experts % groups == 0 && keep >= 1 && keep <= groups), "moe_route: bad groups");
  TP_REQUIRE((score_kind == 0 || score_kind == 1) && group_best >= 1, "moe_route: bad score kind or group_best");
  if (n == 0) return 0;
  const size_t shmem = sizeof(float) * 4 * (size_t)(experts + (groups > 1 ? groups : 1));
  hipLaunchKernelGGL(moe_route_kernel, dim3((n + 3) / 4), dim3(256), shmem, s, logits, logit_stride, correction, experts, top, groups,
                     keep, dense, ids, weights, n, score_kind, group_best, normalize, sum_eps, scale, logit_bias);
  TP_CHECK_LAUNCH("moe_route");
  return 0;
}

// ---- rows sorted by expert --------------------------------------------------------------------
// For steps of many rows the chosen (token, expert) pairs are brought into the order of the experts, so that
// every expert is one product over its own rows.  ids [n, top] lists each token's experts; pair p = t * top + k.
// moe_plan: counts[e] = pairs of expert e, rank[p] = how many pairs of the same expert come before p (in the order
// of p), so the order inside an expert's rows is the order of the tokens whatever else the batch holds; then
// offsets[e] = pairs of the experts before e.  One block per expert walks all pairs; a one-block kernel adds up.
__global__ __launch_bounds__(256) void moe_rank_kernel(const int* __restrict__ ids, int pairs, int* __restrict__ counts,
                                                       int* __restrict__ rank) {
  __shared__ int wave_total[4];
  const int e = blockIdx.x, lane = threadIdx.x % TP_WAVE, wave = threadIdx.x / TP_WAVE;
  int base = 0;
  for (int p0 = 0; p0 < pairs; p0 += 256) {
    const int p = p0 + threadIdx.x;
    const bool mine = p < pairs && ids[p] == e;
    const unsigned long long mask = __ballot(mine);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    __syncthreads();   // (the totals of the chunk before have been read)
    if (lane == 0) wave_total[wave] = __popcll(mask);
    __syncthreads();
    int prior = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) prior += wave_total[w];
      total += wave_total[w];
    }
    if (mine) rank[p] = base + prior + before;
    base += total;
  }
  if (threadIdx.x == 0) counts[e] = base;
}

__global__ void moe_offsets_kernel(const int* __restrict__ counts, int* __restrict__ offsets, int experts) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int acc = 0;
  for (int e = 0; e < experts; ++e) {
    offsets[e] = acc;
    acc += counts[e];
  }
  offsets[experts] = acc;
}

extern "C" int tp_moe_plan(const int* ids, int n, int top, int experts, int* counts, int* offsets, int* rank, hipStream_t s) {
  TP_REQUIRE(n >= 0 && top > 0 && experts > 0 && (long)n * top < 0x7fffffffL, "moe_plan: bad sizes");
  hipLaunchKernelGGL(moe_rank_kernel, dim3(experts), dim3(256), 0, s, ids, n * top, counts, rank);
  hipLaunchKernelGGL(moe_offsets_kernel, dim3(1), dim3(64), 0, s, counts, offsets, experts);
  TP_CHECK_LAUNCH("moe_plan");
  return 0;
}

// xg[offsets[ids[p]] + rank[p]] = x[p / top] (rows of 4-byte words); row_of[p] remembers the place.
__global__ void moe_gather_kernel(const uint32_t* __restrict__ x, const int* __restrict__ ids, const int* __restrict__ rank,
                                  const int* __restrict__ offsets, uint32_t* __restrict__ xg, int* __restrict__ row_of, int top,
                                  int words) {
  const int p = blockIdx.x;
  const int row = offsets[ids[p]] + rank[p];
  if (threadIdx.x == 0) row_of[p] = row;
  const uint32_t* src = x + (size_t)(p / top) * words;
  uint32_t* dst = xg + (size_t)row * words;
  for (int c = threadIdx.x; c < words; c += blockDim.x) dst[c] = src[c];
}

extern "C" int tp_moe_gather(const void* x, const int* ids, const int* rank, const int* offsets, void* xg, int* row_of, int n, int top,
                             int row_bytes, hipStream_t s) {
  TP_REQUIRE(n >= 0 && top > 0 && row_bytes > 0 && row_bytes % 4 == 0, "moe_gather: rows must be a multiple of four bytes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(moe_gather_kernel, dim3(n * top), dim3(row_bytes / 4 >= 256 ? 256 : 64), 0, s, (const uint32_t*)x, ids, rank, offsets,
                     (uint32_t*)xg, row_of, top, row_bytes / 4);
  TP_CHECK_LAUNCH("moe_gather");
  return 0;
}

// y[t] (+)= sum_k weights[t, k] * yg[row_of[t, k]], k ascending.
__global__ void moe_scatter_kernel(const float* __restrict__ yg, const int* __restrict__ row_of, const float* __restrict__ weights,
                                   float* __restrict__ y, int top, int width, int accumulate) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = accumulate ? y[(size_t)t * width + c] : 0.f;
    for (int k = 0; k < top; ++k) acc = fmaf(weights[(size_t)t * top + k], yg[(size_t)row_of[(size_t)t * top + k] * width + c], acc);
    y[(size_t)t * width + c] = acc;
  }
}

extern "C" int tp_moe_scatter(const float* yg, const int* row_of, const float* weights, float* y, int n, int top, int width,
                              int accumulate, hipStream_t s) {
  TP_REQUIRE(n >= 0 && top > 0 && width > 0, "moe_scatter: bad sizes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(moe_scatter_kernel, dim3(n), dim3(width >= 256 ? 256 : 64), 0, s, yg, row_of, weights, y, top, width, accumulate);
  TP_CHECK_LAUNCH("moe_scatter");
  return 0;
}

// out[e][t][c] = a[t][e * ff + c] * dense[t][e]: the activations of all experts of a few rows, each expert's as rows
// of its own, times the token's weight for the expert (zero where it was not chosen); formed in float32, rounded once.
template <typename T>
__global__ void moe_spread_kernel(const T* __restrict__ a, const float* __restrict__ dense, T* __restrict__ out, int n, int experts,
                                  int ff, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % ff);
  const size_t te = i / ff;
  const int e = (int)(te % experts);
  const size_t t = te / experts;
  from_float(out + ((size_t)e * n + t) * ff + c, to_float(a[i]) * dense[t * experts + e]);
}

extern "C" int tp_moe_spread(const void* a, int dt, const float* dense, void* out, int n, int experts, int ff, hipStream_t s) {
  TP_REQUIRE(n >= 0 && experts > 0 && ff > 0, "moe_spread: bad sizes");
  if (n == 0) return 0;
  const size_t total = (size_t)n * experts * ff;
  const dim3 grid((unsigned)((total + 255) / 256));
  if (dt == TP_F32)
    hipLaunchKernelGGL(moe_spread_kernel<float>, grid, dim3(256), 0, s, (const float*)a, dense, (float*)out, n, experts, ff, total);
  else if (dt == TP_BF16)
    hipLaunchKernelGGL(moe_spread_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)a, dense, (bf16_t*)out, n, experts, ff, total);
  else
    TP_REQUIRE(false, "moe_spread: unknown dtype %d", dt);
  TP_CHECK_LAUNCH("moe_spread");
  return 0;
}

// ---- RMS norm in equal parts of a run of columns ----------------------------------------------
// The `width` columns from col0 on of float32 rows [*, x_stride] are split into `groups` equal consecutive parts;
// each part is divided by its own sqrt(mean(part^2) + eps) and the whole multiplied by w [width].  `rows` (optional)
// picks the input row of each output row; out [n_out, width].  One block per output row, a wave per part in turn.
template <typename TO>
__global__ __launch_bounds__(256) void group_rmsnorm_kernel(const float* __restrict__ x, size_t x_stride, int col0,
                                                            const float* __restrict__ w, const int* __restrict__ rows,
                                                            TO* __restrict__ out, int width, int groups, float eps) {
  const int r = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * x_stride + col0;
  TO* o = out + (size_t)r * width;
  const int wave = threadIdx.x / TP_WAVE, lane = threadIdx.x % TP_WAVE, waves = blockDim.x / TP_WAVE;
  const int per = width / groups;
  for (int g = wave; g < groups; g += waves) {
    const float* p = xr + (size_t)g * per;
    float ss = 0.f;
    for (int i = lane; i < per; i += TP_WAVE) ss = fmaf(p[i], p[i], ss);
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)per + eps);
    for (int i = lane; i < per; i += TP_WAVE) from_float(o + (size_t)g * per + i, p[i] * scale * w[(size_t)g * per + i]);
  }
}

extern "C" int tp_group_rmsnorm(const float* x, size_t x_stride, int col0, const float* w, const int* rows, void* out, int out_dt,
                                int n_out, int width, int groups, float eps, hipStream_t s) {
  TP_REQUIRE(n_out >= 0 && width > 0 && groups > 0 && width % groups == 0 && col0 >= 0 && x_stride >= (size_t)col0 + width,
             "group_rmsnorm: bad sizes");
  if (n_out == 0) return 0;
  const int threads = groups >= 4 ? 256 : (groups * TP_WAVE);
  if (out_dt == TP_F32)
    hipLaunchKernelGGL(group_rmsnorm_kernel<float>, dim3(n_out), dim3(threads), 0, s, x, x_stride, col0, w, rows, (float*)out, width, groups, eps);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(group_rmsnorm_kernel<bf16_t>, dim3(n_out), dim3(threads), 0, s, x, x_stride, col0, w, rows, (bf16_t*)out, width, groups, eps);
  else
    TP_REQUIRE(false, "group_rmsnorm: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("group_rmsnorm");
  return 0;
}

// ---- what sublayers read of normed rows: the rows plus a short convolution of them over time ---
// x float32 [n, width]; w [subs, taps, width] (tap-major; the last tap is the current token's).  For sublayer s:
// out_s[t, c] = x[t, c] + sum_k w[s, k, c] * x[t - (taps - 1 - k), c], the rows before a run's first token coming from
// the request's state row (from element state_off on: [taps - 1, width], oldest first; zeros for a fresh request).
// The sublayers read the same rows, so one state serves them all; a second kernel leaves the run's last rows there.
template <typename TO>
__global__ void residual_conv_kernel(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ state,
                                     size_t state_stride, size_t state_off, const int* __restrict__ cu_seqlens,
                                     const int* __restrict__ token_req, const int* __restrict__ state_slots, TO* __restrict__ out,
                                     size_t out_stride_sub, int width, int taps, int subs, int channel_blocks) {
  const int t = blockIdx.x / channel_blocks;
  const int c = (blockIdx.x % channel_blocks) * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int r = token_req[t];
  const int start = cu_seqlens[r];
  const int i = t - start;
  const float* st = state + (size_t)state_slots[r] * state_stride + state_off;
  const float cur = x[(size_t)t * width + c];
  for (int sub = 0; sub < subs; ++sub) {
    float acc = 0.f;
    for (int k = 0; k < taps; ++k) {
      const int src = i - (taps - 1 - k);
      const float v = src >= 0 ? x[(size_t)(start + src) * width + c] : st[(size_t)(taps - 1 + src) * width + c];
      acc = fmaf(w[((size_t)sub * taps + k) * width + c], v, acc);
    }
    from_float(out + (size_t)sub * out_stride_sub + (size_t)t * width + c, cur + acc);
  }
}

// the same, four neighbouring channels a thread (width a multiple of four, at most four sublayers): 16-byte loads of
// the rows and the weights; the request's carried rows are read element by element (their place in the state row
// need not be aligned).  Every channel's sum is formed in the order of the kernel above: the same bits.
#define RCONV_MAX_SUBS 4
template <typename TO>
__global__ void residual_conv4_kernel(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ state,
                                      size_t state_stride, size_t state_off, const int* __restrict__ cu_seqlens,
                                      const int* __restrict__ token_req, const int* __restrict__ state_slots, TO* __restrict__ out,
                                      size_t out_stride_sub, int width, int taps, int subs, int channel_blocks) {
  const int t = blockIdx.x / channel_blocks;
  const int c = ((blockIdx.x % channel_blocks) * blockDim.x + threadIdx.x) * 4;
  if (c >= width) return;
  const int r = token_req[t];
  const int start = cu_seqlens[r];
  const int i = t - start;
  const float* st = state + (size_t)state_slots[r] * state_stride + state_off;
  const float4 cur = *(const float4*)(x + (size_t)t * width + c);
  float4 acc[RCONV_MAX_SUBS];
#pragma unroll
  for (int sub = 0; sub < RCONV_MAX_SUBS; ++sub) acc[sub] = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < taps; ++k) {
    const int src = i - (taps - 1 - k);
    float4 v;
    if (src >= 0) {
      v = *(const float4*)(x + (size_t)(start + src) * width + c);
    } else {
      const float* p = st + (size_t)(taps - 1 + src) * width + c;
      v = make_float4(p[0], p[1], p[2], p[3]);
    }
#pragma unroll
    for (int sub = 0; sub < RCONV_MAX_SUBS; ++sub)
      if (sub < subs) {
        const float4 wv = *(const float4*)(w + ((size_t)sub * taps + k) * width + c);
        acc[sub].x = fmaf(wv.x, v.x, acc[sub].x);
        acc[sub].y = fmaf(wv.y, v.y, acc[sub].y);
        acc[sub].z = fmaf(wv.z, v.z, acc[sub].z);
        acc[sub].w = fmaf(wv.w, v.w, acc[sub].w);
      }
  }
#pragma unroll
  for (int sub = 0; sub < RCONV_MAX_SUBS; ++sub)
    if (sub < subs)
      from_float4(out + (size_t)sub * out_stride_sub + (size_t)t * width + c, cur.x + acc[sub].x, cur.y + acc[sub].y,
                  cur.z + acc[sub].z, cur.w + acc[sub].w);
}

__global__ void residual_conv_state_kernel(const float* __restrict__ x, float* __restrict__ state, size_t state_stride,
                                           size_t state_off, const int* __restrict__ cu_seqlens,
                                           const int* __restrict__ state_slots, int width, int taps) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int start = cu_seqlens[r], len = cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  float* st = state + (size_t)state_slots[r] * state_stride + state_off;
  // in place, ascending: entry j takes entry j + len of the old state or a row of the run; entries below j are never read again
  for (int j = 0; j < taps - 1; ++j) {
    const int src = len - (taps - 1) + j;
    st[(size_t)j * width + c] = src >= 0 ? x[(size_t)(start + src) * width + c] : st[(size_t)(j + len) * width + c];
  }
}

extern "C" int tp_residual_conv(const float* x, const float* w, float* state, size_t state_stride, size_t state_off,
                                const int* cu_seqlens, const int* token_req, const int* state_slots, void* out, int out_dt, int n,
                                int n_req, int width, int taps, int subs, hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_req >= 0 && width > 0 && taps >= 1 && subs >= 1, "residual_conv: bad sizes");
  TP_REQUIRE(state_stride >= state_off + (size_t)(taps - 1) * width, "residual_conv: state rows too short");
  if (n == 0) return 0;
  const int threads = width >= 256 ? 256 : 64;
  const int cb = (width + threads - 1) / threads;
  TP_REQUIRE(cb <= 65535 && (long)n * cb < 0x7fffffffL, "residual_conv: too many channels or tokens");
  const size_t sub_stride = (size_t)n * width;
  TP_REQUIRE(out_dt == TP_F32 || out_dt == TP_BF16, "residual_conv: unknown dtype %d", out_dt);
  if (width % 4 == 0 && subs <= RCONV_MAX_SUBS && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15) == 0) {
    const int quads = width / 4;
    const int qthreads = quads >= 256 ? 256 : 64;
    const int qb = (quads + qthreads - 1) / qthreads;
    if (out_dt == TP_F32)
      hipLaunchKernelGGL(residual_conv4_kernel<float>, dim3((unsigned)((long)n * qb)), dim3(qthreads), 0, s, x, w, state, state_stride,
                         state_off, cu_seqlens, token_req, state_slots, (float*)out, sub_stride, width, taps, subs, qb);
    else
      hipLaunchKernelGGL(residual_conv4_kernel<bf16_t>, dim3((unsigned)((long)n * qb)), dim3(qthreads), 0, s, x, w, state, state_stride,
                         state_off, cu_seqlens, token_req, state_slots, (bf16_t*)out, sub_stride, width, taps, subs, qb);
  } else if (out_dt == TP_F32)
    hipLaunchKernelGGL(residual_conv_kernel<float>, dim3((unsigned)((long)n * cb)), dim3(threads), 0, s, x, w, state, state_stride,
                       state_off, cu_seqlens, token_req, state_slots, (float*)out, sub_stride, width, taps, subs, cb);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(residual_conv_kernel<bf16_t>, dim3((unsigned)((long)n * cb)), dim3(threads), 0, s, x, w, state, state_stride,
                       state_off, cu_seqlens, token_req, state_slots, (bf16_t*)out, sub_stride, width, taps, subs, cb);
  else
    TP_REQUIRE(false, "residual_conv: unknown dtype %d", out_dt);
  if (taps > 1 && n_req > 0)
    hipLaunchKernelGGL(residual_conv_state_kernel, dim3(n_req, cb), dim3(threads), 0, s, x, state, state_stride, state_off, cu_seqlens,
                       state_slots, width, taps);
  TP_CHECK_LAUNCH("residual_conv");
  return 0;
}

// ---- one row of a table added to every row of the stream --------------------------------------
__global__ void add_row_kernel(float* __restrict__ h, const float* __restrict__ row, size_t total, int width) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) h[i] += row[i % width];
}

extern "C" int tp_add_row(float* h, const float* row, int n, int width, hipStream_t s) {
  TP_REQUIRE(n >= 0 && width > 0, "add_row: bad sizes");
  if (n == 0) return 0;
  const size_t total = (size_t)n * width;
  TP_REQUIRE((total + 255) / 256 < 0x7fffffffUL, "add_row: too many elements");
  hipLaunchKernelGGL(add_row_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, h, row, total, width);
  TP_CHECK_LAUNCH("add_row");
  return 0;
}

// ---- rows of q | k | v for an attention whose keys and values are expanded from a latent --------
// Per token: q [heads, key] comes from the projection's rows as it stands (key = rot + dim elements a head, the
// rotated ones first); head h's key is the ONE shared rotated part (rot elements of the projection's rows, not yet
// rotated) followed by its own dim unrotated elements of the expansion `up` ([heads * dim | heads * vdim] a row);
// its value the head's vdim elements of `up`.  out [n, 2 * heads * key + heads * vdim] float32, the layout the
// rotation-and-store kernel takes.
__global__ void latent_rows_kernel(const float* __restrict__ proj, size_t proj_stride, int q_col0, int rot_col0,
                                   const float* __restrict__ up, size_t up_stride, float* __restrict__ out, int heads, int dim,
                                   int rot, int vdim) {
  const int t = blockIdx.x;
  const int key = rot + dim, qk = heads * key, width = 2 * qk + heads * vdim;
  const float* pr = proj + (size_t)t * proj_stride;
  const float* ur = up + (size_t)t * up_stride;
  float* o = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v;
    if (i < qk) {
      v = pr[q_col0 + i];
    } else if (i < 2 * qk) {
      const int h = (i - qk) / key, d = (i - qk) % key;
      v = d < rot ? pr[rot_col0 + d] : ur[h * dim + d - rot];
    } else {
      v = ur[heads * dim + i - 2 * qk];
    }
    o[i] = v;
  }
}

extern "C" int tp_latent_rows(const float* proj, size_t proj_stride, int q_col0, int rot_col0, const float* up, size_t up_stride,
                              float* out, int n, int heads, int dim, int rot, int vdim, hipStream_t s) {
  TP_REQUIRE(n >= 0 && heads > 0 && dim > 0 && rot >= 0 && vdim > 0 && q_col0 >= 0 && rot_col0 >= 0, "latent_rows: bad sizes");
  TP_REQUIRE(proj_stride >= (size_t)q_col0 + (size_t)heads * (rot + dim) && proj_stride >= (size_t)rot_col0 + rot &&
                 up_stride >= (size_t)heads * (dim + vdim), "latent_rows: rows too short");
  if (n == 0) return 0;
  hipLaunchKernelGGL(latent_rows_kernel, dim3(n), dim3(256), 0, s, proj, proj_stride, q_col0, rot_col0, up, up_stride, out, heads, dim,
                     rot, vdim);
  TP_CHECK_LAUNCH("latent_rows");
  return 0;
}

// ---- norm per head on projected rows, in place --------------------------------------------------
// rows float32 [n, stride]: the `heads` heads of `dim` columns from col0 on become x / sqrt(mean(x^2) + eps) * w[d]
// (one weight [dim] for all of them).  Queries and keys of an attention are two calls' worth of columns, so the entry
// point takes two runs of heads, each with its weight.  One wave per (token, head).
__global__ __launch_bounds__(256) void head_rmsnorm_kernel(float* __restrict__ rows, size_t stride, int col_a, int heads_a,
                                                           const float* __restrict__ w_a, int col_b, int heads_b,
                                                           const float* __restrict__ w_b, int dim, float eps, long pairs) {
  const long p = (long)blockIdx.x * 4 + threadIdx.x / TP_WAVE;
  const int lane = threadIdx.x % TP_WAVE;
  if (p >= pairs) return;
  const int per = heads_a + heads_b;
  const long t = p / per;
  const int hh = (int)(p % per);
  float* x = rows + (size_t)t * stride + (hh < heads_a ? col_a + (size_t)hh * dim : col_b + (size_t)(hh - heads_a) * dim);
  const float* w = hh < heads_a ? w_a : w_b;
  float ss = 0.f;
  for (int d = lane; d < dim; d += TP_WAVE) ss = fmaf(x[d], x[d], ss);
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)dim + eps);
  for (int d = lane; d < dim; d += TP_WAVE) x[d] = x[d] * rstd * w[d];
}

extern "C" int tp_head_rmsnorm(float* rows, size_t stride, int col_a, int heads_a, const float* w_a, int col_b, int heads_b,
                               const float* w_b, int dim, float eps, int n, hipStream_t s) {
  TP_REQUIRE(n >= 0 && dim > 0 && heads_a >= 0 && heads_b >= 0 && col_a >= 0 && col_b >= 0, "head_rmsnorm: bad sizes");
  TP_REQUIRE((size_t)col_a + (size_t)heads_a * dim <= stride && (size_t)col_b + (size_t)heads_b * dim <= stride, "head_rmsnorm: rows too short");
  TP_REQUIRE((heads_a == 0 || w_a) && (heads_b == 0 || w_b), "head_rmsnorm: a run of heads needs its weight");
  const long pairs = (long)n * (heads_a + heads_b);
  if (pairs == 0) return 0;
  TP_REQUIRE((pairs + 3) / 4 < 0x7fffffffL, "head_rmsnorm: too many rows");
  hipLaunchKernelGGL(head_rmsnorm_kernel, dim3((unsigned)((pairs + 3) / 4)), dim3(256), 0, s, rows, stride, col_a, heads_a, w_a, col_b,
                     heads_b, w_b, dim, eps, pairs);
  TP_CHECK_LAUNCH("head_rmsnorm");
  return 0;
}

// ---- one vector a token into the cache, as key and as value ------------------------------------------
// c [n, dim] goes to cache place slots[t] of keys [page, 1, page_size, dim] and of transposed values
// [page, 1, dim, page_size]: an attention whose keys are its values reads both with the ordinary kernels.
template <typename T>
__global__ void vector_store_kernel(const T* __restrict__ c, const int* __restrict__ slots, T* __restrict__ k_cache,
                                    T* __restrict__ v_cache, size_t total, int dim, int page_size) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / dim;
  const int d = (int)(i % dim);
  const int slot = slots[t];
  const size_t page = slot / page_size;
  const int off = slot % page_size;
  const T v = c[i];
  k_cache[(page * page_size + off) * dim + d] = v;
  v_cache[(page * dim + d) * page_size + off] = v;
}

extern "C" int tp_vector_store(const void* c, int dt, const int* slots, void* k_cache, void* v_cache, int n, int dim, int page_size,
                               hipStream_t s) {
  TP_REQUIRE(n >= 0 && dim > 0 && page_size > 0, "vector_store: bad sizes");
  const size_t total = (size_t)n * dim;
  if (total == 0) return 0;
  const dim3 grid((unsigned)((total + 255) / 256));
  if (dt == TP_F32)
    hipLaunchKernelGGL(vector_store_kernel<float>, grid, dim3(256), 0, s, (const float*)c, slots, (float*)k_cache, (float*)v_cache, total, dim, page_size);
  else if (dt == TP_BF16)
    hipLaunchKernelGGL(vector_store_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)c, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, total, dim, page_size);
  else
    TP_REQUIRE(false, "vector_store: unknown dtype %d", dt);
  TP_CHECK_LAUNCH("vector_store");
  return 0;
}
