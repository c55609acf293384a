// Mixture of experts: the router's choice and the experts' activation.
//
// Router: scores = softmax of the router's 32-bit logits over all experts; the experts form `n_groups`
// equal groups of neighbours, a group's score is its best expert's, only experts of the `keep` best
// groups can be chosen; the `top` best of those are chosen (ties go to the lower index) and weighted
// by their scores over the sum of the chosen scores (+ 1e-20).  One wave per token.
//
// Expert: g = min(gate, limit), u = clamp(up, -limit, limit), y = g sigmoid(1.702 g) (u + 1).
// `moe_act_kernel` applies it to the gate|up sums of every expert and multiplies by the token's
// weight for that expert (0 where it was not chosen), so that one product with the experts' down
// matrices side by side gives the weighted sum of the chosen experts' outputs.
// `moe_sparse_*`: for steps of few tokens, only the chosen experts' matrices are read: a wave per
// output row of a (token, choice) pair.
#include "common.h"

#define MF_MOE_MAX_EXPERTS 1024

// index of the largest value among a wave's candidates; ties go to the lower index
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, MF_WAVE);
    const int oi = __shfl_xor(idx, o, MF_WAVE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
}

__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, float* __restrict__ dense,
                                                       int* __restrict__ chosen, float* __restrict__ weights, int E,
                                                       int n_groups, int keep, int top) {
  __shared__ float s[MF_MOE_MAX_EXPERTS], ms[MF_MOE_MAX_EXPERTS], gs[MF_MOE_MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* z = logits + (size_t)t * E;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) { const float x = expf(z[e] - mx); s[e] = x; sum += x; }
  sum = wave_sum(sum);
  __syncthreads();
  for (int e = lane; e < E; e += 64) { s[e] = s[e] / sum; dense[(size_t)t * E + e] = 0.f; }
  __syncthreads();
  const int per = E / n_groups;
  for (int g = lane; g < n_groups; g += 64) {
    float b = -1.f;
    for (int i = 0; i < per; ++i) b = fmaxf(b, s[g * per + i]);
    gs[g] = b;
  }
  for (int e = lane; e < E; e += 64) ms[e] = -1.f;
  __syncthreads();
  for (int k = 0; k < keep; ++k) {
    float b = -2.f;
    int bi = 0x7fffffff;
    for (int g = lane; g < n_groups; g += 64)
      if (gs[g] > b) { b = gs[g]; bi = g; }
    wave_argmax(b, bi);
    __syncthreads();
    if (lane == 0) gs[bi] = -3.f;
    for (int i = lane; i < per; i += 64) ms[bi * per + i] = s[bi * per + i];
    __syncthreads();
  }
  float wsum = 0.f;
  int mine = -1;          // lane k keeps the k-th choice (top <= 64)
  for (int k = 0; k < top; ++k) {
    float b = -2.f;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (ms[e] > b) { b = ms[e]; bi = e; }
    wave_argmax(b, bi);
    __syncthreads();
    if (lane == 0) ms[bi] = -3.f;
    if (lane == k) mine = bi;
    wsum += s[bi];
    __syncthreads();
  }
  if (lane < top) {
    const float wgt = s[mine] / (wsum + 1e-20f);
    dense[(size_t)t * E + mine] = wgt;
    chosen[(size_t)t * top + lane] = mine;
    weights[(size_t)t * top + lane] = wgt;
  }
}

__device__ __forceinline__ float expert_act(float g, float u, float limit) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * (1.0f / (1.0f + expf(-1.702f * g))) * (u + 1.0f);
}

// gu [tokens][E][2 F] (an expert's gate sums, then its up sums); dense [tokens][E]; y [tokens][E F]
template <typename OT>
__global__ __launch_bounds__(256) void moe_act_kernel(const float* __restrict__ gu, const float* __restrict__ dense,
                                                      OT* __restrict__ y, int E, int F, float limit) {
  const int t = blockIdx.x;
  const float* row = gu + (size_t)t * E * 2 * F;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < E * F; i += gridDim.y * 256) {
    const int e = i / F, f = i % F;
    const float wgt = dense[(size_t)t * E + e];
    float v = 0.f;
    if (wgt != 0.f) v = wgt * expert_act(row[(size_t)e * 2 * F + f], row[(size_t)e * 2 * F + F + f], limit);
    y[(size_t)t * E * F + i] = from_f32<OT>(v);
  }
}

// ------------------------------------------------------------------ few tokens: the chosen experts only
// gate_up [E][2 F][K], x [tokens][K] -> y [tokens][top][F] (activation applied, not weighted).
// A wave per (token, choice, f): both rows of the pair, lanes over K.
template <typename WT>
__global__ __launch_bounds__(256) void moe_sparse_up_kernel(const WT* __restrict__ x, const WT* __restrict__ gate_up,
                                                            const int* __restrict__ chosen, WT* __restrict__ y,
                                                            int top, int F, int K, float limit) {
  const int t = blockIdx.x, k = blockIdx.y;
  const int f = blockIdx.z * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (f >= F) return;
  const int e = chosen[(size_t)t * top + k];
  const WT* wg = gate_up + ((size_t)e * 2 * F + f) * K;
  const WT* wu = wg + (size_t)F * K;
  const WT* xr = x + (size_t)t * K;
  float g = 0.f, u = 0.f;
  for (int i = lane; i < K; i += 64) {
    const float xv = to_f32(xr[i]);
    g = fmaf(to_f32(wg[i]), xv, g);
    u = fmaf(to_f32(wu[i]), xv, u);
  }
  g = wave_sum(g);
  u = wave_sum(u);
  if (lane == 0) y[((size_t)t * top + k) * F + f] = from_f32<WT>(expert_act(g, u, limit));
}

// down [N][E F] (the experts' down matrices side by side), y [tokens][top][F]:
// out[t][n] += sum_k w[t][k] dot(down[n][e_k F .. e_k F + F), y[t][k]), choices added in their order.
template <typename WT>
__global__ __launch_bounds__(256) void moe_sparse_down_kernel(const WT* __restrict__ y, const WT* __restrict__ down,
                                                              const int* __restrict__ chosen,
                                                              const float* __restrict__ weights, float* __restrict__ out,
                                                              int top, int E, int F, int N) {
  const int t = blockIdx.x;
  const int n = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N) return;
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    const int e = chosen[(size_t)t * top + k];
    const WT* wr = down + (size_t)n * E * F + (size_t)e * F;
    const WT* yr = y + ((size_t)t * top + k) * F;
    float a = 0.f;
    for (int i = lane; i < F; i += 64) a = fmaf(to_f32(wr[i]), to_f32(yr[i]), a);
    total = fmaf(weights[(size_t)t * top + k], wave_sum(a), total);
  }
  if (lane == 0) out[(size_t)t * N + n] += total;
}

// ------------------------------------------------------------------ entry points
MF_API int mf_moe_route(const float* logits, float* dense, int* chosen, float* weights, int n_tok, int E, int n_groups,
                        int keep, int top, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (E <= 0 || E > MF_MOE_MAX_EXPERTS || n_groups <= 0 || E % n_groups || keep <= 0 || keep > n_groups || top <= 0 ||
      top > 64 || top > keep * (E / n_groups))
    return (int)hipErrorInvalidValue;
  moe_route_kernel<<<n_tok, 64, 0, stream>>>(logits, dense, chosen, weights, E, n_groups, keep, top);
  return mf_launch_status();
}

MF_API int mf_moe_act(const float* gu, const float* dense, void* y, int y_is_bf16, int n_tok, int E, int F, float limit,
                      hipStream_t stream) {
  if (n_tok <= 0 || E <= 0 || F <= 0) return 0;
  int by = (E * F + 255) / 256;
  if (by > 64) by = 64;
  dim3 grid(n_tok, by);
  if (y_is_bf16)
    moe_act_kernel<bf16><<<grid, 256, 0, stream>>>(gu, dense, (bf16*)y, E, F, limit);
  else
    moe_act_kernel<float><<<grid, 256, 0, stream>>>(gu, dense, (float*)y, E, F, limit);
  return mf_launch_status();
}

MF_API int mf_moe_sparse(const void* x, const void* gate_up, const void* down, const int* chosen, const float* weights,
                         void* y, float* out, int is_bf16, int n_tok, int top, int E, int F, int K, int N, float limit,
                         hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (top <= 0 || E <= 0 || F <= 0 || K <= 0 || N <= 0) return (int)hipErrorInvalidValue;
  dim3 g1(n_tok, top, (F + 3) / 4), g2(n_tok, (N + 3) / 4);
  if (is_bf16) {
    moe_sparse_up_kernel<bf16><<<g1, 256, 0, stream>>>((const bf16*)x, (const bf16*)gate_up, chosen, (bf16*)y, top, F, K, limit);
    int rc = mf_launch_status();
    if (rc) return rc;
    moe_sparse_down_kernel<bf16><<<g2, 256, 0, stream>>>((const bf16*)y, (const bf16*)down, chosen, weights, out, top, E, F, N);
  } else {
    moe_sparse_up_kernel<float><<<g1, 256, 0, stream>>>((const float*)x, (const float*)gate_up, chosen, (float*)y, top, F, K, limit);
    int rc = mf_launch_status();
    if (rc) return rc;
    moe_sparse_down_kernel<float><<<g2, 256, 0, stream>>>((const float*)y, (const float*)down, chosen, weights, out, top, E, F, N);
  }
  return mf_launch_status();
}
