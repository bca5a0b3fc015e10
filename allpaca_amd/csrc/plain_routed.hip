// Plain kernels of a feed-forward of routed experts: the choice of experts from router logits, the chosen experts'
// gated units, and the weighted sum of their outputs.  All arithmetic in 32-bit float, one fma chain per output, so a
// row's result does not depend on the batch; any element type for rows and matrices.
//
//   z [T][N] router logits over N = experts with matrices + identity experts (the last ones)
//   s = softmax(z), or s = sigmoid(z) each for itself (`score` 1);  chosen: the K largest of s + correction (the
//   lower index wins a tie);  weights: s of the chosen
//   y[t] = sum_k w[t][k] * (expert e = ids[t][k] has matrices ? Wd_e (a(Wg_e h, Wu_e h)) : h)
//   a(g, u) = silu(g) * u  (`act` 0), or with g' = min(g, limit), u' = clamp(u, -limit, limit):
//   g' * sigmoid(alpha g') * (u' + 1)  (`act` 1)
// With `in_weights` the weight multiplies the expert's input instead of its output: y[t] = sum_k expert(w[t][k] h[t]),
// formed as a(w g, w u) from the same sums g = Wg h, u = Wu h (the products are linear in h).
#include "common.h"
#include <math.h>

namespace {

constexpr int MAX_PER_LANE_R = 16;   // up to 1,024 router outputs
constexpr int MAX_TOP = 32;

__global__ __launch_bounds__(64) void route_topk_kernel(const float* __restrict__ z, int ldz,
                                                        const float* __restrict__ correction, int N, int K,
                                                        int renormalize, int score, int* __restrict__ ids,
                                                        float* __restrict__ weights) {
  const int t = blockIdx.x, lane = threadIdx.x;
  float s[MAX_PER_LANE_R], c[MAX_PER_LANE_R];
  float mx = -INFINITY;
#pragma unroll
  for (int e = 0; e < MAX_PER_LANE_R; ++e) {
    const int i = lane + e * WAVE;
    s[e] = i < N ? z[(size_t)t * ldz + i] : -INFINITY;
    mx = fmaxf(mx, s[e]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < MAX_PER_LANE_R; ++e) {
    const int i = lane + e * WAVE;
    if (score == 1) s[e] = i < N ? 1.0f / (1.0f + expf(-s[e])) : 0.f;
    else s[e] = i < N ? expf(s[e] - mx) : 0.f;
    sum += s[e];
  }
  sum = score == 1 ? 1.f : wave_sum(sum);
#pragma unroll
  for (int e = 0; e < MAX_PER_LANE_R; ++e) {
    const int i = lane + e * WAVE;
    s[e] = s[e] / sum;
    c[e] = i < N ? s[e] + (correction ? correction[i] : 0.f) : -INFINITY;
  }
  float total = 0.f;
  float mine = 0.f;      // lane k keeps the k-th weight
  int mine_id = 0;
  for (int k = 0; k < K; ++k) {
    float best = -INFINITY;
    int best_i = 0x7fffffff;
#pragma unroll
    for (int e = 0; e < MAX_PER_LANE_R; ++e) {
      const int i = lane + e * WAVE;
      if (c[e] > best) { best = c[e]; best_i = i; }      // a lane's own candidates come in rising order of index
    }
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, WAVE);
      const int oi = __shfl_xor(best_i, o, WAVE);
      if (ob > best || (ob == best && oi < best_i)) { best = ob; best_i = oi; }
    }
    float w = 0.f;
#pragma unroll
    for (int e = 0; e < MAX_PER_LANE_R; ++e) {
      const int i = lane + e * WAVE;
      if (i == best_i) { w = s[e]; c[e] = -INFINITY; }
    }
    w = wave_sum(w);                                       // one lane holds it, the others 0
    total += w;
    if (lane == k) { mine = w; mine_id = best_i; }
  }
  if (lane < K) {
    ids[(size_t)t * K + lane] = mine_id;
    weights[(size_t)t * K + lane] = renormalize ? mine / total : mine;
  }
}

// act[t * K + k][f] = silu(Wg_e[f] . h[t]) * (Wu_e[f] . h[t]) for e = ids[t][k] with matrices;
// w_gate_up [E][2F][D] (an expert's gate rows, then its up rows).
__global__ __launch_bounds__(256) void routed_glu_kernel(const void* __restrict__ h, int h_dtype, int ldh,
                                                         const void* __restrict__ w_gate_up, int w_dtype, int E, int F,
                                                         int D, const int* __restrict__ ids, int K,
                                                         void* __restrict__ act, int act_dtype, int kind, float alpha,
                                                         float limit, const float* __restrict__ in_weights) {
  extern __shared__ float hs[];
  const int pair = blockIdx.x, t = pair / K;
  const int e = ids[pair];
  if (e >= E) return;                  // an identity expert
  for (int i = threadIdx.x; i < D; i += 256) hs[i] = load_f(h, h_dtype, (size_t)t * ldh + i);
  __syncthreads();
  const int f = blockIdx.y * 256 + threadIdx.x;
  if (f >= F) return;
  const size_t gate_row = ((size_t)e * 2 * F + f) * D, up_row = gate_row + (size_t)F * D;
  float g = 0.f, u = 0.f;
  for (int i = 0; i < D; ++i) {
    g = fmaf(hs[i], load_f(w_gate_up, w_dtype, gate_row + i), g);
    u = fmaf(hs[i], load_f(w_gate_up, w_dtype, up_row + i), u);
  }
  if (in_weights) { g *= in_weights[pair]; u *= in_weights[pair]; }
  float a;
  if (kind == 1) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    a = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
  } else {
    a = (g / (1.0f + expf(-g))) * u;
  }
  store_f(act, act_dtype, (size_t)pair * F + f, a);
}

// y[t][d] = sum_k w[t][k] * (e has matrices ? Wd_e[d] . act[t * K + k] : h[t][d]), k in order; w_down [E][D][F]
__global__ __launch_bounds__(256) void routed_down_kernel(const void* __restrict__ act, int act_dtype,
                                                          const void* __restrict__ w_down, int w_dtype, int E, int F,
                                                          int D, const int* __restrict__ ids,
                                                          const float* __restrict__ weights, int K,
                                                          const void* __restrict__ h, int h_dtype, int ldh,
                                                          float* __restrict__ y, int ldy, int in_lds, int in_weights) {
  extern __shared__ float as[];        // [K][F], if the row's activations fit (else they are read where they lie)
  const int t = blockIdx.x;
  if (in_lds) {
    for (int i = threadIdx.x; i < K * F; i += 256) {
      const int k = i / F;
      as[i] = ids[(size_t)t * K + k] < E ? load_f(act, act_dtype, (size_t)t * K * F + i) : 0.f;
    }
    __syncthreads();
  }
  const int d = blockIdx.y * 256 + threadIdx.x;
  if (d >= D) return;
  float total = 0.f;
  for (int k = 0; k < K; ++k) {
    const int e = ids[(size_t)t * K + k];
    float v;
    if (e < E) {
      const size_t row = ((size_t)e * D + d) * F;
      v = 0.f;
      if (in_lds) {
        for (int f = 0; f < F; ++f) v = fmaf(as[k * F + f], load_f(w_down, w_dtype, row + f), v);
      } else {
        const size_t a0 = ((size_t)t * K + k) * F;
        for (int f = 0; f < F; ++f) v = fmaf(load_f(act, act_dtype, a0 + f), load_f(w_down, w_dtype, row + f), v);
      }
    } else {
      v = load_f(h, h_dtype, (size_t)t * ldh + d);
    }
    // (with the weights on the inputs an expert's output is added as it is; an identity returns its weighted input)
    total = (in_weights && e < E) ? total + v : fmaf(weights[(size_t)t * K + k], v, total);
  }
  y[(size_t)t * ldy + d] = total;
}

}  // namespace

APC_EXPORT int apc_route_topk(const float* z, int ldz, const float* correction, int n_rows, int N, int K,
                              int renormalize, int score, int* ids, float* weights, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (N <= 0 || K <= 0 || K > N || ldz < N || !ids || !weights || score < 0 || score > 1) return APC_ERR_BAD_ARG;
  if (N > MAX_PER_LANE_R * WAVE || K > MAX_TOP) return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(route_topk_kernel, dim3(n_rows), dim3(64), 0, stream, z, ldz, correction, N, K, renormalize, score,
                     ids, weights);
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_routed_glu(const void* h, int h_dtype, int ldh, const void* w_gate_up, int w_dtype, int E, int F,
                              int D, const int* ids, int K, void* act, int act_dtype, int n_rows, int kind, float alpha,
                              float limit, const float* in_weights, hipStream_t stream) {
  if (n_rows <= 0 || E <= 0) return 0;
  if (F <= 0 || D <= 0 || K <= 0 || ldh < D || kind < 0 || kind > 1) return APC_ERR_BAD_ARG;
  if ((size_t)D * sizeof(float) > 64 * 1024 || (long)n_rows * K > 0x7fffffffL || ceil_div(F, 256) > 65535)
    return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(routed_glu_kernel, dim3(n_rows * K, ceil_div(F, 256)), dim3(256), (size_t)D * sizeof(float),
                     stream, h, h_dtype, ldh, w_gate_up, w_dtype, E, F, D, ids, K, act, act_dtype, kind, alpha, limit,
                     in_weights);
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_routed_down(const void* act, int act_dtype, const void* w_down, int w_dtype, int E, int F, int D,
                               const int* ids, const float* weights, int K, const void* h, int h_dtype, int ldh,
                               float* y, int ldy, int n_rows, int in_weights, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (E < 0 || F <= 0 || D <= 0 || K <= 0 || ldh < D || ldy < D) return APC_ERR_BAD_ARG;
  if (ceil_div(D, 256) > 65535) return APC_ERR_UNSUPPORTED;
  const size_t lds = (size_t)K * F * sizeof(float);
  const int in_lds = lds <= 48 * 1024 ? 1 : 0;       // (the same sums in the same order either way)
  hipLaunchKernelGGL(routed_down_kernel, dim3(n_rows, ceil_div(D, 256)), dim3(256), in_lds ? lds : 0, stream, act,
                     act_dtype, w_down, w_dtype, E, F, D, ids, weights, K, h, h_dtype, ldh, y, ldy, in_lds, in_weights);
  APC_LAUNCH_CHECK();
  return 0;
}
