// Plain kernels of a selective state-space mixer and of small row-wise steps: a short causal convolution per channel
// with a bias and an activation behind it, the selective scan with its state per request, an activation over rows,
// a bias added to rows.  One obvious loop nest each, all arithmetic in 32-bit float with an order of additions that
// the row's own place fixes (never the batch), any element type in and out.
#include "common.h"
#include <math.h>

namespace {

constexpr int SCAN_MAX_TAPS = 8;
constexpr int SCAN_MAX_PER_LANE = 4;     // states a lane keeps: up to 256 states a channel

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// Activations by code: 0 none, 1 silu, 2 relu squared, 3 gelu (tanh form).
__device__ __forceinline__ float activate(float z, int kind) {
  if (kind == 1) return silu_f(z);
  if (kind == 2) { const float r = fmaxf(z, 0.f); return r * r; }
  if (kind == 3) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z;
}

// ---------------------------------------------------------------------------
// Short causal convolution over time on every channel, the bias behind it, then an activation:
//   y[t][c] = act(sum_j w[c][j] * u[t - (n-1) + j][c] + b[c]),  u = x[:, c] of the rows of the same segment
// u of the n-1 positions ahead of a segment's first row comes from state[slot][n-1][C] (zero for a new request).
// The state is moved on by `conv_state_kernel` of the attention's convolution afterwards (it keeps inputs, too).
// ---------------------------------------------------------------------------
__global__ void conv_channels_kernel(const void* __restrict__ x, int x_dtype, int ldx, int C,
                                     const float* __restrict__ w, const float* __restrict__ bias, int taps,
                                     const float* __restrict__ state, const int* __restrict__ row_seg,
                                     const int* __restrict__ seg_row0, const int* __restrict__ slots, int act,
                                     void* __restrict__ out, int out_dtype, int ldo) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int seg = row_seg[r];
  const int i_in_seg = r - seg_row0[seg];
  const float* st = taps > 1 ? state + (size_t)slots[seg] * (taps - 1) * C : nullptr;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {              // oldest first
    const int back = taps - 1 - j;
    const float u = back <= i_in_seg ? load_f(x, x_dtype, (size_t)(r - back) * ldx + c)
                                     : st[(size_t)(taps - 1 - (back - i_in_seg)) * C + c];
    acc = fmaf(w[(size_t)c * taps + j], u, acc);
  }
  if (bias) acc += bias[c];
  store_f(out, out_dtype, (size_t)r * ldo + c, activate(acc, act));
}

// The same for bfloat16 rows, 8 consecutive channels a thread on 16-byte accesses (C, the row strides and the addresses
// multiples of 8 elements), ROWS consecutive rows a block: a thread keeps its channels' taps in registers for all of
// them, and a row that follows its predecessor in the same segment takes over that row's inputs and loads one more.
// The same sums in the same order as the kernel above.
template <int TAPS, int ROWS>
__global__ __launch_bounds__(256) void conv_channels_bf16x8_kernel(
    const bf16_t* __restrict__ x, int ldx, int n_rows, int C, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ state, const int* __restrict__ row_seg,
    const int* __restrict__ seg_row0, const int* __restrict__ slots, int act, bf16_t* __restrict__ out, int ldo) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= C) return;
  float wt[8][TAPS], b[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wt[e][j] = w[(size_t)(c + e) * TAPS + j];
    b[e] = bias ? bias[c + e] : 0.f;
  }
  float u[TAPS][8];                               // the inputs of the row and of its TAPS - 1 predecessors, oldest first
  int seg_before = -1;
  for (int rr = 0; rr < ROWS; ++rr) {
    const int r = blockIdx.x * ROWS + rr;
    if (r >= n_rows) return;
    const int seg = row_seg[r];
    const int i_in_seg = r - seg_row0[seg];
    auto load_input = [&](int j) {
      const int back = TAPS - 1 - j;
      if (back <= i_in_seg) {
        const uint4 v = *reinterpret_cast<const uint4*>(x + (size_t)(r - back) * ldx + c);
        const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          u[j][2 * k] = __uint_as_float(p[k] << 16);
          u[j][2 * k + 1] = __uint_as_float(p[k] & 0xffff0000u);
        }
      } else {
        const float* sp = state + ((size_t)slots[seg] * (TAPS - 1) + (TAPS - 1 - (back - i_in_seg))) * C + c;
        const float4 a = *reinterpret_cast<const float4*>(sp), d = *reinterpret_cast<const float4*>(sp + 4);
        u[j][0] = a.x; u[j][1] = a.y; u[j][2] = a.z; u[j][3] = a.w;
        u[j][4] = d.x; u[j][5] = d.y; u[j][6] = d.z; u[j][7] = d.w;
      }
    };
    if (rr > 0 && seg == seg_before) {            // the row before is this row's predecessor
#pragma unroll
      for (int j = 0; j + 1 < TAPS; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) u[j][e] = u[j + 1][e];
      load_input(TAPS - 1);
    } else {
#pragma unroll
      for (int j = 0; j < TAPS; ++j) load_input(j);
    }
    seg_before = seg;
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float v[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int e = 2 * k + h;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) acc = fmaf(wt[e][j], u[j][e], acc);     // oldest first
        if (bias) acc += b[e];
        v[h] = activate(acc, act);
      }
      o[k] = pack_bf16x2(v[0], v[1]);
    }
    *reinterpret_cast<uint4*>(out + (size_t)r * ldo + c) = uint4{o[0], o[1], o[2], o[3]};
  }
}

// ---------------------------------------------------------------------------
// Selective scan.  Per channel c with N states, over the rows of a segment in order:
//   dt = softplus(dt_raw[t][c] + dt_bias[c])
//   S[c][n] <- exp(dt * A[c][n]) * S[c][n] + (dt * x[t][c]) * B[t][n];   y = sum_n S[c][n] * C[t][n] + D[c] * x[t][c]
//   out[t][c] = y * silu(z[t][c])
// S [slots][channels][N] float32 per request.  A group of LPC lanes (a power of two, <= 64) holds one channel's states,
// lane l the states l, l + LPC, ...; the sum over n is added inside the group in an order fixed by N alone.
// ---------------------------------------------------------------------------
template <int LPC>
__global__ __launch_bounds__(256) void selective_scan_kernel(
    const void* __restrict__ x, int x_dtype, int ldx, const float* __restrict__ dt_raw, int lddt,
    const float* __restrict__ dt_bias, const float* __restrict__ A, const float* __restrict__ bc, int ldbc,
    const float* __restrict__ Dw, const void* __restrict__ z, int z_dtype, int ldz, float* __restrict__ state,
    int channels, int N, const int* __restrict__ seg_row0, const int* __restrict__ seg_rows,
    const int* __restrict__ slots, void* __restrict__ out, int out_dtype, int ldo) {
  const int seg = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) / LPC, l = threadIdx.x % LPC;
  if (c >= channels) return;                      // (whole groups leave together: LPC divides 256)
  const int r0 = seg_row0[seg], n_rows = seg_rows[seg];
  float* S = state + ((size_t)slots[seg] * channels + c) * N;
  float s[SCAN_MAX_PER_LANE], a[SCAN_MAX_PER_LANE];
#pragma unroll
  for (int e = 0; e < SCAN_MAX_PER_LANE; ++e) {
    const int n = l + e * LPC;
    s[e] = n < N ? S[n] : 0.f;
    a[e] = n < N ? A[(size_t)c * N + n] : 0.f;
  }
  const float db = dt_bias ? dt_bias[c] : 0.f, dw = Dw ? Dw[c] : 0.f;
  for (int t = 0; t < n_rows; ++t) {
    const size_t r = (size_t)(r0 + t);
    const float dt = softplus_f(dt_raw[r * lddt + c] + db);
    const float xv = load_f(x, x_dtype, r * ldx + c);
    const float dx = dt * xv;
    float y = 0.f;
#pragma unroll
    for (int e = 0; e < SCAN_MAX_PER_LANE; ++e) {
      const int n = l + e * LPC;
      if (n < N) {
        s[e] = fmaf(expf(dt * a[e]), s[e], dx * bc[r * ldbc + n]);
        y = fmaf(s[e], bc[r * ldbc + N + n], y);
      }
    }
#pragma unroll
    for (int o = LPC / 2; o > 0; o >>= 1) y += __shfl_xor(y, o, WAVE);
    if (l == 0) {
      y = fmaf(dw, xv, y);
      store_f(out, out_dtype, r * ldo + c, y * silu_f(load_f(z, z_dtype, r * ldz + c)));
    }
  }
#pragma unroll
  for (int e = 0; e < SCAN_MAX_PER_LANE; ++e) {
    const int n = l + e * LPC;
    if (n < N) S[n] = s[e];
  }
}

// out[t][i] = act(in[t][i])
__global__ void act_rows_kernel(const void* __restrict__ in, int in_dtype, int ldi, void* __restrict__ out,
                                int out_dtype, int ldo, int n, int kind) {
  const int t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i < n) store_f(out, out_dtype, (size_t)t * ldo + i, activate(load_f(in, in_dtype, (size_t)t * ldi + i), kind));
}

// The same for bfloat16 rows whose width is a multiple of 8, 16 bytes a load.
__global__ void act_rows_bf16x8_kernel(const bf16_t* __restrict__ in, int ldi, bf16_t* __restrict__ out, int ldo,
                                       int n, int kind) {
  const int t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= n) return;
  const uint4 v = *reinterpret_cast<const uint4*>(in + (size_t)t * ldi + i);
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
    o[k] = pack_bf16x2(activate(__uint_as_float(w[k] << 16), kind), activate(__uint_as_float(w[k] & 0xffff0000u), kind));
  *reinterpret_cast<uint4*>(out + (size_t)t * ldo + i) = uint4{o[0], o[1], o[2], o[3]};
}

// x[t][i] += b[i]  (x float32)
__global__ void bias_rows_kernel(float* __restrict__ x, int ldx, const float* __restrict__ b, int n) {
  const int t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i < n) x[(size_t)t * ldx + i] += b[i];
}

// x[t][i] = a * u[t][i] + b * v[t][i]  (all float32; x may be u)
__global__ void weighted_pair_kernel(float* __restrict__ x, int ldx, const float* __restrict__ u, int ldu, float a,
                                     const float* __restrict__ v, int ldv, float b, int n) {
  const int t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i < n) x[(size_t)t * ldx + i] = fmaf(b, v[(size_t)t * ldv + i], a * u[(size_t)t * ldu + i]);
}

}  // namespace

APC_EXPORT int apc_conv_channels(const void* x, int x_dtype, int ldx, int n_rows, int C, const float* w,
                                 const float* bias, int taps, const float* state, const int* row_seg,
                                 const int* seg_row0, const int* slots, int act, void* out, int out_dtype, int ldo,
                                 hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (C <= 0 || ldx < C || ldo < C || taps < 1 || !w || act < 0 || act > 3 || !row_seg || !seg_row0) return APC_ERR_BAD_ARG;
  if (taps > 1 && (!state || !slots)) return APC_ERR_BAD_ARG;
  if (taps > SCAN_MAX_TAPS || ceil_div(C, 256) > 65535) return APC_ERR_UNSUPPORTED;
  if (x_dtype == APC_BF16 && out_dtype == APC_BF16 && taps <= 4 && C % 8 == 0 && ldx % 8 == 0 && ldo % 8 == 0 &&
      !((uintptr_t)x & 15u) && !((uintptr_t)out & 15u) && !((uintptr_t)state & 15u)) {
    const int rows_a_block = n_rows >= 512 ? 8 : 1;
    const dim3 grid(ceil_div(n_rows, rows_a_block), ceil_div(C / 8, 256));
#define CC_LAUNCH(TAPS_)                                                                                             \
  do {                                                                                                               \
    if (rows_a_block == 8)                                                                                           \
      hipLaunchKernelGGL((conv_channels_bf16x8_kernel<TAPS_, 8>), grid, dim3(256), 0, stream, (const bf16_t*)x, ldx,  \
                         n_rows, C, w, bias, state, row_seg, seg_row0, slots, act, (bf16_t*)out, ldo);               \
    else                                                                                                             \
      hipLaunchKernelGGL((conv_channels_bf16x8_kernel<TAPS_, 1>), grid, dim3(256), 0, stream, (const bf16_t*)x, ldx,  \
                         n_rows, C, w, bias, state, row_seg, seg_row0, slots, act, (bf16_t*)out, ldo);               \
  } while (0)
    if (taps == 1) CC_LAUNCH(1);
    else if (taps == 2) CC_LAUNCH(2);
    else if (taps == 3) CC_LAUNCH(3);
    else CC_LAUNCH(4);
#undef CC_LAUNCH
    APC_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(conv_channels_kernel, dim3(n_rows, ceil_div(C, 256)), dim3(256), 0, stream, x, x_dtype, ldx, C, w,
                     bias, taps, state, row_seg, seg_row0, slots, act, out, out_dtype, ldo);
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_selective_scan(const void* x, int x_dtype, int ldx, const float* dt_raw, int lddt,
                                  const float* dt_bias, const float* A, const float* bc, int ldbc, const float* Dw,
                                  const void* z, int z_dtype, int ldz, float* state, int channels, int N, int n_segs,
                                  const int* seg_row0, const int* seg_rows, const int* slots, void* out, int out_dtype,
                                  int ldo, hipStream_t stream) {
  if (n_segs <= 0) return 0;
  if (channels <= 0 || N <= 0 || !x || !dt_raw || !A || !bc || !z || !state || !slots || !out || ldx < channels ||
      lddt < channels || ldbc < 2 * N || ldz < channels || ldo < channels)
    return APC_ERR_BAD_ARG;
  if (N > 64 * SCAN_MAX_PER_LANE || n_segs > 65535) return APC_ERR_UNSUPPORTED;
  int lpc = 1;
  while (lpc < N && lpc < 64) lpc *= 2;
  const dim3 grid(ceil_div(channels * lpc, 256), n_segs);
#define SCAN_LAUNCH(LPC_)                                                                                              \
  hipLaunchKernelGGL(selective_scan_kernel<LPC_>, grid, dim3(256), 0, stream, x, x_dtype, ldx, dt_raw, lddt, dt_bias, A, \
                     bc, ldbc, Dw, z, z_dtype, ldz, state, channels, N, seg_row0, seg_rows, slots, out, out_dtype, ldo)
  switch (lpc) {
    case 1: SCAN_LAUNCH(1); break;
    case 2: SCAN_LAUNCH(2); break;
    case 4: SCAN_LAUNCH(4); break;
    case 8: SCAN_LAUNCH(8); break;
    case 16: SCAN_LAUNCH(16); break;
    case 32: SCAN_LAUNCH(32); break;
    default: SCAN_LAUNCH(64); break;
  }
#undef SCAN_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_act_rows(const void* in, int in_dtype, int ldi, void* out, int out_dtype, int ldo, int n_rows, int n,
                            int kind, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (n <= 0 || ldi < n || ldo < n || kind < 0 || kind > 3) return APC_ERR_BAD_ARG;
  if (ceil_div(n, 256) > 65535) return APC_ERR_UNSUPPORTED;
  if (in_dtype == APC_BF16 && out_dtype == APC_BF16 && n % 8 == 0 && ldi % 8 == 0 && ldo % 8 == 0 &&
      !((uintptr_t)in & 15u) && !((uintptr_t)out & 15u)) {
    hipLaunchKernelGGL(act_rows_bf16x8_kernel, dim3(n_rows, ceil_div(n / 8, 256)), dim3(256), 0, stream,
                       (const bf16_t*)in, ldi, (bf16_t*)out, ldo, n, kind);
    APC_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(act_rows_kernel, dim3(n_rows, ceil_div(n, 256)), dim3(256), 0, stream, in, in_dtype, ldi, out,
                     out_dtype, ldo, n, kind);
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_bias_rows(float* x, int ldx, const float* b, int n_rows, int n, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (n <= 0 || ldx < n || !b) return APC_ERR_BAD_ARG;
  if (ceil_div(n, 256) > 65535) return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(bias_rows_kernel, dim3(n_rows, ceil_div(n, 256)), dim3(256), 0, stream, x, ldx, b, n);
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_weighted_pair(float* x, int ldx, const float* u, int ldu, float a, const float* v, int ldv, float b,
                                 int n_rows, int n, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (n <= 0 || ldx < n || ldu < n || ldv < n || !u || !v) return APC_ERR_BAD_ARG;
  if (ceil_div(n, 256) > 65535) return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(weighted_pair_kernel, dim3(n_rows, ceil_div(n, 256)), dim3(256), 0, stream, x, ldx, u, ldu, a, v,
                     ldv, b, n);
  APC_LAUNCH_CHECK();
  return 0;
}
