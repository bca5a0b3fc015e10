// The selective scan (see plain_scan.hip for the formulas) over prompt portions, chunks of rows side by side.
//
// The recurrence S_t = exp(dt_t A) S_(t-1) + dt_t x_t B_t is linear in S, so a segment's rows are cut into chunks of 64
// and three launches replace the walk row by row:
//   summaries  every chunk for itself, from a state of zero: its end state E and the sum of its step sizes (the
//              product of its decays is exp(A * that sum))
//   scan       per segment, channel and state: the state in front of every chunk, S0_(k+1) = exp(A sum_k) S0_k + E_k,
//              starting from the request's state, which is left at the segment's end
//   outputs    every chunk again from the state in front of it: y_t = sum_n S_t[n] C_t[n] + D x_t, times silu(z_t)
// All arithmetic is float32 (exponentials through the hardware's base-2 instruction); x, z and the output are
// bfloat16 rows, the step sizes, B and C float32 rows.  A group of LPC lanes (a power of two) holds a channel's
// states, a lane up to 16 of them in registers; with 16 states or fewer a thread is a channel.  B and C of a chunk's
// rows, which every thread of a block reads, are put into LDS once a block (where they fit 32 KiB), and with exactly 16
// states a thread reads them four at a time without a test of the state's number.  Steps whose segments are all short (decoded rows) stay on the kernel
// that walks row by row, which reads and writes the state once.
#include "mfma.h"
#include <math.h>

namespace {

constexpr int NS = 16;            // states a lane keeps
constexpr int CHUNK = 64;         // rows of a chunk (the step's list of chunks is made for this)
constexpr float LOG2E_F = 1.4426950408889634f;

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(__expf(z)); }
__device__ __forceinline__ float silu_fast(float z) { return z / (1.0f + __expf(-z)); }

template <int MODE, bool FULL>   // MODE 1: summaries, 2: outputs; FULL: 16 states a channel, a thread a channel
__global__ __launch_bounds__(256) void scan_chunk_kernel(
    const bf16_t* __restrict__ x, int ldx, const float* __restrict__ dt_raw, int lddt,
    const float* __restrict__ dt_bias, const float* __restrict__ A, const float* __restrict__ bc, int ldbc,
    const float* __restrict__ Dw, const bf16_t* __restrict__ z, int ldz, float* __restrict__ ws,
    float* __restrict__ sumdt, int channels, int N, int lpc, const int* __restrict__ chunks,
    const int* __restrict__ seg_row0, const int* __restrict__ seg_rows, bf16_t* __restrict__ out, int ldo,
    int staged) {
  extern __shared__ float bcs[];                // [rows of the chunk][2 N], if `staged`
  const int chunk = blockIdx.y;
  const int seg = chunks[2 * chunk], in_seg = chunks[2 * chunk + 1];
  const int gid = blockIdx.x * 256 + threadIdx.x;
  const int c = gid / lpc, l = gid % lpc;
  const int r0 = seg_row0[seg] + in_seg, n_rows = min(CHUNK, seg_rows[seg] - in_seg);
  if (staged) {
    for (int i = threadIdx.x; i < n_rows * 2 * N; i += 256) bcs[i] = bc[(size_t)(r0 + i / (2 * N)) * ldbc + i % (2 * N)];
    __syncthreads();
  }
  if (c >= channels) return;                    // (whole groups leave together: lpc divides 256)
  float* w = ws + ((size_t)chunk * channels + c) * N;
  float s[NS], a2[NS];
#pragma unroll
  for (int e = 0; e < NS; ++e) {
    const int n = l + e * lpc;
    s[e] = (MODE == 2 && n < N) ? w[n] : 0.f;
    a2[e] = n < N ? A[(size_t)c * N + n] * LOG2E_F : 0.f;
  }
  const float db = dt_bias ? dt_bias[c] : 0.f, dw = Dw ? Dw[c] : 0.f;
  float total = 0.f;
  float dt_next = dt_raw[(size_t)r0 * lddt + c];
  float x_next = __uint_as_float((uint32_t)x[(size_t)r0 * ldx + c] << 16);
  for (int t = 0; t < n_rows; ++t) {
    const size_t r = (size_t)(r0 + t);
    const float dt = softplus_f(dt_next + db), xv = x_next;
    if (t + 1 < n_rows) {                       // the next row's own numbers are asked for ahead of this row's work
      dt_next = dt_raw[(r + 1) * lddt + c];
      x_next = __uint_as_float((uint32_t)x[(r + 1) * ldx + c] << 16);
    }
    const float dx = dt * xv;
    total += dt;
    const float* b = staged ? bcs + (size_t)t * 2 * N : bc + r * ldbc;
    float y = 0.f;
    if (FULL) {
#pragma unroll
      for (int e4 = 0; e4 < NS / 4; ++e4) {
        const float4 bv = *reinterpret_cast<const float4*>(b + 4 * e4);
        const float bb[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
          s[4 * e4 + k] = fmaf(__builtin_amdgcn_exp2f(dt * a2[4 * e4 + k]), s[4 * e4 + k], dx * bb[k]);
        if (MODE == 2) {
          const float4 cv = *reinterpret_cast<const float4*>(b + NS + 4 * e4);
          y = fmaf(s[4 * e4], cv.x, y);
          y = fmaf(s[4 * e4 + 1], cv.y, y);
          y = fmaf(s[4 * e4 + 2], cv.z, y);
          y = fmaf(s[4 * e4 + 3], cv.w, y);
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < NS; ++e) {
        const int n = l + e * lpc;
        if (n < N) {
          s[e] = fmaf(__builtin_amdgcn_exp2f(dt * a2[e]), s[e], dx * b[n]);
          if (MODE == 2) y = fmaf(s[e], b[N + n], y);
        }
      }
    }
    if (MODE == 2) {
      for (int o = lpc / 2; o > 0; o >>= 1) y += __shfl_xor(y, o, WAVE);
      if (l == 0) {
        y = fmaf(dw, xv, y);
        const float zv = __uint_as_float((uint32_t)z[r * ldz + c] << 16);
        out[r * ldo + c] = float_to_bf16(y * silu_fast(zv));
      }
    }
  }
  if (MODE == 1) {
#pragma unroll
    for (int e = 0; e < NS; ++e) {
      const int n = l + e * lpc;
      if (n < N) w[n] = s[e];
    }
    if (l == 0) sumdt[(size_t)chunk * channels + c] = total;
  }
}

// ws [chunks][channels][N]: a chunk's end state in, the state in front of it out
__global__ __launch_bounds__(256) void scan_states_kernel(float* __restrict__ ws, const float* __restrict__ sumdt,
                                                          const float* __restrict__ A, float* __restrict__ state,
                                                          const int* __restrict__ seg_chunks,
                                                          const int* __restrict__ slots, int channels, int N) {
  const int seg = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= channels * N) return;
  const int c = i / N;
  const int k0 = seg_chunks[2 * seg], nk = seg_chunks[2 * seg + 1];
  float* S = state + (size_t)slots[seg] * channels * N + i;
  float s = *S;
  const float a2 = A[i] * LOG2E_F;
  for (int k = k0; k < k0 + nk; ++k) {
    float* w = ws + (size_t)k * channels * N + i;
    const float e = *w;
    *w = s;
    s = fmaf(__builtin_amdgcn_exp2f(a2 * sumdt[(size_t)k * channels + c]), s, e);
  }
  *S = s;
}

}  // namespace

// 1 if the kernels take these sizes, else 0 (the caller then runs the plain kernel)
APC_EXPORT int apc_selective_scan_bf16_takes(int channels, int N) {
  return (channels > 0 && N > 0 && N <= NS * 16) ? 1 : 0;
}

// chunks: int32 [n_chunks][2] (segment, first row of the chunk in it), all segments' chunks of 64 rows in order;
// seg_chunks: int32 [n_segs][2] (a segment's first chunk, its chunks); ws: float32 [n_chunks][channels][N];
// sumdt: float32 [n_chunks][channels].
APC_EXPORT int apc_selective_scan_bf16(const void* x, int ldx, const float* dt_raw, int lddt, const float* dt_bias,
                                       const float* A, const float* bc, int ldbc, const float* Dw, const void* z,
                                       int ldz, float* state, int channels, int N, int n_segs, const int* seg_row0,
                                       const int* seg_rows, const int* slots, int n_chunks, const int* chunks,
                                       const int* seg_chunks, float* ws, float* sumdt, void* out, int ldo,
                                       hipStream_t stream) {
  if (n_segs <= 0 || n_chunks <= 0) return 0;
  if (!apc_selective_scan_bf16_takes(channels, N)) return APC_ERR_UNSUPPORTED;
  if (!x || !dt_raw || !A || !bc || !z || !state || !slots || !chunks || !seg_chunks || !ws || !sumdt || !out ||
      ldx < channels || lddt < channels || ldbc < 2 * N || ldz < channels || ldo < channels)
    return APC_ERR_BAD_ARG;
  int lpc = 1;
  while (lpc * NS < N) lpc *= 2;
  const long threads = (long)channels * lpc;
  if (n_chunks > 65535 || n_segs > 65535 || (threads + 255) / 256 > 0x7fffffffL) return APC_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)((threads + 255) / 256), n_chunks);
  // B and C of a chunk's rows in LDS (rows of the staged copy are 2 N floats: 16-byte reads need N a multiple of 2)
  const size_t lds = (size_t)CHUNK * 2 * N * sizeof(float);
  const int staged = lds <= 32 * 1024 ? 1 : 0;
  const bool full = N == NS && staged;
#define SCAN_LAUNCH(MODE_)                                                                                            \
  do {                                                                                                                \
    if (full)                                                                                                         \
      hipLaunchKernelGGL((scan_chunk_kernel<MODE_, true>), grid, dim3(256), lds, stream, (const bf16_t*)x, ldx, dt_raw, \
                         lddt, dt_bias, A, bc, ldbc, Dw, (const bf16_t*)z, ldz, ws, sumdt, channels, N, lpc, chunks,    \
                         seg_row0, seg_rows, (bf16_t*)out, ldo, staged);                                              \
    else                                                                                                              \
      hipLaunchKernelGGL((scan_chunk_kernel<MODE_, false>), grid, dim3(256), staged ? lds : 0, stream,                \
                         (const bf16_t*)x, ldx, dt_raw, lddt, dt_bias, A, bc, ldbc, Dw, (const bf16_t*)z, ldz, ws,      \
                         sumdt, channels, N, lpc, chunks, seg_row0, seg_rows, (bf16_t*)out, ldo, staged);              \
    APC_LAUNCH_CHECK();                                                                                               \
  } while (0)
  SCAN_LAUNCH(1);
  hipLaunchKernelGGL(scan_states_kernel, dim3(ceil_div(channels * N, 256), n_segs), dim3(256), 0, stream, ws, sumdt, A,
                     state, seg_chunks, slots, channels, N);
  APC_LAUNCH_CHECK();
  SCAN_LAUNCH(2);
#undef SCAN_LAUNCH
  return 0;
}
