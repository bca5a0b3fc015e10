// Routed experts (see plain_routed.hip for the formulas) in bfloat16 on MFMA.
//
//   sort      one block: the (row, choice) pairs that chose an expert with matrices are put side by side per expert
//             (`order`: sorted place -> pair, `place`: pair -> sorted place), and every expert's run is cut into tiles
//             of `tile_rows` rows (`tiles`: expert, first place, rows).  The order inside a run is whatever the
//             atomics give; no result depends on it, since every pair's output is computed for itself.
//   With many rows an expert (tiles of 64 or 128 rows) the rows are copied side by side first (`gather`) and the two
//   products run on the tiled kernel of the other products in its grouped mode (gemm_bf16.hip): the same tiles through
//   LDS, the matrix chosen per row tile.  With few (tiles of 16 rows: decoded rows) they run on the kernels below,
//   which stream an expert's matrices once a tile straight into the MFMA operands:
//   gate/up   a block takes a tile x 4 bands of 16 outputs, a wave one band of the gate matrix and the same band of the
//             up matrix: the weights' tiles (1 KiB each, in the lane order of the MFMA operand) stream from memory once
//             a tile, the rows are gathered through `order`; the activation a(g, u) leaves in bfloat16 at the sorted
//             place (a = silu(g) * u, or the clamped unit min(g, limit) * sigmoid(alpha min(g, limit)) *
//             (clamp(u, -limit, limit) + 1)).
//   down      the same over the activations at their sorted places; float32 out.
//   combine   y[row] = sum_k weight[row][k] * (down's row at the pair's place, or the input row for an identity
//             expert), k in order.
// With the weights on the experts' inputs (`in_weights`: y[row] = sum_k expert(weight * h)) the streaming kernel
// multiplies the float32 sums of gate and up with the pair's weight ahead of the activation (the products are linear
// in h), the copy for the tiled kernel writes weight * h, and the last kernel adds the experts' outputs as they are.
// Experts' matrices: gate_up [E][2][bands(F)][chunks(D)][64][8] and down [E][bands(D)][chunks(F)][64][8] in the tiled
// layout of the other products.  The grid is made for the most tiles the step can have; a block beyond the tiles that
// exist leaves at once.
#include "mfma.h"
#include <math.h>

namespace {

constexpr int TILE_ELEMS = 512;
constexpr int MAX_EXPERTS = 1024;
constexpr int STREAM_U = 4;       // chunks of 32 columns a wave asks for together

__device__ __forceinline__ float unit_act(float g, float u, int kind, float alpha, float limit) {
  return gated_unit_act(g, u, kind, alpha, limit);
}

__global__ __launch_bounds__(1024) void routed_sort_kernel(const int* __restrict__ ids, int n_pairs, int E,
                                                           int tile_rows, int* __restrict__ order,
                                                           int* __restrict__ place, int* __restrict__ tiles,
                                                           int* __restrict__ n_tiles) {
  __shared__ int cnt[MAX_EXPERTS], start[MAX_EXPERTS], tstart[MAX_EXPERTS + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int p = tid; p < n_pairs; p += 1024) {
    const int e = ids[p];
    if (e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0, t = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      tstart[e] = t;
      at += cnt[e];
      t += (cnt[e] + tile_rows - 1) / tile_rows;
    }
    tstart[E] = t;
    *n_tiles = t;
  }
  __syncthreads();
  for (int e = tid; e < E; e += 1024) {
    const int c = cnt[e];
    for (int k = 0, t = tstart[e]; t < tstart[e + 1]; ++k, ++t) {
      tiles[3 * t] = e;
      tiles[3 * t + 1] = start[e] + k * tile_rows;
      tiles[3 * t + 2] = min(tile_rows, c - k * tile_rows);
    }
    cnt[e] = 0;        // now the count of pairs placed
  }
  __syncthreads();
  for (int p = tid; p < n_pairs; p += 1024) {
    const int e = ids[p];
    if (e < E) {
      const int at = start[e] + atomicAdd(&cnt[e], 1);
      order[at] = p;
      place[p] = at;
    } else {
      place[p] = -1;
    }
  }
}

// RT tiles of 16 rows a wave: a weight tile read from memory feeds RT MFMAs (the launches use 1: more rows an expert
// go to the tiled kernel)
template <int RT>
__global__ __launch_bounds__(256) void routed_glu_bf16_kernel(const bf16_t* __restrict__ h, int ldh,
                                                              const bf16_t* __restrict__ w_gate_up, int F, int D,
                                                              const int* __restrict__ order, int K,
                                                              const int* __restrict__ tiles,
                                                              const int* __restrict__ n_tiles,
                                                              bf16_t* __restrict__ act, int kind, float alpha,
                                                              float limit, const float* __restrict__ in_weights) {
  const int ti = blockIdx.x;
  if (ti >= *n_tiles) return;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, li = lane % 16, lc = lane / 16;
  const int bands = (F + 15) / 16, chunks = (D + 31) / 32, full = D / 32;
  const int band = blockIdx.y * 4 + wave;
  if (band >= bands) return;
  const int e = tiles[3 * ti], p0 = tiles[3 * ti + 1], rows = tiles[3 * ti + 2];
  const bf16_t* wg = w_gate_up + (((size_t)e * 2) * bands + band) * chunks * TILE_ELEMS + lane * 8;
  const bf16_t* wu = wg + (size_t)bands * chunks * TILE_ELEMS;
  const bf16_t* arow[RT];
  bool on[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int r = rt * 16 + li;
    on[rt] = r < rows;
    arow[rt] = h + (size_t)(on[rt] ? order[p0 + r] / K : 0) * ldh + lc * 8;
  }
  floatx4 g[RT], u[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) g[rt] = u[rt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // The weights are read once a tile: loads that the caches do not keep, STREAM_U chunks asked for together so that a
  // wave has 8 KiB of them in flight (one chunk at a time a wave waited a trip to memory for every 2 KiB).
  int c = 0;
  for (; c + STREAM_U <= chunks; c += STREAM_U) {
    Frag fg[STREAM_U], fu[STREAM_U], a[STREAM_U][RT];
#pragma unroll
    for (int x = 0; x < STREAM_U; ++x) {
      fg[x] = load_frag_once(wg + (size_t)(c + x) * TILE_ELEMS);
      fu[x] = load_frag_once(wu + (size_t)(c + x) * TILE_ELEMS);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        // (a last chunk that reaches beyond D: the weights' tile is zero there, the row's elements must not be read)
        a[x][rt] = (on[rt] && (c + x < full || (c + x) * 32 + lc * 8 < D)) ? load_frag(arow[rt] + (c + x) * 32)
                                                                          : zero_frag();
    }
#pragma unroll
    for (int x = 0; x < STREAM_U; ++x)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        g[rt] = mfma16(fg[x], a[x][rt], g[rt]);
        u[rt] = mfma16(fu[x], a[x][rt], u[rt]);
      }
  }
  for (; c < chunks; ++c) {
    const Frag fg = load_frag_once(wg + (size_t)c * TILE_ELEMS), fu = load_frag_once(wu + (size_t)c * TILE_ELEMS);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const Frag a = (on[rt] && (c < full || c * 32 + lc * 8 < D)) ? load_frag(arow[rt] + c * 32) : zero_frag();
      g[rt] = mfma16(fg, a, g[rt]);
      u[rt] = mfma16(fu, a, u[rt]);
    }
  }
  // lane: outputs band * 16 + lc * 4 + 0..3 of row rt * 16 + li
  const int f0 = band * 16 + lc * 4;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (!on[rt] || f0 >= F) continue;
    bf16_t* dst = act + (size_t)(p0 + rt * 16 + li) * F + f0;
    float v[4];
    const float w = in_weights ? in_weights[order[p0 + rt * 16 + li]] : 1.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = unit_act(g[rt][r] * w, u[rt][r] * w, kind, alpha, limit);
    if (f0 + 4 <= F && F % 4 == 0) {
      uint2 pk;
      pk.x = pack_bf16x2(v[0], v[1]);
      pk.y = pack_bf16x2(v[2], v[3]);
      *reinterpret_cast<uint2*>(dst) = pk;
    } else {
      for (int r = 0; r < 4 && f0 + r < F; ++r) dst[r] = float_to_bf16(v[r]);
    }
  }
}

template <int RT>
__global__ __launch_bounds__(256) void routed_down_bf16_kernel(const bf16_t* __restrict__ act, int F, int D,
                                                               const bf16_t* __restrict__ w_down,
                                                               const int* __restrict__ tiles,
                                                               const int* __restrict__ n_tiles,
                                                               float* __restrict__ ys) {
  const int ti = blockIdx.x;
  if (ti >= *n_tiles) return;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, li = lane % 16, lc = lane / 16;
  const int bands = (D + 15) / 16, chunks = (F + 31) / 32, full = F / 32;
  const int band = blockIdx.y * 4 + wave;
  if (band >= bands) return;
  const int e = tiles[3 * ti], p0 = tiles[3 * ti + 1], rows = tiles[3 * ti + 2];
  const bf16_t* wd = w_down + ((size_t)e * bands + band) * chunks * TILE_ELEMS + lane * 8;
  const bf16_t* arow[RT];
  bool on[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int r = rt * 16 + li;
    on[rt] = r < rows;
    arow[rt] = act + (size_t)(p0 + (on[rt] ? r : 0)) * F + lc * 8;
  }
  floatx4 acc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = floatx4{0.f, 0.f, 0.f, 0.f};
  int c = 0;
  for (; c + 2 * STREAM_U <= chunks; c += 2 * STREAM_U) {
    Frag fw[2 * STREAM_U], a[2 * STREAM_U][RT];
#pragma unroll
    for (int x = 0; x < 2 * STREAM_U; ++x) {
      fw[x] = load_frag_once(wd + (size_t)(c + x) * TILE_ELEMS);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        a[x][rt] = (on[rt] && (c + x < full || (c + x) * 32 + lc * 8 < F)) ? load_frag(arow[rt] + (c + x) * 32)
                                                                          : zero_frag();
    }
#pragma unroll
    for (int x = 0; x < 2 * STREAM_U; ++x)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) acc[rt] = mfma16(fw[x], a[x][rt], acc[rt]);
  }
  for (; c < chunks; ++c) {
    const Frag fw = load_frag_once(wd + (size_t)c * TILE_ELEMS);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const Frag a = (on[rt] && (c < full || c * 32 + lc * 8 < F)) ? load_frag(arow[rt] + c * 32) : zero_frag();
      acc[rt] = mfma16(fw, a, acc[rt]);
    }
  }
  const int d0 = band * 16 + lc * 4;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (!on[rt] || d0 >= D) continue;
    float* dst = ys + (size_t)(p0 + rt * 16 + li) * D + d0;
    if (D % 4 == 0) *reinterpret_cast<float4*>(dst) = float4{acc[rt][0], acc[rt][1], acc[rt][2], acc[rt][3]};
    else for (int r = 0; r < 4 && d0 + r < D; ++r) dst[r] = acc[rt][r];
  }
}

// rows side by side in the sorted order: hs[place] = h[row of the pair at that place], 16 bytes a thread
__global__ __launch_bounds__(256) void routed_gather_kernel(const bf16_t* __restrict__ h, int ldh, int D,
                                                            const int* __restrict__ order, int K,
                                                            const int* __restrict__ tiles,
                                                            const int* __restrict__ n_tiles, int tile_rows,
                                                            bf16_t* __restrict__ hs,
                                                            const float* __restrict__ in_weights) {
  const int ti = blockIdx.x;
  if (ti >= *n_tiles) return;
  const int p0 = tiles[3 * ti + 1], rows = tiles[3 * ti + 2];
  const int pieces = D / 8;
  for (int idx = blockIdx.y * 256 + threadIdx.x; idx < rows * pieces; idx += gridDim.y * 256) {
    const int r = idx / pieces, c = (idx % pieces) * 8;
    const int pair = order[p0 + r];
    Frag f = load_frag(h + (size_t)(pair / K) * ldh + c);
    if (in_weights) {
      const float w = in_weights[pair];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        f.w[k] = pack_bf16x2(__uint_as_float(f.w[k] << 16) * w, __uint_as_float(f.w[k] & 0xffff0000u) * w);
    }
    *reinterpret_cast<Frag*>(hs + (size_t)(p0 + r) * D + c) = f;
  }
}

__global__ __launch_bounds__(256) void routed_combine_kernel(const float* __restrict__ ys, const int* __restrict__ place,
                                                             const float* __restrict__ weights, int K,
                                                             const bf16_t* __restrict__ h, int ldh,
                                                             float* __restrict__ y, int ldy, int D, int in_weights) {
  const int t = blockIdx.x;
  for (int d = threadIdx.x; d < D; d += 256) {
    float total = 0.f;
    for (int k = 0; k < K; ++k) {
      const int at = place[(size_t)t * K + k];
      const float v = at >= 0 ? ys[(size_t)at * D + d] : bf16_to_float(h[(size_t)t * ldh + d]);
      total = (in_weights && at >= 0) ? total + v : fmaf(weights[(size_t)t * K + k], v, total);
    }
    y[(size_t)t * ldy + d] = total;
  }
}

}  // namespace

// 1 if the kernels take these sizes, else 0 (the caller then keeps the matrices row-major for the plain kernels)
APC_EXPORT int apc_routed_bf16_takes(int E, int F, int D) {
  return (E >= 1 && E <= MAX_EXPERTS && F >= 8 && D >= 8 && F % 8 == 0 && D % 8 == 0) ? 1 : 0;
}

// most tiles a step of n_pairs pairs can have
APC_EXPORT int apc_routed_max_tiles(int n_pairs, int E, int tile_rows) {
  return (n_pairs + tile_rows - 1) / tile_rows + (E < n_pairs ? E : n_pairs);
}

extern "C" int apc_gemm_grouped_bf16(const void* A, int lda, const void* W, const void* W2, size_t w_stride, void* C,
                                     int ldc, const int* tiles, const int* n_tiles, int max_tiles, int tile_rows,
                                     int N, int K, int mode, int act, float alpha, float limit, hipStream_t stream);

// work: int32 [2 * n_pairs + 3 * max_tiles + 1] (order, place, tiles, the tiles' count); act: bfloat16 [n_pairs, F];
// ys: float32 [n_pairs, D]; hs: bfloat16 [n_pairs, D] (tiles of 64 and 128 rows only).  tile_rows: 16, 64 or 128.
// kind, alpha, limit: the activation (0: silu(g) * u; 1: the clamped unit), applied where gate and up are formed.
APC_EXPORT int apc_routed_experts_bf16(const void* h, int ldh, const void* w_gate_up, const void* w_down, int E, int F,
                                       int D, const int* ids, const float* weights, int K, int n_rows, int tile_rows,
                                       int* work, void* act, float* ys, void* hs, float* y, int ldy, int kind,
                                       float alpha, float limit, int in_weights, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!apc_routed_bf16_takes(E, F, D)) return APC_ERR_UNSUPPORTED;
  if (kind < 0 || kind > 1) return APC_ERR_BAD_ARG;
  if (K <= 0 || ldh < D || ldy < D || ldh % 8 || (tile_rows != 16 && tile_rows != 64 && tile_rows != 128) || !work ||
      !act || !ys || (tile_rows != 16 && (!hs || ((uintptr_t)hs & 15u))) ||
      ((uintptr_t)h & 15u) || ((uintptr_t)w_gate_up & 15u) || ((uintptr_t)w_down & 15u) || ((uintptr_t)act & 15u) ||
      ((uintptr_t)ys & 15u) || (long)n_rows * K > 0x3fffffffL)
    return APC_ERR_BAD_ARG;
  const int n_pairs = n_rows * K;
  const int max_tiles = apc_routed_max_tiles(n_pairs, E, tile_rows);
  int* order = work;
  int* place = work + n_pairs;
  int* tiles = work + 2 * (size_t)n_pairs;
  int* n_tiles = tiles + 3 * (size_t)max_tiles;
  hipLaunchKernelGGL(routed_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, n_pairs, E, tile_rows, order, place,
                     tiles, n_tiles);
  APC_LAUNCH_CHECK();
  const dim3 g1(max_tiles, ceil_div(ceil_div(F, 16), 4)), g2(max_tiles, ceil_div(ceil_div(D, 16), 4));
  if (g1.y > 65535 || g2.y > 65535) return APC_ERR_UNSUPPORTED;
  if (tile_rows == 16) {
    hipLaunchKernelGGL(routed_glu_bf16_kernel<1>, g1, dim3(256), 0, stream, (const bf16_t*)h, ldh,
                       (const bf16_t*)w_gate_up, F, D, order, K, tiles, n_tiles, (bf16_t*)act, kind, alpha, limit,
                       in_weights ? weights : nullptr);
    APC_LAUNCH_CHECK();
    hipLaunchKernelGGL(routed_down_bf16_kernel<1>, g2, dim3(256), 0, stream, (const bf16_t*)act, F, D,
                       (const bf16_t*)w_down, tiles, n_tiles, ys);
    APC_LAUNCH_CHECK();
  } else {
    if (max_tiles > 65535) return APC_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(routed_gather_kernel, dim3(max_tiles, 16), dim3(256), 0, stream, (const bf16_t*)h, ldh, D, order, K,
                       tiles, n_tiles, tile_rows, (bf16_t*)hs, in_weights ? weights : nullptr);
    APC_LAUNCH_CHECK();
    const size_t gate_elems = (size_t)ceil_div(F, 16) * ceil_div(D, 32) * TILE_ELEMS;
    const size_t down_elems = (size_t)ceil_div(D, 16) * ceil_div(F, 32) * TILE_ELEMS;
    int e = apc_gemm_grouped_bf16(hs, D, w_gate_up, (const bf16_t*)w_gate_up + gate_elems, 2 * gate_elems, act, F,
                                  tiles, n_tiles, max_tiles, tile_rows, F, D, /* gated unit */ 3, kind, alpha, limit,
                                  stream);
    if (e) return e;
    e = apc_gemm_grouped_bf16(act, F, w_down, nullptr, down_elems, ys, D, tiles, n_tiles, max_tiles, tile_rows, D, F,
                              /* float32 out */ 1, 0, 1.0f, 0.0f, stream);
    if (e) return e;
  }
  hipLaunchKernelGGL(routed_combine_kernel, dim3(n_rows), dim3(256), 0, stream, ys, place, weights, K,
                     (const bf16_t*)h, ldh, y, ldy, D, in_weights);
  APC_LAUNCH_CHECK();
  return 0;
}
