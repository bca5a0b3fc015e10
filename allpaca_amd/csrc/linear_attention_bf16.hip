// Linear attention with a decay (see plain_recurrent.hip for the formulas) for bfloat16 rows on MFMA, a segment's rows
// in chunks of 64.  With S0 the state in front of a chunk, lam the head's decay, rows t, s = 0 .. n-1 of the chunk:
//   A[t][s] = (q_t . k_s) lam^(t-s) for s <= t                      (scores and decay in float32)
//   o_t     = lam^(t+1) S0^T q_t + sum_s A[t][s] v_s
//   S       = lam^n S0 + sum_s (lam^(n-1-s) k_s) v_s^T
// The chunks of all segments run side by side in three launches: every chunk's own contribution to the state (a block
// a chunk x head x 64 value columns), then every state element's walk over its segment's chunks, which leaves the
// state in front of each chunk, then every chunk's outputs.  q, k and v are bfloat16 (through silu if asked,
// rounded once); everything that is float32 in the formulas and has to be an MFMA operand (S0, the decayed keys, A)
// goes in as two bfloat16 pieces, value = hi + lo, so that a product keeps 16 bits of it and not 8.
// All products are transposed (keys or value columns as the rows of a tile) so that a lane holds 4 consecutive
// elements of what it stores.
#include "mfma.h"
#include <math.h>

namespace {

constexpr int C = 64;      // rows of a chunk
constexpr int VT = 64;     // value columns of a block
constexpr int PAD = 8;
constexpr int SR = C + PAD;

__device__ __forceinline__ void unpack8f(const Frag& f, float* v) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    v[2 * w] = __uint_as_float(f.w[w] << 16);
    v[2 * w + 1] = __uint_as_float(f.w[w] & 0xffff0000u);
  }
}
__device__ __forceinline__ float round_bf16(float v) { return bf16_to_float(float_to_bf16(v)); }

// four consecutive float32 as two bfloat16 pieces each: hi to `ph`, lo to `pl`
__device__ __forceinline__ void store_split4(bf16_t* ph, bf16_t* pl, float a, float b, float c, float d) {
  uint2 hi, lo;
  hi.x = pack_bf16x2(a, b);
  hi.y = pack_bf16x2(c, d);
  const float ha = __uint_as_float(hi.x << 16), hb = __uint_as_float(hi.x & 0xffff0000u);
  const float hc = __uint_as_float(hi.y << 16), hd = __uint_as_float(hi.y & 0xffff0000u);
  lo.x = pack_bf16x2(a - ha, b - hb);
  lo.y = pack_bf16x2(c - hc, d - hd);
  *reinterpret_cast<uint2*>(ph) = hi;
  *reinterpret_cast<uint2*>(pl) = lo;
}

// MODE 1: the chunk's own contribution to the state, sum_s (lam^(n-1-s) k_s) v_s^T, into `ws` [chunk][head][dk][dv].
// MODE 2: the chunk's outputs from the state in front of it, which the scan kernel below has put into `ws` in the
// contribution's place.  `chunks` [n][2]: a chunk's segment and its first row inside the segment.
template <int DKP, int MODE>  // key size rounded up to a multiple of 64
__global__ __launch_bounds__(256) void linear_attention_chunk_kernel(
    const bf16_t* __restrict__ proj, int ld, int q_off, int k_off, int v_off, int H, int dk, int dv, int act,
    const float* __restrict__ powers, const int* __restrict__ chunks, float* __restrict__ ws,
    const int* __restrict__ seg_row0, const int* __restrict__ seg_rows, float* __restrict__ out, int ldo) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  constexpr int QR = DKP + PAD;
  constexpr int IT = DKP / 64;               // tiles of 16 state rows a wave owns
  bf16_t* Vt = reinterpret_cast<bf16_t*>(lds);   // [VT][SR]  v, a column's rows side by side
  // MODE 1
  bf16_t* KtH = Vt + VT * SR;                    // [DKP][SR] decayed k, a key element's rows side by side (hi, lo)
  bf16_t* KtL = KtH + DKP * SR;
  // MODE 2
  bf16_t* Ks = Vt + VT * SR;                     // [C][QR]   k of the chunk's rows
  bf16_t* AsH = Ks + C * QR;                     // [C][SR]   A[t][s] (hi, lo)
  bf16_t* AsL = AsH + C * SR;
  bf16_t* StH = AsL + C * SR;                    // [VT][QR]  the state in front of the chunk, S0[i][j] at [j][i]
  bf16_t* StL = StH + VT * QR;
  bf16_t* last = MODE == 1 ? KtL + DKP * SR : StL + VT * QR;
  float* pw = reinterpret_cast<float*>(last);    // [C + 1] powers of the decay

  const int seg = chunks[2 * blockIdx.x], c0 = chunks[2 * blockIdx.x + 1];
  const int h = blockIdx.y, j0 = blockIdx.z * VT;
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int li = lane % 16, lc = lane / 16;
  const int r0 = seg_row0[seg] + c0, nc = min(C, seg_rows[seg] - c0);
  float* W = ws + (((size_t)blockIdx.x * H + h) * dk) * dv;
  // (every element of LDS that is read below is written below: rows beyond the chunk's and columns beyond the sizes
  // as zeros)
  if (tid <= C) pw[tid] = powers[(size_t)h * (C + 1) + tid];
  __syncthreads();

  // ---- the chunk's v (both modes), decayed k (1) or k (2)
  for (int idx = tid; idx < C * (VT / 8); idx += 256) {
    const int s = idx % C, e = (idx / C) * 8;
    float vv[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) vv[x] = 0.f;
    if (s < nc && j0 + e < dv) {
      unpack8f(load_frag(proj + (size_t)(r0 + s) * ld + v_off + (size_t)h * dv + j0 + e), vv);
      if (act) {
#pragma unroll
        for (int x = 0; x < 8; ++x) vv[x] = silu_f(vv[x]);
      }
    }
#pragma unroll
    for (int x = 0; x < 8; ++x) Vt[(e + x) * SR + s] = float_to_bf16(vv[x]);
  }
  for (int idx = tid; idx < C * (DKP / 8); idx += 256) {
    const int s = idx % C, e = (idx / C) * 8;
    float kv[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) kv[x] = 0.f;
    if (s < nc && e < dk) {
      unpack8f(load_frag(proj + (size_t)(r0 + s) * ld + (size_t)h * dk + e + k_off), kv);
      if (act) {
#pragma unroll
        for (int x = 0; x < 8; ++x) kv[x] = silu_f(kv[x]);
      }
    }
    Frag fk;
#pragma unroll
    for (int w = 0; w < 4; ++w) fk.w[w] = pack_bf16x2(kv[2 * w], kv[2 * w + 1]);
    if (MODE == 2) {
      *reinterpret_cast<Frag*>(Ks + s * QR + e) = fk;
    } else {
      const float d = s < nc ? pw[nc - 1 - s] : 0.f;
      float kr[8];
      unpack8f(fk, kr);                       // the rounded keys, as the scores see them
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float kd = kr[x] * d;
        const bf16_t hi = float_to_bf16(kd);
        KtH[(e + x) * SR + s] = hi;
        KtL[(e + x) * SR + s] = float_to_bf16(kd - bf16_to_float(hi));
      }
    }
  }

  if constexpr (MODE == 1) {
    __syncthreads();
    // ---- tile rows key elements i (the wave's own), columns j
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int i = (wave * IT + it) * 16 + li;
      Frag kh[2], kl[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        kh[kk] = *reinterpret_cast<const Frag*>(KtH + i * SR + kk * 32 + lc * 8);
        kl[kk] = *reinterpret_cast<const Frag*>(KtL + i * SR + kk * 32 + lc * 8);
      }
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
        floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const Frag vf = *reinterpret_cast<const Frag*>(Vt + (jt * 16 + li) * SR + kk * 32 + lc * 8);
          acc = mfma16(kh[kk], vf, acc);
          acc = mfma16(kl[kk], vf, acc);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {      // element r: [i0 + lc * 4 + r][j0 + jt * 16 + li]
          const int ii = (wave * IT + it) * 16 + lc * 4 + r, j = j0 + jt * 16 + li;
          if (ii < dk && j < dv) W[(size_t)ii * dv + j] = acc[r];
        }
      }
    }
  } else {
    // ---- the state in front of the chunk, as an operand (S0[i][j] at [j][i], hi and lo)
#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = (wave * IT + it) * 16 + lc * 4 + r, j = j0 + jt * 16 + li;
          v[r] = (i < dk && j < dv) ? W[(size_t)i * dv + j] : 0.f;
        }
        const int at = (jt * 16 + li) * QR + (wave * IT + it) * 16 + lc * 4;
        store_split4(StH + at, StL + at, v[0], v[1], v[2], v[3]);
      }
    __syncthreads();

    // ---- scores of the wave's 16 rows t with all 64 rows s, transposed: tile rows s, columns t
    const int t = wave * 16 + li;              // the lane's row of the chunk as a column of the tiles
    // (its q as the second operand of every product comes straight from memory: no other wave needs it)
    Frag qf[DKP / 32];
#pragma unroll
    for (int ks = 0; ks < DKP / 32; ++ks) {
      const int e = ks * 32 + lc * 8;
      float qv[8];
#pragma unroll
      for (int x = 0; x < 8; ++x) qv[x] = 0.f;
      if (t < nc && e < dk) {
        unpack8f(load_frag(proj + (size_t)(r0 + t) * ld + (size_t)h * dk + e + q_off), qv);
        if (act) {
#pragma unroll
          for (int x = 0; x < 8; ++x) qv[x] = silu_f(qv[x]);
        }
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) qf[ks].w[w] = pack_bf16x2(qv[2 * w], qv[2 * w + 1]);
    }
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
      if (st <= wave) {                        // (tiles of later rows s hold nothing the rows t see)
#pragma unroll
        for (int ks = 0; ks < DKP / 32; ++ks) {
          const Frag kf = *reinterpret_cast<const Frag*>(Ks + (st * 16 + li) * QR + ks * 32 + lc * 8);
          acc = mfma16(kf, qf[ks], acc);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int s_ = st * 16 + lc * 4 + r;
          acc[r] = s_ <= t ? acc[r] * pw[t - s_] : 0.f;
        }
      }
      const int at = t * SR + st * 16 + lc * 4;
      store_split4(AsH + at, AsL + at, acc[0], acc[1], acc[2], acc[3]);
    }
    wave_lds_order();

    // ---- outputs of the wave's rows, transposed: tile rows value columns j, columns t
    const float from_state = pw[t + 1];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) {
      floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DKP / 32; ++ks) {
        const int at = (jt * 16 + li) * QR + ks * 32 + lc * 8;
        acc = mfma16(*reinterpret_cast<const Frag*>(StH + at), qf[ks], acc);
        acc = mfma16(*reinterpret_cast<const Frag*>(StL + at), qf[ks], acc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] *= from_state;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        if (kk * 32 > wave * 16 + 15) continue;
        const Frag vf = *reinterpret_cast<const Frag*>(Vt + (jt * 16 + li) * SR + kk * 32 + lc * 8);
        const int at = t * SR + kk * 32 + lc * 8;
        acc = mfma16(vf, *reinterpret_cast<const Frag*>(AsH + at), acc);
        acc = mfma16(vf, *reinterpret_cast<const Frag*>(AsL + at), acc);
      }
      const int j = j0 + jt * 16 + lc * 4;
      if (t < nc && j < dv)
        *reinterpret_cast<float4*>(out + (size_t)(r0 + t) * ldo + (size_t)h * dv + j) =
            float4{acc[0], acc[1], acc[2], acc[3]};
    }
  }
}

// Between the two: every element of a request's state walks its segment's chunks in order.  `ws` holds a chunk's
// contribution U_c on the way in and the state in front of the chunk on the way out: S <- lam^(rows of c) S + U_c.
// seg_chunks [segments][2]: a segment's first chunk and its chunks.
__global__ __launch_bounds__(256) void linear_attention_scan_kernel(float* __restrict__ ws, float* __restrict__ state,
                                                                    const float* __restrict__ powers,
                                                                    const int* __restrict__ seg_chunks,
                                                                    const int* __restrict__ seg_rows,
                                                                    const int* __restrict__ slots, int H, int dk,
                                                                    int dv) {
  const int seg = blockIdx.y, per_head = dk * dv;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= H * per_head) return;
  const int h = idx / per_head;
  const int first = seg_chunks[2 * seg], n = seg_chunks[2 * seg + 1], rows = seg_rows[seg];
  const float whole = powers[(size_t)h * (C + 1) + C], rest = powers[(size_t)h * (C + 1) + rows - (n - 1) * C];
  float* S = state + (size_t)slots[seg] * H * per_head + idx;
  float s = *S;
  for (int c = 0; c < n; ++c) {
    float* w = ws + (size_t)(first + c) * H * per_head + idx;
    const float u = *w;
    *w = s;
    s = fmaf(c + 1 < n ? whole : rest, s, u);
  }
  *S = s;
}

template <int DKP, int MODE>
constexpr size_t lds_bytes() {
  return (MODE == 1 ? (size_t)(VT * SR + 2 * DKP * SR) : (size_t)(VT * SR + C * (DKP + PAD) + 2 * C * SR + 2 * VT * (DKP + PAD))) * 2 +
         (C + 1) * 4;
}

// q and k of every row rotated by the row's position where they lie, k multiplied by k_scale behind the rotation:
// what the chunk kernels then read.  A thread takes 8 consecutive elements of a head; in the first half of the rotated
// range it takes its partner piece (rot / 2 further on) too, reads both and writes both; the thread of a piece in the
// second half does nothing.
__global__ __launch_bounds__(256) void linear_rotate_kernel(bf16_t* __restrict__ proj, int ld, int q_off, int k_off,
                                                            int H, int dk, int rot, const float* __restrict__ cos_sin,
                                                            const int* __restrict__ positions, float k_scale) {
  const int r = blockIdx.x, per = dk / 8, half = rot / 2;
  const int item = blockIdx.y * 256 + threadIdx.x;
  if (item >= 2 * H * per) return;
  const bool is_k = item >= H * per;
  const int it = is_k ? item - H * per : item, h = it / per, e = (it % per) * 8;
  bf16_t* head = proj + (size_t)r * ld + (is_k ? k_off : q_off) + (size_t)h * dk;
  const float sc = is_k ? k_scale : 1.f;
  float x[8], y[8];
  if (e >= rot) {
    if (sc != 1.f) {
      unpack8f(load_frag(head + e), x);
      Frag f;
#pragma unroll
      for (int i = 0; i < 4; ++i) f.w[i] = pack_bf16x2(x[2 * i] * sc, x[2 * i + 1] * sc);
      *reinterpret_cast<Frag*>(head + e) = f;
    }
    return;
  }
  if (e >= half) return;
  unpack8f(load_frag(head + e), x);
  unpack8f(load_frag(head + e + half), y);
  const float* cs = cos_sin + (size_t)positions[r] * rot;
  Frag fa, fb;
  float a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float c = cs[e + i], sn = cs[half + e + i];
    a[i] = (x[i] * c - y[i] * sn) * sc;
    b[i] = (y[i] * c + x[i] * sn) * sc;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    fa.w[i] = pack_bf16x2(a[2 * i], a[2 * i + 1]);
    fb.w[i] = pack_bf16x2(b[2 * i], b[2 * i + 1]);
  }
  *reinterpret_cast<Frag*>(head + e) = fa;
  *reinterpret_cast<Frag*>(head + e + half) = fb;
}

}  // namespace

// q and k heads of bfloat16 rows rotated (and k scaled) in place; rot a multiple of 16, dk and the offsets of 8.
APC_EXPORT int apc_linear_rotate_bf16(void* proj, int ld, int q_off, int k_off, int H, int dk, int rot,
                                      const float* cos_sin, const int* positions, float k_scale, int n_rows,
                                      hipStream_t stream) {
  if (n_rows <= 0 || (rot == 0 && k_scale == 1.f)) return 0;
  if (H <= 0 || dk <= 0 || rot < 0 || rot > dk || (rot && (!cos_sin || !positions))) return APC_ERR_BAD_ARG;
  if (dk % 8 || rot % 16 || ld % 8 || q_off % 8 || k_off % 8 || ((uintptr_t)proj & 15u)) return APC_ERR_UNSUPPORTED;
  const int items = 2 * H * (dk / 8);
  if (ceil_div(items, 256) > 65535) return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(linear_rotate_kernel, dim3(n_rows, ceil_div(items, 256)), dim3(256), 0, stream, (bf16_t*)proj, ld,
                     q_off, k_off, H, dk, rot, cos_sin, positions, k_scale);
  APC_LAUNCH_CHECK();
  return 0;
}

// 1 if the kernel takes these sizes, else 0 (the caller then runs the plain kernel)
APC_EXPORT int apc_linear_attention_bf16_takes(int ld, int q_off, int k_off, int v_off, int H, int dk, int dv) {
  if (H <= 0 || dk <= 0 || dv <= 0 || dk > 128 || dk % 8 || dv % 8 || ld % 8 || q_off % 8 || k_off % 8 || v_off % 8) return 0;
  return 1;
}

// powers: float32 [H][65], decay[h]^0 .. decay[h]^64 (rounded from double precision once, by the caller).
// chunks: int32 [n_chunks][2] (segment, first row of the chunk in it), all segments' chunks in order; seg_chunks: int32
// [n_segs][2] (a segment's first chunk, its chunks); ws: float32 [n_chunks][H][dk][dv].
APC_EXPORT int apc_linear_attention_bf16(const void* proj, int ld, int q_off, int k_off, int v_off, int H, int dk,
                                         int dv, int act, const float* powers, float* state, int n_segs,
                                         const int* seg_row0, const int* seg_rows, const int* slots, int n_chunks,
                                         const int* chunks, const int* seg_chunks, float* ws, float* out, int ldo,
                                         hipStream_t stream) {
  if (n_segs <= 0 || n_chunks <= 0) return 0;
  if (!apc_linear_attention_bf16_takes(ld, q_off, k_off, v_off, H, dk, dv)) return APC_ERR_UNSUPPORTED;
  if (!powers || !state || !slots || !chunks || !seg_chunks || !ws || ldo < H * dv || ldo % 4 ||
      ((uintptr_t)proj & 15u) || ((uintptr_t)out & 15u))
    return APC_ERR_BAD_ARG;
  dim3 grid(n_chunks, H, ceil_div(dv, VT));
  if (H > 65535 || grid.z > 65535 || n_segs > 65535) return APC_ERR_UNSUPPORTED;
#define LAC_LAUNCH(DKP_, MODE_)                                                                                     \
  do {                                                                                                              \
    static bool set_ = false;                                                                                       \
    if (!set_) {                                                                                                    \
      hipError_t e_ = hipFuncSetAttribute(                                                                          \
          reinterpret_cast<const void*>(&linear_attention_chunk_kernel<DKP_, MODE_>),                               \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes<DKP_, MODE_>());                               \
      if (e_ != hipSuccess) return (int)e_;                                                                         \
      set_ = true;                                                                                                  \
    }                                                                                                               \
    hipLaunchKernelGGL((linear_attention_chunk_kernel<DKP_, MODE_>), grid, dim3(256), (lds_bytes<DKP_, MODE_>()),   \
                       stream, (const bf16_t*)proj, ld, q_off, k_off, v_off, H, dk, dv, act, powers, chunks, ws,    \
                       seg_row0, seg_rows, out, ldo);                                                               \
    APC_LAUNCH_CHECK();                                                                                             \
  } while (0)
  if (dk <= 64) LAC_LAUNCH(64, 1);
  else LAC_LAUNCH(128, 1);
  hipLaunchKernelGGL(linear_attention_scan_kernel, dim3(ceil_div(H * dk * dv, 256), n_segs), dim3(256), 0, stream, ws,
                     state, powers, seg_chunks, seg_rows, slots, H, dk, dv);
  APC_LAUNCH_CHECK();
  if (dk <= 64) LAC_LAUNCH(64, 2);
  else LAC_LAUNCH(128, 2);
#undef LAC_LAUNCH
  return 0;
}
