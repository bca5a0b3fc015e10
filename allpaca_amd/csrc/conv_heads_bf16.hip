// The short convolution on the heads of projected rows (see plain_mixers.hip for the formulas) for bfloat16 rows, 16
// bytes a thread: a block takes 8 or 4 consecutive rows whole, a thread PPT pieces of 8 channels of each, with the taps of
// its channels in registers.  Sums of squares of the pieces go through LDS, so a head may be any multiple of 8 wide,
// and so may the width the norm is taken over (`norm_dim`, which divides a head; the normed values are multiplied with
// q_norm_w / k_norm_w [norm_dim] if given).
// `norm_rows`: the norm is taken over all heads of q (of k) at once, with weights of the projection's size; the
// pieces' sums of a row are added by one wave for q and one for k.  `qt_every` > 0: q of the row at position p is
// multiplied by 1 + qt_coef * ln(floor((p + 1) / qt_every) + 1).
// The row holds q heads, then k heads, then v heads.  The state of the convolution is moved on by the plain kernel,
// or here (`fold_state`) in a step of few rows in which every segment is a single row (decoded tokens).
#include "mfma.h"
#include <math.h>

namespace {

constexpr int MAXT = 4;   // taps

__device__ __forceinline__ void unpack8(const Frag& f, float* v) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    v[2 * w] = __uint_as_float(f.w[w] << 16);
    v[2 * w + 1] = __uint_as_float(f.w[w] & 0xffff0000u);
  }
}

template <int NT, int PPT, int ROWS, int TAPS>
__global__ __launch_bounds__(NT) void conv_heads_bf16_kernel(
    const bf16_t* __restrict__ proj, int ld, int n_rows, int H, int G, int dk, int dv, const float* __restrict__ bias,
    const float* __restrict__ conv_w, float* __restrict__ state, int fold_state, int width,
    const int* __restrict__ row_seg, const int* __restrict__ seg_row0, const int* __restrict__ slots,
    const int* __restrict__ positions, int unit_norm, float eps, int norm_dim, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, int norm_rows, float qt_coef, int qt_every, bf16_t* __restrict__ q_out, int ldq,
    const int* __restrict__ block_table, int max_blocks, bf16_t* __restrict__ cache, int P) {
  extern __shared__ float ssum[];            // [ROWS][pieces], then [ROWS][2] (the sums over all of q and all of k)
  constexpr int taps = TAPS;
  const int tid = threadIdx.x;
  const int pieces = width / 8;
  const int r0 = blockIdx.x * ROWS;
  int seg[ROWS], in_seg[ROWS];
  const float* st[ROWS];
#pragma unroll
  for (int rr = 0; rr < ROWS; ++rr) {
    const int r = min(r0 + rr, n_rows - 1);
    seg[rr] = row_seg[r];
    in_seg[rr] = r - seg_row0[seg[rr]];
    st[rr] = taps > 1 ? state + (size_t)slots[seg[rr]] * (taps - 1) * width : nullptr;
  }
  bool block_all_in = r0 >= TAPS - 1;
#pragma unroll
  for (int rr = 0; rr < ROWS; ++rr) block_all_in = block_all_in && in_seg[rr] >= TAPS - 1;
  float y[PPT][ROWS][8];
#pragma unroll
  for (int k = 0; k < PPT; ++k) {
    const int p = tid + NT * k;
    if (p >= pieces) continue;
    const int c0 = p * 8;
    float b[8], w[8 * TAPS];                         // w[e * TAPS + j], as the taps lie in memory
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = 0.f;
    if (bias) {
      const float4 a = *reinterpret_cast<const float4*>(bias + c0), c = *reinterpret_cast<const float4*>(bias + c0 + 4);
      b[0] = a.x; b[1] = a.y; b[2] = a.z; b[3] = a.w; b[4] = c.x; b[5] = c.y; b[6] = c.z; b[7] = c.w;
    }
    if (conv_w) {
#pragma unroll
      for (int i = 0; i < 2 * TAPS; ++i) {
        const float4 a = *reinterpret_cast<const float4*>(conv_w + (size_t)c0 * TAPS + 4 * i);
        w[4 * i] = a.x; w[4 * i + 1] = a.y; w[4 * i + 2] = a.z; w[4 * i + 3] = a.w;
      }
    } else {                                         // no convolution (one tap of 1)
#pragma unroll
      for (int i = 0; i < 8 * TAPS; ++i) w[i] = 1.f;
    }
    // The rows' inputs are asked for together and used afterwards, so the loads are in flight at once.  When every row
    // of the block has its TAPS - 1 predecessors in its own segment (all but the first rows of a prompt portion), the
    // ROWS + TAPS - 1 rows from r0 - (TAPS - 1) on serve all of them.
    if (block_all_in) {
      Frag src[ROWS + TAPS - 1];
#pragma unroll
      for (int i = 0; i < ROWS + TAPS - 1; ++i)
        src[i] = load_frag(proj + (size_t)min(r0 - (TAPS - 1) + i, n_rows - 1) * ld + c0);
#pragma unroll
      for (int rr = 0; rr < ROWS; ++rr) {
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {               // oldest first, as the plain kernel adds
          float u[8];
          unpack8(src[rr + j], u);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = fmaf(w[e * TAPS + j], u[e] + b[e], acc[e]);
        }
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { y[k][rr][e] = acc[e]; ss = fmaf(acc[e], acc[e], ss); }
        ssum[rr * pieces + p] = ss;
      }
    } else {
#pragma unroll
      for (int rr = 0; rr < ROWS; ++rr) {
        const int r = min(r0 + rr, n_rows - 1);
        Frag raw[TAPS];
        float4 sa[TAPS], sb[TAPS];
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
          const int back = TAPS - 1 - j;
          if (back <= in_seg[rr]) {
            raw[j] = load_frag(proj + (size_t)(r - back) * ld + c0);
          } else {
            const float* sp = st[rr] + (size_t)(TAPS - 1 - (back - in_seg[rr])) * width + c0;
            sa[j] = *reinterpret_cast<const float4*>(sp);
            sb[j] = *reinterpret_cast<const float4*>(sp + 4);
          }
        }
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
          const int back = TAPS - 1 - j;
          float u[8];
          if (back <= in_seg[rr]) {
            unpack8(raw[j], u);
#pragma unroll
            for (int e = 0; e < 8; ++e) u[e] += b[e];
          } else {
            u[0] = sa[j].x; u[1] = sa[j].y; u[2] = sa[j].z; u[3] = sa[j].w;
            u[4] = sb[j].x; u[5] = sb[j].y; u[6] = sb[j].z; u[7] = sb[j].w;
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = fmaf(w[e * TAPS + j], u[e], acc[e]);
          // A step in which every segment is one row: the row's state moves on here (this thread alone reads and
          // writes these channels of the row's slot, and it has read them all): rows 1 .. of the old state become
          // rows 0 .., the row's own input the last.
          if (TAPS > 1 && fold_state && r0 + rr < n_rows && j >= 1) {
            float* sp = state + ((size_t)slots[seg[rr]] * (TAPS - 1) + (j - 1)) * width + c0;
            *reinterpret_cast<float4*>(sp) = float4{u[0], u[1], u[2], u[3]};
            *reinterpret_cast<float4*>(sp + 4) = float4{u[4], u[5], u[6], u[7]};
          }
        }
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { y[k][rr][e] = acc[e]; ss = fmaf(acc[e], acc[e], ss); }
        ssum[rr * pieces + p] = ss;
      }
    }
  }
  __syncthreads();
  const int kq = H * dk, kk = (H + G) * dk;
  float* totals = ssum + ROWS * pieces;
  if (norm_rows) {
    // wave w adds the pieces of (row, q or k) number w, w + waves, ..: an order that the sizes alone fix
    const int lane = tid % WAVE;
    for (int job = tid / WAVE; job < ROWS * 2; job += NT / WAVE) {
      const int rr = job / 2, first = (job % 2) ? kq / 8 : 0, n = (job % 2) ? (kk - kq) / 8 : kq / 8;
      float t = 0.f;
      for (int i = lane; i < n; i += WAVE) t += ssum[rr * pieces + first + i];
      t = wave_sum(t);
      if (lane == 0) totals[job] = t;
    }
    __syncthreads();
  }
#pragma unroll
  for (int k = 0; k < PPT; ++k) {
    const int p = tid + NT * k;
    if (p >= pieces) continue;
    const int c0 = p * 8;
    const int kind = c0 < kq ? 0 : c0 < kk ? 1 : 2;
    const int d = kind == 2 ? dv : dk;
    const int rel = c0 - (kind == 0 ? 0 : kind == 1 ? kq : kk);
    const int head = rel / d, off = rel % d;
    // the piece's place in the range its norm is taken over (and in that range's weights)
    const int noff = norm_rows ? rel : off % norm_dim;
    float nw[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) nw[e] = 1.f;
    const float* nwp = kind == 0 ? q_norm_w : kind == 1 ? k_norm_w : nullptr;
    if (nwp) {
      const float4 a = *reinterpret_cast<const float4*>(nwp + noff), c = *reinterpret_cast<const float4*>(nwp + noff + 4);
      nw[0] = a.x; nw[1] = a.y; nw[2] = a.z; nw[3] = a.w; nw[4] = c.x; nw[5] = c.y; nw[6] = c.z; nw[7] = c.w;
    }
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
      const int r = r0 + rr;
      if (r >= n_rows) continue;
      float inv = 1.f;
      if (unit_norm && kind != 2 && norm_rows) {
        inv = 1.0f / sqrtf(totals[rr * 2 + kind] / (float)(kind == 0 ? kq : kk - kq) + eps);
      } else if (unit_norm && kind != 2) {
        const float* sp = ssum + rr * pieces + (c0 - noff) / 8;
        float ss = 0.f;
        for (int i = 0; i < norm_dim / 8; ++i) ss += sp[i];
        inv = 1.0f / sqrtf(ss / (float)norm_dim + eps);
      }
      if (kind == 0 && qt_every > 0)      // (behind the weights in the plain kernel; a product of three either way)
        inv *= 1.0f + qt_coef * logf((float)((positions[r] + 1) / qt_every) + 1.0f);
      Frag o;
#pragma unroll
      for (int wd = 0; wd < 4; ++wd)
        o.w[wd] = pack_bf16x2((y[k][rr][2 * wd] * inv) * nw[2 * wd], (y[k][rr][2 * wd + 1] * inv) * nw[2 * wd + 1]);
      if (kind == 0) {
        *reinterpret_cast<Frag*>(q_out + (size_t)r * ldq + c0) = o;
        continue;
      }
      const int pos = positions[r];
      const int page = block_table[(size_t)seg[rr] * max_blocks + pos / P];
      bf16_t* base = cache + ((size_t)page * G + head) * (size_t)P * (dk + dv);
      if (kind == 1) {
        *reinterpret_cast<Frag*>(base + (size_t)(pos % P) * dk + off) = o;
      } else {
        bf16_t* vp = base + (size_t)P * dk + (size_t)off * P + (pos % P);
#pragma unroll
        for (int e = 0; e < 8; ++e) vp[(size_t)e * P] = (bf16_t)((e & 1) ? (o.w[e / 2] >> 16) : (o.w[e / 2] & 0xffffu));
      }
    }
  }
}

}  // namespace

// 1 if the kernel takes these sizes (q, k and v heads side by side from column 0 on), else 0
APC_EXPORT int apc_conv_heads_bf16_takes(int ld, int width, int H, int G, int dk, int dv, int taps, int ldq) {
  if (H <= 0 || G < 0 || dk % 8 || (G && dv % 8) || taps < 1 || taps > MAXT || ld % 8 || ldq % 8) return 0;
  if (width != H * dk + G * (dk + dv) || width / 8 > 2 * 768) return 0;
  return 1;
}

APC_EXPORT int apc_conv_heads_bf16(const void* proj, int ld, int n_rows, int H, int G, int dk, int dv, const float* bias,
                                   const float* conv_w, int taps, float* state, int fold_state, int width, const int* row_seg,
                                   const int* seg_row0, const int* slots, const int* positions, int unit_norm, float eps,
                                   int norm_dim, const float* q_norm_w, const float* k_norm_w, int norm_rows,
                                   float qt_coef, int qt_every, void* q_out, int ldq, const int* block_table,
                                   int max_blocks, void* cache, int page_tokens, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!apc_conv_heads_bf16_takes(ld, width, H, G, dk, dv, taps, ldq)) return APC_ERR_UNSUPPORTED;
  if (((uintptr_t)proj & 15u) || ((uintptr_t)q_out & 15u) || ((uintptr_t)cache & 15u) || ((uintptr_t)state & 15u) ||
      ((uintptr_t)bias & 15u) || ((uintptr_t)conv_w & 15u))
    return APC_ERR_UNSUPPORTED;
  if (taps > 1 && (!conv_w || !state || !slots)) return APC_ERR_BAD_ARG;
  if (norm_dim <= 0) norm_dim = dk;
  if (dk % norm_dim || qt_every < 0 || (norm_rows && (!unit_norm || norm_dim != dk))) return APC_ERR_BAD_ARG;
  if (norm_dim % 8 || ((uintptr_t)q_norm_w & 15u) || ((uintptr_t)k_norm_w & 15u)) return APC_ERR_UNSUPPORTED;
  if (!conv_w && taps != 1) return APC_ERR_BAD_ARG;
  if (G > 0 && (!cache || !block_table || page_tokens <= 0 || max_blocks <= 0)) return APC_ERR_BAD_ARG;
  // A row's pieces of 8 channels are spread over up to 768 threads (a block of 1,024 would leave a thread too few
  // registers): a thread's pieces come one after the other, each with loads of its own to wait for.
  const int pieces = width / 8;
  const int nt = pieces <= 256 ? 256 : pieces <= 512 ? 512 : pieces <= 768 ? 768 : pieces <= 1024 ? 512 : 768;
  // (a thread keeps its channels' taps for all rows of the block: 8 rows where a thread has one piece, else 4; a step
  // of few rows, decoded ones, has a block a row: the rows of a block come one after the other)
  const bool few = n_rows <= 32 || fold_state;
  const int rows_a_block = few ? 1 : pieces <= 768 ? 8 : 4;
  dim3 grid((n_rows + rows_a_block - 1) / rows_a_block), block(nt);
  const size_t lds = (size_t)rows_a_block * (pieces + 2) * sizeof(float);
#define CH_LAUNCH(NT_, PPT_, ROWS_, TAPS_)                                                                          \
  hipLaunchKernelGGL((conv_heads_bf16_kernel<NT_, PPT_, ROWS_, TAPS_>), grid, block, lds, stream,                   \
                     (const bf16_t*)proj, ld, n_rows, H, G, dk, dv, bias, conv_w, state, fold_state, width, row_seg, seg_row0,  \
                     slots, positions, unit_norm, eps, norm_dim, q_norm_w, k_norm_w, norm_rows, qt_coef, qt_every, (bf16_t*)q_out, ldq, block_table, max_blocks, (bf16_t*)cache, \
                     page_tokens)
#define CH_TAPS(NT_, PPT_, ROWS_)                            \
  do {                                                       \
    if (taps == 1) CH_LAUNCH(NT_, PPT_, ROWS_, 1);           \
    else if (taps == 2) CH_LAUNCH(NT_, PPT_, ROWS_, 2);      \
    else if (taps == 3) CH_LAUNCH(NT_, PPT_, ROWS_, 3);      \
    else CH_LAUNCH(NT_, PPT_, ROWS_, 4);                     \
  } while (0)
#define CH_ROWS(NT_, PPT_, ROWS_)            \
  do {                                       \
    if (few) CH_TAPS(NT_, PPT_, 1);          \
    else CH_TAPS(NT_, PPT_, ROWS_);          \
  } while (0)
  if (pieces <= 256) CH_ROWS(256, 1, 8);
  else if (pieces <= 512) CH_ROWS(512, 1, 8);
  else if (pieces <= 768) CH_ROWS(768, 1, 8);
  else if (pieces <= 1024) CH_ROWS(512, 2, 4);
  else CH_ROWS(768, 2, 4);
#undef CH_ROWS
#undef CH_TAPS
#undef CH_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}
