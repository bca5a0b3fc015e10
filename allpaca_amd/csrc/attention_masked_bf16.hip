// Attention with a mask of chunks or a sliding window, an optional sink, and keys and values of different sizes, in
// bfloat16 on MFMA with float32 softmax.
//
//   the row at position p sees keys lo(p) .. p:  lo = 0 (causal), max(0, p - n + 1) (window of n), p - p % n (chunks of
//   n positions counted from position 0);  s = (q . k) * scale;  weights exp(s) / (sink + sum exp(s)), sink = 1 (a key
//   of score 0 without a value) or 0;  query head h reads kv head h / (H / G).
//
// `key_parts` = M > 1: a cached key of dk elements is M keys of dk / M side by side, one for each of M softmax maps over
// the same values; q holds H heads of dk / M, head j uses part j % M of the keys (M consecutive heads are the maps of
// one head).  The kernels keep the whole key as the summed axis and give a head's query zeros outside its own part, so
// nothing else changes; `out_f32`: the heads' outputs leave in float32 (for a caller that combines the maps).
//
// `softcap` c > 0: s <- c * tanh(s / c).  `r1`, `r2` [H]: s <- s - r1[h] * ln(1 + r2[h] * (p - t)) for the key at
// position t, a learned penalty on the distance (behind the cap).  Both are applied to the float32 scores where they
// leave the first product, ahead of the maximum; a launch without them runs as before.
//
// Pages: one row per kv head, first the page's keys [slot][dk], then its values [dv][slot]; a page is
// G * P * (dk + dv) elements.
//
//   prompt portions  a block of 4 waves takes up to 64 consecutive rows of one request x one head, 16 rows a wave on
//                    v_mfma_f32_16x16x32_bf16; keys and values in tiles of 64 through LDS; online softmax whose running
//                    maximum starts at the sink's score.  The products are transposed (S^T = K Q^T, O^T = V^T P^T), as
//                    in attention_bf16.hip, so a row's maximum and sum are registers of 4 lanes.
//   decoded rows     one row x one kv head x one range of its keys a block; the query heads of the group are the 16
//                    columns of an MFMA tile, so keys and values are read once a group, straight from the pages into
//                    the operands.  A second kernel adds the ranges and the sink.
#include "mfma.h"
#include <math.h>

namespace {

constexpr int KT = 64;
constexpr int QT = 64;
constexpr int KPAD = 8;
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ int first_seen(int pos, int mask, int size) {
  if (mask == 1) return pos - size + 1 > 0 ? pos - size + 1 : 0;
  if (mask == 2) return pos - pos % size;
  return 0;
}
__device__ __forceinline__ float row4_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, WAVE));
  return fmaxf(v, __shfl_xor(v, 32, WAVE));
}
__device__ __forceinline__ float row4_sum(float v) {
  v += __shfl_xor(v, 16, WAVE);
  return v + __shfl_xor(v, 32, WAVE);
}
// all but the positions lo <= p < hi of a value operand's 8 are cleared (what lies there may be anything, and
// 0 x NaN is NaN)
__device__ __forceinline__ void keep_positions(Frag& v, int lo, int hi) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t a = (2 * w >= lo && 2 * w < hi) ? 0x0000ffffu : 0u;
    const uint32_t b = (2 * w + 1 >= lo && 2 * w + 1 < hi) ? 0xffff0000u : 0u;
    v.w[w] &= a | b;
  }
}
__device__ __forceinline__ float exp2_neg(float x) { return __builtin_amdgcn_exp2f(x); }
// A product q . k through the scale, the soft cap and the distance penalty, in units of `unit` (1: natural, log2(e):
// the exponent's base 2), with the constants folded by the caller:
//   no cap:  dot * mul;                      mul = scale * unit
//   cap c:   out * tanh(dot * scale / c) = out * (1 - 2 / (2^(dot * in) + 1));   in = 2 log2(e) scale / c, out = c * unit
//   penalty: less pen * log2(1 + r2 * d);    pen = r1 * ln 2 * unit  (d: how far back the key lies, not negative)
struct ScoreShape {
  float mul, in, out, pen, r2;
  bool capped, penalty;
};
__device__ __forceinline__ ScoreShape score_shape(float scale, float cap, const float* r1, const float* r2, int head,
                                                  float unit) {
  ScoreShape f;
  f.capped = cap > 0.f;
  f.penalty = r1 != nullptr;
  f.mul = scale * unit;
  f.in = f.capped ? 2.0f * LOG2E * scale / cap : 0.f;
  f.out = cap * unit;
  f.pen = f.penalty ? r1[head] * 0.6931471805599453f * unit : 0.f;
  f.r2 = f.penalty ? r2[head] : 0.f;
  return f;
}
__device__ __forceinline__ float shape_score(float dot, const ScoreShape& f, int d) {
  float v = dot * f.mul;
  if (f.capped) v = f.out * (1.0f - 2.0f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(dot * f.in) + 1.0f));
  if (f.penalty) v = fmaf(-f.pen, __log2f(fmaf(f.r2, (float)d, 1.0f)), v);
  return v;
}

// ------------------------------------------------------------------------------------------ prompt portions
template <int DKP, int DVP>  // key and value sizes rounded up to a multiple of 32
__global__ __launch_bounds__(256) void attn_masked_prefill_kernel(
    const bf16_t* __restrict__ q, int ldq, void* __restrict__ out, int ldo, int H, int G, int dk, int dv,
    const bf16_t* __restrict__ cache, int P, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ row_seg, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, int n_tiles, int mask, int mask_size, int sink, const float* __restrict__ sinks,
    const float* __restrict__ gate, int ldg, float scale, int key_parts, int out_f32, float softcap,
    const float* __restrict__ r1, const float* __restrict__ r2) {
  constexpr int KROW = DKP + (DKP % 128 == 0 ? 72 : DKP % 128 == 64 ? 8 : DKP % 128 == 32 ? 40 : 104);
  __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KROW];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[DVP * (KT + KPAD)];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4 * 16 * (KT + KPAD)];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int li = lane % 16, lc = lane / 16;
  // all heads that read one kv head run on one XCD (blocks go to the 8 XCDs in turn), tiles from the last to the first
  int tile, h;
  {
    const int id = blockIdx.x, per = H / G;
    if (G % 8 == 0) {
      const int xcd = id % 8, slot = id / 8;
      const int lh = slot / n_tiles;
      tile = n_tiles - 1 - slot % n_tiles;
      h = (xcd + 8 * (lh / per)) * per + lh % per;
    } else {
      tile = n_tiles - 1 - id % n_tiles;
      h = id / n_tiles;
    }
  }
  // the step's tiles have up to 2 QT rows; this kernel takes them in halves (n_tiles counts halves)
  const int nrows = min(tile_rows[tile / 2] - (tile % 2) * QT, QT);
  if (nrows <= 0) return;
  const int row0 = tile_row0[tile / 2] + (tile % 2) * QT;
  const int g = h / (H / G);
  const int pos0 = positions[row0];
  const int* bt = block_table + (size_t)row_seg[row0] * max_blocks;
  const int last = pos0 + nrows - 1;
  const int first = first_seen(pos0, mask, mask_size);   // the smallest of the rows' first keys
  const size_t page_stride = (size_t)G * P * (dk + dv);
  const int dchunks = dk / 8;

  for (int idx = tid; idx < KT * KROW; idx += 256) Ks[idx] = 0;
  for (int idx = tid; idx < DVP * (KT + KPAD); idx += 256) Vs[idx] = 0;

  const int my_row = wave * 16 + li;
  Frag qf[DKP / 32];
  {
    const int dq = dk / key_parts, part0 = (h % key_parts) * dq;     // the head's own part of a key
    const bf16_t* qrow = q + (size_t)(row0 + min(my_row, nrows - 1)) * ldq + (size_t)h * dq;
#pragma unroll
    for (int ks = 0; ks < DKP / 32; ++ks) {
      const int e = ks * 32 + lc * 8;
      qf[ks] = (my_row < nrows && e >= part0 && e < part0 + dq) ? load_frag(qrow + (e - part0)) : zero_frag();
    }
  }
  const int my_pos = pos0 + my_row;
  const int my_lo = first_seen(my_pos, mask, mask_size);
  const int wave_hi = pos0 + wave * 16;                        // smallest position of the wave's rows
  const int wave_lo = first_seen(wave_hi + 15, mask, mask_size);  // largest first key of the wave's rows
  const bool shaped = softcap > 0.f || r1 != nullptr;       // scores are then finished (in base 2) before the maximum
  const ScoreShape shape = score_shape(scale, softcap, r1, r2, h, LOG2E);
  const float sc2 = shaped ? 1.f : scale * LOG2E;
  floatx4 o[DVP / 16];
#pragma unroll
  for (int dt = 0; dt < DVP / 16; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the sink is the row's first "key": its score (0, or the head's learned one; in the exponent's base 2)
  float m_run = sink ? (sinks ? sinks[h] * LOG2E : 0.f) : -INFINITY, l_run = sink ? 1.f : 0.f;
  bf16_t* pw = Ps + wave * 16 * (KT + KPAD) + li * (KT + KPAD);
  const bf16_t* krd = Ks + li * KROW + lc * 8;
  const bf16_t* vrd = Vs + li * (KT + KPAD) + lc * 8;

  // A tile is 8 groups of 8 consecutive keys, a group lies in one page; the 32 threads of group tid / 32 copy its keys
  // (8 x dk elements, consecutive in the page) and its values (dv rows of 8 slots).
  constexpr int KP = DKP / 32, VP = DVP / 32;
  const int grp = tid / 32, gl = tid % 32;
  const int last_group = (last / 8) * 8;
  int k_ldst[KP], v_ldst[VP];
  bool k_on[KP], v_on[VP];
#pragma unroll
  for (int j = 0; j < KP; ++j) {
    const int idx = gl + 32 * j;
    k_on[j] = idx < dk;
    const int key = k_on[j] ? idx / dchunks : 0, ch = k_on[j] ? idx % dchunks : 0;
    k_ldst[j] = (grp * 8 + key) * KROW + ch * 8;
  }
#pragma unroll
  for (int j = 0; j < VP; ++j) {
    const int idx = gl + 32 * j;
    v_on[j] = idx < dv;
    v_ldst[j] = (v_on[j] ? idx : 0) * (KT + KPAD) + grp * 8;
  }
  const bf16_t* k_head = cache + (size_t)g * P * (dk + dv);
  const bf16_t* v_head = k_head + (size_t)P * dk;
  int page_next = 0;
  auto lookup_tile = [&](int t0) { page_next = bt[min(t0 + grp * 8, last_group) / P]; };
  Frag kreg[KP], vreg[VP];
  int v_lo = 0, v_hi = 8;
  auto load_tile = [&](int t0) {
    const int tg = min(t0 + grp * 8, last_group), slot0 = tg % P;
    v_lo = first - tg;
    v_hi = last - tg + 1;
    const bf16_t* kp = k_head + (size_t)page_next * page_stride + (size_t)slot0 * dk;
    const bf16_t* vp = v_head + (size_t)page_next * page_stride + slot0;
#pragma unroll
    for (int j = 0; j < KP; ++j) kreg[j] = load_frag(kp + (k_on[j] ? gl + 32 * j : 0) * 8);
#pragma unroll
    for (int j = 0; j < VP; ++j) vreg[j] = load_frag(vp + (size_t)(v_on[j] ? gl + 32 * j : 0) * P);
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < KP; ++j)
      if (k_on[j]) *reinterpret_cast<Frag*>(Ks + k_ldst[j]) = kreg[j];
#pragma unroll
    for (int j = 0; j < VP; ++j) {
      if (v_on[j]) {
        if (v_lo > 0 || v_hi < 8) keep_positions(vreg[j], v_lo, v_hi);
        *reinterpret_cast<Frag*>(Vs + v_ldst[j]) = vreg[j];
      }
    }
  };

  const int t_begin = (first / KT) * KT;
  lookup_tile(t_begin);
  load_tile(t_begin);
  lookup_tile(t_begin + KT);
  __syncthreads();
  store_tile();
  __syncthreads();
  for (int t0 = t_begin; t0 <= last; t0 += KT) {
    load_tile(t0 + KT);
    lookup_tile(t0 + 2 * KT);

    floatx4 s[KT / 16];
#pragma unroll
    for (int nt = 0; nt < KT / 16; ++nt) {
      s[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DKP / 32; ++ks) {
        const Frag kf = *reinterpret_cast<const Frag*>(krd + nt * 16 * KROW + ks * 32);
        s[nt] = mfma16(kf, qf[ks], s[nt]);
      }
    }
    if (shaped) {
#pragma unroll
      for (int nt = 0; nt < KT / 16; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int d = my_pos - (t0 + nt * 16 + lc * 4 + r);
          s[nt][r] = shape_score(s[nt][r], shape, d > 0 ? d : 0);
        }
    }
    float mx = -INFINITY;
    if (t0 >= wave_lo && t0 + KT - 1 <= wave_hi) {
#pragma unroll
      for (int nt = 0; nt < KT / 16; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[nt][r]);
    } else {
#pragma unroll
      for (int nt = 0; nt < KT / 16; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int t = t0 + nt * 16 + lc * 4 + r;
          const float v = (t >= my_lo && t <= my_pos) ? s[nt][r] : -INFINITY;
          s[nt][r] = v;
          mx = fmaxf(mx, v);
        }
    }
    mx = row4_max(mx) * sc2;
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2_neg(m_run - m_safe);
    float sum = 0.f;
#pragma unroll
    for (int nt = 0; nt < KT / 16; ++nt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[nt][r] = exp2_neg(fmaf(s[nt][r], sc2, -m_safe));
        sum += s[nt][r];
      }
      uint2 pk;
      pk.x = pack_bf16x2(s[nt][0], s[nt][1]);
      pk.y = pack_bf16x2(s[nt][2], s[nt][3]);
      *reinterpret_cast<uint2*>(pw + nt * 16 + lc * 4) = pk;
    }
    l_run = l_run * alpha + row4_sum(sum);
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < DVP / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
    }
    wave_lds_order();
#pragma unroll
    for (int kstep = 0; kstep < KT / 32; ++kstep) {
      const Frag pf = *reinterpret_cast<const Frag*>(pw + kstep * 32 + lc * 8);
#pragma unroll
      for (int dt = 0; dt < DVP / 16; ++dt) {
        const Frag vf = *reinterpret_cast<const Frag*>(vrd + dt * 16 * (KT + KPAD) + kstep * 32);
        o[dt] = mfma16(vf, pf, o[dt]);
      }
    }
    __syncthreads();
    store_tile();
    __syncthreads();
  }
  if (my_row < nrows) {
    float inv = 1.0f / l_run;
    if (gate) inv *= 1.0f / (1.0f + __expf(-gate[(size_t)(row0 + my_row) * ldg + h]));
    const size_t at = (size_t)(row0 + my_row) * ldo + (size_t)h * dv;
    bf16_t* orow = (bf16_t*)out + at;
#pragma unroll
    for (int dt = 0; dt < DVP / 16; ++dt) {
      const int e = dt * 16 + lc * 4;
      if (e < dv && out_f32) {
        *reinterpret_cast<float4*>((float*)out + at + e) =
            float4{o[dt][0] * inv, o[dt][1] * inv, o[dt][2] * inv, o[dt][3] * inv};
      } else if (e < dv) {
        uint2 pk;
        pk.x = pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv);
        pk.y = pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv);
        *reinterpret_cast<uint2*>(orow + e) = pk;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------ decoded rows
constexpr int DT = 256;       // keys of a block's pass: 64 a wave
constexpr int DMAX = 256;     // largest key and value size
constexpr int HGMAX = 16;     // query heads of a kv head: the 16 columns of an MFMA tile
constexpr int SROW = 64 + 4;  // floats of a row of a wave's scores in LDS (heads then fall into different banks)
constexpr int PROW = 64 + 8;  // bfloat16 of a row of a wave's weights in LDS
constexpr int NW = DT / WAVE;

// grid: rows x G x n_splits, 4 waves a block.  Split s of a row takes the keys at positions a0 + s * kps ..
// a0 + (s + 1) * kps - 1 that the row sees, a0 being the row's first key rounded down to a multiple of 256 and kps the
// multiple of 256 that spreads this row's keys over the splits (pages are powers of two up to 256, so 8 consecutive positions from a multiple of 8 on lie in one
// page); of every 256 of them wave w takes keys 64 w .. 64 w + 63.  A wave works for itself, with a running maximum
// and sum of its own, and no wave waits for another until the end, where the block's 4 add up through LDS: the block
// leaves, per query head of the group, the maximum score m, sum exp(s - m) and sum exp(s - m) v of its keys in
// `parts` [row][head][split][2 + dv].
// 64 keys: scores with all heads of the group as S = K Q^T (keys as the rows of 4 tiles, straight from the pages into
// the operand), maxima and sums with a key a lane, weights to LDS in bfloat16, then O^T += V^T P^T over the 64 keys for
// every 16 value elements (8 slots of an element a lane, straight from the pages).
template <int KS, int ET>  // 32-element steps over a key; tiles of 16 value elements
__global__ __launch_bounds__(DT) void attn_masked_decode_kernel(
    const bf16_t* __restrict__ q, int ldq, int H, int G, int dk, int dv, const bf16_t* __restrict__ cache, int P,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ positions,
    const int* __restrict__ row_seg, const int* __restrict__ rows, int mask, int mask_size, float scale, int n_splits,
    float* __restrict__ parts, int key_parts, float softcap, const float* __restrict__ r1,
    const float* __restrict__ r2) {
  __shared__ __attribute__((aligned(16))) float sc_all[NW][HGMAX * SROW];
  __shared__ __attribute__((aligned(16))) bf16_t ps_all[NW][HGMAX * PROW];
  __shared__ float ml_all[NW][HGMAX][3];        // running maximum, running sum, the last pass's factor
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int li = lane % 16, lc = lane / 16;
  float* sc = sc_all[wave];
  bf16_t* ps = ps_all[wave];
  float(*ml)[3] = ml_all[wave];
  const int split = blockIdx.x % n_splits, g = (blockIdx.x / n_splits) % G, ri = blockIdx.x / (n_splits * G);
  const int r = rows ? rows[ri] : ri;
  const int per = H / G;                        // query heads of this kv head (<= HGMAX)
  const int pos = positions[r];
  const int first = first_seen(pos, mask, mask_size);
  const int a0 = (first / DT) * DT;
  const int* bt = block_table + (size_t)row_seg[r] * max_blocks;
  const size_t page_stride = (size_t)G * P * (dk + dv);
  const bf16_t* head = cache + (size_t)g * P * (dk + dv);

  // the heads' queries as the second operand: column li = head, 8 elements from (ks * 32 + lc * 8) on
  Frag qf[KS];
  const int dq = dk / key_parts, part0 = (li % key_parts) * dq;      // (per is a multiple of key_parts)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int c = ks * 32 + lc * 8;
    qf[ks] = (li < per && c >= part0 && c < part0 + dq)
                 ? load_frag(q + (size_t)r * ldq + (size_t)(g * per + li) * dq + (c - part0)) : zero_frag();
  }
  const bool shaped = softcap > 0.f || r1 != nullptr;
  const ScoreShape shape = score_shape(scale, softcap, r1, r2, g * per + (li < per ? li : 0), 1.0f);
  for (int idx = lane; idx < HGMAX * PROW; idx += WAVE) ps[idx] = 0;    // rows of heads that do not exist stay 0
  if (lane < HGMAX) { ml[lane][0] = -INFINITY; ml[lane][1] = 0.f; ml[lane][2] = 1.f; }
  floatx4 o[ET];
#pragma unroll
  for (int i = 0; i < ET; ++i) o[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  wave_lds_order();

  // the row's own keys in n_splits ranges of whole passes: a step's rows differ in length, and the launch is made for
  // the longest the step may hold
  const int row_passes = (pos + 1 - a0 + DT - 1) / DT;
  const int kps = (row_passes + n_splits - 1) / n_splits * DT;
  const int lo_t = a0 + split * kps;
  const int hi_t = min(lo_t + kps, pos + 1);
  for (int t0 = lo_t + wave * WAVE; t0 < hi_t; t0 += DT) {
    if (t0 + WAVE <= first) continue;           // (only in front of the row's first key)
    // ---- scores of keys t0 .. t0 + 63: 4 tiles of 16 keys
    {
      Frag kf[4][KS];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        const int t = t0 + tt * 16 + li;
        const bool seen = t >= first && t <= pos;
        const bf16_t* kp = head + (size_t)(seen ? bt[t / P] : 0) * page_stride + (size_t)(t % P) * dk;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int c = ks * 32 + lc * 8;
          kf[tt][ks] = (seen && c < dk) ? load_frag_once(kp + c) : zero_frag();
        }
      }
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) acc = mfma16(kf[tt][ks], qf[ks], acc);
        // lane: keys tt * 16 + lc * 4 + 0..3 of the 64, head li
        float4 sv = float4{acc[0] * scale, acc[1] * scale, acc[2] * scale, acc[3] * scale};
        if (shaped) {
          const int d0 = pos - (t0 + tt * 16 + lc * 4);       // how far back the first of the four keys lies
          sv.x = shape_score(acc[0], shape, d0 > 0 ? d0 : 0);
          sv.y = shape_score(acc[1], shape, d0 > 1 ? d0 - 1 : 0);
          sv.z = shape_score(acc[2], shape, d0 > 2 ? d0 - 2 : 0);
          sv.w = shape_score(acc[3], shape, d0 > 3 ? d0 - 3 : 0);
        }
        *reinterpret_cast<float4*>(sc + li * SROW + tt * 16 + lc * 4) = sv;
      }
    }
    // ---- the value pieces are asked for now: they do not wait for the weights
    Frag vf[ET][2];
#pragma unroll
    for (int i = 0; i < ET; ++i) {
      const int e = i * 16 + li;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const int tp = t0 + kk * 32 + lc * 8;
        if (e < dv && tp <= pos && tp + 8 > first) {
          vf[i][kk] = load_frag_once(head + (size_t)bt[tp / P] * page_stride + (size_t)P * dk + (size_t)e * P + tp % P);
          if (tp < first || tp + 8 > pos + 1) keep_positions(vf[i][kk], first - tp, pos - tp + 1);
        } else {
          vf[i][kk] = zero_frag();
        }
      }
    }
    wave_lds_order();
    // ---- softmax, a key a lane
    const int t = t0 + lane;
    const bool valid = t >= first && t <= pos;
    for (int j = 0; j < per; ++j) {
      const float s = valid ? sc[j * SROW + lane] : -INFINITY;
      const float m_old = ml[j][0], l_old = ml[j][1];
      const float m_new = fmaxf(m_old, wave_max(s));   // finite: the 64 keys hold one the row sees
      const float alpha = __expf(m_old - m_new);
      const float p = valid ? __expf(s - m_new) : 0.f;
      ps[j * PROW + lane] = float_to_bf16(p);
      const float l_new = l_old * alpha + wave_sum(p);
      wave_lds_order();                           // every lane has read the old values
      if (lane == 0) { ml[j][0] = m_new; ml[j][1] = l_new; ml[j][2] = alpha; }
    }
    wave_lds_order();
    // ---- values
    const float my_alpha = li < per ? ml[li][2] : 1.f;
    Frag pf[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) pf[kk] = *reinterpret_cast<const Frag*>(ps + li * PROW + kk * 32 + lc * 8);
#pragma unroll
    for (int i = 0; i < ET; ++i) {
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) o[i][rr] *= my_alpha;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) o[i] = mfma16(vf[i][kk], pf[kk], o[i]);
    }
    wave_lds_order();
  }
  // The block's 4 waves add up through LDS, 4 heads at a time, and leave one part.
  // lane: elements i * 16 + lc * 4 + 0..3 of head li
  constexpr int HR = 4;
  __shared__ __attribute__((aligned(16))) float ox[NW][HR][ET * 16];
  for (int j0 = 0; j0 < per; j0 += HR) {
    if (li >= j0 && li < j0 + HR) {
#pragma unroll
      for (int i = 0; i < ET; ++i)
        *reinterpret_cast<float4*>(&ox[wave][li - j0][i * 16 + lc * 4]) = float4{o[i][0], o[i][1], o[i][2], o[i][3]};
    }
    __syncthreads();
    const int nh = min(HR, per - j0);
    for (int idx = tid; idx < nh * dv; idx += DT) {
      const int jj = idx / dv, e = idx % dv, j = j0 + jj;
      float M = -INFINITY;
#pragma unroll
      for (int w = 0; w < NW; ++w) M = fmaxf(M, ml_all[w][j][0]);
      float a = 0.f, l = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float m = ml_all[w][j][0];
        const float f = m == -INFINITY ? 0.f : __expf(m - M);
        a = fmaf(f, ox[w][jj][e], a);
        l = fmaf(f, ml_all[w][j][1], l);
      }
      float* p = parts + (((size_t)ri * H + g * per + j) * n_splits + split) * (dv + 2);
      p[2 + e] = a;
      if (e == 0) { p[0] = M; p[1] = l; }
    }
    __syncthreads();
  }
}

// out[row][head] = sum_s e^(m_s - M) o_s / (sink e^(z - M) + sum_s e^(m_s - M) l_s),  M = max(m_s, z with a sink), z the
// sink's score (0, or sinks[head]); times sigmoid(gate[row][head]) with a gate;
// at most 64 parts: lane s holds part s's maximum and sum.  The parts' elements are asked for 16 parts at a time, with
// no condition on the way (a part beyond the last one is read as the last one, with weight 0).
__global__ __launch_bounds__(64) void attn_masked_merge_kernel(const float* __restrict__ parts, int n_parts, int H,
                                                               int dv, const int* __restrict__ rows, int sink,
                                                               const float* __restrict__ sinks,
                                                               const float* __restrict__ gate, int ldg,
                                                               void* __restrict__ out, int ldo, int out_f32) {
  const int ri = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = rows ? rows[ri] : ri;
  const float* p = parts + ((size_t)ri * H + h) * n_parts * (dv + 2);
  const float m = lane < n_parts ? p[(size_t)lane * (dv + 2)] : -INFINITY;
  const float l = lane < n_parts ? p[(size_t)lane * (dv + 2) + 1] : 0.f;
  float M = wave_max(m);
  const float z = sinks ? sinks[h] : 0.f;
  if (sink) M = fmaxf(M, z);
  const float w = m == -INFINITY ? 0.f : __expf(m - M);
  const float L = wave_sum(w * l) + (sink ? __expf(z - M) : 0.f);
  float inv = 1.0f / L;
  if (gate) inv *= 1.0f / (1.0f + __expf(-gate[(size_t)r * ldg + h]));
  for (int e0 = 0; e0 < dv; e0 += WAVE) {
    const int e = min(e0 + lane, dv - 1);
    float a = 0.f;
    for (int s0 = 0; s0 < n_parts; s0 += 16) {
      float v[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) v[k] = p[(size_t)min(s0 + k, n_parts - 1) * (dv + 2) + 2 + e];
#pragma unroll
      for (int k = 0; k < 16; ++k) a = fmaf(s0 + k < n_parts ? __shfl(w, (s0 + k) & 63, WAVE) : 0.f, v[k], a);
    }
    if (e0 + lane < dv) store_f(out, out_f32 ? APC_F32 : APC_BF16, (size_t)r * ldo + (size_t)h * dv + e, a * inv);
  }
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

int check_sizes(const void* q, int ldq, const void* out, int ldo, const void* cache, int H, int G, int dk, int dv, int P,
                int mask, int mask_size, float scale, int key_parts, int out_f32) {
  if (H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0 || P <= 0 || mask < 0 || mask > 2 || (mask && mask_size <= 0) ||
      key_parts < 1 || dk % key_parts || (H / G) % key_parts)
    return APC_ERR_BAD_ARG;
  if (dk % (8 * key_parts) || dv % 4 || dk > DMAX || dv > DMAX || P % 8 || ldq % 8 || ldo % 4 || !aligned16(q) ||
      !aligned16(cache) || ((uintptr_t)out & (out_f32 ? 15u : 7u)) || !(scale > 0.f))
    return APC_ERR_UNSUPPORTED;
  return 0;
}

}  // namespace

// 1 if the kernels take these sizes, else 0 (the caller then runs the plain kernel)
APC_EXPORT int apc_attention_masked_takes(int H, int G, int dk, int dv, int page_tokens, int key_parts) {
  if (H <= 0 || G <= 0 || H % G || H / G > 16 || key_parts < 1 || (H / G) % key_parts) return 0;
  if (dk % (8 * key_parts) || dv % 8 || dk > DMAX || dv > DMAX) return 0;
  if (page_tokens < 8 || page_tokens > DT || (page_tokens & (page_tokens - 1))) return 0;
  return 1;
}

APC_EXPORT int apc_attention_masked_prefill_bf16(const void* q, int ldq, void* out, int ldo, int H, int G, int dk,
                                                 int dv, const void* cache, int page_tokens, const int* block_table,
                                                 int max_blocks, const int* positions, const int* row_seg,
                                                 const int* tile_row0, const int* tile_rows, int n_tiles, int mask,
                                                 int mask_size, int sink, const float* sinks, const float* gate,
                                                 int ldg, float scale, int key_parts, int out_f32, float softcap,
                                                 const float* r1, const float* r2, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if ((sinks && !sink) || (gate && ldg < H) || softcap < 0.f || (!r1) != (!r2)) return APC_ERR_BAD_ARG;
  int e = check_sizes(q, ldq, out, ldo, cache, H, G, dk, dv, page_tokens, mask, mask_size, scale, key_parts, out_f32);
  if (e) return e;
  n_tiles *= 2;  // halves
  if (max_blocks <= 0 || (long)n_tiles * H > 0x7fffffffL) return APC_ERR_BAD_ARG;
  dim3 grid(n_tiles * H), block(256);
#define MP_LAUNCH(DK_, DV_)                                                                                         \
  hipLaunchKernelGGL((attn_masked_prefill_kernel<DK_, DV_>), grid, block, 0, stream, (const bf16_t*)q, ldq,          \
                     out, ldo, H, G, dk, dv, (const bf16_t*)cache, page_tokens, block_table, max_blocks,             \
                     positions, row_seg, tile_row0, tile_rows, n_tiles, mask, mask_size, sink, sinks, gate, ldg,     \
                     scale, key_parts, out_f32, softcap, r1, r2)
#define MP_VALUES(DK_)                       \
  do {                                       \
    if (dv <= 64) MP_LAUNCH(DK_, 64);        \
    else if (dv <= 128) MP_LAUNCH(DK_, 128); \
    else MP_LAUNCH(DK_, 256);                \
  } while (0)
  if (dk <= 64) MP_VALUES(64);
  else if (dk <= 128) MP_VALUES(128);
  else MP_VALUES(256);
#undef MP_VALUES
#undef MP_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

// `rows`: the step's rows that are decoded ones (nullptr: all n_rows rows); at most 64 splits; `parts`: room for n_rows * H * n_splits * (dv + 2) floats.
APC_EXPORT int apc_attention_masked_decode_bf16(const void* q, int ldq, void* out, int ldo, int n_rows, int H, int G,
                                                int dk, int dv, const void* cache, int page_tokens,
                                                const int* block_table, int max_blocks, const int* positions,
                                                const int* row_seg, const int* rows, int mask, int mask_size, int sink,
                                                const float* sinks, const float* gate, int ldg, float scale,
                                                int n_splits, float* parts, int key_parts, int out_f32,
                                                float softcap, const float* r1, const float* r2,
                                                hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if ((sinks && !sink) || (gate && ldg < H) || softcap < 0.f || (!r1) != (!r2)) return APC_ERR_BAD_ARG;
  int e = check_sizes(q, ldq, out, ldo, cache, H, G, dk, dv, page_tokens, mask, mask_size, scale, key_parts, out_f32);
  if (e) return e;
  if (!apc_attention_masked_takes(H, G, dk, dv, page_tokens, key_parts)) return APC_ERR_UNSUPPORTED;
  if (n_splits <= 0 || n_splits > WAVE || !parts || max_blocks <= 0 ||
      (long)n_rows * G * n_splits > 0x7fffffffL || H > 65535)
    return APC_ERR_BAD_ARG;
  dim3 grid(n_rows * G * n_splits), block(DT);
#define MD_LAUNCH(KS_, ET_)                                                                                       \
  hipLaunchKernelGGL((attn_masked_decode_kernel<KS_, ET_>), grid, block, 0, stream, (const bf16_t*)q, ldq, H, G, dk, \
                     dv, (const bf16_t*)cache, page_tokens, block_table, max_blocks, positions, row_seg, rows, mask,  \
                     mask_size, scale, n_splits, parts, key_parts, softcap, r1, r2)
#define MD_VALUES(KS_)                     \
  do {                                     \
    if (dv <= 64) MD_LAUNCH(KS_, 4);       \
    else if (dv <= 128) MD_LAUNCH(KS_, 8); \
    else MD_LAUNCH(KS_, 16);               \
  } while (0)
  if (dk <= 64) MD_VALUES(2);
  else if (dk <= 128) MD_VALUES(4);
  else MD_VALUES(8);
#undef MD_VALUES
#undef MD_LAUNCH
  APC_LAUNCH_CHECK();
  hipLaunchKernelGGL(attn_masked_merge_kernel, dim3(n_rows, H), dim3(64), 0, stream, parts, n_splits, H, dv, rows, sink,
                     sinks, gate, ldg, out, ldo, out_f32);
  APC_LAUNCH_CHECK();
  return 0;
}
