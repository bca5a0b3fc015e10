// Heads put together from several projected rows, rotated on a range of their elements and written into pages whose
// keys and values have different sizes (see plain_heads.hip for the formulas), 16 bytes a thread.
//
// A row's work is cut into pieces of 8 consecutive elements of one head: the pieces of the H query heads, of the G
// keys and of the G values.  A piece outside the rotated range is copied.  A piece in the first half of the rotated
// range is handled together with its partner, the piece rot/2 elements further on (rot/2 is a multiple of 8, so the
// partners of a piece's elements are a piece): the thread reads both, turns the 8 pairs and writes both, so q may be
// rotated where it lies; the thread of a piece in the second half does nothing.  A key's piece goes into the page
// as one 16-byte store; a value's 8 elements go to 8 rows of the transposed value block, slot by slot.  In steps of
// many rows the values go through rotary_pages_values_kernel instead (16 rows x 128 columns through LDS, 8 slots of a
// column in one store).
// The second part of a key (the part all heads share, or a head's own) may be float32 rows.
//
// With a norm on the heads (q_norm_w / k_norm_w: a head over its root mean square, times weights all heads share,
// ahead of the rotation) a wave takes a whole head of one row, a lane a piece: the sum of squares is the wave's, a lane
// reads its piece and its partner's and writes its own, after all lanes have read (rotary_pages_norm_bf16_kernel).
#include "mfma.h"
#include <math.h>

namespace {

struct F8 { float v[8]; };

__device__ __forceinline__ F8 load8_bf16(const bf16_t* p) {
  const Frag f = load_frag(p);
  F8 o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o.v[2 * i] = __uint_as_float(f.w[i] << 16);
    o.v[2 * i + 1] = __uint_as_float(f.w[i] & 0xffff0000u);
  }
  return o;
}
__device__ __forceinline__ F8 load8_f32(const float* p) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  return F8{{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w}};
}
__device__ __forceinline__ void store8_bf16(bf16_t* p, const F8& x) {
  Frag f;
#pragma unroll
  for (int i = 0; i < 4; ++i) f.w[i] = pack_bf16x2(x.v[2 * i], x.v[2 * i + 1]);
  *reinterpret_cast<Frag*>(p) = f;
}

__global__ __launch_bounds__(256) void rotary_pages_bf16_kernel(
    const bf16_t* __restrict__ q, int ldq, int q_off, int H, int dq, int q_rot0, bf16_t* __restrict__ q_out, int ldqo,
    const bf16_t* __restrict__ ka, int ldka, int ka_off, int da, const void* __restrict__ kb, int kb_f32, int ldkb,
    int kb_off, int db, int kb_shared, int k_rot0, const bf16_t* __restrict__ v, int ldv, int v_off, int dv, int G,
    int rot, const float* __restrict__ cos_sin, const int* __restrict__ positions, const int* __restrict__ row_seg,
    const int* __restrict__ block_table, int max_blocks, bf16_t* __restrict__ cache, int P, int with_values) {
  const int r = blockIdx.x;
  const int dk = da + db, half = rot / 2;
  const int nq = H * (dq / 8), nk = G * (dk / 8), nv = with_values ? G * (dv / 8) : 0;
  const int item = blockIdx.y * 256 + threadIdx.x;
  if (item >= nq + nk + nv) return;
  const int pos = positions[r];
  const float* cs = cos_sin + (size_t)pos * rot;
  if (item < nq) {
    const int h = item / (dq / 8), e = (item % (dq / 8)) * 8, j = e - q_rot0;
    const bf16_t* src = q + (size_t)r * ldq + q_off + (size_t)h * dq;
    bf16_t* dst = q_out + (size_t)r * ldqo + (size_t)h * dq;
    if (j < 0 || j >= rot) {
      if (dst != src) store8_bf16(dst + e, load8_bf16(src + e));
    } else if (j < half) {
      const F8 x = load8_bf16(src + e), y = load8_bf16(src + e + half);
      const F8 c = load8_f32(cs + j), s = load8_f32(cs + half + j);
      F8 a, b;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        a.v[i] = x.v[i] * c.v[i] - y.v[i] * s.v[i];
        b.v[i] = y.v[i] * c.v[i] + x.v[i] * s.v[i];
      }
      store8_bf16(dst + e, a);
      store8_bf16(dst + e + half, b);
    }
    return;
  }
  const size_t page = (size_t)block_table[(size_t)row_seg[r] * max_blocks + pos / P];
  const int slot = pos % P;
  if (item < nq + nk) {
    const int it = item - nq, g = it / (dk / 8), e = (it % (dk / 8)) * 8, j = e - k_rot0;
    bf16_t* dst = cache + (page * G + g) * (size_t)P * (dk + dv) + (size_t)slot * dk;
    auto piece = [&](int at) -> F8 {
      if (at < da) return load8_bf16(ka + (size_t)r * ldka + ka_off + (size_t)g * da + at);
      const size_t col = (size_t)kb_off + (kb_shared ? 0 : (size_t)g * db) + (at - da);
      return kb_f32 ? load8_f32((const float*)kb + (size_t)r * ldkb + col)
                    : load8_bf16((const bf16_t*)kb + (size_t)r * ldkb + col);
    };
    if (j < 0 || j >= rot) {
      store8_bf16(dst + e, piece(e));
    } else if (j < half) {
      const F8 x = piece(e), y = piece(e + half);
      const F8 c = load8_f32(cs + j), s = load8_f32(cs + half + j);
      F8 a, b;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        a.v[i] = x.v[i] * c.v[i] - y.v[i] * s.v[i];
        b.v[i] = y.v[i] * c.v[i] + x.v[i] * s.v[i];
      }
      store8_bf16(dst + e, a);
      store8_bf16(dst + e + half, b);
    }
    return;
  }
  const int it = item - nq - nk, g = it / (dv / 8), e = (it % (dv / 8)) * 8;
  const Frag f = load_frag(v + (size_t)r * ldv + v_off + (size_t)g * dv + e);
  bf16_t* dst = cache + (page * G + g) * (size_t)P * (dk + dv) + (size_t)P * dk + (size_t)e * P + slot;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    dst[(size_t)(2 * i) * P] = (bf16_t)(f.w[i] & 0xffffu);
    dst[(size_t)(2 * i + 1) * P] = (bf16_t)(f.w[i] >> 16);
  }
}

// A group of `lph` lanes (a power of two from 8 on, at least a head's pieces) a (row, head), 256 / lph heads a block:
// heads 0 .. H-1 are query heads, H .. H+G-1 keys (and their values).  d <= 512.
__global__ __launch_bounds__(256) void rotary_pages_norm_bf16_kernel(
    const bf16_t* q, int ldq, int q_off, int H, int dq, int q_rot0, bf16_t* q_out, int ldqo,     // (q_out may be q)
    const bf16_t* __restrict__ ka, int ldka, int ka_off, int dk, int k_rot0, const bf16_t* __restrict__ v, int ldv,
    int v_off, int dv, int G, int rot, const float* __restrict__ cos_sin, const int* __restrict__ positions,
    const int* __restrict__ row_seg, const int* __restrict__ block_table, int max_blocks, bf16_t* __restrict__ cache,
    int P, int with_values, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    int lph) {
  const int r = blockIdx.x, hh = blockIdx.y * (256 / lph) + threadIdx.x / lph, lane = threadIdx.x % lph;
  if (hh >= H + G) return;                      // (whole groups leave together; a wave holds whole groups)
  const bool is_q = hh < H;
  const int g = hh - H;
  const int d = is_q ? dq : dk, rot0 = is_q ? q_rot0 : k_rot0, half = rot / 2;
  const bf16_t* src = is_q ? q + (size_t)r * ldq + q_off + (size_t)hh * dq : ka + (size_t)r * ldka + ka_off + (size_t)g * dk;
  const float* nw = is_q ? q_norm_w : k_norm_w;
  const int pos = positions[r];
  const int e = lane * 8;
  const bool on = e < d;
  F8 x = F8{{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}}, y = x;
  if (on) x = load8_bf16(src + e);
  const int j = e - rot0;
  const bool turn = on && j >= 0 && j < rot, first = j < half;
  const int pe = first ? e + half : e - half;        // the partner piece
  if (turn) y = load8_bf16(src + pe);
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss = fmaf(x.v[i], x.v[i], ss);
  for (int o = lph / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);
  if (nw) {
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    if (on) {
      const F8 w = load8_f32(nw + e);
#pragma unroll
      for (int i = 0; i < 8; ++i) x.v[i] = (x.v[i] * inv) * w.v[i];
    }
    if (turn) {
      const F8 w = load8_f32(nw + pe);
#pragma unroll
      for (int i = 0; i < 8; ++i) y.v[i] = (y.v[i] * inv) * w.v[i];
    }
  }
  if (turn) {
    const int jj = first ? j : j - half;
    const float* cs = cos_sin + (size_t)pos * rot;
    const F8 c = load8_f32(cs + jj), sn = load8_f32(cs + half + jj);
#pragma unroll
    for (int i = 0; i < 8; ++i) x.v[i] = first ? x.v[i] * c.v[i] - y.v[i] * sn.v[i] : x.v[i] * c.v[i] + y.v[i] * sn.v[i];
  }
  if (is_q) {
    if (on) store8_bf16(q_out + (size_t)r * ldqo + (size_t)hh * dq + e, x);
    return;
  }
  const size_t page = (size_t)block_table[(size_t)row_seg[r] * max_blocks + pos / P];
  const int slot = pos % P;
  bf16_t* head = cache + (page * G + g) * (size_t)P * (dk + dv);
  if (on) store8_bf16(head + (size_t)slot * dk + e, x);
  if (with_values && e < dv) {
    const Frag f = load_frag(v + (size_t)r * ldv + v_off + (size_t)g * dv + e);
    bf16_t* dst = head + (size_t)P * dk + (size_t)e * P + slot;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dst[(size_t)(2 * i) * P] = (bf16_t)(f.w[i] & 0xffffu);
      dst[(size_t)(2 * i + 1) * P] = (bf16_t)(f.w[i] >> 16);
    }
  }
}

// The values of 16 rows x 128 columns (kv head * dv + element) through LDS into the transposed value blocks: where 8
// rows are 8 consecutive slots of one page that start at a multiple of 8, a column's 8 values leave as one 16-byte
// store; else slot by slot.
constexpr int VR = 16, VC = 128, VPAD = 8;

__global__ __launch_bounds__(256) void rotary_pages_values_kernel(
    const bf16_t* __restrict__ v, int ldv, int v_off, int dk, int dv, int G, const int* __restrict__ positions,
    const int* __restrict__ row_seg, const int* __restrict__ block_table, int max_blocks, bf16_t* __restrict__ cache,
    int P, int n_rows) {
  __shared__ __attribute__((aligned(16))) bf16_t vt[VR][VC + VPAD];
  __shared__ long long base_s[VR];      // element offset of the row's page; -1: no such row
  __shared__ int slot_s[VR];
  const int tid = threadIdx.x, r0 = blockIdx.x * VR, c0 = blockIdx.y * VC;
  if (tid < VR) {
    const int t = r0 + tid;
    long long base = -1;
    int slot = 0;
    if (t < n_rows) {
      const int pos = positions[t];
      base = (long long)block_table[(size_t)row_seg[t] * max_blocks + pos / P] * G * P * (dk + dv);
      slot = pos % P;
    }
    base_s[tid] = base;
    slot_s[tid] = slot;
  }
  __syncthreads();
  const int h = tid % 2;                // the half (8 rows) whose columns this thread stores
  bool run = P % 8 == 0 && slot_s[8 * h] % 8 == 0;
#pragma unroll
  for (int r = 0; r < 8; ++r)
    run = run && base_s[8 * h + r] >= 0 && base_s[8 * h + r] == base_s[8 * h] && slot_s[8 * h + r] == slot_s[8 * h] + r;
  const int cw = min(VC, G * dv - c0), pieces = cw / 8;
  for (int item = tid; item < VR * pieces; item += 256) {
    const int r = item / pieces, p = item % pieces;
    if (r0 + r < n_rows)
      *reinterpret_cast<Frag*>(&vt[r][p * 8]) = load_frag(v + (size_t)(r0 + r) * ldv + v_off + c0 + p * 8);
  }
  __syncthreads();
  for (int item = tid; item < 2 * cw; item += 256) {      // item % 2 == h: 256 is even
    const int col = c0 + item / 2, g = col / dv, e = col % dv;
    const size_t at = ((size_t)g * (dk + dv) + dk + e) * P;   // the column's row of slots inside a page
    if (run) {
      Frag f;
#pragma unroll
      for (int w = 0; w < 4; ++w)
        f.w[w] = (uint32_t)vt[8 * h + 2 * w][item / 2] | ((uint32_t)vt[8 * h + 2 * w + 1][item / 2] << 16);
      *reinterpret_cast<Frag*>(cache + base_s[8 * h] + at + slot_s[8 * h]) = f;
    } else {
#pragma unroll
      for (int r = 0; r < 8; ++r)
        if (base_s[8 * h + r] >= 0) cache[base_s[8 * h + r] + at + slot_s[8 * h + r]] = vt[8 * h + r][item / 2];
    }
  }
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace

// 1 if the kernel takes these sizes (every size, offset and row stride a multiple of 8 elements), else 0
APC_EXPORT int apc_rotary_pages_bf16_takes(int ldq, int q_off, int dq, int q_rot0, int ldqo, int ldka, int ka_off,
                                           int da, int ldkb, int kb_off, int db, int k_rot0, int ldv, int v_off,
                                           int dv, int rot) {
  const int all = ldq | q_off | dq | q_rot0 | ldqo | ldka | ka_off | da | ldkb | kb_off | db | k_rot0 | ldv | v_off | dv;
  return (all % 8 == 0 && rot % 16 == 0 && dq > 0 && da + db > 0 && dv > 0) ? 1 : 0;
}

APC_EXPORT int apc_rotary_pages_bf16(const void* q, int ldq, int q_off, int H, int dq, int q_rot0, void* q_out,
                                     int ldqo, const void* ka, int ldka, int ka_off, int da, const void* kb, int kb_f32,
                                     int ldkb, int kb_off, int db, int kb_shared, int k_rot0, const void* v, int ldv,
                                     int v_off, int dv, int G, int rot, const float* cos_sin, const int* positions,
                                     const int* row_seg, const int* block_table, int max_blocks, void* cache,
                                     int page_tokens, int n_rows, const float* q_norm_w, const float* k_norm_w,
                                     float norm_eps, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || G <= 0 || rot < 0 || (rot && !cos_sin) || !positions || !row_seg || !block_table || !cache || !q ||
      !q_out || !ka || !v || (db && !kb) || q_rot0 < 0 || q_rot0 + rot > dq || k_rot0 < 0 || k_rot0 + rot > da + db ||
      page_tokens <= 0 || max_blocks <= 0 || ldqo < H * dq)
    return APC_ERR_BAD_ARG;
  if (!apc_rotary_pages_bf16_takes(ldq, q_off, dq, q_rot0, ldqo, ldka, ka_off, da, ldkb, kb_off, db, k_rot0, ldv, v_off,
                                   dv, rot) ||
      !aligned16(q) || !aligned16(q_out) || !aligned16(ka) || !aligned16(v) || (db && !aligned16(kb)) ||
      !aligned16(cache) || (rot && !aligned16(cos_sin)))
    return APC_ERR_UNSUPPORTED;
  // Steps of many rows (prompt portions): the values go through a kernel of their own that gathers 8 slots of a
  // column into one store.  Both ways write the same bits.
  const bool apart = n_rows >= 2 * VR && page_tokens % 8 == 0 && ((long)G * dv + VC - 1) / VC <= 65535;
  const long items = (long)H * (dq / 8) + (long)G * ((da + db) / 8) + (apart ? 0 : (long)G * (dv / 8));
  if (items > 65535L * 256) return APC_ERR_UNSUPPORTED;
  const bool normed = q_norm_w || k_norm_w;
  int lph = 8;                                  // lanes a head: its pieces of 8 elements, rounded up to a power of two
  while (lph * 8 < dq || lph * 8 < da || lph * 8 < dv) lph *= 2;
  const int heads_a_block = 256 / (lph > 64 ? 64 : lph);
  if (normed && (db || lph > 64 || (H + G + heads_a_block - 1) / heads_a_block > 65535 || !aligned16(q_norm_w) ||
                 !aligned16(k_norm_w)))
    return APC_ERR_UNSUPPORTED;
  if (apart) {
    hipLaunchKernelGGL(rotary_pages_values_kernel, dim3((n_rows + VR - 1) / VR, (unsigned)((G * dv + VC - 1) / VC)),
                       dim3(256), 0, stream, (const bf16_t*)v, ldv, v_off, da + db, dv, G, positions, row_seg,
                       block_table, max_blocks, (bf16_t*)cache, page_tokens, n_rows);
    APC_LAUNCH_CHECK();
  }
  if (normed) {
    hipLaunchKernelGGL(rotary_pages_norm_bf16_kernel,
                       dim3(n_rows, (unsigned)((H + G + heads_a_block - 1) / heads_a_block)), dim3(256), 0, stream,
                       (const bf16_t*)q, ldq, q_off, H, dq, q_rot0, (bf16_t*)q_out, ldqo, (const bf16_t*)ka, ldka,
                       ka_off, da, k_rot0, (const bf16_t*)v, ldv, v_off, dv, G, rot, cos_sin, positions, row_seg,
                       block_table, max_blocks, (bf16_t*)cache, page_tokens, apart ? 0 : 1, q_norm_w, k_norm_w, norm_eps,
                       lph);
    APC_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(rotary_pages_bf16_kernel, dim3(n_rows, (unsigned)((items + 255) / 256)), dim3(256), 0, stream,
                     (const bf16_t*)q, ldq, q_off, H, dq, q_rot0, (bf16_t*)q_out, ldqo, (const bf16_t*)ka, ldka, ka_off,
                     da, kb, kb_f32, ldkb, kb_off, db, kb_shared, k_rot0, (const bf16_t*)v, ldv, v_off, dv, G, rot,
                     cos_sin, positions, row_seg, block_table, max_blocks, (bf16_t*)cache, page_tokens, apart ? 0 : 1);
  APC_LAUNCH_CHECK();
  return 0;
}
