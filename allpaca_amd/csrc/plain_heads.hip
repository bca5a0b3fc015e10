// Plain kernel for attentions whose heads are put together from several projected rows before they are rotated and
// cached: a rotation on a range of a head's elements, keys that are a head's own part followed by a part shared by
// all heads, and values that may be the keys' own columns as projected.  All arithmetic in 32-bit float, any element
// type in and out.
#include "common.h"
#include <math.h>

namespace {

constexpr int MAX_HEAD = 1024;

// One wave per (row, head).  Heads 0 .. H-1 are query heads, heads H .. H+G-1 the key and value of a kv head.
//   q:  q[t][q_off + h * dq + i], i < dq; elements [q_rot0, q_rot0 + rot) are rotated; the result goes to q_out
//       [t][h * dq + i] (q_out may be q itself: a head is read whole before any of it is written)
//   key of kv head g, dk = da + db elements: first ka[t][ka_off + g * da + i] (i < da), then
//       kb[t][kb_off + (kb_shared ? 0 : g * db) + i] (i < db); elements [k_rot0, k_rot0 + rot) of the whole are rotated
//   value of kv head g: v[t][v_off + g * dv + e], as it is
// With `q_norm_w` [dq] (`k_norm_w` [da + db]) a query (key) head is first divided by its root mean square over the
// head, sqrt(mean(x^2) + eps), and multiplied with the weights, which all heads share; values are never normed.
// The rotation pairs element i with element i + rot/2 of the range: (x, y) -> (x c - y s, y c + x s), c and s from
// cos_sin[position][2][rot/2].
// pages: page = block_table[seg][pos / P]; keys page[g][slot * dk + i], values page[g][P * dk + e * P + slot], a page
// being G * P * (dk + dv) elements.
__global__ __launch_bounds__(64) void rotary_pages_kernel(
    const void* __restrict__ q, int q_dtype, int ldq, int q_off, int H, int dq, int q_rot0, void* __restrict__ q_out,
    int qo_dtype, int ldqo, const void* __restrict__ ka, int ka_dtype, int ldka, int ka_off, int da,
    const void* __restrict__ kb, int kb_dtype, int ldkb, int kb_off, int db, int kb_shared, int k_rot0,
    const void* __restrict__ v, int v_dtype, int ldv, int v_off, int dv, int G, int rot,
    const float* __restrict__ cos_sin, const int* __restrict__ positions, const int* __restrict__ row_seg,
    const int* __restrict__ block_table, int max_blocks, void* __restrict__ cache, int cache_dtype, int P,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps) {
  __shared__ float xs[MAX_HEAD];
  const int r = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[r];
  const int half = rot / 2;
  const float* cs = cos_sin + (size_t)pos * rot;     // [2][half]
  const bool is_q = hh < H;
  const int g = hh - H;
  const int d = is_q ? dq : da + db;
  const int rot0 = is_q ? q_rot0 : k_rot0;
  for (int i = lane; i < d; i += WAVE) {
    float x;
    if (is_q) x = load_f(q, q_dtype, (size_t)r * ldq + q_off + (size_t)hh * dq + i);
    else if (i < da) x = load_f(ka, ka_dtype, (size_t)r * ldka + ka_off + (size_t)g * da + i);
    else x = load_f(kb, kb_dtype, (size_t)r * ldkb + kb_off + (kb_shared ? 0 : (size_t)g * db) + (i - da));
    xs[i] = x;
  }
  __syncthreads();
  const float* nw = is_q ? q_norm_w : k_norm_w;
  if (nw) {
    float ss = 0.f;
    for (int i = lane; i < d; i += WAVE) ss = fmaf(xs[i], xs[i], ss);
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
    for (int i = lane; i < d; i += WAVE) xs[i] = (xs[i] * inv) * nw[i];      // (a lane's own elements)
    __syncthreads();
  }
  size_t key_base = 0, val_base = 0;
  if (!is_q) {
    const int dk = da + db;
    const size_t page = (size_t)block_table[(size_t)row_seg[r] * max_blocks + pos / P];
    const size_t head = (page * G + g) * (size_t)P * (dk + dv);
    key_base = head + (size_t)(pos % P) * dk;
    val_base = head + (size_t)P * dk + (pos % P);
  }
  for (int i = lane; i < d; i += WAVE) {
    float x = xs[i];
    const int j = i - rot0;
    if (j >= 0 && j < rot) {
      const bool first = j < half;
      const int f = first ? j : j - half;
      const float c = cs[f], s = cs[half + f];
      const float y = xs[first ? i + half : i - half];
      x = first ? x * c - y * s : x * c + y * s;
    }
    if (is_q) store_f(q_out, qo_dtype, (size_t)r * ldqo + (size_t)hh * dq + i, x);
    else store_f(cache, cache_dtype, key_base + i, x);
  }
  if (!is_q) {
    for (int e = lane; e < dv; e += WAVE)
      store_f(cache, cache_dtype, val_base + (size_t)e * P, load_f(v, v_dtype, (size_t)r * ldv + v_off + (size_t)g * dv + e));
  }
}

}  // namespace

APC_EXPORT int apc_rotary_pages(const void* q, int q_dtype, int ldq, int q_off, int H, int dq, int q_rot0, void* q_out,
                                int qo_dtype, int ldqo, const void* ka, int ka_dtype, int ldka, int ka_off, int da,
                                const void* kb, int kb_dtype, int ldkb, int kb_off, int db, int kb_shared, int k_rot0,
                                const void* v, int v_dtype, int ldv, int v_off, int dv, int G, int rot,
                                const float* cos_sin, const int* positions, const int* row_seg, const int* block_table,
                                int max_blocks, void* cache, int cache_dtype, int page_tokens, int n_rows,
                                const float* q_norm_w, const float* k_norm_w, float eps, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H < 0 || G < 0 || H + G <= 0 || rot < 0 || rot % 2 || (rot && !cos_sin) || !positions) return APC_ERR_BAD_ARG;
  if (H && (!q || !q_out || dq <= 0 || q_rot0 < 0 || q_rot0 + rot > dq || ldqo < H * dq)) return APC_ERR_BAD_ARG;
  if (G && (!ka || da <= 0 || db < 0 || (db && !kb) || k_rot0 < 0 || k_rot0 + rot > da + db || !v || dv <= 0 ||
            !cache || !block_table || !row_seg || page_tokens <= 0 || max_blocks <= 0))
    return APC_ERR_BAD_ARG;
  if (dq > MAX_HEAD || da + db > MAX_HEAD || H + G > 65535) return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(rotary_pages_kernel, dim3(n_rows, H + G), dim3(64), 0, stream, q, q_dtype, ldq, q_off, H, dq,
                     q_rot0, q_out, qo_dtype, ldqo, ka, ka_dtype, ldka, ka_off, da, kb, kb_dtype, ldkb, kb_off, db,
                     kb_shared, k_rot0, v, v_dtype, ldv, v_off, dv, G, rot, cos_sin, positions, row_seg, block_table,
                     max_blocks, cache, cache_dtype, page_tokens, q_norm_w, k_norm_w, eps);
  APC_LAUNCH_CHECK();
  return 0;
}
