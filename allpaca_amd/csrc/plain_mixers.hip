// Plain kernels of the mechanisms beside the llama layer: a short causal convolution over time with per-request
// state, unit RMS norm of heads, attention with a chunked or sliding mask and an optional sink over pages whose keys
// and values have different sizes, residual streams with learned read / write weights, a clamped gated activation.
// One obvious loop nest each, all arithmetic in 32-bit float with an order of additions that the row's own place
// fixes (never the batch), any element type in and out.
#include "common.h"
#include <math.h>

constexpr int MAX_TAPS = 8;
constexpr int MAX_PER_LANE = 4;   // head sizes up to 256
constexpr int MAX_STREAMS = 16;

// ---------------------------------------------------------------------------
// Short convolution on the heads of a projected row, then (q, k) unit RMS norm per head, then q to `q_out` and k, v
// into the pages.
//
// proj [T, ld]: q heads at column q_off (H of dk), k heads at k_off (G of dk), v heads at v_off (G of dv); with
// G == 0 the row holds q only.  Channel c of the convolution is column c of the row:
//   u[t][c] = proj[t][c] + bias[c]
//   y[t][c] = sum_j w[c][j] * u[t - (n-1) + j][c]            (n taps, n = 1 too; without w: y = u)
// u of the n-1 positions ahead of a segment's first row comes from state[slot][n-1][width] (zero for a new request:
// the sequence starts with zeros).  `conv_state_kernel` moves the state on afterwards.
//   q, k:  y / sqrt(mean(y^2) + eps)  if `unit_norm`, the mean over the head, or over each piece of `norm_dim`
//          elements of it (norm_dim divides dk; 0: the whole head); times q_norm_w / k_norm_w [norm_dim] if given.
//          `norm_rows`: the mean is taken over all heads of q (of k) at once and the weights are [H * dk] ([G * dk]);
//          every wave forms the sum over the whole projection for itself, in one order
//   q:     times 1 + qt_coef * ln(floor((pos + 1) / qt_every) + 1) at position pos, if qt_every > 0
// pages: page = block_table[seg][pos / P]; keys page[g][slot * dk + i], values page[g][P * dk + e * P + slot]
// (a key's elements lie together, a value element's slots lie together), a page being G * P * (dk + dv) elements.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void conv_heads_kernel(
    const void* __restrict__ proj, int in_dtype, int ld, int q_off, int k_off, int v_off, int H, int G, int dk, int dv,
    const float* __restrict__ bias, const float* __restrict__ conv_w, int taps, const float* __restrict__ state,
    int width, const int* __restrict__ row_seg, const int* __restrict__ seg_row0, const int* __restrict__ slots,
    const int* __restrict__ positions, int unit_norm, float eps, int norm_dim, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, int norm_rows, float qt_coef, int qt_every, void* __restrict__ q_out,
    int q_dtype, int ldq, const int* __restrict__ block_table, int max_blocks, void* __restrict__ cache,
    int cache_dtype, int P) {
  const int r = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
  int kind, head, d, col0;
  if (hh < H) { kind = 0; head = hh; d = dk; col0 = q_off + head * dk; }
  else if (hh < H + G) { kind = 1; head = hh - H; d = dk; col0 = k_off + head * dk; }
  else { kind = 2; head = hh - H - G; d = dv; col0 = v_off + head * dv; }
  const int seg = row_seg[r];
  const int i_in_seg = r - seg_row0[seg];
  const float* st = (taps > 1) ? state + (size_t)slots[seg] * (taps - 1) * width : nullptr;

  auto channel = [&](int c) -> float {         // the convolution's output of column c of this row
    const float b = bias ? bias[c] : 0.f;
    if (!conv_w) return load_f(proj, in_dtype, (size_t)r * ld + c) + b;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {            // oldest first: the order of the sum is that of the taps
      const int back = taps - 1 - j;
      const float u = back <= i_in_seg ? load_f(proj, in_dtype, (size_t)(r - back) * ld + c) + b
                                       : st[(size_t)(taps - 1 - (back - i_in_seg)) * width + c];
      acc = fmaf(conv_w[(size_t)c * taps + j], u, acc);
    }
    return acc;
  };
  float y[MAX_PER_LANE];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < MAX_PER_LANE; ++e) {
    const int i = lane + e * WAVE;
    y[e] = 0.f;
    if (i < d) {
      y[e] = channel(col0 + i);
      ss = fmaf(y[e], y[e], ss);
    }
  }
  if (unit_norm && kind != 2 && norm_rows) {
    const int n = (kind == 0 ? H : G) * dk, c0 = kind == 0 ? q_off : k_off;
    float tot = 0.f;
    for (int i = lane; i < n; i += WAVE) {
      const float v = channel(c0 + i);
      tot = fmaf(v, v, tot);
    }
    const float inv = 1.0f / sqrtf(wave_sum(tot) / (float)n + eps);
    const float* nw = kind == 0 ? q_norm_w : k_norm_w;
#pragma unroll
    for (int e = 0; e < MAX_PER_LANE; ++e) {
      const int i = lane + e * WAVE;
      y[e] = y[e] * inv;
      if (nw && i < d) y[e] *= nw[(size_t)head * dk + i];
    }
  } else if (unit_norm && kind != 2) {
    const int nd = norm_dim > 0 ? norm_dim : d;
    const float* nw = kind == 0 ? q_norm_w : k_norm_w;
    if (nd == d) {
      const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
      for (int e = 0; e < MAX_PER_LANE; ++e) {
        const int i = lane + e * WAVE;
        y[e] = y[e] * inv;
        if (nw && i < d) y[e] *= nw[i];
      }
    } else {
      float inv_mine[MAX_PER_LANE];
#pragma unroll
      for (int e = 0; e < MAX_PER_LANE; ++e) inv_mine[e] = 1.f;
      for (int piece = 0; piece < d / nd; ++piece) {
        float part = 0.f;
#pragma unroll
        for (int e = 0; e < MAX_PER_LANE; ++e) {
          const int i = lane + e * WAVE;
          if (i < d && i / nd == piece) part = fmaf(y[e], y[e], part);
        }
        const float inv = 1.0f / sqrtf(wave_sum(part) / (float)nd + eps);
#pragma unroll
        for (int e = 0; e < MAX_PER_LANE; ++e) {
          const int i = lane + e * WAVE;
          if (i < d && i / nd == piece) inv_mine[e] = inv;
        }
      }
#pragma unroll
      for (int e = 0; e < MAX_PER_LANE; ++e) {
        const int i = lane + e * WAVE;
        y[e] = y[e] * inv_mine[e];
        if (nw && i < d) y[e] *= nw[i % nd];
      }
    }
  }
  const int pos = positions[r];
  const float inv = (kind == 0 && qt_every > 0) ? 1.0f + qt_coef * logf((float)((pos + 1) / qt_every) + 1.0f) : 1.f;

  if (kind == 0) {
#pragma unroll
    for (int e = 0; e < MAX_PER_LANE; ++e) {
      const int i = lane + e * WAVE;
      if (i < d) store_f(q_out, q_dtype, (size_t)r * ldq + (size_t)head * dk + i, y[e] * inv);
    }
    return;
  }
  const int page = block_table[(size_t)seg * max_blocks + pos / P];
  const size_t base = ((size_t)page * G + head) * (size_t)P * (dk + dv);
#pragma unroll
  for (int e = 0; e < MAX_PER_LANE; ++e) {
    const int i = lane + e * WAVE;
    if (i < d) {
      if (kind == 1) store_f(cache, cache_dtype, base + (size_t)(pos % P) * dk + i, y[e] * inv);
      else store_f(cache, cache_dtype, base + (size_t)P * dk + (size_t)i * P + (pos % P), y[e]);
    }
  }
}

// The state after a step: u of the last n-1 positions of every segment (older ones shift down when the segment
// brought fewer rows than that).  Every thread reads what it needs of the old state before it writes.
__global__ void conv_state_kernel(const void* __restrict__ proj, int in_dtype, int ld, const float* __restrict__ bias,
                                  int taps, float* __restrict__ state, int width, const int* __restrict__ seg_row0,
                                  const int* __restrict__ seg_rows, const int* __restrict__ slots) {
  const int seg = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int n = seg_rows[seg], r0 = seg_row0[seg];
  float* st = state + (size_t)slots[seg] * (taps - 1) * width;
  const float b = bias ? bias[c] : 0.f;
  float keep[MAX_TAPS - 1];
#pragma unroll
  for (int k = 0; k < MAX_TAPS - 1; ++k) {
    if (k < taps - 1) {
      const int back = taps - 1 - k;              // new row k holds the position `back` before the segment's end
      keep[k] = back <= n ? load_f(proj, in_dtype, (size_t)(r0 + n - back) * ld + c) + b
                          : st[(size_t)(k + n) * width + c];
    }
  }
#pragma unroll
  for (int k = 0; k < MAX_TAPS - 1; ++k)
    if (k < taps - 1) st[(size_t)k * width + c] = keep[k];
}

APC_EXPORT int apc_conv_heads(const void* proj, int in_dtype, int ld, int q_off, int k_off, int v_off, int n_rows,
                              int n_segs, int H, int G, int dk, int dv, const float* bias, const float* conv_w,
                              int taps, float* state, int width, const int* row_seg, const int* seg_row0,
                              const int* seg_rows, const int* slots, const int* positions, int unit_norm, float eps,
                              int norm_dim, const float* q_norm_w, const float* k_norm_w, int norm_rows,
                              float qt_coef, int qt_every,
                              void* q_out, int q_dtype, int ldq, const int* block_table, int max_blocks, void* cache,
                              int cache_dtype, int page_tokens, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (norm_dim < 0 || (norm_dim > 0 && dk % norm_dim) || qt_every < 0 || (norm_rows && !unit_norm)) return APC_ERR_BAD_ARG;
  if (H <= 0 || G < 0 || dk <= 0 || (G > 0 && dv <= 0) || taps < 1 || width <= 0 || n_segs <= 0) return APC_ERR_BAD_ARG;
  if (taps > 1 && (!conv_w || !state)) return APC_ERR_BAD_ARG;
  if (G > 0 && (!cache || !block_table || page_tokens <= 0 || max_blocks <= 0)) return APC_ERR_BAD_ARG;
  if (taps > MAX_TAPS || dk > MAX_PER_LANE * WAVE || dv > MAX_PER_LANE * WAVE || H + 2 * G > 65535 || n_segs > 65535)
    return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(conv_heads_kernel, dim3(n_rows, H + 2 * G), dim3(64), 0, stream, proj, in_dtype, ld, q_off,
                     k_off, v_off, H, G, dk, dv, bias, conv_w, taps, state, width, row_seg, seg_row0, slots, positions,
                     unit_norm, eps, norm_dim, q_norm_w, k_norm_w, norm_rows, qt_coef, qt_every, q_out, q_dtype, ldq,
                     block_table, max_blocks, cache, cache_dtype, page_tokens);
  APC_LAUNCH_CHECK();
  if (taps > 1) {
    hipLaunchKernelGGL(conv_state_kernel, dim3(ceil_div(width, 256), n_segs), dim3(256), 0, stream, proj, in_dtype,
                       ld, bias, taps, state, width, seg_row0, seg_rows, slots);
    APC_LAUNCH_CHECK();
  }
  return 0;
}

// The second half alone: for callers that ran the first half on another kernel.
APC_EXPORT int apc_conv_state(const void* proj, int in_dtype, int ld, const float* bias, int taps, float* state,
                              int width, int n_segs, const int* seg_row0, const int* seg_rows, const int* slots,
                              hipStream_t stream) {
  if (n_segs <= 0 || taps <= 1) return 0;
  if (!state || width <= 0 || taps > MAX_TAPS || n_segs > 65535) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(conv_state_kernel, dim3(ceil_div(width, 256), n_segs), dim3(256), 0, stream, proj, in_dtype, ld,
                     bias, taps, state, width, seg_row0, seg_rows, slots);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Attention over pages with a mask and an optional sink: one wave per (query row, head), keys in order in groups of
// 64 anchored at key 0, online softmax in float32.
//   the row at position pos sees keys t in [first, pos]:
//     mask 0: first = 0;  mask 1 (window of n): first = max(0, pos - n + 1);  mask 2 (chunks of n): first = pos - pos % n
//   s_t = (q . K[t]) * scale;  p_t = exp(s_t) / (sink + sum exp(s_t)),  sink = 0, 1 (a key of score 0 without a value)
//   or exp(sinks[h]) (`sinks`: a learned score per query head, not scaled)
//   out = sum p_t V[t] (times sigmoid(gate[row][h]) with `gate`: logits [rows][>= H]);  query head h reads key/value
//   head h / (H / G).
// With `key_parts` = M > 1 a key of dk elements is M keys of dk / M side by side, one for each of M maps over the same
// values: q holds H heads of dk / M elements, head j computes its scores with part j % M of the keys of kv head
// j / (H / G) (the M heads of a group of M are the maps of one head), and `out` holds H heads of dv.
// `softcap` c > 0: s_t <- c * tanh(s_t / c).  `bias_r1`, `bias_r2` [H]: s_t <- s_t - r1[h] * ln(1 + r2[h] * (pos - t)), a
// learned penalty on the distance (behind the cap, if both are asked for).
// The running maximum starts at the sink's score and the running sum at 1 with a sink (the sink is the first "key"),
// at -inf and 0 without.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void masked_attention_plain_kernel(
    const void* __restrict__ q, int q_dtype, int ldq, void* __restrict__ out, int out_dtype, int ldo, int H, int G,
    int dk, int dv, const void* __restrict__ cache, int cache_dtype, int P, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ positions, const int* __restrict__ row_seg, int mask, int mask_size,
    int sink, const float* __restrict__ sinks, const void* __restrict__ gate, int gate_dtype, int ldg, float scale,
    int key_parts, float softcap, const float* __restrict__ bias_r1, const float* __restrict__ bias_r2) {
  __shared__ float qs[MAX_PER_LANE * WAVE];
  __shared__ float ps[WAVE];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  const int pos = positions[r];
  const int* bt = block_table + (size_t)row_seg[r] * max_blocks;
  int first = 0;
  if (mask == 1) first = pos - mask_size + 1 > 0 ? pos - mask_size + 1 : 0;
  else if (mask == 2) first = pos - pos % mask_size;
  const size_t page_elems = (size_t)G * P * (dk + dv);
  const size_t head_off = (size_t)g * P * (dk + dv);

  const int dq = dk / key_parts, part0 = (h % key_parts) * dq;    // the head's own part of a key
  for (int i = lane; i < dq; i += WAVE) qs[i] = load_f(q, q_dtype, (size_t)r * ldq + (size_t)h * dq + i);
  __syncthreads();

  float o[MAX_PER_LANE];
#pragma unroll
  for (int e = 0; e < MAX_PER_LANE; ++e) o[e] = 0.f;
  float m = sink ? (sinks ? sinks[h] : 0.f) : -INFINITY, l = sink ? 1.f : 0.f;

  for (int c = first / WAVE; c <= pos / WAVE; ++c) {
    const int t = c * WAVE + lane;
    const bool valid = t >= first && t <= pos;
    float s = -INFINITY;
    if (valid) {
      const size_t kb = (size_t)bt[t / P] * page_elems + head_off + (size_t)(t % P) * dk + part0;
      float dot = 0.f;
      for (int i = 0; i < dq; ++i) dot = fmaf(qs[i], load_f(cache, cache_dtype, kb + i), dot);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      if (bias_r1) s -= bias_r1[h] * logf(1.0f + bias_r2[h] * (float)(pos - t));
    }
    const float m_new = fmaxf(m, wave_max(s));   // finite: every group in the range holds a visible key
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int e = 0; e < MAX_PER_LANE; ++e) o[e] *= alpha;
    __syncthreads();
    ps[lane] = p;
    __syncthreads();
    const int j_end = min(WAVE, pos - c * WAVE + 1);
    const int j_begin = max(0, first - c * WAVE);
    for (int j = j_begin; j < j_end; ++j) {
      const float pj = ps[j];
      const int tj = c * WAVE + j;
      const size_t vb = (size_t)bt[tj / P] * page_elems + head_off + (size_t)P * dk + (tj % P);
#pragma unroll
      for (int e = 0; e < MAX_PER_LANE; ++e) {
        const int i = lane + e * WAVE;
        if (i < dv) o[e] = fmaf(pj, load_f(cache, cache_dtype, vb + (size_t)i * P), o[e]);
      }
    }
  }
  float inv = 1.0f / l;
  if (gate) inv *= 1.0f / (1.0f + expf(-load_f(gate, gate_dtype, (size_t)r * ldg + h)));
#pragma unroll
  for (int e = 0; e < MAX_PER_LANE; ++e) {
    const int i = lane + e * WAVE;
    if (i < dv) store_f(out, out_dtype, (size_t)r * ldo + (size_t)h * dv + i, o[e] * inv);
  }
}

APC_EXPORT int apc_masked_attention_plain(const void* q, int q_dtype, int ldq, void* out, int out_dtype, int ldo,
                                          int n_rows, int H, int G, int dk, int dv, const void* cache, int cache_dtype,
                                          int page_tokens, const int* block_table, int max_blocks,
                                          const int* positions, const int* row_seg, int mask, int mask_size, int sink,
                                          const float* sinks, const void* gate, int gate_dtype, int ldg, float scale,
                                          int key_parts, float softcap, const float* bias_r1, const float* bias_r2,
                                          hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0 || page_tokens <= 0 || max_blocks <= 0 || mask < 0 || mask > 2 ||
      (mask != 0 && mask_size <= 0) || key_parts < 1 || dk % key_parts || (H / G) % key_parts || (sinks && !sink) ||
      (gate && ldg < H) || softcap < 0.f || (!bias_r1) != (!bias_r2))
    return APC_ERR_BAD_ARG;
  if (dk > MAX_PER_LANE * WAVE || dv > MAX_PER_LANE * WAVE || H > 65535) return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(masked_attention_plain_kernel, dim3(n_rows, H), dim3(64), 0, stream, q, q_dtype, ldq, out,
                     out_dtype, ldo, H, G, dk, dv, cache, cache_dtype, page_tokens, block_table, max_blocks, positions,
                     row_seg, mask, mask_size, sink, sinks, gate, gate_dtype, ldg, scale, key_parts, softcap, bias_r1,
                     bias_r2);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Residual streams.  x [T, S, D] float32: S copies of the residual of every row.
//   write (with y):   x[t][b] <- sum_a mix[a][b] x[t][a] + out_w[b] y[t]      (all b from the old copies)
//   read  (with in_w): u = sum_a in_w[a] x[t][a];  h[t] = u / sqrt(mean(u^2) + eps) * norm_w   (norm_w may be absent)
// One launch does the write, the read, or the write and then the read of the new copies.  `rows` (read only):
// h[r] is made from x[rows[r]].
// ---------------------------------------------------------------------------
template <int NT>
__global__ __launch_bounds__(NT) void streams_step_kernel(float* __restrict__ x, int S, int D, const void* __restrict__ y,
                                                          int y_dtype, int ldy, const float* __restrict__ mix,
                                                          const float* __restrict__ out_w,
                                                          const float* __restrict__ in_w,
                                                          const float* __restrict__ norm_w, float eps,
                                                          void* __restrict__ h, int h_dtype, int ldh,
                                                          const int* __restrict__ rows) {
  __shared__ float red[NT / WAVE];
  __shared__ float w_mix[MAX_STREAMS * MAX_STREAMS], w_out[MAX_STREAMS], w_in[MAX_STREAMS];
  const int r = blockIdx.x;
  const size_t t = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + t * (size_t)S * D;
  if (threadIdx.x < S * S && y) w_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (y) w_out[threadIdx.x] = out_w[threadIdx.x];
    if (in_w) w_in[threadIdx.x] = in_w[threadIdx.x];
  }
  __syncthreads();
  float ss = 0.f;
  for (int i = threadIdx.x; i < D; i += NT) {
    float v[MAX_STREAMS];
#pragma unroll
    for (int a = 0; a < MAX_STREAMS; ++a)
      if (a < S) v[a] = xr[(size_t)a * D + i];
    if (y) {
      const float yy = load_f(y, y_dtype, t * ldy + i);
      float nv[MAX_STREAMS];
#pragma unroll
      for (int b = 0; b < MAX_STREAMS; ++b) {
        if (b < S) {
          float acc = 0.f;
#pragma unroll
          for (int a = 0; a < MAX_STREAMS; ++a)
            if (a < S) acc = fmaf(w_mix[a * S + b], v[a], acc);
          nv[b] = fmaf(w_out[b], yy, acc);
        }
      }
#pragma unroll
      for (int b = 0; b < MAX_STREAMS; ++b)
        if (b < S) { v[b] = nv[b]; xr[(size_t)b * D + i] = nv[b]; }
    }
    if (in_w) {
      float u = 0.f;
#pragma unroll
      for (int a = 0; a < MAX_STREAMS; ++a)
        if (a < S) u = fmaf(w_in[a], v[a], u);
      ss = fmaf(u, u, ss);
    }
  }
  if (!in_w) return;
  ss = block_sum<NT>(ss, red);            // (its barriers also order this thread's writes of x before the reads below)
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += NT) {   // the same thread re-reads the elements it wrote
    float u = 0.f;
#pragma unroll
    for (int a = 0; a < MAX_STREAMS; ++a)
      if (a < S) u = fmaf(w_in[a], xr[(size_t)a * D + i], u);
    store_f(h, h_dtype, (size_t)r * ldh + i, norm_w ? (u * inv) * norm_w[i] : u * inv);
  }
}

// The same for widths that are a multiple of 4 and at most NT * 4 * VPT, 16 bytes a load: what a thread reads of the
// row stays in registers between the sum of squares and the scaling.  Which of the two kernels runs is fixed by the
// width and the alignment alone, never by the batch.
template <int NT, int VPT>
__global__ __launch_bounds__(NT) void streams_step_f4_kernel(float* __restrict__ x, int S, int D,
                                                             const void* __restrict__ y, int y_dtype, int ldy,
                                                             const float* __restrict__ mix,
                                                             const float* __restrict__ out_w,
                                                             const float* __restrict__ in_w,
                                                             const float* __restrict__ norm_w, float eps,
                                                             void* __restrict__ h, int h_dtype, int ldh,
                                                             const int* __restrict__ rows) {
  __shared__ float red[NT / WAVE];
  __shared__ float w_mix[MAX_STREAMS * MAX_STREAMS], w_out[MAX_STREAMS], w_in[MAX_STREAMS];
  const int r = blockIdx.x;
  const size_t t = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + t * (size_t)S * D;
  if (threadIdx.x < S * S && y) w_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (y) w_out[threadIdx.x] = out_w[threadIdx.x];
    if (in_w) w_in[threadIdx.x] = in_w[threadIdx.x];
  }
  __syncthreads();
  const int n4 = D / 4;
  float4 u[VPT];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * NT;
    u[k] = float4{0.f, 0.f, 0.f, 0.f};
    if (i >= n4) continue;
    float4 v[MAX_STREAMS];
#pragma unroll
    for (int a = 0; a < MAX_STREAMS; ++a)
      if (a < S) v[a] = reinterpret_cast<const float4*>(xr + (size_t)a * D)[i];
    if (y) {
      float4 yy;
      if (y_dtype == APC_F32) {
        yy = reinterpret_cast<const float4*>((const float*)y + t * ldy)[i];
      } else {
        const uint2 p = reinterpret_cast<const uint2*>((const bf16_t*)y + t * ldy)[i];
        yy = float4{__uint_as_float(p.x << 16), __uint_as_float(p.x & 0xffff0000u), __uint_as_float(p.y << 16),
                    __uint_as_float(p.y & 0xffff0000u)};
      }
      float4 nv[MAX_STREAMS];
#pragma unroll
      for (int b = 0; b < MAX_STREAMS; ++b) {
        if (b < S) {
          float4 acc = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int a = 0; a < MAX_STREAMS; ++a) {
            if (a < S) {
              const float m = w_mix[a * S + b];
              acc.x = fmaf(m, v[a].x, acc.x); acc.y = fmaf(m, v[a].y, acc.y);
              acc.z = fmaf(m, v[a].z, acc.z); acc.w = fmaf(m, v[a].w, acc.w);
            }
          }
          const float o = w_out[b];
          nv[b] = float4{fmaf(o, yy.x, acc.x), fmaf(o, yy.y, acc.y), fmaf(o, yy.z, acc.z), fmaf(o, yy.w, acc.w)};
        }
      }
#pragma unroll
      for (int b = 0; b < MAX_STREAMS; ++b)
        if (b < S) { v[b] = nv[b]; reinterpret_cast<float4*>(xr + (size_t)b * D)[i] = nv[b]; }
    }
    if (in_w) {
      float4 acc = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int a = 0; a < MAX_STREAMS; ++a) {
        if (a < S) {
          const float m = w_in[a];
          acc.x = fmaf(m, v[a].x, acc.x); acc.y = fmaf(m, v[a].y, acc.y);
          acc.z = fmaf(m, v[a].z, acc.z); acc.w = fmaf(m, v[a].w, acc.w);
        }
      }
      u[k] = acc;
      ss = fmaf(acc.x, acc.x, ss); ss = fmaf(acc.y, acc.y, ss); ss = fmaf(acc.z, acc.z, ss); ss = fmaf(acc.w, acc.w, ss);
    }
  }
  if (!in_w) return;
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * NT;
    if (i >= n4) continue;
    float4 g = float4{1.f, 1.f, 1.f, 1.f};
    if (norm_w) g = reinterpret_cast<const float4*>(norm_w)[i];
    const float4 o = float4{(u[k].x * inv) * g.x, (u[k].y * inv) * g.y, (u[k].z * inv) * g.z, (u[k].w * inv) * g.w};
    if (h_dtype == APC_F32) {
      reinterpret_cast<float4*>((float*)h + (size_t)r * ldh)[i] = o;
    } else {
      uint2 p;
      p.x = pack_bf16x2(o.x, o.y);
      p.y = pack_bf16x2(o.z, o.w);
      reinterpret_cast<uint2*>((bf16_t*)h + (size_t)r * ldh)[i] = p;
    }
  }
}

// One stream (S = 1) with a sublayer's output to add: x <- mix x + out_w y, h = rms_norm(in_w x) * norm_w.  The same
// arithmetic in the same order as the kernel above; every load of the row is issued before the first store, so a
// thread waits for memory once and not once a piece.
template <int NT, int VPT>
__global__ __launch_bounds__(NT) void stream_add_f4_kernel(float* __restrict__ x, int D, const void* __restrict__ y,
                                                           int y_dtype, int ldy, const float* __restrict__ mix,
                                                           const float* __restrict__ out_w,
                                                           const float* __restrict__ in_w,
                                                           const float* __restrict__ norm_w, float eps,
                                                           void* __restrict__ h, int h_dtype, int ldh) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x, n4 = D / 4;
  float4* xr = reinterpret_cast<float4*>(x + (size_t)r * D);
  const float m = mix[0], o = out_w[0], wi = in_w ? in_w[0] : 0.f;
  float4 v[VPT], yy[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * NT;
    v[k] = yy[k] = float4{0.f, 0.f, 0.f, 0.f};
    if (i >= n4) continue;
    v[k] = xr[i];
    if (y_dtype == APC_F32) {
      yy[k] = reinterpret_cast<const float4*>((const float*)y + (size_t)r * ldy)[i];
    } else {
      const uint2 p = reinterpret_cast<const uint2*>((const bf16_t*)y + (size_t)r * ldy)[i];
      yy[k] = float4{__uint_as_float(p.x << 16), __uint_as_float(p.x & 0xffff0000u), __uint_as_float(p.y << 16),
                     __uint_as_float(p.y & 0xffff0000u)};
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * NT;
    if (i >= n4) continue;
    float4 a = float4{fmaf(m, v[k].x, 0.f), fmaf(m, v[k].y, 0.f), fmaf(m, v[k].z, 0.f), fmaf(m, v[k].w, 0.f)};
    a = float4{fmaf(o, yy[k].x, a.x), fmaf(o, yy[k].y, a.y), fmaf(o, yy[k].z, a.z), fmaf(o, yy[k].w, a.w)};
    xr[i] = a;
    if (in_w) {
      a = float4{fmaf(wi, a.x, 0.f), fmaf(wi, a.y, 0.f), fmaf(wi, a.z, 0.f), fmaf(wi, a.w, 0.f)};
      ss = fmaf(a.x, a.x, ss); ss = fmaf(a.y, a.y, ss); ss = fmaf(a.z, a.z, ss); ss = fmaf(a.w, a.w, ss);
    }
    v[k] = a;
  }
  if (!in_w) return;
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * NT;
    if (i >= n4) continue;
    float4 g = float4{1.f, 1.f, 1.f, 1.f};
    if (norm_w) g = reinterpret_cast<const float4*>(norm_w)[i];
    const float4 u = float4{(v[k].x * inv) * g.x, (v[k].y * inv) * g.y, (v[k].z * inv) * g.z, (v[k].w * inv) * g.w};
    if (h_dtype == APC_F32) {
      reinterpret_cast<float4*>((float*)h + (size_t)r * ldh)[i] = u;
    } else {
      uint2 p;
      p.x = pack_bf16x2(u.x, u.y);
      p.y = pack_bf16x2(u.z, u.w);
      reinterpret_cast<uint2*>((bf16_t*)h + (size_t)r * ldh)[i] = p;
    }
  }
}

APC_EXPORT int apc_streams_step(float* x, int n_rows, int S, int D, const void* y, int y_dtype, int ldy,
                                const float* mix, const float* out_w, const float* in_w, const float* norm_w, float eps,
                                void* h, int h_dtype, int ldh, const int* rows, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (S <= 0 || D <= 0 || (y && (!mix || !out_w || ldy < D)) || (in_w && (!h || ldh < D)) || (!y && !in_w) ||
      (rows && y))
    return APC_ERR_BAD_ARG;
  if (S > MAX_STREAMS) return APC_ERR_UNSUPPORTED;
  const bool wide = D % 4 == 0 && D <= 256 * 4 * 8 && !((uintptr_t)x & 15u) && !((uintptr_t)norm_w & 15u) &&
                    (!y || (ldy % 4 == 0 && !((uintptr_t)y & 15u))) && (!in_w || (ldh % 4 == 0 && !((uintptr_t)h & 15u)));
  if (wide && S == 1 && y && !rows) {
#define SA_LAUNCH(VPT_)                                                                                           \
  hipLaunchKernelGGL((stream_add_f4_kernel<256, VPT_>), dim3(n_rows), dim3(256), 0, stream, x, D, y, y_dtype, ldy, \
                     mix, out_w, in_w, norm_w, eps, h, h_dtype, ldh)
    if (D <= 1024) SA_LAUNCH(1);
    else if (D <= 2048) SA_LAUNCH(2);
    else if (D <= 4096) SA_LAUNCH(4);
    else SA_LAUNCH(8);
#undef SA_LAUNCH
    APC_LAUNCH_CHECK();
    return 0;
  }
  if (wide) {
#define ST_LAUNCH(VPT_)                                                                                              \
  hipLaunchKernelGGL((streams_step_f4_kernel<256, VPT_>), dim3(n_rows), dim3(256), 0, stream, x, S, D, y, y_dtype, ldy, \
                     mix, out_w, in_w, norm_w, eps, h, h_dtype, ldh, rows)
    if (D <= 1024) ST_LAUNCH(1);
    else if (D <= 2048) ST_LAUNCH(2);
    else if (D <= 4096) ST_LAUNCH(4);
    else ST_LAUNCH(8);
#undef ST_LAUNCH
    APC_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(streams_step_kernel<256>, dim3(n_rows), dim3(256), 0, stream, x, S, D, y, y_dtype, ldy, mix, out_w,
                     in_w, norm_w, eps, h, h_dtype, ldh, rows);
  APC_LAUNCH_CHECK();
  return 0;
}

// Token rows through an RMS norm into every stream: x[t][a] = e / sqrt(mean(e^2) + eps) * w, e = table[tokens[t]]
// (without w: x[t][a] = e).
template <int NT>
__global__ __launch_bounds__(NT) void embed_streams_kernel(const void* __restrict__ table, int table_dtype,
                                                           const int* __restrict__ tokens,
                                                           const float* __restrict__ w, float eps,
                                                           float* __restrict__ x, int S, int D) {
  __shared__ float red[NT / WAVE];
  const int t = blockIdx.x;
  const size_t src = (size_t)tokens[t] * D;
  float inv = 1.f;
  if (w) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) {
      const float v = load_f(table, table_dtype, src + i);
      ss = fmaf(v, v, ss);
    }
    ss = block_sum<NT>(ss, red);
    inv = 1.0f / sqrtf(ss / (float)D + eps);
  }
  for (int i = threadIdx.x; i < D; i += NT) {
    const float e = load_f(table, table_dtype, src + i);
    const float v = w ? (e * inv) * w[i] : e;
    for (int a = 0; a < S; ++a) x[((size_t)t * S + a) * D + i] = v;
  }
}

APC_EXPORT int apc_embed_streams(const void* table, int table_dtype, const int* tokens, const float* w, float eps,
                                 float* x, int n_tok, int S, int D, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (S <= 0 || D <= 0) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(embed_streams_kernel<256>, dim3(n_tok), dim3(256), 0, stream, table, table_dtype, tokens, w, eps,
                     x, S, D);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Clamped gated activation: g = min(gu[t][f], limit), u = clamp(gu[t][F + f], -limit, limit),
// out = g * sigmoid(alpha g) * (u + 1).
// ---------------------------------------------------------------------------
__global__ void clamped_glu_kernel(const void* __restrict__ gu, int in_dtype, int ldg, void* __restrict__ out,
                                   int out_dtype, int ldo, int F, float alpha, float limit) {
  const int t = blockIdx.y;
  const int f = blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= F) return;
  const float g = fminf(load_f(gu, in_dtype, (size_t)t * ldg + f), limit);
  const float u = fminf(fmaxf(load_f(gu, in_dtype, (size_t)t * ldg + F + f), -limit), limit);
  store_f(out, out_dtype, (size_t)t * ldo + f, (g / (1.0f + expf(-alpha * g))) * (u + 1.0f));
}

// The same for bfloat16 rows whose width is a multiple of 8, 16 bytes a load.
__global__ void clamped_glu_bf16x8_kernel(const bf16_t* __restrict__ gu, int ldg, bf16_t* __restrict__ out, int ldo,
                                          int F, float alpha, float limit) {
  const int t = blockIdx.y;
  const int f = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (f >= F) return;
  const uint4 g4 = *reinterpret_cast<const uint4*>(gu + (size_t)t * ldg + f);
  const uint4 u4 = *reinterpret_cast<const uint4*>(gu + (size_t)t * ldg + F + f);
  const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
  uint32_t ow[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    float r[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const float g = fminf(__uint_as_float(k ? (gw[w] & 0xffff0000u) : (gw[w] << 16)), limit);
      const float u = fminf(fmaxf(__uint_as_float(k ? (uw[w] & 0xffff0000u) : (uw[w] << 16)), -limit), limit);
      r[k] = (g / (1.0f + expf(-alpha * g))) * (u + 1.0f);
    }
    ow[w] = pack_bf16x2(r[0], r[1]);
  }
  *reinterpret_cast<uint4*>(out + (size_t)t * ldo + f) = uint4{ow[0], ow[1], ow[2], ow[3]};
}

APC_EXPORT int apc_clamped_glu(const void* gu, int in_dtype, int ldg, void* out, int out_dtype, int ldo, int n_rows,
                               int F, float alpha, float limit, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (F <= 0 || ldg < 2 * F || ldo < F || n_rows > 65535) return APC_ERR_BAD_ARG;
  if (in_dtype == APC_BF16 && out_dtype == APC_BF16 && F % 8 == 0 && ldg % 8 == 0 && ldo % 8 == 0 &&
      !((uintptr_t)gu & 15u) && !((uintptr_t)out & 15u)) {
    hipLaunchKernelGGL(clamped_glu_bf16x8_kernel, dim3(ceil_div(F / 8, 256), n_rows), dim3(256), 0, stream,
                       (const bf16_t*)gu, ldg, (bf16_t*)out, ldo, F, alpha, limit);
    APC_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(clamped_glu_kernel, dim3(ceil_div(F, 256), n_rows), dim3(256), 0, stream, gu, in_dtype, ldg, out,
                     out_dtype, ldo, F, alpha, limit);
  APC_LAUNCH_CHECK();
  return 0;
}

// x *= s (float32, contiguous)
__global__ void scale_kernel(float* __restrict__ x, float s, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] *= s;
}

APC_EXPORT int apc_scale(float* x, float s, size_t n, hipStream_t stream) {
  if (n == 0) return 0;
  const size_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffu) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(scale_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, s, n);
  APC_LAUNCH_CHECK();
  return 0;
}
