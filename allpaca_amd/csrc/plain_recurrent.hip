// Plain kernels of: an embedding with a scale and learned position vectors; a residual sum that takes a sublayer's
// output through an RMS norm first; linear attention with a decay per head and a matrix of state per request; an RMS
// norm over concatenated heads with a sigmoid gate; the combination of the maps of a differential attention.
// One obvious loop nest each, all arithmetic in 32-bit float with an order of additions that the row's own place
// fixes (never the batch), any element type in and out.
#include "common.h"
#include <math.h>

namespace {

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// silu of a projected value, held in the rows' own element type like every activation of a run
__device__ __forceinline__ float act_silu(float z, int dtype) {
  const float a = z * sigmoid_f(z);
  return dtype == APC_BF16 ? bf16_to_float(float_to_bf16(a)) : a;
}

// x[t] = table[tokens[t]] * scale + pos_table[positions[t]]
__global__ void embed_positions_kernel(const void* __restrict__ table, int table_dtype, const int* __restrict__ tokens,
                                       const void* __restrict__ pos_table, int pos_dtype,
                                       const int* __restrict__ positions, float scale, float* __restrict__ out, int ldo,
                                       int dim) {
  const int t = blockIdx.x;
  const size_t a = (size_t)tokens[t] * dim, b = (size_t)positions[t] * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x)
    out[(size_t)t * ldo + i] = load_f(table, table_dtype, a + i) * scale + load_f(pos_table, pos_dtype, b + i);
}

// x[t] += mult * (y[t] / sqrt(mean(y[t]^2) + eps)) * w ;  optionally copy[t] = x[t] in another element type (what the
// next sublayer multiplies with)
template <int NT>
__global__ __launch_bounds__(NT) void rmsnorm_add_kernel(const void* __restrict__ y, int y_dtype, int ldy,
                                                         const float* __restrict__ w, float eps, float mult,
                                                         float* __restrict__ x, int ldx, void* __restrict__ copy,
                                                         int copy_dtype, int ldc, int dim) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += NT) {
    const float v = load_f(y, y_dtype, (size_t)r * ldy + i);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  for (int i = threadIdx.x; i < dim; i += NT) {
    const float v = load_f(y, y_dtype, (size_t)r * ldy + i);
    const float nx = x[(size_t)r * ldx + i] + mult * ((v * inv) * w[i]);
    x[(size_t)r * ldx + i] = nx;
    if (copy) store_f(copy, copy_dtype, (size_t)r * ldc + i, nx);
  }
}

// The same for float32 rows whose width is a multiple of 4 and at most NT*4*VPT: every thread keeps its elements of
// y in registers between the sum and the scaling, and all its loads are in flight together.  Which of the two kernels
// runs, and so the order of the additions, is fixed by the width and the alignment of the rows alone.
template <int NT, int VPT>
__global__ __launch_bounds__(NT) void rmsnorm_add_f4_kernel(const float* __restrict__ y, int ldy,
                                                            const float* __restrict__ w, float eps, float mult,
                                                            float* __restrict__ x, int ldx, void* __restrict__ copy,
                                                            int copy_dtype, int ldc, int dim) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x, n4 = dim / 4;
  const float4* src = reinterpret_cast<const float4*>(y + (size_t)r * ldy);
  float4* xr = reinterpret_cast<float4*>(x + (size_t)r * ldx);
  float4 v[VPT], old[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * NT;
    v[j] = i < n4 ? src[i] : float4{0.f, 0.f, 0.f, 0.f};
    old[j] = i < n4 ? xr[i] : float4{0.f, 0.f, 0.f, 0.f};
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    ss = fmaf(v[j].x, v[j].x, ss);
    ss = fmaf(v[j].y, v[j].y, ss);
    ss = fmaf(v[j].z, v[j].z, ss);
    ss = fmaf(v[j].w, v[j].w, ss);
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  const float4* w4 = reinterpret_cast<const float4*>(w);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * NT;
    if (i >= n4) continue;
    const float4 g = w4[i];
    const float4 nx = float4{old[j].x + mult * ((v[j].x * inv) * g.x), old[j].y + mult * ((v[j].y * inv) * g.y),
                             old[j].z + mult * ((v[j].z * inv) * g.z), old[j].w + mult * ((v[j].w * inv) * g.w)};
    xr[i] = nx;
    if (copy) {
      const size_t at = (size_t)r * ldc + (size_t)i * 4;
      if (copy_dtype == APC_F32) {
        *reinterpret_cast<float4*>((float*)copy + at) = nx;
      } else {
        uint2 pk;
        pk.x = pack_bf16x2(nx.x, nx.y);
        pk.y = pack_bf16x2(nx.z, nx.w);
        *reinterpret_cast<uint2*>((bf16_t*)copy + at) = pk;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Linear attention with a decay: per head S <- decay * S + k_t v_t^T, o_t = S^T q_t, S [dk][dv] float32 per request.
// proj [T, ld] holds q heads at q_off (H of dk), k heads at k_off (H of dk), v heads at v_off (H of dv); with `act`
// q, k and v pass silu first.  A block takes one segment x one head x 64 value columns and walks the segment's rows
// in order; thread (rg, j) keeps rows rg, rg + 4, ... of column j of S in registers.  The sum over a column's rows
// is added in an order fixed by dk alone.
// With `rot` > 0 the first rot elements of every q and k head are rotated by the row's position (pairs i, i + rot/2:
// (x, y) -> (x c - y s, y c + x s), c and s from cos_sin[position][2][rot/2]); k is multiplied by `k_scale` behind the
// rotation.  Both in 32-bit: what enters the state is never rounded.
// ---------------------------------------------------------------------------
template <int RPT>   // rows of S a thread keeps: dk <= 4 * RPT
__global__ __launch_bounds__(256) void linear_attention_kernel(
    const void* __restrict__ proj, int in_dtype, int ld, int q_off, int k_off, int v_off, int H, int dk, int dv, int act,
    const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ seg_row0,
    const int* __restrict__ seg_rows, const int* __restrict__ slots, float* __restrict__ out, int ldo, int rot,
    const float* __restrict__ cos_sin, const int* __restrict__ positions, float k_scale) {
  __shared__ float qs[2][4 * RPT], ks[2][4 * RPT];
  __shared__ float red[4][64];
  const int seg = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * 64;
  const int tid = threadIdx.x, j = tid % 64, rg = tid / 64;
  const int col = j0 + j;
  const bool on = col < dv;
  const int r0 = seg_row0[seg], n = seg_rows[seg];
  float* S = state + (((size_t)slots[seg] * H + h) * dk) * dv;
  const float lam = decay[h];
  float s[RPT];
#pragma unroll
  for (int ii = 0; ii < RPT; ++ii) {
    const int i = rg + 4 * ii;
    s[ii] = (on && i < dk) ? S[(size_t)i * dv + col] : 0.f;
  }
  for (int t = 0; t < n; ++t) {
    const size_t row = (size_t)(r0 + t) * ld;
    const int b = t & 1;
    for (int i = tid; i < dk; i += 256) {
      float qv = load_f(proj, in_dtype, row + q_off + (size_t)h * dk + i);
      float kv = load_f(proj, in_dtype, row + k_off + (size_t)h * dk + i);
      if (act) { qv = act_silu(qv, in_dtype); kv = act_silu(kv, in_dtype); }
      if (i < rot) {
        const int half = rot / 2;
        const bool first = i < half;
        const int f = first ? i : i - half, other = first ? i + half : i - half;
        const float* cs = cos_sin + (size_t)positions[r0 + t] * rot;
        const float c = cs[f], sn = cs[half + f];
        float qo = load_f(proj, in_dtype, row + q_off + (size_t)h * dk + other);
        float ko = load_f(proj, in_dtype, row + k_off + (size_t)h * dk + other);
        if (act) { qo = act_silu(qo, in_dtype); ko = act_silu(ko, in_dtype); }
        qv = first ? qv * c - qo * sn : qv * c + qo * sn;
        kv = first ? kv * c - ko * sn : kv * c + ko * sn;
      }
      qs[b][i] = qv;
      ks[b][i] = kv * k_scale;
    }
    float vv = on ? load_f(proj, in_dtype, row + v_off + (size_t)h * dv + col) : 0.f;
    if (act) vv = act_silu(vv, in_dtype);
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int ii = 0; ii < RPT; ++ii) {
      const int i = rg + 4 * ii;
      if (i < dk) {
        s[ii] = fmaf(lam, s[ii], ks[b][i] * vv);
        acc = fmaf(s[ii], qs[b][i], acc);
      }
    }
    red[rg][j] = acc;
    __syncthreads();
    if (rg == 0 && on) out[(size_t)(r0 + t) * ldo + (size_t)h * dv + col] = ((red[0][j] + red[1][j]) + red[2][j]) + red[3][j];
    // (the next row writes the other halves of qs / ks, and `red` only after its own barrier, which every thread
    // reaches after it has read `red` here)
  }
  if (on) {
#pragma unroll
    for (int ii = 0; ii < RPT; ++ii) {
      const int i = rg + 4 * ii;
      if (i < dk) S[(size_t)i * dv + col] = s[ii];
    }
  }
}

// The same with the mean taken over each group of `group` consecutive elements (a head) for itself: one wave a group.
// `w` [dim] may be absent; gate_kind 0: times sigmoid(gate), 1: times silu(gate).
__global__ __launch_bounds__(64) void gated_groupnorm_kernel(const float* __restrict__ o, int ldo_in,
                                                             const float* __restrict__ w, float eps,
                                                             const void* __restrict__ gate, int gate_dtype, int ldg,
                                                             int gate_kind, void* __restrict__ out, int out_dtype,
                                                             int ldo, int group) {
  const int r = blockIdx.x, c0 = blockIdx.y * group, lane = threadIdx.x;
  float ss = 0.f;
  for (int i = lane; i < group; i += WAVE) {
    const float v = o[(size_t)r * ldo_in + c0 + i];
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)group + eps);
  for (int i = lane; i < group; i += WAVE) {
    float v = o[(size_t)r * ldo_in + c0 + i] * inv;
    if (w) v *= w[c0 + i];
    if (gate) {
      const float z = load_f(gate, gate_dtype, (size_t)r * ldg + c0 + i);
      v *= gate_kind == 1 ? z * sigmoid_f(z) : sigmoid_f(z);
    }
    store_f(out, out_dtype, (size_t)r * ldo + c0 + i, v);
  }
}

// out[t] = (o[t] / sqrt(mean(o[t]^2) + eps)) * w * sigmoid(gate[t]), over the whole row of concatenated heads
template <int NT>
__global__ __launch_bounds__(NT) void gated_rmsnorm_kernel(const float* __restrict__ o, int ldo_in,
                                                           const float* __restrict__ w, float eps,
                                                           const void* __restrict__ gate, int gate_dtype, int ldg,
                                                           void* __restrict__ out, int out_dtype, int ldo, int dim) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += NT) {
    const float v = o[(size_t)r * ldo_in + i];
    ss = fmaf(v, v, ss);
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  for (int i = threadIdx.x; i < dim; i += NT) {
    const float v = (o[(size_t)r * ldo_in + i] * inv) * w[i];
    const float g = gate ? sigmoid_f(load_f(gate, gate_dtype, (size_t)r * ldg + i)) : 1.f;
    store_f(out, out_dtype, (size_t)r * ldo + i, v * g);
  }
}

// ---------------------------------------------------------------------------
// Two softmax maps of a head over the same values, a [T][H][2][dv] float32:
//   o = a1 - lam * a2;  out = o / sqrt(mean_dv(o^2) + eps) * post * sigmoid(gate[t][h])   (gate: one number a head)
// One wave per (row, head).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void diff_combine_kernel(const float* __restrict__ a, int lda, float lam, float post,
                                                          float eps, const void* __restrict__ gate, int gate_dtype,
                                                          int ldg, void* __restrict__ out, int out_dtype, int ldo,
                                                          int H, int dv) {
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* a1 = a + (size_t)r * lda + (size_t)h * 2 * dv;
  const float* a2 = a1 + dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += WAVE) {
    const float o = a1[i] - lam * a2[i];
    ss = fmaf(o, o, ss);
  }
  ss = wave_sum(ss);
  float f = post / sqrtf(ss / (float)dv + eps);
  if (gate) f *= sigmoid_f(load_f(gate, gate_dtype, (size_t)r * ldg + h));
  for (int i = lane; i < dv; i += WAVE)
    store_f(out, out_dtype, (size_t)r * ldo + (size_t)h * dv + i, (a1[i] - lam * a2[i]) * f);
}

}  // namespace

APC_EXPORT int apc_embed_positions(const void* table, int table_dtype, const int* tokens, const void* pos_table,
                                   int pos_dtype, const int* positions, float scale, float* out, int ldo, int n_rows,
                                   int dim, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (dim <= 0 || ldo < dim || !table || !pos_table || !tokens || !positions) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(embed_positions_kernel, dim3(n_rows), dim3(256), 0, stream, table, table_dtype, tokens, pos_table,
                     pos_dtype, positions, scale, out, ldo, dim);
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_rmsnorm_add(const void* y, int y_dtype, int ldy, const float* w, float eps, float mult, float* x,
                               int ldx, void* copy, int copy_dtype, int ldc, int n_rows, int dim, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (dim <= 0 || ldy < dim || ldx < dim || (copy && ldc < dim)) return APC_ERR_BAD_ARG;
  const bool vec = y_dtype == APC_F32 && dim % 4 == 0 && ldy % 4 == 0 && ldx % 4 == 0 && (!copy || ldc % 4 == 0) &&
                   dim <= 256 * 4 * 8 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)x % 16) == 0 &&
                   ((uintptr_t)w % 16) == 0 && ((uintptr_t)copy % 16) == 0;
  if (vec) {
    const int n4 = dim / 4;
#define RA_LAUNCH(VPT_)                                                                                          \
  hipLaunchKernelGGL((rmsnorm_add_f4_kernel<256, VPT_>), dim3(n_rows), dim3(256), 0, stream, (const float*)y, ldy, \
                     w, eps, mult, x, ldx, copy, copy_dtype, ldc, dim)
    if (n4 <= 256) RA_LAUNCH(1);
    else if (n4 <= 512) RA_LAUNCH(2);
    else if (n4 <= 1024) RA_LAUNCH(4);
    else RA_LAUNCH(8);
#undef RA_LAUNCH
  } else {
    hipLaunchKernelGGL(rmsnorm_add_kernel<256>, dim3(n_rows), dim3(256), 0, stream, y, y_dtype, ldy, w, eps, mult, x,
                       ldx, copy, copy_dtype, ldc, dim);
  }
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_linear_attention(const void* proj, int in_dtype, int ld, int q_off, int k_off, int v_off, int H,
                                    int dk, int dv, int act, const float* decay, float* state, int n_segs,
                                    const int* seg_row0, const int* seg_rows, const int* slots, float* out, int ldo,
                                    int rot, const float* cos_sin, const int* positions, float k_scale,
                                    hipStream_t stream) {
  if (n_segs <= 0) return 0;
  if (H <= 0 || dk <= 0 || dv <= 0 || !decay || !state || !slots || ldo < H * dv) return APC_ERR_BAD_ARG;
  if (rot < 0 || rot % 2 || rot > dk || (rot && (!cos_sin || !positions))) return APC_ERR_BAD_ARG;
  if (dk > 256 || H > 65535 || n_segs > 0x7fffffff / 1) return APC_ERR_UNSUPPORTED;
  dim3 grid(n_segs, H, ceil_div(dv, 64));
  if (grid.z > 65535) return APC_ERR_UNSUPPORTED;
#define LA_LAUNCH(RPT_)                                                                                            \
  hipLaunchKernelGGL(linear_attention_kernel<RPT_>, grid, dim3(256), 0, stream, proj, in_dtype, ld, q_off, k_off, \
                     v_off, H, dk, dv, act, decay, state, seg_row0, seg_rows, slots, out, ldo, rot, cos_sin, positions,  \
                     k_scale)
  if (dk <= 32) LA_LAUNCH(8);
  else if (dk <= 64) LA_LAUNCH(16);
  else if (dk <= 128) LA_LAUNCH(32);
  else LA_LAUNCH(64);
#undef LA_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_gated_rmsnorm(const float* o, int ldo_in, const float* w, float eps, const void* gate, int gate_dtype,
                                 int ldg, void* out, int out_dtype, int ldo, int n_rows, int dim, int group,
                                 int gate_kind, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (dim <= 0 || ldo_in < dim || ldo < dim || (gate && ldg < dim)) return APC_ERR_BAD_ARG;
  if (group < 0 || (group && dim % group) || gate_kind < 0 || gate_kind > 1) return APC_ERR_BAD_ARG;
  if (group || !w || gate_kind) {
    const int g = group ? group : dim;
    if (dim / g > 65535) return APC_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(gated_groupnorm_kernel, dim3(n_rows, dim / g), dim3(64), 0, stream, o, ldo_in, w, eps, gate,
                       gate_dtype, ldg, gate_kind, out, out_dtype, ldo, g);
    APC_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(gated_rmsnorm_kernel<256>, dim3(n_rows), dim3(256), 0, stream, o, ldo_in, w, eps, gate, gate_dtype,
                     ldg, out, out_dtype, ldo, dim);
  APC_LAUNCH_CHECK();
  return 0;
}

APC_EXPORT int apc_diff_combine(const float* a, int lda, float lam, float post, float eps, const void* gate,
                                int gate_dtype, int ldg, void* out, int out_dtype, int ldo, int n_rows, int H, int dv,
                                hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || dv <= 0 || lda < 2 * H * dv || ldo < H * dv || H > 65535) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(diff_combine_kernel, dim3(n_rows, H), dim3(64), 0, stream, a, lda, lam, post, eps, gate,
                     gate_dtype, ldg, out, out_dtype, ldo, H, dv);
  APC_LAUNCH_CHECK();
  return 0;
}
