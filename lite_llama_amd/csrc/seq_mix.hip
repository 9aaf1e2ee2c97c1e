// Sequence-mixing layers over RAGGED steps (several sequences, each bringing a run of consecutive tokens: a portion of a
// prompt, or one decoded token) with a 32-bit residual stream:
//
//   ll_add_rmsnorm_shift   residual add (fp32) + RMS norm (fp32) + optional token shift against the previous token's normed
//                          row (carried per sequence in a state slot) -> activations in the storage dtype; the update may come
//                          as one row plus several part rows per token (sublayers that ran side by side, experts' slots)
//   ll_embed_pair          token embedding times a scale plus a row of a hashed (previous token, token) table -> fp32 residual;
//                          the previous token of a run's first token is carried per sequence in a state slot
//   ll_xielu               the xIELU activation with its two learned numbers
//   ll_cast_pair / ll_residual_set   the two ends of a projection over [x ; x0] that re-enters the residual stream
//   ll_gated_linear_scan   per-head linear recurrence S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t with a
//                          lower-bounded forget gate and a per-head RMS norm of o (HGRN2), state in fp32 slots
//   ll_mingru_scan         per-channel gated recurrence S_t = (1 - z_t) S_(t-1) + z_t c_t whose gates read the current token
//                          only (minGRU), silu-gated read-out, state in fp32 slots
//
// Storage dtype DT = LL_F16 / LL_BF16 / LL_F32 for activations and weights; everything that the recurrence, the norms and
// the residual touch is fp32.  A step is described by   seq_start[b + 1] (first flat token of each sequence's run),
// seq_first_pos[b] (position of that token inside its sequence: 0 = the sequence starts here and carries no state yet),
// seq_slot[b] (state slot), and for per-token kernels tok_seq[n].
#include "common.h"

namespace {

template <int DT> struct Store { typedef uint16_t type; };
template <> struct Store<LL_F32> { typedef float type; };

template <int DT>
__device__ __forceinline__ float ldv(const void* p, int64_t i) {
  if constexpr (DT == LL_F32) return ((const float*)p)[i];
  else return to_f32<DT>(((const uint16_t*)p)[i]);
}
template <int DT>
__device__ __forceinline__ void stv(void* p, int64_t i, float v) {
  if constexpr (DT == LL_F32) ((float*)p)[i] = v;
  else ((uint16_t*)p)[i] = from_f32<DT>(v);
}

// sum over a 256-thread workgroup, same order for every caller (wave sums, then the four waves in order): the value a
// row's norm gets does not depend on which workgroup computes it
__device__ __forceinline__ float block_sum256(float v, float* lds4) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds4[wave] = v;
  __syncthreads();
  return ((lds4[0] + lds4[1]) + lds4[2]) + lds4[3];
}

// the update of row t at element i: delta row + the row's parts in order (either may be absent), fp32
template <int DT>
__device__ __forceinline__ float update_at(const void* delta, const void* parts, int num_parts, int64_t t, int width, int i) {
  float u = delta ? ldv<DT>(delta, t * width + i) : 0.f;
  if (parts) {
    float p = ldv<DT>(parts, (t * num_parts) * width + i);
    for (int k = 1; k < num_parts; ++k) p += ldv<DT>(parts, (t * num_parts + k) * width + i);
    u = delta ? u + p : p;
  }
  return u;
}

// One workgroup per token.  s = x_in + delta (fp32; written to x_out when delta is given), h = s / sqrt(mean(s^2) + eps) * w,
// y = h + (h_prev - h) * shift, h_prev = the same h of the previous token of the sequence: recomputed from the previous row
// when that token is part of this step, read from the sequence's state slot when the run starts inside the sequence, zero
// at position 0.  The last token of a run leaves its h in the other half of the slot pair (state is double-buffered by the
// per-sequence parity: a run's first token reads while its last token writes).
template <int DT>
__global__ __launch_bounds__(256) void add_rmsnorm_shift_kernel(
    const float* __restrict__ x_in, const void* __restrict__ delta, float* __restrict__ x_out, const void* __restrict__ weight,
    const void* __restrict__ shift, void* __restrict__ y, int64_t n, int width, float eps, const int32_t* __restrict__ tok_seq,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ seq_parity, float* __restrict__ state, int64_t state_half, const void* __restrict__ parts,
    int num_parts, float out_scale) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const float* xr = x_in + t * width;
  const bool upd = delta || parts;
  float ss = 0.f;
  for (int i = tid; i < width; i += 256) {
    float s = xr[i];
    if (upd) s += update_at<DT>(delta, parts, num_parts, t, width, i);
    ss += s * s;
  }
  ss = block_sum256(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  int mode = 0;  // 0: no shift, 1: previous row of this step, 2: state slot, 3: zeros
  int b = 0;
  const float* prev_state = nullptr;
  float inv_prev = 0.f;
  if (shift) {
    b = tok_seq[t];
    const int start = seq_start[b];
    if (t > start) {
      mode = 1;
      const float* pr = x_in + (t - 1) * width;
      float sp = 0.f;
      for (int i = tid; i < width; i += 256) {
        float s = pr[i];
        if (upd) s += update_at<DT>(delta, parts, num_parts, t - 1, width, i);
        sp += s * s;
      }
      sp = block_sum256(sp, red);
      inv_prev = 1.0f / sqrtf(sp / (float)width + eps);
    } else if (seq_first_pos[b] > 0) {
      mode = 2;
      prev_state = state + (int64_t)seq_parity[b] * state_half + (int64_t)seq_slot[b] * width;
    } else {
      mode = 3;
    }
  }
  float* keep = nullptr;
  if (shift && t == seq_start[b + 1] - 1)
    keep = state + (int64_t)(1 - seq_parity[b]) * state_half + (int64_t)seq_slot[b] * width;
  for (int i = tid; i < width; i += 256) {
    float s = xr[i];
    if (upd) {
      s += update_at<DT>(delta, parts, num_parts, t, width, i);
      x_out[t * width + i] = s;
    }
    const float w = ldv<DT>(weight, i);
    const float h = s * inv * w;
    float out = h;
    if (mode) {
      float hp = 0.f;
      if (mode == 1) {
        float s1 = x_in[(t - 1) * width + i];
        if (upd) s1 += update_at<DT>(delta, parts, num_parts, t - 1, width, i);
        hp = s1 * inv_prev * w;
      } else if (mode == 2) {
        hp = prev_state[i];
      }
      out = h + (hp - h) * ldv<DT>(shift, i);
      if (keep) keep[i] = h;
    }
    stv<DT>(y, t * width + i, out * out_scale);
  }
}


// Register-cached form of the kernel above for widths <= 4096 that are multiples of 4: every thread keeps its 4-element
// pieces of the row's sum (and of the previous row's) in registers -- one pass over global memory, 16-byte residual
// accesses, 8-byte (16-bit storage) activation accesses.  Same arithmetic and the same reduction order as the plain form.
template <int DT>
__device__ __forceinline__ f32x4 ld4(const void* p, int64_t i) {  // four storage-dtype values at element i (multiple of 4)
  if constexpr (DT == LL_F32) {
    return *reinterpret_cast<const f32x4*>((const float*)p + i);
  } else {
    const uint2 u = *reinterpret_cast<const uint2*>((const uint16_t*)p + i);
    return f32x4{to_f32<DT>((uint16_t)(u.x & 0xffff)), to_f32<DT>((uint16_t)(u.x >> 16)), to_f32<DT>((uint16_t)(u.y & 0xffff)),
                 to_f32<DT>((uint16_t)(u.y >> 16))};
  }
}
template <int DT>
__device__ __forceinline__ void st4(void* p, int64_t i, f32x4 v) {
  if constexpr (DT == LL_F32) {
    *reinterpret_cast<f32x4*>((float*)p + i) = v;
  } else {
    uint2 u;
    u.x = (uint32_t)from_f32<DT>(v[0]) | ((uint32_t)from_f32<DT>(v[1]) << 16);
    u.y = (uint32_t)from_f32<DT>(v[2]) | ((uint32_t)from_f32<DT>(v[3]) << 16);
    *reinterpret_cast<uint2*>((uint16_t*)p + i) = u;
  }
}

// update_at for four elements at i (a multiple of 4): the same sums in the same order
template <int DT>
__device__ __forceinline__ f32x4 update4(const void* delta, const void* parts, int num_parts, int64_t t, int width, int i) {
  f32x4 u = {0.f, 0.f, 0.f, 0.f};
  if (delta) u = ld4<DT>(delta, t * width + i);
  if (parts) {
    f32x4 p = ld4<DT>(parts, (t * num_parts) * width + i);
    for (int k = 1; k < num_parts; ++k) {
      const f32x4 q = ld4<DT>(parts, (t * num_parts + k) * width + i);
      p[0] += q[0]; p[1] += q[1]; p[2] += q[2]; p[3] += q[3];
    }
    if (delta) { u[0] += p[0]; u[1] += p[1]; u[2] += p[2]; u[3] += p[3]; }
    else u = p;
  }
  return u;
}

template <int DT, int NV>
__global__ __launch_bounds__(256) void add_rmsnorm_shift_vec_kernel(
    const float* __restrict__ x_in, const void* __restrict__ delta, float* __restrict__ x_out, const void* __restrict__ weight,
    const void* __restrict__ shift, void* __restrict__ y, int64_t n, int width, float eps, const int32_t* __restrict__ tok_seq,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ seq_parity, float* __restrict__ state, int64_t state_half, const void* __restrict__ parts,
    int num_parts, float out_scale) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  f32x4 s[NV], sp[NV];
  const bool upd = delta || parts;
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (tid + 256 * j) * 4;
    s[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (i < width) {
      s[j] = *reinterpret_cast<const f32x4*>(x_in + t * width + i);
      if (upd) {
        const f32x4 d = update4<DT>(delta, parts, num_parts, t, width, i);
        s[j][0] += d[0]; s[j][1] += d[1]; s[j][2] += d[2]; s[j][3] += d[3];
      }
      // (element order i, i + 1, ..: the plain form adds the same values thread by thread in steps of 256 -- the per-thread
      // partial sums differ, so the two forms agree to rounding, and each is deterministic on its own)
      ss += s[j][0] * s[j][0]; ss += s[j][1] * s[j][1]; ss += s[j][2] * s[j][2]; ss += s[j][3] * s[j][3];
    }
  }
  ss = block_sum256(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  int mode = 0, b = 0;
  const float* prev_state = nullptr;
  float inv_prev = 0.f;
  if (shift) {
    b = tok_seq[t];
    if (t > seq_start[b]) {
      mode = 1;
      float q = 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int i = (tid + 256 * j) * 4;
        sp[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (i < width) {
          sp[j] = *reinterpret_cast<const f32x4*>(x_in + (t - 1) * width + i);
          if (upd) {
            const f32x4 d = update4<DT>(delta, parts, num_parts, t - 1, width, i);
            sp[j][0] += d[0]; sp[j][1] += d[1]; sp[j][2] += d[2]; sp[j][3] += d[3];
          }
          q += sp[j][0] * sp[j][0]; q += sp[j][1] * sp[j][1]; q += sp[j][2] * sp[j][2]; q += sp[j][3] * sp[j][3];
        }
      }
      q = block_sum256(q, red);
      inv_prev = 1.0f / sqrtf(q / (float)width + eps);
    } else if (seq_first_pos[b] > 0) {
      mode = 2;
      prev_state = state + (int64_t)seq_parity[b] * state_half + (int64_t)seq_slot[b] * width;
    } else {
      mode = 3;
    }
  }
  float* keep = nullptr;
  if (shift && t == seq_start[b + 1] - 1)
    keep = state + (int64_t)(1 - seq_parity[b]) * state_half + (int64_t)seq_slot[b] * width;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (tid + 256 * j) * 4;
    if (i < width) {
      if (upd) *reinterpret_cast<f32x4*>(x_out + t * width + i) = s[j];
      const f32x4 w = ld4<DT>(weight, i);
      f32x4 h, o;
#pragma unroll
      for (int e = 0; e < 4; ++e) h[e] = s[j][e] * inv * w[e];
      o = h;
      if (mode) {
        f32x4 hp = {0.f, 0.f, 0.f, 0.f};
        if (mode == 1) {
#pragma unroll
          for (int e = 0; e < 4; ++e) hp[e] = sp[j][e] * inv_prev * w[e];
        } else if (mode == 2) {
          hp = *reinterpret_cast<const f32x4*>(prev_state + i);
        }
        const f32x4 mu = ld4<DT>(shift, i);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = h[e] + (hp[e] - h[e]) * mu[e];
        if (keep) *reinterpret_cast<f32x4*>(keep + i) = h;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] *= out_scale;
      st4<DT>(y, t * width + i, o);
    }
  }
}

__device__ __forceinline__ float softplus_f32(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// xIELU: z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2
// (16-bit storage: exp(v) - 1 through the hardware exp2 -- its absolute error of ~1e-7 sits under the z / 2 term by more than the
// storage format resolves; fp32 storage: libm's expm1)
template <int DT>
__device__ __forceinline__ float xielu_f32(float v, float ap, float an) {
  if (v > 0.f) return ap * v * v + 0.5f * v;
  float em1;
  if constexpr (DT == LL_F32) em1 = expm1f(v);
  else em1 = __builtin_amdgcn_exp2f(v * 1.44269504088896341f) - 1.0f;
  return an * (em1 - v) + 0.5f * v;
}

// VEC: 16-byte pieces (8 sixteen-bit values / 4 floats) when the count and both pointers allow it
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void xielu_kernel(void* __restrict__ y, const void* __restrict__ z, const void* __restrict__ pq,
                                                    int64_t n) {
  const float ap = softplus_f32(ldv<DT>(pq, 0));
  const float an = 0.5f + softplus_f32(ldv<DT>(pq, 1));
  if constexpr (!VEC) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
      stv<DT>(y, i, xielu_f32<DT>(ldv<DT>(z, i), ap, an));
  } else if constexpr (DT == LL_F32) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n / 4; i += (int64_t)gridDim.x * 256) {
      f32x4 a = ((const f32x4*)z)[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) a[j] = xielu_f32<DT>(a[j], ap, an);
      ((f32x4*)y)[i] = a;
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n / 8; i += (int64_t)gridDim.x * 256) {
      U16x8 a = ((const U16x8*)z)[i];
#pragma unroll
      for (int j = 0; j < 8; ++j) a.v[j] = from_f32<DT>(xielu_f32<DT>(to_f32<DT>(a.v[j]), ap, an));
      ((U16x8*)y)[i] = a;
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void cast_pair_kernel(void* __restrict__ out, const float* __restrict__ a,
                                                        const void* __restrict__ a_delta, const float* __restrict__ b, int64_t n,
                                                        int width) {
  const int64_t total = n * 2 * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t row = i / (2 * width);
    const int c = (int)(i - row * 2 * width);
    float val;
    if (c < width) {
      val = a[row * width + c];
      if (a_delta) val += ldv<DT>(a_delta, row * width + c);
    } else {
      val = b[row * width + c - width];
    }
    stv<DT>(out, i, val);
  }
}

template <int DT>
__global__ __launch_bounds__(256) void residual_set_kernel(float* __restrict__ x, const void* __restrict__ y,
                                                           const void* __restrict__ bias, int64_t n, int width) {
  const int64_t total = n * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    float v = ldv<DT>(y, i);
    if (bias) v += ldv<DT>(bias, i % width);
    x[i] = v;
  }
}

// One workgroup per token: x = embed[token] * scale + pair[row], row = (previous token * mul_prev + token * mul_cur) mod buckets,
// or row `buckets` (the table's last) for a sequence's first token.  The previous token of a run's first token comes from the
// sequence's state slot (half seq_parity is read); a run's last token leaves itself in the other half.  pair == NULL: no table.
template <int DT>
__global__ __launch_bounds__(256) void embed_pair_kernel(
    float* __restrict__ x, const int32_t* __restrict__ tokens, const void* __restrict__ embed, int64_t vocab, float scale,
    const void* __restrict__ pair, int64_t buckets, int64_t mul_prev, int64_t mul_cur, int width,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos,
    const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ seq_parity, int32_t* __restrict__ prev_state,
    int64_t state_half) {
  const int64_t t = blockIdx.x;
  int64_t tok = tokens[t];
  tok = tok < 0 ? 0 : tok >= vocab ? vocab - 1 : tok;   // (the host refuses ids outside the table; never read past it)
  int64_t row = buckets;
  if (pair) {
    const int b = tok_seq[t];
    int64_t prev = -1;
    if (t > seq_start[b]) prev = tokens[t - 1];
    else if (seq_first_pos[b] > 0) prev = prev_state[(int64_t)seq_parity[b] * state_half + seq_slot[b]];
    if (prev >= 0) row = (prev * mul_prev + tok * mul_cur) % buckets;
    if (t == seq_start[b + 1] - 1 && threadIdx.x == 0)
      prev_state[(int64_t)(1 - seq_parity[b]) * state_half + seq_slot[b]] = (int32_t)tok;
  }
  for (int i = threadIdx.x; i < width; i += 256) {
    float v = ldv<DT>(embed, tok * width + i) * scale;
    if (pair) v += ldv<DT>(pair, row * width + i);
    x[t * width + i] = v;
  }
}

// --------------------------------------------------------------------------------------------------------------------- //
// Gated linear recurrence.  One workgroup per (sequence of the step, head).  Thread (g, c): column c of the head's state
// (c < dv) and rows g, g + KG, ... (KG = 256 / dv column groups), R rows in registers.  Tokens are taken TB at a time:
// their gates, queries and values are staged in LDS (gate and silu evaluated once, in fp32), every thread walks the TB
// tokens over its rows (state update + partial o), the partials of the KG groups are added in group order, o is RMS-normed
// over dv and stored.  The state is read when the run starts inside the sequence (first_pos > 0), zero otherwise, and
// written back at the end of the run.
// --------------------------------------------------------------------------------------------------------------------- //
constexpr int kScanTB = 8;

// sigmoid of the gate and of silu: libm's exp for fp32 storage, the hardware exp2 / reciprocal (1 ulp each) for 16-bit storage
template <int DT>
__device__ __forceinline__ float gate_sigmoid(float v) {
  if constexpr (DT == LL_F32) return 1.0f / (1.0f + expf(-v));
  else return ll_sigmoidf(v);
}

template <int DT, int RMAX>
__global__ __launch_bounds__(256) void gated_linear_scan_kernel(
    const void* __restrict__ q, const void* __restrict__ f, const void* __restrict__ v, int64_t ld, const void* __restrict__ f_bias,
    const void* __restrict__ lower, const void* __restrict__ norm_w, float eps, void* __restrict__ out, int heads, int dk, int dv,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
    float* __restrict__ state) {
  extern __shared__ float lds[];
  const int b = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x;
  const int kg = 256 / dv > 0 ? (256 / dv < dk ? 256 / dv : dk) : 1;
  const int c = tid % dv, g = tid / dv;
  const bool active = g < kg;
  const int rows = active ? (dk - g + kg - 1) / kg : 0;  // rows g, g + kg, ...
  float* sf = lds;                        // [TB][dk] forget gates
  float* sq = sf + kScanTB * dk;          // [TB][dk] queries
  float* sv = sq + kScanTB * dk;          // [TB][dv] values
  float* sp = sv + kScanTB * dv;          // [TB][kg][dv] partial outputs
  float* so = sp + kScanTB * kg * dv;     // [TB][dv] outputs
  float* sn = so + kScanTB * dv;          // [TB] inverse rms
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  float* st = state + ((int64_t)seq_slot[b] * heads + head) * dk * dv;
  float S[RMAX];
  const bool carry = seq_first_pos[b] > 0;
#pragma unroll
  for (int r = 0; r < RMAX; ++r) S[r] = (r < rows && carry) ? st[(int64_t)(g + r * kg) * dv + c] : 0.f;
  for (int base = t0; base < t1; base += kScanTB) {
    const int nt = t1 - base < kScanTB ? t1 - base : kScanTB;
    __syncthreads();
    for (int i = tid; i < nt * dk; i += 256) {
      const int tt = i / dk, k = i - tt * dk;
      const int64_t at = (int64_t)(base + tt) * ld + head * dk + k;
      const float lo = ldv<DT>(lower, head * dk + k);
      const float raw = ldv<DT>(f, at) + ldv<DT>(f_bias, head * dk + k);
      sf[i] = lo + (1.0f - lo) * gate_sigmoid<DT>(raw);
      const float qv = ldv<DT>(q, at);
      sq[i] = qv * gate_sigmoid<DT>(qv);
    }
    for (int i = tid; i < nt * dv; i += 256) {
      const int tt = i / dv, cc = i - tt * dv;
      sv[i] = ldv<DT>(v, (int64_t)(base + tt) * ld + head * dv + cc);
    }
    __syncthreads();
    if (active) {
      for (int tt = 0; tt < nt; ++tt) {
        const float val = sv[tt * dv + c];
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
          if (r < rows) {
            const int k = g + r * kg;
            const float fg = sf[tt * dk + k];
            S[r] = __builtin_fmaf(fg, S[r], (1.0f - fg) * val);
            acc = __builtin_fmaf(S[r], sq[tt * dk + k], acc);
          }
        }
        sp[(tt * kg + g) * dv + c] = acc;
      }
    }
    __syncthreads();
    for (int i = tid; i < nt * dv; i += 256) {
      const int tt = i / dv, cc = i - tt * dv;
      float o = 0.f;
      for (int gg = 0; gg < kg; ++gg) o += sp[(tt * kg + gg) * dv + cc];
      so[i] = o;
    }
    __syncthreads();
    {
      // one wave per token: mean of squares over dv in lane order
      const int wave = tid >> 6, lane = tid & 63;
      for (int tt = wave; tt < nt; tt += 4) {
        float ss = 0.f;
        for (int cc = lane; cc < dv; cc += 64) ss += so[tt * dv + cc] * so[tt * dv + cc];
        ss = wave_sum(ss);
        if (lane == 0) sn[tt] = 1.0f / sqrtf(ss / (float)dv + eps);
      }
    }
    __syncthreads();
    for (int i = tid; i < nt * dv; i += 256) {
      const int tt = i / dv, cc = i - tt * dv;
      stv<DT>(out, ((int64_t)(base + tt) * heads + head) * dv + cc, so[i] * sn[tt] * ldv<DT>(norm_w, cc));
    }
  }
#pragma unroll
  for (int r = 0; r < RMAX; ++r)
    if (r < rows) st[(int64_t)(g + r * kg) * dv + c] = S[r];
}


// Wide form for runs of many tokens: one workgroup per (sequence, head, 16 columns of the state) -- dv / 16 times the
// workgroups of the form above and dk / 16 state rows per thread instead of dk dv / 256, which is what a run's serial walk
// costs per token.  Thread (kg, c): column c of the slice, rows kg, kg + 16, ...  The per-head output norm needs all dv
// columns: o goes to an fp32 scratch [n, heads dv] and head_rmsnorm_kernel finishes.  The state update is the expression of
// the form above, so both leave the same state bits.
template <int DT, int RMAX, bool EXACT>   // EXACT: dk == 16 RMAX, every thread owns RMAX rows (no per-row guards)
__global__ __launch_bounds__(256) void gated_linear_scan_wide_kernel(
    const void* __restrict__ q, const void* __restrict__ f, const void* __restrict__ v, int64_t ld, const void* __restrict__ f_bias,
    const void* __restrict__ lower, float* __restrict__ o_scratch, int heads, int dk, int dv, int tb,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
    float* __restrict__ state) {
  extern __shared__ float lds[];
  const int b = blockIdx.x, head = blockIdx.y, c0 = blockIdx.z * 16;
  const int tid = threadIdx.x, col = tid & 15, kg = tid >> 4;
  const bool active = c0 + col < dv && kg < dk;
  const int rows = kg < dk ? (dk - kg + 15) / 16 : 0;
  f32x4* sg = reinterpret_cast<f32x4*>(lds);          // [tb][dk] (gate, 1 - gate, query, -): one 16-byte read per state row
  float* sv = lds + 4 * tb * dk;                       // [tb][16] values of the slice
  float* sp = sv + tb * 16;                            // [tb][16 groups][16] partial outputs
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  float* st = state + ((int64_t)seq_slot[b] * heads + head) * dk * dv + c0 + col;
  const bool carry = seq_first_pos[b] > 0;
  float S[RMAX];
#pragma unroll
  for (int r = 0; r < RMAX; ++r) S[r] = (active && r < rows && carry) ? st[(int64_t)(kg + 16 * r) * dv] : 0.f;
  for (int base = t0; base < t1; base += tb) {
    const int nt = t1 - base < tb ? t1 - base : tb;
    __syncthreads();
    for (int i = tid; i < nt * dk; i += 256) {
      const int tt = i / dk, k = i - tt * dk;
      const int64_t at = (int64_t)(base + tt) * ld + head * dk + k;
      const float lo = ldv<DT>(lower, head * dk + k);
      const float fg = lo + (1.0f - lo) * gate_sigmoid<DT>(ldv<DT>(f, at) + ldv<DT>(f_bias, head * dk + k));
      const float qv = ldv<DT>(q, at);
      sg[i] = f32x4{fg, 1.0f - fg, qv * gate_sigmoid<DT>(qv), 0.f};
    }
    for (int i = tid; i < nt * 16; i += 256) {
      const int tt = i >> 4, cc = i & 15;
      sv[i] = c0 + cc < dv ? ldv<DT>(v, (int64_t)(base + tt) * ld + head * dv + c0 + cc) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float val = sv[tt * 16 + col];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < RMAX; ++r) {
        if (EXACT || r < rows) {
          const f32x4 gq = sg[tt * dk + kg + 16 * r];
          S[r] = __builtin_fmaf(gq[0], S[r], gq[1] * val);   // (the expression of the fused form: both leave the same bits)
          acc = __builtin_fmaf(S[r], gq[2], acc);
        }
      }
      sp[(tt * 16 + kg) * 16 + col] = acc;
    }
    __syncthreads();
    for (int i = tid; i < nt * 16; i += 256) {
      const int tt = i >> 4, cc = i & 15;
      float o = 0.f;
#pragma unroll
      for (int g2 = 0; g2 < 16; ++g2) o += sp[(tt * 16 + g2) * 16 + cc];
      if (c0 + cc < dv) o_scratch[((int64_t)(base + tt) * heads + head) * dv + c0 + cc] = o;
    }
  }
#pragma unroll
  for (int r = 0; r < RMAX; ++r)
    if (active && r < rows) st[(int64_t)(kg + 16 * r) * dv] = S[r];
}

// one wave per (token, head): out = o / sqrt(mean_dv(o^2) + eps) * w
template <int DT>
__global__ __launch_bounds__(256) void head_rmsnorm_kernel(void* __restrict__ out, const float* __restrict__ o,
                                                           const void* __restrict__ w, float eps, int64_t items, int dv) {
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int lane = threadIdx.x & 63;
  const float* src = o + item * dv;
  float ss = 0.f;
  for (int cc = lane; cc < dv; cc += 64) ss += src[cc] * src[cc];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int cc = lane; cc < dv; cc += 64) stv<DT>(out, item * dv + cc, src[cc] * inv * ldv<DT>(w, cc));
}

inline unsigned flat_grid(int64_t total) {
  const int64_t g = (total + 255) / 256;
  return (unsigned)(g < 1 ? 1 : (g > (1 << 20) ? (1 << 20) : g));  // (one piece per thread up to 2^28 pieces: no ragged second pass)
}

// minGRU: S_t = (1 - z_t) S_(t-1) + z_t c_t per channel, with z = sigmoid(z_raw + z_bias), u = x_raw + x_bias and the candidate
// c = u + 1/2 for u >= 0, sigmoid(u) below; the read-out is S_t * silu(g_raw).  Rows hold [z_raw | x_raw | g_raw] (stride ld).
// One thread per (sequence, channel) walks the run's tokens in order; neighbouring threads read neighbouring channels.  The
// loads of four tokens are issued before the four dependent state updates.  State fp32 [slots][width].
template <int DT>
__global__ __launch_bounds__(256) void mingru_scan_kernel(const void* __restrict__ z, const void* __restrict__ x,
                                                          const void* __restrict__ g, int64_t ld, const void* __restrict__ z_bias,
                                                          const void* __restrict__ x_bias, void* __restrict__ out, int width,
                                                          const int32_t* __restrict__ seq_start,
                                                          const int32_t* __restrict__ seq_first_pos,
                                                          const int32_t* __restrict__ seq_slot, float* __restrict__ state) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int b = blockIdx.y;
  const int start = seq_start[b], stop = seq_start[b + 1];
  float* slot = state + (int64_t)seq_slot[b] * width + c;
  float S = seq_first_pos[b] > 0 ? *slot : 0.f;
  const float zb = z_bias ? ldv<DT>(z_bias, c) : 0.f, xb = x_bias ? ldv<DT>(x_bias, c) : 0.f;
  auto update = [&](float zr, float xr, float gr, int64_t t) {
    const float zt = 1.0f / (1.0f + expf(-(zr + zb)));
    const float u = xr + xb;
    const float cand = u >= 0.f ? u + 0.5f : 1.0f / (1.0f + expf(-u));
    S = (1.0f - zt) * S + zt * cand;
    stv<DT>(out, t * width + c, S * (gr / (1.0f + expf(-gr))));
  };
  int t = start;
  for (; t + 4 <= stop; t += 4) {
    float zr[4], xr[4], gr[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t at = (int64_t)(t + k) * ld + c;
      zr[k] = ldv<DT>(z, at);
      xr[k] = ldv<DT>(x, at);
      gr[k] = ldv<DT>(g, at);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) update(zr[k], xr[k], gr[k], t + k);
  }
  for (; t < stop; ++t) {
    const int64_t at = (int64_t)t * ld + c;
    update(ldv<DT>(z, at), ldv<DT>(x, at), ldv<DT>(g, at), t);
  }
  *slot = S;
}

// Chunked form of the minGRU scan for long runs.  The walk above keeps one wave per 64 channels of a sequence busy for the
// whole run; here a run is cut into chunks of kGruChunk tokens that are walked side by side:
//   pass 1   thread per (sequence, chunk, channel): the chunk's map S -> A S + B (A = product of (1 - z), B = the chunk walked
//            from a zero state), into scratch
//   pass 2   thread per (sequence, channel): the state that enters every chunk (S <- A S + B, chunk by chunk), the final state
//            into the slot
//   pass 3   thread per (sequence, chunk, channel): the chunk walked again from its entering state, outputs written
// Inside a chunk the expression is the token-by-token one; across chunks the state passes through A S + B (one more rounding
// per chunk than the plain walk).
constexpr int kGruChunk = 32;

template <int DT>
__device__ __forceinline__ void mingru_gates(float zr, float xr, float zb, float xb, float& zt, float& cand) {
  zt = 1.0f / (1.0f + expf(-(zr + zb)));
  const float u = xr + xb;
  cand = u >= 0.f ? u + 0.5f : 1.0f / (1.0f + expf(-u));
}

template <int DT, int PASS>
__global__ __launch_bounds__(256) void mingru_chunk_kernel(const void* __restrict__ z, const void* __restrict__ x,
                                                           const void* __restrict__ g, int64_t ld, const void* __restrict__ z_bias,
                                                           const void* __restrict__ x_bias, void* __restrict__ out, int width,
                                                           const int32_t* __restrict__ seq_start, int max_chunks,
                                                           float* __restrict__ scratch) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int b = blockIdx.y / max_chunks, k = blockIdx.y - b * max_chunks;
  const int start = seq_start[b] + k * kGruChunk, stop_run = seq_start[b + 1];
  if (start >= stop_run) return;
  const int stop = start + kGruChunk < stop_run ? start + kGruChunk : stop_run;
  const float zb = z_bias ? ldv<DT>(z_bias, c) : 0.f, xb = x_bias ? ldv<DT>(x_bias, c) : 0.f;
  float* rec = scratch + ((int64_t)blockIdx.y * width + c) * 2;
  if (PASS == 1) {
    float A = 1.0f, B = 0.f;
    for (int t = start; t < stop; ++t) {
      const int64_t at = (int64_t)t * ld + c;
      float zt, cand;
      mingru_gates<DT>(ldv<DT>(z, at), ldv<DT>(x, at), zb, xb, zt, cand);
      A = (1.0f - zt) * A;
      B = (1.0f - zt) * B + zt * cand;
    }
    rec[0] = A;
    rec[1] = B;
  } else {
    float S = rec[0];   // (pass 2 left the entering state here)
    for (int t = start; t < stop; ++t) {
      const int64_t at = (int64_t)t * ld + c;
      float zt, cand;
      mingru_gates<DT>(ldv<DT>(z, at), ldv<DT>(x, at), zb, xb, zt, cand);
      S = (1.0f - zt) * S + zt * cand;
      const float gr = ldv<DT>(g, at);
      stv<DT>(out, (int64_t)t * width + c, S * (gr / (1.0f + expf(-gr))));
    }
  }
}

__global__ __launch_bounds__(256) void mingru_carry_kernel(int width, const int32_t* __restrict__ seq_start,
                                                           const int32_t* __restrict__ seq_first_pos,
                                                           const int32_t* __restrict__ seq_slot, float* __restrict__ state,
                                                           int max_chunks, float* __restrict__ scratch) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int b = blockIdx.y;
  const int count = seq_start[b + 1] - seq_start[b];
  const int chunks = (count + kGruChunk - 1) / kGruChunk;
  float* slot = state + (int64_t)seq_slot[b] * width + c;
  float S = seq_first_pos[b] > 0 ? *slot : 0.f;
  for (int k = 0; k < chunks; ++k) {
    float* rec = scratch + (((int64_t)b * max_chunks + k) * width + c) * 2;
    const float A = rec[0], B = rec[1];
    rec[0] = S;
    S = A * S + B;
  }
  if (count > 0) *slot = S;
}

}  // namespace

#define LL_BY_DTYPE(dtype, CALL)             \
  do {                                       \
    if (dtype == LL_F16) { CALL(LL_F16); }   \
    else if (dtype == LL_BF16) { CALL(LL_BF16); } \
    else { CALL(LL_F32); }                   \
  } while (0)

extern "C" int ll_add_rmsnorm_shift(const float* x_in, const void* delta, float* x_out, const void* weight, const void* shift,
                                    void* y, int64_t n, int64_t width, float eps, const int32_t* tok_seq,
                                    const int32_t* seq_start, const int32_t* seq_first_pos, const int32_t* seq_slot,
                                    const int32_t* seq_parity, float* state, int64_t state_half, const void* parts,
                                    int64_t num_parts, float out_scale, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || width < 1 || width > (1 << 20) || num_parts < 0 || num_parts > 64 || (parts && num_parts < 1)) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!x_in || !weight || !y || ((delta || parts) && !x_out)) return LL_ERR_ARG;
  if ((delta || parts) && x_out == x_in && shift) return LL_ERR_ARG;  // the previous row is re-read: it must still hold the old sum
  if (shift && (!tok_seq || !seq_start || !seq_first_pos || !seq_slot || !seq_parity || !state)) return LL_ERR_ARG;
#define LL_NORM_ARGS \
  x_in, delta, x_out, weight, shift, y, n, (int)width, eps, tok_seq, seq_start, seq_first_pos, seq_slot, seq_parity, state, state_half, \
      parts, (int)num_parts, out_scale
  const bool vec = width % 4 == 0 && width <= 4096 && ll_aligned16(x_in) && (!delta || ll_aligned16(delta)) &&
                   (!parts || ll_aligned16(parts)) && (!(delta || parts) || ll_aligned16(x_out)) &&
                   ll_aligned16(weight) && ll_aligned16(y) && (!shift || (ll_aligned16(shift) && ll_aligned16(state)));
  const dim3 grid((unsigned)n);
  hipStream_t st = (hipStream_t)stream;
#define CALL(DT)                                                                                   \
  if (!vec) add_rmsnorm_shift_kernel<DT><<<grid, 256, 0, st>>>(LL_NORM_ARGS);                      \
  else if (width <= 1024) add_rmsnorm_shift_vec_kernel<DT, 1><<<grid, 256, 0, st>>>(LL_NORM_ARGS); \
  else if (width <= 2048) add_rmsnorm_shift_vec_kernel<DT, 2><<<grid, 256, 0, st>>>(LL_NORM_ARGS); \
  else add_rmsnorm_shift_vec_kernel<DT, 4><<<grid, 256, 0, st>>>(LL_NORM_ARGS)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef LL_NORM_ARGS
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_xielu(void* y, const void* z, const void* pq, int64_t n, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!y || !z || !pq) return LL_ERR_ARG;
  const int per = dtype == LL_F32 ? 4 : 8;
  const bool vec = n % per == 0 && ll_aligned16(y) && ll_aligned16(z);
#define CALL(DT)                                                                                           \
  if (vec) xielu_kernel<DT, true><<<dim3(flat_grid(n / per)), 256, 0, (hipStream_t)stream>>>(y, z, pq, n); \
  else xielu_kernel<DT, false><<<dim3(flat_grid(n)), 256, 0, (hipStream_t)stream>>>(y, z, pq, n)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_cast_pair(void* out, const float* a, const void* a_delta, const float* b, int64_t n, int64_t width, int dtype,
                            void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || width < 1 || width > (1 << 20)) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!out || !a || !b) return LL_ERR_ARG;
#define CALL(DT) cast_pair_kernel<DT><<<dim3(flat_grid(n * 2 * width)), 256, 0, (hipStream_t)stream>>>(out, a, a_delta, b, n, (int)width)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_residual_set(float* x, const void* y, const void* bias, int64_t n, int64_t width, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || width < 1 || width > (1 << 20)) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!x || !y) return LL_ERR_ARG;
#define CALL(DT) residual_set_kernel<DT><<<dim3(flat_grid(n * width)), 256, 0, (hipStream_t)stream>>>(x, y, bias, n, (int)width)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_embed_pair(float* x, const int32_t* tokens, const void* embed, int64_t vocab, float scale, const void* pair,
                             int64_t buckets, int64_t mul_prev, int64_t mul_cur, int64_t n, int64_t width, const int32_t* tok_seq,
                             const int32_t* seq_start, const int32_t* seq_first_pos, const int32_t* seq_slot,
                             const int32_t* seq_parity, int32_t* prev_state, int64_t state_half, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || width < 1 || width > (1 << 20) || vocab < 1 || (pair && (buckets < 1 || mul_prev < 0 || mul_cur < 0))) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!x || !tokens || !embed) return LL_ERR_ARG;
  if (pair && (!tok_seq || !seq_start || !seq_first_pos || !seq_slot || !seq_parity || !prev_state)) return LL_ERR_ARG;
#define CALL(DT)                                                                                                              \
  embed_pair_kernel<DT><<<dim3((unsigned)n), 256, 0, (hipStream_t)stream>>>(x, tokens, embed, vocab, scale, pair, buckets, mul_prev, \
                                                                            mul_cur, (int)width, tok_seq, seq_start, seq_first_pos, \
                                                                            seq_slot, seq_parity, prev_state, state_half)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_gated_linear_scan_supported(int64_t dk, int64_t dv) {
  if (dk < 1 || dv < 1 || dv > 256) return 0;
  const int64_t kg = 256 / dv < dk ? 256 / dv : dk;
  return (dk + kg - 1) / kg <= 128 ? 1 : 0;
}

extern "C" int ll_gated_linear_scan(const void* q, const void* f, const void* v, int64_t ld, const void* f_bias, const void* lower,
                                    const void* norm_w, float eps, void* out, int64_t batch, int64_t heads, int64_t dk, int64_t dv,
                                    const int32_t* seq_start, const int32_t* seq_first_pos, const int32_t* seq_slot, float* state,
                                    int64_t n, int64_t longest_run, float* scratch, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (batch < 0 || n < 0 || heads < 1 || heads > 65535 || !ll_gated_linear_scan_supported(dk, dv)) return LL_ERR_SHAPE;
  if (batch == 0) return LL_OK;
  if (!q || !f || !v || !f_bias || !lower || !norm_w || !out || !seq_start || !seq_first_pos || !seq_slot || !state)
    return LL_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (scratch && dk <= 256 && (longest_run > 2 || batch * heads < 1024)) {
    // wide form + output norm: runs of several tokens (prompt portions, mixed steps), and decode batches too small to fill the
    // chip with one workgroup per (sequence, head)
    const int tb = dk <= 128 ? 16 : 8;
    const size_t lds = sizeof(float) * (size_t)(tb * (4 * dk + 16 + 256));
    const dim3 grid((unsigned)batch, (unsigned)heads, (unsigned)((dv + 15) / 16));
    const int rmax = (int)((dk + 15) / 16);
#define CALL_W(DT, R, E)                                                                                                       \
  gated_linear_scan_wide_kernel<DT, R, E><<<grid, 256, lds, st>>>(q, f, v, ld, f_bias, lower, scratch, (int)heads, (int)dk,    \
                                                                  (int)dv, tb, seq_start, seq_first_pos, seq_slot, state)
#define CALL(DT)                                \
  if (dk == 64) CALL_W(DT, 4, true);            \
  else if (dk == 128) CALL_W(DT, 8, true);      \
  else if (dk == 256) CALL_W(DT, 16, true);     \
  else if (rmax <= 4) CALL_W(DT, 4, false);     \
  else if (rmax <= 8) CALL_W(DT, 8, false);     \
  else CALL_W(DT, 16, false)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef CALL_W
    const int64_t items = n * heads;
#define CALL(DT) head_rmsnorm_kernel<DT><<<dim3((unsigned)((items + 3) / 4)), 256, 0, st>>>(out, scratch, norm_w, eps, items, (int)dv)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
    return LL_LAUNCH_CHECK();
  }
  const int kg = (int)(256 / dv < dk ? 256 / dv : dk);
  const int rmax = (int)((dk + kg - 1) / kg);
  const size_t lds = sizeof(float) * (size_t)(kScanTB * (2 * dk + dv) + kScanTB * kg * dv + kScanTB * dv + kScanTB);
  if (lds > 64 * 1024) return LL_ERR_SHAPE;
  const dim3 grid((unsigned)batch, (unsigned)heads);
#define CALL_R(DT, R)                                                                                                        \
  gated_linear_scan_kernel<DT, R><<<grid, 256, lds, st>>>(q, f, v, ld, f_bias, lower, norm_w, eps, out, (int)heads, (int)dk, \
                                                          (int)dv, seq_start, seq_first_pos, seq_slot, state)
#define CALL(DT)                       \
  if (rmax <= 4) CALL_R(DT, 4);        \
  else if (rmax <= 16) CALL_R(DT, 16); \
  else if (rmax <= 32) CALL_R(DT, 32); \
  else if (rmax <= 64) CALL_R(DT, 64); \
  else CALL_R(DT, 128)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef CALL_R
  return LL_LAUNCH_CHECK();
}

extern "C" int64_t ll_mingru_scan_scratch_floats(int64_t batch, int64_t width, int64_t longest_run) {
  static const bool plain = getenv("LL_MINGRU_PLAIN") != nullptr;   // A/B knob, read once
  if (plain || longest_run < 4 * kGruChunk || batch < 1) return 0;   // short runs: the plain walk
  return batch * ((longest_run + kGruChunk - 1) / kGruChunk) * width * 2;
}

// scratch: fp32, ll_mingru_scan_scratch_floats(batch, width, longest_run) floats (NULL or longest_run = 0: the plain walk)
extern "C" int ll_mingru_scan(const void* z, const void* x, const void* g, int64_t ld, const void* z_bias, const void* x_bias,
                              void* out, int64_t batch, int64_t width, const int32_t* seq_start, const int32_t* seq_first_pos,
                              const int32_t* seq_slot, float* state, int64_t longest_run, float* scratch, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (batch < 0 || batch > 65535 || width < 1 || ld < width || longest_run < 0) return LL_ERR_SHAPE;
  if (batch == 0) return LL_OK;
  if (!z || !x || !g || !out || !seq_start || !seq_first_pos || !seq_slot || !state) return LL_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  const int64_t max_chunks = (longest_run + kGruChunk - 1) / kGruChunk;
  if (scratch && ll_mingru_scan_scratch_floats(batch, width, longest_run) > 0 && batch * max_chunks <= 65535) {
    const dim3 grid_c((unsigned)((width + 255) / 256), (unsigned)(batch * max_chunks)), grid_b((unsigned)((width + 255) / 256), (unsigned)batch);
#define CALL(DT)                                                                                                                \
  mingru_chunk_kernel<DT, 1><<<grid_c, 256, 0, st>>>(z, x, g, ld, z_bias, x_bias, out, (int)width, seq_start, (int)max_chunks, scratch); \
  mingru_carry_kernel<<<grid_b, 256, 0, st>>>((int)width, seq_start, seq_first_pos, seq_slot, state, (int)max_chunks, scratch);         \
  mingru_chunk_kernel<DT, 2><<<grid_c, 256, 0, st>>>(z, x, g, ld, z_bias, x_bias, out, (int)width, seq_start, (int)max_chunks, scratch)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
    return LL_LAUNCH_CHECK();
  }
  const dim3 grid((unsigned)((width + 255) / 256), (unsigned)batch);
#define CALL(DT) \
  mingru_scan_kernel<DT><<<grid, 256, 0, st>>>(z, x, g, ld, z_bias, x_bias, out, (int)width, seq_start, seq_first_pos, seq_slot, state)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}
