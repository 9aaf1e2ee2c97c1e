// Layers whose sublayers are wrapped in TWO norms and a learned gate on the residual branch (32-bit residual stream):
//
//     x <- x + norm_b( f(norm_a(x)) * sigmoid(W_r norm_a(x) + b_r) )
//
// with RMS norms taken over GROUPS: the row is cut into `groups` equal consecutive parts, each divided by its own root mean
// square, then the whole is multiplied by the weight.
//
//   ll_gated_group_norm   closes one sublayer and opens the next in ONE launch: the sublayer's result (one row per token, or the
//                         sum of several rows -- the experts a token chose -- plus a scaled shared row) times the sigmoid of its
//                         gate logits, grouped norm with the post weight, residual add in fp32, then the grouped norm that feeds
//                         the next sublayer (or the output head).  Without a pending result it is the plain grouped norm.
//   ll_glu_act            act(gate) * up, gate and up two row-strided column ranges (act: silu, the tanh form of gelu, sigmoid),
//                         or the clamped form g sigmoid(a g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit);
//                         the result may be a column range of wider rows
//
// Storage dtype DT = LL_F16 / LL_BF16 / LL_F32 for activations and weights; sums, norms, gates and the residual are fp32.
#include "common.h"

namespace {

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

// sum over a 256-thread workgroup in a fixed order (wave sums, then the four waves in order)
__device__ __forceinline__ float block_sum256(float v, float* lds4) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds4[wave] = v;
  __syncthreads();
  return ((lds4[0] + lds4[1]) + lds4[2]) + lds4[3];
}

template <bool EXACT>
__device__ __forceinline__ float sigmoid_f(float v) {
  if constexpr (EXACT) return 1.0f / (1.0f + expf(-v));
  else return ll_sigmoidf(v);
}

// One workgroup per token; thread i owns elements i, i + 256, ... of every group (the same elements in every pass, so a
// thread re-reads only what it wrote itself).  NV > 0: the gated value of a thread's elements stays in registers between the
// passes (rows of up to 256 NV elements per group pass); NV == 0: recomputed from memory.
template <int DT>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    const float* x_in, float* x_out, void* __restrict__ h_out, const void* __restrict__ y, int parts,
    const void* __restrict__ shared, const float* __restrict__ shared_scale, const void* __restrict__ gate, int64_t gate_ld,
    const void* __restrict__ gate_bias, const void* __restrict__ post_w, const void* __restrict__ next_w, int width, int groups,
    float eps, const void* __restrict__ y_bias) {
  constexpr bool EXACT = DT == LL_F32;
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const int gs = width / groups;
  const float* xr = x_in + t * width;
  float* xo = x_out + t * width;
  const float sscale = shared ? shared_scale[t] : 0.f;

  auto branch = [&](int i) -> float {   // the sublayer's gated result at element i
    float s = 0.f;
    for (int p = 0; p < parts; ++p) s += ldv<DT>(y, (t * parts + p) * (int64_t)width + i);
    if (y_bias) s += ldv<DT>(y_bias, i);
    if (shared) s += sscale * ldv<DT>(shared, t * (int64_t)width + i);
    if (gate) {
      float r = ldv<DT>(gate, t * gate_ld + i);
      if (gate_bias) r += ldv<DT>(gate_bias, i);
      s *= sigmoid_f<EXACT>(r);
    }
    return s;
  };

  for (int g = 0; g < groups; ++g) {
    const int lo = g * gs, hi = lo + gs;
    if (y) {
      float ss = 0.f;
      for (int i = lo + tid; i < hi; i += 256) {
        const float s = branch(i);
        ss += s * s;
      }
      ss = block_sum256(ss, red);
      const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
      float s2 = 0.f;
      for (int i = lo + tid; i < hi; i += 256) {
        const float v = xr[i] + branch(i) * inv * ldv<DT>(post_w, i);
        xo[i] = v;
        s2 += v * v;
      }
      s2 = block_sum256(s2, red);
      if (h_out) {
        const float inv2 = 1.0f / sqrtf(s2 / (float)gs + eps);
        for (int i = lo + tid; i < hi; i += 256)
          stv<DT>(h_out, t * (int64_t)width + i, next_w ? xo[i] * inv2 * ldv<DT>(next_w, i) : xo[i]);
      }
    } else {
      float s2 = 0.f;
      for (int i = lo + tid; i < hi; i += 256) {
        const float v = xr[i];
        s2 += v * v;
      }
      s2 = block_sum256(s2, red);
      const float inv2 = 1.0f / sqrtf(s2 / (float)gs + eps);
      for (int i = lo + tid; i < hi; i += 256)
        stv<DT>(h_out, t * (int64_t)width + i, next_w ? xr[i] * inv2 * ldv<DT>(next_w, i) : xr[i]);
    }
  }
}

// Register-cached form: a thread keeps the gated values of its elements (and then the new residual) between the passes, so
// every input is read once.  Same arithmetic and reduction order as the plain form.  Needs width / groups <= 256 NV.
template <int DT, int NV>
__global__ __launch_bounds__(256) void gated_group_norm_cached_kernel(
    const float* x_in, float* x_out, void* __restrict__ h_out, const void* __restrict__ y, int parts,
    const void* __restrict__ shared, const float* __restrict__ shared_scale, const void* __restrict__ gate, int64_t gate_ld,
    const void* __restrict__ gate_bias, const void* __restrict__ post_w, const void* __restrict__ next_w, int width, int groups,
    float eps, const void* __restrict__ y_bias) {
  constexpr bool EXACT = DT == LL_F32;
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const int gs = width / groups;
  const float* xr = x_in + t * width;
  float* xo = x_out + t * width;
  const float sscale = shared ? shared_scale[t] : 0.f;
  for (int g = 0; g < groups; ++g) {
    const int lo = g * gs, hi = lo + gs;
    float val[NV];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = lo + tid + 256 * k;
      float s = 0.f;
      if (i < hi) {
        for (int p = 0; p < parts; ++p) s += ldv<DT>(y, (t * parts + p) * (int64_t)width + i);
        if (y_bias) s += ldv<DT>(y_bias, i);
        if (shared) s += sscale * ldv<DT>(shared, t * (int64_t)width + i);
        if (gate) {
          float r = ldv<DT>(gate, t * gate_ld + i);
          if (gate_bias) r += ldv<DT>(gate_bias, i);
          s *= sigmoid_f<EXACT>(r);
        }
      }
      val[k] = s;
      ss += s * s;
    }
    ss = block_sum256(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    float s2 = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = lo + tid + 256 * k;
      float v = 0.f;
      if (i < hi) {
        v = xr[i] + val[k] * inv * ldv<DT>(post_w, i);
        xo[i] = v;
      }
      val[k] = v;
      s2 += v * v;
    }
    s2 = block_sum256(s2, red);
    if (h_out) {
      const float inv2 = 1.0f / sqrtf(s2 / (float)gs + eps);
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int i = lo + tid + 256 * k;
        if (i < hi) stv<DT>(h_out, t * (int64_t)width + i, next_w ? val[k] * inv2 * ldv<DT>(next_w, i) : val[k]);
      }
    }
  }
}

// four storage-dtype values at element i (a multiple of 4; 8-byte / 16-byte aligned)
template <int DT>
__device__ __forceinline__ f32x4 ld4(const void* p, int64_t i) {
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

// Vector form of the register-cached kernel: a thread owns pieces of four consecutive channels (16-byte residual accesses,
// 8-byte accesses of 16-bit rows).  Needs group sizes that are multiples of 4 and at most 1024 NV channels, aligned rows.
template <int DT, int NV>
__global__ __launch_bounds__(256) void gated_group_norm_vec_kernel(
    const float* x_in, float* x_out, void* __restrict__ h_out, const void* __restrict__ y, int parts,
    const void* __restrict__ shared, const float* __restrict__ shared_scale, const void* __restrict__ gate, int64_t gate_ld,
    const void* __restrict__ gate_bias, const void* __restrict__ post_w, const void* __restrict__ next_w, int width, int groups,
    float eps, const void* __restrict__ y_bias) {
  constexpr bool EXACT = DT == LL_F32;
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const int gs = width / groups;
  const float* xr = x_in + t * width;
  float* xo = x_out + t * width;
  const float sscale = shared ? shared_scale[t] : 0.f;
  for (int g = 0; g < groups; ++g) {
    const int lo = g * gs, hi = lo + gs;
    f32x4 val[NV];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = lo + 4 * (tid + 256 * k);
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
      if (i < hi) {
        for (int p = 0; p < parts; ++p) s += ld4<DT>(y, (t * parts + p) * (int64_t)width + i);
        if (y_bias) s += ld4<DT>(y_bias, i);
        if (shared) s += sscale * ld4<DT>(shared, t * (int64_t)width + i);
        if (gate) {
          f32x4 r = ld4<DT>(gate, t * gate_ld + i);
          if (gate_bias) r += ld4<DT>(gate_bias, i);
#pragma unroll
          for (int e = 0; e < 4; ++e) s[e] *= sigmoid_f<EXACT>(r[e]);
        }
      }
      val[k] = s;
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += s[e] * s[e];
    }
    ss = block_sum256(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    float s2 = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int i = lo + 4 * (tid + 256 * k);
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (i < hi) {
        const f32x4 pw = ld4<DT>(post_w, i);
        const f32x4 xv = *reinterpret_cast<const f32x4*>(xr + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = xv[e] + val[k][e] * inv * pw[e];
        *reinterpret_cast<f32x4*>(xo + i) = v;
      }
      val[k] = v;
#pragma unroll
      for (int e = 0; e < 4; ++e) s2 += v[e] * v[e];
    }
    s2 = block_sum256(s2, red);
    if (h_out) {
      const float inv2 = 1.0f / sqrtf(s2 / (float)gs + eps);
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int i = lo + 4 * (tid + 256 * k);
        if (i < hi) {
          f32x4 o = val[k];   // (no next weight: the new residual itself, cast)
          if (next_w) {
            const f32x4 nw = ld4<DT>(next_w, i);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = val[k][e] * inv2 * nw[e];
          }
          st4<DT>(h_out, t * (int64_t)width + i, o);
        }
      }
    }
  }
}

template <int DT>
__device__ __forceinline__ float glu_value(float g, float u, int kind);

// out[t][j] = act(gate[t][j]) * up[t][j]; gate and up rows have their own strides (two column ranges of one projection, or two
// tensors).  kind 0: silu, 1: gelu (tanh form), 2: sigmoid, 3: clamped (p0 = limit, p1 = slope inside the sigmoid)
template <int DT>
__device__ __forceinline__ float glu_value(float g, float u, int kind, float p0, float p1) {
  constexpr bool EXACT = DT == LL_F32;
  float a;
  if (kind == 0) {
    a = g * sigmoid_f<EXACT>(g);
  } else if (kind == 2) {
    a = sigmoid_f<EXACT>(g);
  } else if (kind == 3) {
    g = fminf(g, p0);
    u = fminf(fmaxf(u, -p0), p0) + 1.0f;
    a = g * sigmoid_f<EXACT>(p1 * g);
  } else {
    const float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    const float th = EXACT ? tanhf(inner) : 2.0f * ll_sigmoidf(2.0f * inner) - 1.0f;
    a = 0.5f * g * (1.0f + th);
  }
  return a * u;
}

template <int DT>
__global__ __launch_bounds__(256) void glu_act_kernel(void* __restrict__ out, int64_t out_ld, const void* __restrict__ gate,
                                                      int64_t gate_ld, const void* __restrict__ up, int64_t up_ld, int64_t n, int ff,
                                                      int kind, float p0, float p1) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n * ff) return;
  const int64_t t = idx / ff;
  const int j = (int)(idx - t * ff);
  stv<DT>(out, t * out_ld + j, glu_value<DT>(ldv<DT>(gate, t * gate_ld + j), ldv<DT>(up, t * up_ld + j), kind, p0, p1));
}

// 16-byte form: a thread owns one piece (8 sixteen-bit / 4 fp32 values) of a row; same values as the plain form
template <int DT>
__global__ __launch_bounds__(256) void glu_act_vec_kernel(void* __restrict__ out, int64_t out_ld, const void* __restrict__ gate,
                                                          int64_t gate_ld, const void* __restrict__ up, int64_t up_ld, int64_t n,
                                                          int ff, int kind, float p0, float p1) {
  constexpr int VEC = DT == LL_F32 ? 4 : 8;
  const int pieces = ff / VEC;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n * pieces) return;
  const int64_t t = idx / pieces;
  const int j = (int)(idx - t * pieces) * VEC;
  if constexpr (DT == LL_F32) {
    const f32x4 g = *reinterpret_cast<const f32x4*>((const float*)gate + t * gate_ld + j);
    const f32x4 u = *reinterpret_cast<const f32x4*>((const float*)up + t * up_ld + j);
    f32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = glu_value<DT>(g[i], u[i], kind, p0, p1);
    *reinterpret_cast<f32x4*>((float*)out + t * out_ld + j) = o;
  } else {
    const U16x8 g = *reinterpret_cast<const U16x8*>((const uint16_t*)gate + t * gate_ld + j);
    const U16x8 u = *reinterpret_cast<const U16x8*>((const uint16_t*)up + t * up_ld + j);
    U16x8 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o.v[i] = from_f32<DT>(glu_value<DT>(to_f32<DT>(g.v[i]), to_f32<DT>(u.v[i]), kind, p0, p1));
    *reinterpret_cast<U16x8*>((uint16_t*)out + t * out_ld + j) = o;
  }
}

// logits <- cap tanh(logits / cap), fp32 arithmetic
template <int DT>
__global__ __launch_bounds__(256) void softcap_kernel(void* __restrict__ x, int64_t n, float cap) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  stv<DT>(x, idx, cap * tanhf(ldv<DT>(x, idx) / cap));
}

}  // namespace

#define LL_BY_DTYPE(dtype, CALL)             \
  do {                                       \
    if (dtype == LL_F16) { CALL(LL_F16); }   \
    else if (dtype == LL_BF16) { CALL(LL_BF16); } \
    else { CALL(LL_F32); }                   \
  } while (0)

extern "C" int ll_gated_group_norm(const float* x_in, float* x_out, void* h_out, const void* y, int64_t parts, const void* shared,
                                   const float* shared_scale, const void* gate, int64_t gate_ld, const void* gate_bias,
                                   const void* post_w, const void* next_w, int64_t n, int64_t width, int64_t groups, float eps,
                                   const void* y_bias, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || width < 1 || width > (1 << 20) || groups < 1 || width % groups || parts < 0 || parts > 64) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!x_in) return LL_ERR_ARG;
  if (y && (!x_out || !post_w || parts < 1)) return LL_ERR_ARG;
  if (!y && (!h_out || shared || gate)) return LL_ERR_ARG;
  if (y_bias && !y) return LL_ERR_ARG;
  if (shared && !shared_scale) return LL_ERR_ARG;
  if (gate && gate_ld < width) return LL_ERR_SHAPE;
  if (!y) x_out = const_cast<float*>(x_in);
  const dim3 grid((unsigned)n);
  hipStream_t st = (hipStream_t)stream;
  const int64_t gs = width / groups;
#define LL_GN_ARGS \
  x_in, x_out, h_out, y, (int)parts, shared, shared_scale, gate, gate_ld, gate_bias, post_w, next_w, (int)width, (int)groups, eps, \
  y_bias
  const int al = dtype == LL_F32 ? 16 : 8;   // bytes a four-channel piece of a storage-dtype row must be aligned to
  auto ok = [&](const void* p) { return !p || (reinterpret_cast<uintptr_t>(p) % al) == 0; };
  const bool vec = y && gs % 4 == 0 && gs <= 4096 && (!gate || gate_ld % 4 == 0) && ll_aligned16(x_in) && ll_aligned16(x_out) && ok(h_out) &&
                   ok(y) && ok(shared) && ok(gate) && ok(gate_bias) && ok(post_w) && ok(next_w) && ok(y_bias);
#define CALL(DT)                                                                                          \
  if (vec && gs <= 1024) gated_group_norm_vec_kernel<DT, 1><<<grid, 256, 0, st>>>(LL_GN_ARGS);            \
  else if (vec && gs <= 2048) gated_group_norm_vec_kernel<DT, 2><<<grid, 256, 0, st>>>(LL_GN_ARGS);       \
  else if (vec) gated_group_norm_vec_kernel<DT, 4><<<grid, 256, 0, st>>>(LL_GN_ARGS);                     \
  else if (y && gs <= 256) gated_group_norm_cached_kernel<DT, 1><<<grid, 256, 0, st>>>(LL_GN_ARGS);       \
  else if (y && gs <= 1024) gated_group_norm_cached_kernel<DT, 4><<<grid, 256, 0, st>>>(LL_GN_ARGS);      \
  else if (y && gs <= 4096) gated_group_norm_cached_kernel<DT, 16><<<grid, 256, 0, st>>>(LL_GN_ARGS);     \
  else gated_group_norm_kernel<DT><<<grid, 256, 0, st>>>(LL_GN_ARGS)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef LL_GN_ARGS
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_glu_act(void* out, int64_t out_ld, const void* gate, int64_t gate_ld, const void* up, int64_t up_ld, int64_t n,
                          int64_t ff, int kind, float p0, float p1, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || ff < 1 || out_ld < ff || gate_ld < ff || up_ld < ff || ff > (1 << 24) || kind < 0 || kind > 3) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!out || !gate || !up) return LL_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  const int vec = dtype == LL_F32 ? 4 : 8;
  if (ff % vec == 0 && out_ld % vec == 0 && gate_ld % vec == 0 && up_ld % vec == 0 && ll_aligned16(out) && ll_aligned16(gate) && ll_aligned16(up)) {
    const dim3 grid((unsigned)((n * (ff / vec) + 255) / 256));
#define CALL(DT) glu_act_vec_kernel<DT><<<grid, 256, 0, st>>>(out, out_ld, gate, gate_ld, up, up_ld, n, (int)ff, kind, p0, p1)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
    return LL_LAUNCH_CHECK();
  }
  const dim3 grid((unsigned)((n * ff + 255) / 256));
#define CALL(DT) glu_act_kernel<DT><<<grid, 256, 0, st>>>(out, out_ld, gate, gate_ld, up, up_ld, n, (int)ff, kind, p0, p1)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_softcap(void* x, int64_t n, float cap, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || !(cap > 0.f)) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!x) return LL_ERR_ARG;
  const dim3 grid((unsigned)((n + 255) / 256));
  hipStream_t st = (hipStream_t)stream;
#define CALL(DT) softcap_kernel<DT><<<grid, 256, 0, st>>>(x, n, cap)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}
