// Linear-attention family over RAGGED steps (several sequences, each bringing a run of consecutive tokens against the state
// its earlier steps left), and what stands around such a recurrence:
//
//   ll_linear_scan          per head  S_t = diag(a_t) S_(t-1) + k_t (b_t v_t)^T,  o_t = S_t^T q_t (+ skip_h v_t)  over an fp32
//                           state [dk, dv] per (sequence slot, head).  The decay a_t is, by `kind`:
//                             0  one number per head, fixed                                   (retention / lightning attention)
//                             1  per key entry, sigmoid(z_t + bias)^(1 / tau) from projected rows z   (gated linear attention)
//                             2  one number per head and token, exp(-exp(A_log_h) dt_t) with dt_t = softplus(dt_raw + dt_bias_h),
//                                and b_t = dt_t  (state-space duality: k = B, q = C, v = x, shared by the heads of a group)
//                           q / k / v may pass through silu first; q is multiplied by a constant.
//   ll_gated_out_norm       o (fp32) -> RMS norm over equal consecutive parts of the row, times a weight (one per channel, or a
//                           shorter vector repeated), times silu / sigmoid of a gate row -- before or after the norm --, times a
//                           constant -> storage dtype, into a column range of the next projection's input
//   ll_conv_act             causal convolution over time per channel (+ bias) and silu, the raw rows of a sequence's last
//                           taps - 1 positions carried per sequence slot
//   ll_rownorm_rope_cache   [q | k | v] rows -> q and k RMS-normed over their WHOLE row (all heads at once, a weight per entry),
//                           entry i of a head's first `dims` entries rotated with entry i + dims / 2 by position * f_i; k and
//                           v (times a constant) land in the cache rows of the step
//
// Storage dtype DT = LL_F16 / LL_BF16 / LL_F32 for activations and weights.  fp32 whatever DT: decays, their logarithms and
// exponentials, step sizes, the state and its read-out, norms, angles.  A sequence whose run starts at position 0 starts from
// a zero state whatever an earlier owner of its slot left; state is never cleared on release.
#include "common.h"

#include <math.h>

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

// sigmoid inside an activation: libm's exp for fp32 storage, the hardware exp2 / reciprocal (1 ulp each) for 16-bit storage
template <int DT>
__device__ __forceinline__ float act_sigmoid(float v) {
  if constexpr (DT == LL_F32) return 1.0f / (1.0f + expf(-v));
  else return ll_sigmoidf(v);
}

// ln(sigmoid(z)) without cancellation on either side
__device__ __forceinline__ float log_sigmoid(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }
__device__ __forceinline__ float softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
// sigmoid(z)^(1 / tau): ONE definition for the scan and for the pass that evaluates a step's decays ahead of it
__device__ __forceinline__ float entry_decay(float z, float inv_tau) { return expf(log_sigmoid(z) * inv_tau); }

struct ScanArgs {
  const void* q;   // [n, q_ld]: head j's entries at columns j dk ..
  const void* k;
  const void* v;   // [n, v_ld]: head h's entries at columns h dv ..
  int64_t q_ld, k_ld, v_ld;
  int heads, dk, dv;
  int qk_rep;      // value head h reads query / key head h / qk_rep
  int kind, act;
  float q_scale;
  const float* head_decay;   // kind 0: fp32 [heads]
  const void* gate;          // kind 1: rows [n, gate_ld] of heads dk decay logits, + gate_bias [heads dk]
  int64_t gate_ld;
  const void* gate_bias;
  float inv_tau;
  const float* decay_pre;    // kind 1: the decays of this step [n, heads dk], evaluated ahead of the scan (or NULL: evaluated here)
  const void* dt;            // kind 2: rows [n, dt_ld] of one raw step size per head; dt_bias, a_log, skip: [heads]
  int64_t dt_ld;
  const void* dt_bias;
  const void* a_log;
  const void* skip;
  float* o;                  // fp32 [n, heads dv]
  int tb;                    // tokens staged per pass
  const int32_t* seq_start;
  const int32_t* seq_first_pos;
  const int32_t* seq_slot;
  float* state;              // fp32 [slots, heads, dk, dv]
};

// The decays of a step's tokens per key entry, once per token: the scan's dv / 16 column workgroups of a head would each evaluate
// them again (two exponentials and a logarithm per entry), which for runs of many tokens costs more than the walk over the state.
template <int DT>
__global__ __launch_bounds__(256) void entry_decay_kernel(float* __restrict__ out, const void* __restrict__ gate, int64_t gate_ld,
                                                          const void* __restrict__ gate_bias, float inv_tau, int64_t total, int cols) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / cols;
  const int c = (int)(i - t * cols);
  out[i] = entry_decay(ldv<DT>(gate, t * gate_ld + c) + ldv<DT>(gate_bias, c), inv_tau);
}

// One workgroup per (sequence of the step, head, 16 columns of the state).  Thread (kg, col): column col of the slice, state
// rows kg, kg + 16, ... in registers.  Tokens are taken tb at a time: decay, key and query of every key entry are staged in
// LDS as one 16-byte record (all transcendental work happens here, once per token and entry), the slice's values beside
// them; every thread then walks the tb tokens over its rows (state update + partial read-out), and the partials of the 16 row
// groups are added in group order.  The walk is the same token-by-token expression whatever the step's cut.
template <int DT, int RMAX, bool EXACT>   // EXACT: dk == 16 RMAX, every thread owns RMAX rows (no per-row guards)
__global__ __launch_bounds__(256) void linear_scan_kernel(const ScanArgs a) {
  extern __shared__ float lds[];
  const int b = blockIdx.x, head = blockIdx.y, c0 = blockIdx.z * 16;
  const int tid = threadIdx.x, col = tid & 15, kg = tid >> 4;
  const int dk = a.dk, dv = a.dv, tb = a.tb, heads = a.heads;
  const bool active = c0 + col < dv && kg < dk;
  const int rows = kg < dk ? (dk - kg + 15) / 16 : 0;
  f32x4* sg = reinterpret_cast<f32x4*>(lds);   // [tb][dk] (decay, key, query, -)
  float* sv = lds + 4 * tb * dk;                // [tb][16] what enters the state: value (times the step size)
  float* sx = sv + tb * 16;                     // [tb][16] skip path: skip_h * value
  float* sp = sx + tb * 16;                     // [tb][16 groups][16] partial read-outs
  float* sd = sp + tb * 256;                    // [tb][2] kind 2: (decay, step size) of the token
  const int t0 = a.seq_start[b], t1 = a.seq_start[b + 1];
  float* st = a.state + ((int64_t)a.seq_slot[b] * heads + head) * dk * dv + c0 + col;
  const bool carry = a.seq_first_pos[b] > 0;
  const int qh = head / a.qk_rep;
  const int kind = a.kind;
  float S[RMAX];
#pragma unroll
  for (int r = 0; r < RMAX; ++r) S[r] = (active && r < rows && carry) ? st[(int64_t)(kg + 16 * r) * dv] : 0.f;
  for (int base = t0; base < t1; base += tb) {
    const int nt = t1 - base < tb ? t1 - base : tb;
    __syncthreads();
    if (kind == 2) {
      for (int tt = tid; tt < nt; tt += 256) {
        const float step = softplus(ldv<DT>(a.dt, (int64_t)(base + tt) * a.dt_ld + head) + ldv<DT>(a.dt_bias, head));
        sd[2 * tt] = expf(-expf(ldv<DT>(a.a_log, head)) * step);
        sd[2 * tt + 1] = step;
      }
      __syncthreads();
    }
    for (int i = tid; i < nt * dk; i += 256) {
      const int tt = i / dk, kk = i - tt * dk;
      const int64_t row = base + tt;
      float qv = ldv<DT>(a.q, row * a.q_ld + qh * dk + kk);
      float kv = ldv<DT>(a.k, row * a.k_ld + qh * dk + kk);
      if (a.act) {
        qv *= act_sigmoid<DT>(qv);
        kv *= act_sigmoid<DT>(kv);
      }
      float dec;
      if (kind == 0) dec = a.head_decay[head];
      else if (kind == 1)
        dec = a.decay_pre ? a.decay_pre[(row * heads + head) * dk + kk]
                          : entry_decay(ldv<DT>(a.gate, row * a.gate_ld + head * dk + kk) + ldv<DT>(a.gate_bias, head * dk + kk), a.inv_tau);
      else dec = sd[2 * tt];
      sg[i] = f32x4{dec, kv, qv * a.q_scale, 0.f};
    }
    for (int i = tid; i < nt * 16; i += 256) {
      const int tt = i >> 4, cc = i & 15;
      float x = c0 + cc < dv ? ldv<DT>(a.v, (int64_t)(base + tt) * a.v_ld + head * dv + c0 + cc) : 0.f;
      if (a.act) x *= act_sigmoid<DT>(x);
      sv[i] = kind == 2 ? sd[2 * tt + 1] * x : x;
      sx[i] = (kind == 2 && a.skip) ? ldv<DT>(a.skip, head) * x : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float val = sv[tt * 16 + col];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < RMAX; ++r) {
        if (EXACT || r < rows) {
          const f32x4 g = sg[tt * dk + kg + 16 * r];
          S[r] = __builtin_fmaf(g[0], S[r], g[1] * val);
          acc = __builtin_fmaf(S[r], g[2], acc);
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
      if (c0 + cc < dv) a.o[((int64_t)(base + tt) * heads + head) * dv + c0 + cc] = o + sx[i];
    }
  }
#pragma unroll
  for (int r = 0; r < RMAX; ++r)
    if (active && r < rows) st[(int64_t)(kg + 16 * r) * dv] = S[r];
}

// One wave per (token, part): out = [o * act(gate)] / sqrt(mean_part(.^2) + eps) * w [* act(gate)] * out_scale.
// gate_kind 0: none, 1: silu, 2: sigmoid; gate_first: the gate multiplies before the norm.  w has w_len entries and is read
// at (channel mod w_len): a weight per channel, or one short vector for every head.
template <int DT>
__global__ __launch_bounds__(256) void gated_out_norm_kernel(void* __restrict__ out, int64_t out_ld, const float* __restrict__ o,
                                                             const void* __restrict__ gate, int64_t gate_ld, int gate_kind,
                                                             int gate_first, const void* __restrict__ w, int w_len, float eps,
                                                             float out_scale, int64_t items, int parts, int ps) {
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = item / parts;
  const int c0 = (int)(item - t * parts) * ps;
  const float* src = o + t * (int64_t)parts * ps + c0;
  auto gate_at = [&](int cc) -> float {
    const float g = ldv<DT>(gate, t * gate_ld + c0 + cc);
    const float s = act_sigmoid<DT>(g);
    return gate_kind == 1 ? g * s : s;
  };
  float ss = 0.f;
  for (int cc = lane; cc < ps; cc += 64) {
    float v = src[cc];
    if (gate_kind && gate_first) v *= gate_at(cc);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)ps + eps);
  for (int cc = lane; cc < ps; cc += 64) {
    float v = src[cc];
    const float g = gate_kind ? gate_at(cc) : 1.0f;
    if (gate_first) v *= g;
    v = v * inv * (w ? ldv<DT>(w, (c0 + cc) % w_len) : 1.0f);
    if (!gate_first) v *= g;
    stv<DT>(out, t * out_ld + c0 + cc, v * out_scale);
  }
}

// Thread per (token, channel): y = silu(bias + sum_j w[c][j] u_(p - taps + 1 + j)), positions in front of the sequence count
// as zero.  A predecessor that rides in the same step is read from the step's rows, an earlier one from the carried rows
// (state [2][slots][taps - 1][channels]: the half named by the sequence's parity is read, the other written by the run's last
// token from the same two sources, so runs shorter than the taps shift the old rows forward).
template <int DT>
__global__ __launch_bounds__(256) void conv_act_kernel(void* __restrict__ out, int64_t out_ld, const void* __restrict__ rows, int64_t ld,
                                                       const void* __restrict__ w, const void* __restrict__ bias, int channels, int taps,
                                                       void* __restrict__ state, int64_t state_half, const int32_t* __restrict__ tok_seq,
                                                       const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ seq_start,
                                                       const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
                                                       const int32_t* __restrict__ seq_parity) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int seq = tok_seq[t], pos = tok_pos[t];
  const int start = seq_start[seq], first = seq_first_pos[seq];
  const int64_t slot_at = (int64_t)seq_slot[seq] * (taps - 1) * channels;
  const int par = seq_parity[seq] & 1;
  const int64_t in_at = par * state_half + slot_at, out_at = (par ^ 1) * state_half + slot_at;
  auto raw_at = [&](int p) -> float {   // the projected row of position p >= 0 of this sequence, channel c
    if (p >= first) return ldv<DT>(rows, (int64_t)(start + (p - first)) * ld + c);
    return ldv<DT>(state, in_at + (int64_t)(p - first + taps - 1) * channels + c);
  };
  float acc = bias ? ldv<DT>(bias, c) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int p = pos - (taps - 1 - j);
    if (p < 0) continue;
    acc += ldv<DT>(w, (int64_t)c * taps + j) * raw_at(p);
  }
  stv<DT>(out, t * out_ld + c, acc * act_sigmoid<DT>(acc));
  if (taps > 1 && t == seq_start[seq + 1] - 1) {
    for (int s = 0; s < taps - 1; ++s) {
      const int p = pos + 1 - (taps - 1) + s;
      stv<DT>(state, out_at + (int64_t)s * channels + c, p >= 0 ? raw_at(p) : 0.f);
    }
  }
}

// One workgroup per token.  q and k: RMS norm over the whole row (mean over all heads' entries) times a weight per entry,
// then the rotation of (i, i + half) pairs inside each head; k and value_scale * v go to cache row select[t].
template <int DT>
__global__ __launch_bounds__(256) void rownorm_rope_cache_kernel(
    const void* __restrict__ rows, int64_t ld, const void* __restrict__ q_w, const void* __restrict__ k_w, float eps,
    const float* __restrict__ freq, int half, float value_scale, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ select,
    void* __restrict__ q_out, void* __restrict__ k_cache, void* __restrict__ v_cache, int heads, int kv_heads, int dk, int dv) {
  extern __shared__ float cs[];   // [half] cos, [half] sin
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const int qn = heads * dk, kn = kv_heads * dk, vn = kv_heads * dv;
  const int64_t at = t * ld;
  const float pos = (float)tok_pos[t];
  for (int i = tid; i < half; i += 256) {
    float s, c;
    sincosf(pos * freq[i], &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
  float sq = 0.f, sk = 0.f;
  for (int i = tid; i < qn; i += 256) {
    const float v = ldv<DT>(rows, at + i);
    sq += v * v;
  }
  for (int i = tid; i < kn; i += 256) {
    const float v = ldv<DT>(rows, at + qn + i);
    sk += v * v;
  }
  sq = block_sum256(sq, red);
  sk = block_sum256(sk, red);   // (its first barrier also publishes cs)
  const float inv_q = q_w ? 1.0f / sqrtf(sq / (float)qn + eps) : 1.0f;
  const float inv_k = k_w ? 1.0f / sqrtf(sk / (float)kn + eps) : 1.0f;
  auto normed = [&](int64_t base, const void* w, float inv, int i) -> float {
    const float v = ldv<DT>(rows, base + i);
    return w ? v * inv * ldv<DT>(w, i) : v;
  };
  auto rotated = [&](int64_t base, const void* w, float inv, int idx) -> float {
    const int i = idx % dk;
    const float v = normed(base, w, inv, idx);
    if (i >= 2 * half) return v;
    if (i < half) return v * cs[i] - normed(base, w, inv, idx + half) * cs[half + i];
    return v * cs[i - half] + normed(base, w, inv, idx - half) * cs[i];
  };
  for (int i = tid; i < qn; i += 256) stv<DT>(q_out, t * qn + i, rotated(at, q_w, inv_q, i));
  const int64_t row = select[t];
  for (int i = tid; i < kn; i += 256) stv<DT>(k_cache, row * kn + i, rotated(at + qn, k_w, inv_k, i));
  for (int i = tid; i < vn; i += 256) stv<DT>(v_cache, row * vn + i, ldv<DT>(rows, at + qn + kn + i) * value_scale);
}

// eight consecutive storage-dtype values at element i (a multiple of 8 from a 16-byte aligned base) as fp32
template <int DT>
__device__ __forceinline__ void ld8(const void* p, int64_t i, float (&o)[8]) {
  if constexpr (DT == LL_F32) {
    const f32x4 a = *reinterpret_cast<const f32x4*>((const float*)p + i), b = *reinterpret_cast<const f32x4*>((const float*)p + i + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { o[e] = a[e]; o[4 + e] = b[e]; }
  } else {
    const U16x8 u = *reinterpret_cast<const U16x8*>((const uint16_t*)p + i);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = to_f32<DT>(u.v[e]);
  }
}
template <int DT>
__device__ __forceinline__ void st8(void* p, int64_t i, const float (&o)[8]) {
  if constexpr (DT == LL_F32) {
    *reinterpret_cast<f32x4*>((float*)p + i) = f32x4{o[0], o[1], o[2], o[3]};
    *reinterpret_cast<f32x4*>((float*)p + i + 4) = f32x4{o[4], o[5], o[6], o[7]};
  } else {
    U16x8 u;
#pragma unroll
    for (int e = 0; e < 8; ++e) u.v[e] = from_f32<DT>(o[e]);
    *reinterpret_cast<U16x8*>((uint16_t*)p + i) = u;
  }
}

// The read-out norm for long parts: one workgroup per (token, part), same arithmetic per element as the wave form.
template <int DT>
__global__ __launch_bounds__(256) void gated_out_norm_block_kernel(void* __restrict__ out, int64_t out_ld, const float* __restrict__ o,
                                                                   const void* __restrict__ gate, int64_t gate_ld, int gate_kind,
                                                                   int gate_first, const void* __restrict__ w, int w_len, float eps,
                                                                   float out_scale, int parts, int ps) {
  __shared__ float red[4];
  const int64_t item = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t t = item / parts;
  const int c0 = (int)(item - t * parts) * ps;
  const float* src = o + t * (int64_t)parts * ps + c0;
  auto gate_at = [&](int cc) -> float {
    const float g = ldv<DT>(gate, t * gate_ld + c0 + cc);
    const float s = act_sigmoid<DT>(g);
    return gate_kind == 1 ? g * s : s;
  };
  float ss = 0.f;
  for (int cc = tid; cc < ps; cc += 256) {
    float v = src[cc];
    if (gate_kind && gate_first) v *= gate_at(cc);
    ss += v * v;
  }
  ss = block_sum256(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)ps + eps);
  for (int cc = tid; cc < ps; cc += 256) {
    float v = src[cc];
    const float g = gate_kind ? gate_at(cc) : 1.0f;
    if (gate_first) v *= g;
    v = v * inv * (w ? ldv<DT>(w, (c0 + cc) % w_len) : 1.0f);
    if (!gate_first) v *= g;
    stv<DT>(out, t * out_ld + c0 + cc, v * out_scale);
  }
}

// The convolution in 16-byte pieces: a thread owns eight consecutive channels of one token; the taps' weights of those
// channels are one contiguous run of 8 TAPS values.  Same sums in the same order as the plain form.
template <int DT, int TAPS>
__global__ __launch_bounds__(256) void conv_act_vec_kernel(void* __restrict__ out, int64_t out_ld, const void* __restrict__ rows, int64_t ld,
                                                           const void* __restrict__ w, const void* __restrict__ bias, int channels,
                                                           void* __restrict__ state, int64_t state_half, const int32_t* __restrict__ tok_seq,
                                                           const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ seq_start,
                                                           const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
                                                           const int32_t* __restrict__ seq_parity, int64_t pieces) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= pieces) return;
  const int per = channels >> 3;
  const int64_t t = idx / per;
  const int c = (int)(idx - t * per) << 3;
  const int seq = tok_seq[t], pos = tok_pos[t];
  const int start = seq_start[seq], first = seq_first_pos[seq];
  const int64_t slot_at = (int64_t)seq_slot[seq] * (TAPS - 1) * channels;
  const int par = seq_parity[seq] & 1;
  const int64_t in_at = par * state_half + slot_at, out_at = (par ^ 1) * state_half + slot_at;
  auto raw_at = [&](int p, float (&u)[8]) {
    if (p >= first) ld8<DT>(rows, (int64_t)(start + (p - first)) * ld + c, u);
    else ld8<DT>(state, in_at + (int64_t)(p - first + TAPS - 1) * channels + c, u);
  };
  float wl[8 * TAPS];
#pragma unroll
  for (int j = 0; j < TAPS; ++j) {
    float piece[8];
    ld8<DT>(w, (int64_t)c * TAPS + 8 * j, piece);
#pragma unroll
    for (int e = 0; e < 8; ++e) wl[8 * j + e] = piece[e];
  }
  float acc[8];
  if (bias) ld8<DT>(bias, c, acc);
  else {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < TAPS; ++j) {
    const int p = pos - (TAPS - 1 - j);
    if (p < 0) continue;
    float u[8];
    raw_at(p, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += wl[e * TAPS + j] * u[e];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = acc[e] * act_sigmoid<DT>(acc[e]);
  st8<DT>(out, t * out_ld + c, acc);
  if (TAPS > 1 && t == seq_start[seq + 1] - 1) {
#pragma unroll
    for (int s = 0; s < TAPS - 1; ++s) {
      const int p = pos + 1 - (TAPS - 1) + s;
      float u[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (p >= 0) raw_at(p, u);
      st8<DT>(state, out_at + (int64_t)s * channels + c, u);
    }
  }
}

// The whole-row norms and the rotation in 16-byte pieces (head widths, rotated halves and row strides multiples of 8): a
// thread sums the squares of its pieces, then -- after the two workgroup sums -- reads each piece again with the piece it is
// rotated with.  Same arithmetic per entry as the plain form; the sums of squares are taken in piece order.
template <int DT>
__global__ __launch_bounds__(256) void rownorm_rope_cache_vec_kernel(
    const void* __restrict__ rows, int64_t ld, const void* __restrict__ q_w, const void* __restrict__ k_w, float eps,
    const float* __restrict__ freq, int half, float value_scale, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ select,
    void* __restrict__ q_out, void* __restrict__ k_cache, void* __restrict__ v_cache, int heads, int kv_heads, int dk, int dv) {
  extern __shared__ float cs[];   // [half] cos, [half] sin
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const int qn = heads * dk, kn = kv_heads * dk, vn = kv_heads * dv;
  const int64_t at = t * ld;
  const float pos = (float)tok_pos[t];
  for (int i = tid; i < half; i += 256) {
    float s, c;
    sincosf(pos * freq[i], &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
  float sq = 0.f, sk = 0.f;
  for (int i = tid * 8; i < qn + kn; i += 2048) {
    float u[8];
    ld8<DT>(rows, at + i, u);
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s += u[e] * u[e];
    if (i < qn) sq += s;
    else sk += s;
  }
  sq = block_sum256(sq, red);
  sk = block_sum256(sk, red);   // (its first barrier also publishes cs)
  const float inv_q = q_w ? 1.0f / sqrtf(sq / (float)qn + eps) : 1.0f;
  const float inv_k = k_w ? 1.0f / sqrtf(sk / (float)kn + eps) : 1.0f;
  const int64_t row = select[t];
  for (int i = tid * 8; i < qn + kn; i += 2048) {
    const bool is_q = i < qn;
    const int idx = is_q ? i : i - qn;                 // entry inside the q (k) row
    const int64_t base = is_q ? at : at + qn;
    const void* w = is_q ? q_w : k_w;
    const float inv = is_q ? inv_q : inv_k;
    float v[8];
    ld8<DT>(rows, base + idx, v);
    if (w) {
      float wv[8];
      ld8<DT>(w, idx, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = v[e] * inv * wv[e];
    }
    const int in_head = idx % dk;
    if (in_head < 2 * half) {
      const bool low = in_head < half;
      const int other = low ? idx + half : idx - half;
      const int a0 = low ? in_head : in_head - half;   // first angle of the piece
      float p[8];
      ld8<DT>(rows, base + other, p);
      if (w) {
        float wv[8];
        ld8<DT>(w, other, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = p[e] * inv * wv[e];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = low ? v[e] * cs[a0 + e] - p[e] * cs[half + a0 + e] : v[e] * cs[a0 + e] + p[e] * cs[half + a0 + e];
    }
    if (is_q) st8<DT>(q_out, t * qn + idx, v);
    else st8<DT>(k_cache, row * kn + idx, v);
  }
  for (int i = tid * 8; i < vn; i += 2048) {
    float v[8];
    ld8<DT>(rows, at + qn + kn + i, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= value_scale;
    st8<DT>(v_cache, row * vn + i, v);
  }
}

}  // namespace

#define LL_BY_DTYPE(dtype, CALL)                  \
  do {                                            \
    if (dtype == LL_F16) { CALL(LL_F16); }        \
    else if (dtype == LL_BF16) { CALL(LL_BF16); } \
    else { CALL(LL_F32); }                        \
  } while (0)

extern "C" int ll_linear_scan_supported(int64_t dk, int64_t dv) { return dk >= 1 && dk <= 256 && dv >= 1 ? 1 : 0; }

extern "C" int ll_linear_scan(const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld, int64_t heads,
                              int64_t dk, int64_t dv, int64_t qk_rep, int kind, int act, float q_scale, const float* head_decay,
                              const void* gate, int64_t gate_ld, const void* gate_bias, float inv_tau, const void* dt, int64_t dt_ld,
                              const void* dt_bias, const void* a_log, const void* skip, float* o, int64_t batch,
                              const int32_t* seq_start, const int32_t* seq_first_pos, const int32_t* seq_slot, float* state,
                              float* decay_scratch, int64_t n, int64_t longest_run, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (batch < 0 || heads < 1 || heads > 65535 || !ll_linear_scan_supported(dk, dv) || qk_rep < 1 || heads % qk_rep || kind < 0 ||
      kind > 2 || (dv + 15) / 16 > 65535)
    return LL_ERR_SHAPE;
  const int64_t qk_cols = heads / qk_rep * dk;
  if (q_ld < qk_cols || k_ld < qk_cols || v_ld < heads * dv) return LL_ERR_SHAPE;
  if (batch == 0) return LL_OK;
  if (!q || !k || !v || !o || !seq_start || !seq_first_pos || !seq_slot || !state) return LL_ERR_ARG;
  if (kind == 0 && !head_decay) return LL_ERR_ARG;
  if (kind == 1 && (!gate || !gate_bias || gate_ld < heads * dk)) return LL_ERR_ARG;
  if (kind == 2 && (!dt || !dt_bias || !a_log || dt_ld < heads)) return LL_ERR_ARG;
  ScanArgs a;
  a.q = q; a.k = k; a.v = v; a.q_ld = q_ld; a.k_ld = k_ld; a.v_ld = v_ld;
  a.heads = (int)heads; a.dk = (int)dk; a.dv = (int)dv; a.qk_rep = (int)qk_rep; a.kind = kind; a.act = act; a.q_scale = q_scale;
  a.head_decay = head_decay; a.gate = gate; a.gate_ld = gate_ld; a.gate_bias = gate_bias; a.inv_tau = inv_tau;
  a.decay_pre = nullptr;
  a.dt = dt; a.dt_ld = dt_ld; a.dt_bias = dt_bias; a.a_log = a_log; a.skip = skip; a.o = o;
  a.tb = dk <= 128 ? 16 : 8;   // tokens staged per pass; a step of short runs asks for less LDS and fits more workgroups per CU
  if (longest_run > 0 && longest_run < a.tb) a.tb = (int)longest_run;
  a.seq_start = seq_start; a.seq_first_pos = seq_first_pos; a.seq_slot = seq_slot; a.state = state;
  const size_t lds = sizeof(float) * (size_t)(a.tb * (4 * dk + 16 + 16 + 256 + 2));
  const dim3 grid((unsigned)batch, (unsigned)heads, (unsigned)((dv + 15) / 16));
  hipStream_t st = (hipStream_t)stream;
  if (kind == 1 && decay_scratch && n > 0) {   // decays once per token and entry, ahead of the scan: fp32 [n, heads dk]
    const int64_t total = n * heads * dk;
    if ((total + 255) / 256 > 0x7fffffffll) return LL_ERR_SHAPE;
#define CALL(DT) \
  entry_decay_kernel<DT><<<dim3((unsigned)((total + 255) / 256)), 256, 0, st>>>(decay_scratch, gate, gate_ld, gate_bias, inv_tau, total, (int)(heads * dk))
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
    a.decay_pre = decay_scratch;
  }
  const int rmax = (int)((dk + 15) / 16);
#define CALL_W(DT, R, E) linear_scan_kernel<DT, R, E><<<grid, 256, lds, st>>>(a)
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
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_gated_out_norm(void* out, int64_t out_ld, const float* o, const void* gate, int64_t gate_ld, int gate_kind,
                                 int gate_first, const void* w, int64_t w_len, float eps, float out_scale, int64_t n, int64_t width,
                                 int64_t parts, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || width < 1 || parts < 1 || width % parts || out_ld < width || gate_kind < 0 || gate_kind > 2 ||
      (w && (w_len < 1 || w_len > width)) || width > (1 << 24))
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!out || !o || (gate_kind && (!gate || gate_ld < width))) return LL_ERR_ARG;
  const int64_t items = n * parts;
  if (items > 0x7fffffffll) return LL_ERR_SHAPE;
  if (width / parts >= 512) {   // long parts: a workgroup each (the form depends on the part's length only)
#define CALL(DT)                                                                                                                   \
  gated_out_norm_block_kernel<DT><<<dim3((unsigned)items), 256, 0, (hipStream_t)stream>>>(                                         \
      out, out_ld, o, gate, gate_ld, gate_kind, gate_first ? 1 : 0, w, (int)(w ? w_len : 1), eps, out_scale, (int)parts, (int)(width / parts))
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
    return LL_LAUNCH_CHECK();
  }
#define CALL(DT)                                                                                                                 \
  gated_out_norm_kernel<DT><<<dim3((unsigned)((items + 3) / 4)), 256, 0, (hipStream_t)stream>>>(                                 \
      out, out_ld, o, gate, gate_ld, gate_kind, gate_first ? 1 : 0, w, (int)(w ? w_len : 1), eps, out_scale, items, (int)parts, \
      (int)(width / parts))
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_conv_act(void* out, int64_t out_ld, const void* rows, int64_t ld, const void* w, const void* bias, int64_t channels,
                           int64_t taps, void* state, int64_t state_half, const int32_t* tok_seq, const int32_t* tok_pos,
                           const int32_t* seq_start, const int32_t* seq_first_pos, const int32_t* seq_slot, const int32_t* seq_parity,
                           int64_t n, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || channels < 1 || taps < 1 || taps > 64 || ld < channels || out_ld < channels || (channels + 255) / 256 > 65535)
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!out || !rows || !w || !tok_seq || !tok_pos || !seq_start || !seq_first_pos || !seq_slot || !seq_parity || (taps > 1 && !state))
    return LL_ERR_ARG;
  const int al = dtype == LL_F32 ? 4 : 8;   // elements per 16 bytes
  if (taps <= 4 && channels % 8 == 0 && ld % al == 0 && out_ld % al == 0 && ll_aligned16(rows) && ll_aligned16(out) && ll_aligned16(w) &&
      (!bias || ll_aligned16(bias)) && (taps == 1 || ll_aligned16(state)) ) {
    // (fp32 pieces of eight are two 16-byte accesses: strides that are multiples of 4 keep both aligned)
    const int64_t pieces = n * (channels / 8);
    const dim3 vgrid((unsigned)((pieces + 255) / 256));
#define CALL_T(DT, T)                                                                                                                \
  conv_act_vec_kernel<DT, T><<<vgrid, 256, 0, (hipStream_t)stream>>>(out, out_ld, rows, ld, w, bias, (int)channels, state, state_half, \
                                                                     tok_seq, tok_pos, seq_start, seq_first_pos, seq_slot, seq_parity, pieces)
#define CALL(DT)                      \
  if (taps == 1) CALL_T(DT, 1);       \
  else if (taps == 2) CALL_T(DT, 2);  \
  else if (taps == 3) CALL_T(DT, 3);  \
  else CALL_T(DT, 4)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef CALL_T
    return LL_LAUNCH_CHECK();
  }
  const dim3 grid((unsigned)n, (unsigned)((channels + 255) / 256));
#define CALL(DT)                                                                                                                     \
  conv_act_kernel<DT><<<grid, 256, 0, (hipStream_t)stream>>>(out, out_ld, rows, ld, w, bias, (int)channels, (int)taps, state, state_half, \
                                                             tok_seq, tok_pos, seq_start, seq_first_pos, seq_slot, seq_parity)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_rownorm_rope_cache(const void* rows, int64_t ld, const void* q_w, const void* k_w, float eps, const float* freq,
                                     int64_t pairs, float value_scale, const int32_t* tok_pos, const int32_t* select, void* q_out,
                                     void* k_cache, void* v_cache, int64_t n, int64_t heads, int64_t kv_heads, int64_t dk, int64_t dv,
                                     int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || heads < 1 || kv_heads < 1 || dk < 1 || dv < 1 || pairs < 0 || 2 * pairs > dk || pairs > 8192 ||
      ld < (heads + kv_heads) * dk + kv_heads * dv)
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!rows || !tok_pos || !select || !q_out || !k_cache || !v_cache || (pairs && !freq)) return LL_ERR_ARG;
  const size_t lds = sizeof(float) * (size_t)(2 * pairs + 1);
  const int al = dtype == LL_F32 ? 4 : 8;
  if (dk % 8 == 0 && dv % 8 == 0 && pairs % 8 == 0 && ld % al == 0 && ll_aligned16(rows) && ll_aligned16(q_out) && ll_aligned16(k_cache) &&
      ll_aligned16(v_cache) && (!q_w || ll_aligned16(q_w)) && (!k_w || ll_aligned16(k_w))) {
#define CALL(DT)                                                                                                                 \
  rownorm_rope_cache_vec_kernel<DT><<<dim3((unsigned)n), 256, lds, (hipStream_t)stream>>>(                                       \
      rows, ld, q_w, k_w, eps, freq, (int)pairs, value_scale, tok_pos, select, q_out, k_cache, v_cache, (int)heads, (int)kv_heads, \
      (int)dk, (int)dv)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
    return LL_LAUNCH_CHECK();
  }
#define CALL(DT)                                                                                                                 \
  rownorm_rope_cache_kernel<DT><<<dim3((unsigned)n), 256, lds, (hipStream_t)stream>>>(                                           \
      rows, ld, q_w, k_w, eps, freq, (int)pairs, value_scale, tok_pos, select, q_out, k_cache, v_cache, (int)heads, (int)kv_heads, \
      (int)dk, (int)dv)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}
