// Softmax attention over RAGGED steps against a paged cache, for head geometries the rotary llama kernels do not cover:
// separate key and value widths, per-head RMS norm of queries and keys, a position-dependent query temperature instead of a
// rotation, and a learned per-head SINK in the softmax denominator.
//
//   ll_qk_norm_cache     fused projection rows [q | k | v] -> normed, temperature-scaled queries; normed keys and raw values
//                        written to the cache rows of their tokens
//   ll_conv_rope_cache   fused projection rows [q | k | v] -> bias, a short causal convolution over time per channel (the last
//                        taps - 1 projected rows of a sequence are carried in a state slot), rotation of entry pairs of q / k
//                        heads, unit RMS norm of q / k heads, values blended with the values another layer cached for the same
//                        token; queries out, keys and values into the cache rows of their tokens
//   ll_rotation_table    cos / sin (times an amplitude) of position * frequency per token and entry pair, once per step for all
//                        layers and heads that rotate alike
//   ll_ragged_attention  every token of the step against keys 0 .. its own position of its sequence, read through the
//                        per-token row table; scores, softmax and the running output in fp32; optionally only the last
//                        `window` keys plus the sequence's first `keep_first`
//
// The sink is a virtual key with score sink_h (not scaled) and a zero value: the running softmax simply STARTS at
// (max = sink, sum = 1, output = 0).  A token's result depends only on its own position and on the cache rows of its
// sequence, visited in a fixed order: how a prompt was cut into steps, or what else rides in the step, cannot change it.
#include <type_traits>

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

// One wave per (token, item): items 0 .. H - 1 = query heads, H .. H + G - 1 = key heads, then G value heads.
template <int DT>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(
    const void* __restrict__ qkv, int64_t ld, const void* __restrict__ q_w, const void* __restrict__ k_w, float eps,
    float temp_coef, int temp_every, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ select,
    void* __restrict__ q_out, void* __restrict__ k_cache, void* __restrict__ v_cache, int64_t n, int heads, int kv_heads, int dk,
    int dv) {
  const int items = heads + 2 * kv_heads;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= n * items) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = w / items;
  const int item = (int)(w - t * items);
  const int64_t row = select[t];
  if (item >= heads + kv_heads) {  // value head: copy
    const int gidx = item - heads - kv_heads;
    const int64_t src = t * ld + (int64_t)(heads + kv_heads) * dk + (int64_t)gidx * dv;
    for (int c = lane; c < dv; c += 64) stv<DT>(v_cache, (row * kv_heads + gidx) * dv + c, ldv<DT>(qkv, src + c));
    return;
  }
  const bool is_q = item < heads;
  const int64_t src = t * ld + (int64_t)item * dk;
  float ss = 0.f;
  for (int c = lane; c < dk; c += 64) {
    const float x = ldv<DT>(qkv, src + c);
    ss += x * x;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dk + eps);
  float temp = 1.0f;
  if (is_q && temp_coef != 0.f) temp = 1.0f + temp_coef * logf((float)((tok_pos[t] + 1) / temp_every) + 1.0f);
  const void* wt = is_q ? q_w : k_w;
  for (int c = lane; c < dk; c += 64) {
    float r = ldv<DT>(qkv, src + c) * inv;
    if (wt) r *= ldv<DT>(wt, c);
    if (is_q) stv<DT>(q_out, (t * heads + item) * dk + c, r * temp);
    else stv<DT>(k_cache, (row * kv_heads + (item - heads)) * dk + c, r);
  }
}

// floats per token of a rotation table: (cos, sin) per pair, the pairs padded to a multiple of four (32-byte pieces stay inside)
__host__ __device__ __forceinline__ int64_t rot_stride(int64_t pairs) { return 2 * ((pairs + 3) & ~(int64_t)3); }

// One wave per (token, item): items 0 .. H - 1 = query heads, H .. H + G - 1 = key heads, then G value heads.  Lane l owns the
// entry pairs l, l + 64, .. of its head (NP of them).  Per channel, in fp32:
//   u_p   = projected row of position p (+ bias): this step's rows, or -- in front of the run -- the sequence's state slot, which
//           holds the RAW projected rows of its last taps - 1 positions (row d - 1 = position length - d); zeros in front of
//           position 0
//   y     = sum_j w[c][j] u_(pos - taps + 1 + j)                       (taps == 0: y = u)
//   q, k  : pairs (2i, 2i + 1), i < pairs, rotated by pos * freq[i] with cos / sin times amp; then the head divided by
//           sqrt(mean(y^2) + eps) when unit_norm
//   v     : (1 - lam) y + lam v_src[select[t]] when a source cache is given
// The wave of a run's LAST token also writes its item's channels of the state slot for the next step (other half of the pair).
template <int DT, int NP>
__global__ __launch_bounds__(256) void conv_rope_cache_kernel(
    const void* __restrict__ qkv, int64_t ld, const void* __restrict__ bias, const void* __restrict__ conv_w, int taps,
    void* __restrict__ conv_state, int64_t state_half, const float* __restrict__ freq, int pairs, float amp,
    const float* __restrict__ rot_table, int unit_norm,
    float eps, const void* __restrict__ v_src, int64_t v_src_stride, const void* __restrict__ v_lam,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ select,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ seq_parity, void* __restrict__ q_out, void* __restrict__ k_cache, void* __restrict__ v_cache,
    int64_t n, int heads, int kv_heads, int dk, int dv) {
  const int items = heads + 2 * kv_heads;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= n * items) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = w / items;
  const int item = (int)(w - t * items);
  const bool is_q = item < heads, is_v = item >= heads + kv_heads;
  const int width = is_v ? dv : dk;
  const int64_t col0 = is_v ? (int64_t)(heads + kv_heads) * dk + (int64_t)(item - heads - kv_heads) * dv : (int64_t)item * dk;
  const int64_t channels = (int64_t)(heads + kv_heads) * dk + (int64_t)kv_heads * dv;
  const int b = tok_seq[t];
  const int pos = tok_pos[t], first = seq_first_pos[b];
  const int in_run = pos - first;                       // tokens of the run in front of this one
  const int back = taps > 1 ? taps - 1 : 0;
  const uint8_t* old_state = nullptr;
  if (back) old_state = (const uint8_t*)conv_state + ((int64_t)seq_parity[b] * state_half + (int64_t)seq_slot[b] * back * channels) *
                                                         (DT == LL_F32 ? 4 : 2);
  // projected value (+ bias) of channel c at `d` positions in front of this token (d = 0: its own); 0 in front of position 0
  auto u_at = [&](int64_t c, int d) -> float {
    if (d > pos) return 0.f;
    float v;
    if (d <= in_run) v = ldv<DT>(qkv, (t - d) * ld + c);
    else v = ldv<DT>(old_state, (int64_t)(d - in_run - 1) * channels + c);
    return bias ? v + ldv<DT>(bias, c) : v;
  };
  auto conv_at = [&](int64_t c) -> float {
    if (taps <= 0) return u_at(c, 0);
    float y = 0.f;
    for (int j = 0; j < taps; ++j) y += ldv<DT>(conv_w, c * taps + j) * u_at(c, taps - 1 - j);
    return y;
  };
  float a[NP], bb[NP];
  float ss = 0.f;
  const float fpos = (float)pos;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int pi = lane + 64 * i;
    a[i] = bb[i] = 0.f;
    if (2 * pi < width) {
      a[i] = conv_at(col0 + 2 * pi);
      if (2 * pi + 1 < width) bb[i] = conv_at(col0 + 2 * pi + 1);
      if (!is_v && pi < pairs) {
        float cs, sn;
        if (rot_table) {   // (the same two values, computed once per token by rotation_table_kernel)
          cs = rot_table[t * rot_stride(pairs) + 2 * pi];
          sn = rot_table[t * rot_stride(pairs) + 2 * pi + 1];
        } else {
          const float ang = fpos * freq[pi];
          cs = cosf(ang) * amp;
          sn = sinf(ang) * amp;
        }
        const float x0 = a[i], x1 = bb[i];
        a[i] = x0 * cs - x1 * sn;
        bb[i] = x1 * cs + x0 * sn;
      }
      ss += a[i] * a[i];
      ss += bb[i] * bb[i];
    }
  }
  float mul = 1.0f, lam = 0.f;
  if (!is_v && unit_norm) {
    ss = wave_sum(ss);
    mul = 1.0f / sqrtf(ss / (float)dk + eps);
  }
  const int64_t crow = select[t];
  const bool blend = is_v && v_src != nullptr;
  if (blend) lam = ldv<DT>(v_lam, 0);
  const int64_t dst = is_q ? (t * heads + item) * dk
                           : is_v ? (crow * kv_heads + (item - heads - kv_heads)) * dv : (crow * kv_heads + (item - heads)) * dk;
  void* dstp = is_q ? q_out : is_v ? v_cache : k_cache;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int pi = lane + 64 * i;
    if (2 * pi < width) {
      float y0 = a[i] * mul, y1 = bb[i] * mul;
      if (blend) {
        const int64_t src = crow * v_src_stride + (int64_t)(item - heads - kv_heads) * dv + 2 * pi;
        y0 = (1.0f - lam) * y0 + lam * ldv<DT>(v_src, src);
        if (2 * pi + 1 < width) y1 = (1.0f - lam) * y1 + lam * ldv<DT>(v_src, src + 1);
      }
      stv<DT>(dstp, dst + 2 * pi, y0);
      if (2 * pi + 1 < width) stv<DT>(dstp, dst + 2 * pi + 1, y1);
    }
  }
  // the run's last token leaves the raw projected rows of the sequence's last taps - 1 positions
  if (back && t == seq_start[b + 1] - 1) {
    uint8_t* new_state = (uint8_t*)conv_state + ((int64_t)(1 - seq_parity[b]) * state_half + (int64_t)seq_slot[b] * back * channels) *
                                                    (DT == LL_F32 ? 4 : 2);
    for (int d = 1; d <= back; ++d) {                   // state row d - 1 = the position d - 1 in front of this token
      for (int c = lane; c < width; c += 64) {
        float v = 0.f;
        if (d - 1 <= in_run) v = ldv<DT>(qkv, (t - (d - 1)) * ld + col0 + c);
        else if (d - 1 <= pos) v = ldv<DT>(old_state, (int64_t)(d - 1 - in_run - 1) * channels + col0 + c);
        stv<DT>(new_state, (int64_t)(d - 1) * channels + col0 + c, v);
      }
    }
  }
}

// sum over the 16 lanes of a DPP row (every lane of the row active); the result is in every lane of the row
__device__ __forceinline__ float row16_sum(float v) {
  float t;
  t = ll_dpp_f32<0xB1>(v); v += t;   // quad_perm [1,0,3,2]
  t = ll_dpp_f32<0x4E>(v); v += t;   // quad_perm [2,3,0,1]
  t = ll_dpp_f32<0x124>(v); v += t;  // row_ror:4
  t = ll_dpp_f32<0x128>(v); v += t;  // row_ror:8
  return v;
}

// 16-byte form of the kernel above.  A workgroup owns 16 CONSECUTIVE TOKENS -- one per 16-lane row -- and a few items, which
// its rows take in step: the tap weights and the bias of an item are fetched once for the sixteen tokens, and the rows a tap
// reads are the neighbouring rows' own.  Lane r of a row owns the 16-byte pieces r, r + 16, .. of the head (up to four: widths
// <= 512 sixteen-bit / 256 fp32 channels, multiples of 8 / 4; how many is a template constant, as are the taps (0 .. 4), so a
// piece's tap weights sit in registers.  A token's cos / sin come from the step's rotation table.  The same sums in the
// same order as the plain form.
template <int DT, int TAPS, int NPC>   // NPC: 16-byte pieces per lane (1, 2 or 4)
__global__ __launch_bounds__(256) void conv_rope_cache_vec_kernel(
    const void* __restrict__ qkv, int64_t ld, const void* __restrict__ bias, const void* __restrict__ conv_w,
    void* __restrict__ conv_state, int64_t state_half, const float* __restrict__ rot_table, int pairs, int unit_norm,
    float eps, const void* __restrict__ v_src, int64_t v_src_stride, const void* __restrict__ v_lam,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ select,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ seq_parity, void* __restrict__ q_out, void* __restrict__ k_cache, void* __restrict__ v_cache,
    int64_t n, int heads, int kv_heads, int dk, int dv, int items_per_wg) {
  constexpr int EPC = DT == LL_F32 ? 4 : 8;  // elements per 16-byte piece
  typedef typename std::conditional<DT == LL_F32, float, uint16_t>::type elem;
  struct alignas(16) Piece { elem e[EPC]; };
  constexpr int BACK = TAPS > 1 ? TAPS - 1 : 0;
  constexpr int WN = TAPS > 0 ? TAPS : 1;
  const int items = heads + 2 * kv_heads;
  const int trow = threadIdx.x >> 4, r = threadIdx.x & 15;
  const int64_t t = (int64_t)blockIdx.x * 16 + trow;
  if (t >= n) return;   // (whole 16-lane rows leave; nothing below synchronises across rows)
  const int64_t channels = (int64_t)(heads + kv_heads) * dk + (int64_t)kv_heads * dv;
  const int b = tok_seq[t];
  const int pos = tok_pos[t], first = seq_first_pos[b];
  const int in_run = pos - first;
  const int item_lo = blockIdx.y * items_per_wg;
  const int item_hi = item_lo + items_per_wg < items ? item_lo + items_per_wg : items;
  const float* my_cs = rot_table + t * rot_stride(pairs);   // (cos, sin) of the token's angles, times the amplitude
  const bool last_of_run = t == seq_start[b + 1] - 1;
  float lam = 0.f;
  if (v_src) lam = ldv<DT>(v_lam, 0);
  const int64_t crow = select[t];
  const elem* rows = (const elem*)qkv;
  const elem* old_state = rows;   // (never read without carried rows)
  if constexpr (BACK > 0) old_state = (const elem*)conv_state + (int64_t)seq_parity[b] * state_half + (int64_t)seq_slot[b] * BACK * channels;
  for (int item = item_lo; item < item_hi; ++item) {
    const bool is_q = item < heads, is_v = item >= heads + kv_heads;
    const int width = is_v ? dv : dk;
    const int64_t col0 = is_v ? (int64_t)(heads + kv_heads) * dk + (int64_t)(item - heads - kv_heads) * dv : (int64_t)item * dk;
    const int pieces = width / EPC;
    float val[NPC][EPC];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NPC; ++j) {
      const int pc = r + 16 * j;
      if (pc < pieces) {
        const int64_t c = col0 + (int64_t)pc * EPC;
        float bv[EPC], acc[EPC];
#pragma unroll
        for (int e = 0; e < EPC; ++e) bv[e] = acc[e] = 0.f;
        // every load of the piece is issued before the first sum: the bias, the taps' rows (this step's, or the carried ones;
        // a tap in front of position 0 re-reads the token's own row and counts as zero) and the EPC * TAPS contiguous tap
        // weights of these channels (channel e, tap j at e * TAPS + j)
        Piece braw, raw[WN], wraw[WN];
        if (bias) braw = *reinterpret_cast<const Piece*>((const elem*)bias + c);
#pragma unroll
        for (int jt = 0; jt < WN; ++jt) {
          const int dist = WN - 1 - jt;
          const elem* src = rows + t * ld + c;
          if constexpr (BACK > 0) {
            if (dist <= pos && dist > in_run) src = old_state + (int64_t)(dist - in_run - 1) * channels + c;
            else if (dist <= pos) src = rows + (t - dist) * ld + c;
          }
          raw[jt] = *reinterpret_cast<const Piece*>(src);
          if constexpr (TAPS > 0) wraw[jt] = *reinterpret_cast<const Piece*>((const elem*)conv_w + c * TAPS + jt * EPC);
        }
        if (bias) {
#pragma unroll
          for (int e = 0; e < EPC; ++e) {
            if constexpr (DT == LL_F32) bv[e] = braw.e[e];
            else bv[e] = to_f32<DT>(braw.e[e]);
          }
        }
#pragma unroll
        for (int jt = 0; jt < WN; ++jt) {
          const bool seen = WN - 1 - jt <= pos;
#pragma unroll
          for (int e = 0; e < EPC; ++e) {
            float u;
            if constexpr (DT == LL_F32) u = raw[jt].e[e];
            else u = to_f32<DT>(raw[jt].e[e]);
            if (bias) u += bv[e];
            if constexpr (TAPS > 0) {   // (weights widened where they are used: fewer live registers)
              const int flat = e * TAPS + jt;
              float wt;
              if constexpr (DT == LL_F32) wt = wraw[flat / EPC].e[flat % EPC];
              else wt = to_f32<DT>(wraw[flat / EPC].e[flat % EPC]);
              acc[e] += wt * (seen ? u : 0.f);
            } else {
              acc[e] = u;
            }
          }
        }
        if (!is_v && pc * (EPC / 2) < pairs) {
          float rot[EPC];   // (cos, sin) of this piece's pairs: EPC floats at pc * EPC, inside the padded row
#pragma unroll
          for (int k = 0; k < EPC / 4; ++k) {
            const f32x4 v4 = *reinterpret_cast<const f32x4*>(my_cs + pc * EPC + 4 * k);
            rot[4 * k] = v4[0]; rot[4 * k + 1] = v4[1]; rot[4 * k + 2] = v4[2]; rot[4 * k + 3] = v4[3];
          }
#pragma unroll
          for (int m = 0; m < EPC / 2; ++m) {
            const int pi = pc * (EPC / 2) + m;
            if (pi < pairs) {
              const float cs = rot[2 * m], sn = rot[2 * m + 1];
              const float x0 = acc[2 * m], x1 = acc[2 * m + 1];
              acc[2 * m] = x0 * cs - x1 * sn;
              acc[2 * m + 1] = x1 * cs + x0 * sn;
            }
          }
        }
#pragma unroll
        for (int e = 0; e < EPC; ++e) {
          val[j][e] = acc[e];
          ss += acc[e] * acc[e];
        }
      }
    }
    float mul = 1.0f;
    if (!is_v && unit_norm) {
      ss = row16_sum(ss);
      mul = 1.0f / sqrtf(ss / (float)dk + eps);
    }
    const bool blend = is_v && v_src != nullptr;
    elem* dst = is_q ? (elem*)q_out + (t * heads + item) * dk
                     : is_v ? (elem*)v_cache + (crow * kv_heads + (item - heads - kv_heads)) * dv
                            : (elem*)k_cache + (crow * kv_heads + (item - heads)) * dk;
#pragma unroll
    for (int j = 0; j < NPC; ++j) {
      const int pc = r + 16 * j;
      if (pc < pieces) {
        Piece sraw;
        if (blend) sraw = *reinterpret_cast<const Piece*>((const elem*)v_src + crow * v_src_stride + (int64_t)(item - heads - kv_heads) * dv + pc * EPC);
        Piece o;
#pragma unroll
        for (int e = 0; e < EPC; ++e) {
          float y = val[j][e] * mul;
          if (blend) {
            float sv;
            if constexpr (DT == LL_F32) sv = sraw.e[e];
            else sv = to_f32<DT>(sraw.e[e]);
            y = (1.0f - lam) * y + lam * sv;
          }
          if constexpr (DT == LL_F32) o.e[e] = y;
          else o.e[e] = from_f32<DT>(y);
        }
        *reinterpret_cast<Piece*>(dst + pc * EPC) = o;
      }
    }
    if constexpr (BACK > 0) if (last_of_run) {   // the run's last token leaves the raw rows of the sequence's last TAPS - 1 positions
      elem* new_state = (elem*)conv_state + (int64_t)(1 - seq_parity[b]) * state_half + (int64_t)seq_slot[b] * BACK * channels;
#pragma unroll
      for (int dist = 0; dist < BACK; ++dist) {             // state row `dist` = the position `dist` in front of this token
        for (int pc = r; pc < pieces; pc += 16) {
          const int64_t c = col0 + (int64_t)pc * EPC;
          Piece v;
#pragma unroll
          for (int e = 0; e < EPC; ++e) v.e[e] = 0;
          if (dist <= in_run) v = *reinterpret_cast<const Piece*>(rows + (t - dist) * ld + c);
          else if (dist <= pos) v = *reinterpret_cast<const Piece*>(old_state + (int64_t)(dist - in_run - 1) * channels + c);
          *reinterpret_cast<Piece*>(new_state + (int64_t)dist * channels + c) = v;
        }
      }
    }
  }
}

// 16-byte form of qk_norm_cache_kernel: one 16-lane row per (token, item), lane r of the row owns the 16-byte pieces r, r + 16, ..
// of the head (up to four: widths <= 512 sixteen-bit / 256 fp32 channels, multiples of 8 / 4).
template <int DT>
__global__ __launch_bounds__(256) void qk_norm_cache_vec_kernel(
    const void* __restrict__ qkv, int64_t ld, const void* __restrict__ q_w, const void* __restrict__ k_w, float eps,
    float temp_coef, int temp_every, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ select,
    void* __restrict__ q_out, void* __restrict__ k_cache, void* __restrict__ v_cache, int64_t n, int heads, int kv_heads, int dk,
    int dv) {
  constexpr int EPC = DT == LL_F32 ? 4 : 8;  // elements per 16-byte piece
  typedef typename std::conditional<DT == LL_F32, float, uint16_t>::type elem;
  const int items = heads + 2 * kv_heads;
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
  if (row >= n * items) return;
  const int r = threadIdx.x & 15;
  const int64_t t = row / items;
  const int item = (int)(row - t * items);
  const bool is_q = item < heads, is_v = item >= heads + kv_heads;
  const int width = is_v ? dv : dk;
  const int64_t src = t * ld + (is_v ? (int64_t)(heads + kv_heads) * dk + (int64_t)(item - heads - kv_heads) * dv : (int64_t)item * dk);
  const int pieces = width / EPC;
  float val[4][EPC];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = r + 16 * j;
    if (c < pieces) {
      struct alignas(16) Piece { elem e[EPC]; };
      const Piece pc = *reinterpret_cast<const Piece*>((const elem*)qkv + src + c * EPC);
#pragma unroll
      for (int e = 0; e < EPC; ++e) {
        if constexpr (DT == LL_F32) val[j][e] = pc.e[e];
        else val[j][e] = to_f32<DT>(pc.e[e]);
        ss += val[j][e] * val[j][e];
      }
    }
  }
  float mul = 1.0f;
  const void* wt = nullptr;
  if (!is_v) {
    ss = row16_sum(ss);
    mul = 1.0f / sqrtf(ss / (float)dk + eps);
    wt = is_q ? q_w : k_w;
  }
  float temp = 1.0f;
  if (is_q && temp_coef != 0.f) temp = 1.0f + temp_coef * logf((float)((tok_pos[t] + 1) / temp_every) + 1.0f);
  const int64_t crow = select[t];
  elem* dst = is_q ? (elem*)q_out + (t * heads + item) * dk
                   : is_v ? (elem*)v_cache + (crow * kv_heads + (item - heads - kv_heads)) * dv
                          : (elem*)k_cache + (crow * kv_heads + (item - heads)) * dk;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = r + 16 * j;
    if (c < pieces) {
      struct alignas(16) Piece { elem e[EPC]; };
      Piece o;
#pragma unroll
      for (int e = 0; e < EPC; ++e) {
        float x = val[j][e];
        if (!is_v) {
          x *= mul;
          if (wt) x *= ldv<DT>(wt, c * EPC + e);
          if (is_q) x *= temp;
        }
        if constexpr (DT == LL_F32) o.e[e] = x;
        else o.e[e] = from_f32<DT>(x);
      }
      *reinterpret_cast<Piece*>(dst + c * EPC) = o;
    }
  }
}

// dot of an fp32 LDS vector with a contiguous cache row, channels in order; 16-byte loads when the row allows them
template <int DT>
__device__ __forceinline__ float dot_row(const float* __restrict__ a, const void* __restrict__ rowp, int64_t at, int dk, bool vec) {
  float d = 0.f;
  if constexpr (DT == LL_F32) {
    const float* r = (const float*)rowp + at;
    if (vec) {
      for (int c = 0; c < dk; c += 4) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(r + c);
        d += a[c] * x[0]; d += a[c + 1] * x[1]; d += a[c + 2] * x[2]; d += a[c + 3] * x[3];
      }
    } else {
      for (int c = 0; c < dk; ++c) d += a[c] * r[c];
    }
  } else {
    const uint16_t* r = (const uint16_t*)rowp + at;
    if (vec) {
      for (int c = 0; c < dk; c += 8) {
        const U16x8 x = *reinterpret_cast<const U16x8*>(r + c);
#pragma unroll
        for (int i = 0; i < 8; ++i) d += a[c + i] * to_f32<DT>(x.v[i]);
      }
    } else {
      for (int c = 0; c < dk; ++c) d += a[c] * to_f32<DT>(r[c]);
    }
  }
  return d;
}

// One wave per (token, query head).  Keys in tiles of 64: lane j scores key base + j (a contiguous dk-row of the cache),
// the tile's weights go through LDS, then lane c accumulates channel c (and c + 64, ...) of the output over the tile.
template <int DT, int VPL>
__global__ __launch_bounds__(256) void ragged_attention_kernel(
    const void* __restrict__ q, const void* __restrict__ k_cache, const void* __restrict__ v_cache,
    const int32_t* __restrict__ token_table, int64_t tt_stride, const int32_t* __restrict__ seq_req,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const void* __restrict__ sink, float scale,
    void* __restrict__ out, int64_t n, int heads, int kv_heads, int dk, int dv, int64_t k_stride, int64_t v_stride, int window,
    int keep_first, int64_t out_stride) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* sq = lds + wave * (dk + 128);  // [dk] query
  float* sp = sq + dk;                  // [64] weights of the tile
  int* sr = (int*)(sp + 64);            // [64] cache rows of the tile
  const int64_t w = (int64_t)blockIdx.x * 4 + wave;
  if (w >= n * heads) return;  // (no workgroup barrier below: waves are independent)
  const int64_t t = w / heads;
  const int h = (int)(w - t * heads);
  const int g = h / (heads / kv_heads);
  const int pos = tok_pos[t];
  const bool vec = (dk % (DT == LL_F32 ? 4 : 8) == 0) && (k_stride % (DT == LL_F32 ? 4 : 8) == 0) &&
                   ((reinterpret_cast<uintptr_t>(k_cache) & 15u) == 0);
  const int first_key = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;   // a window keeps the last `window` keys
  const int32_t* table = token_table + (int64_t)seq_req[tok_seq[t]] * tt_stride;
  for (int c = lane; c < dk; c += 64) sq[c] = ldv<DT>(q, (t * heads + h) * dk + c);
  float m = -INFINITY, l = 0.f;
  if (sink) {
    m = ldv<DT>(sink, h);
    l = 1.0f;
  }
  float acc[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) acc[i] = 0.f;
  __builtin_amdgcn_wave_barrier();
  // keys in position order: the sequence's first `keep_first` keys that lie in front of the window, then the window
  const int kept = keep_first < first_key ? keep_first : first_key;
  for (int base = kept > 0 ? 0 : first_key; base <= pos; base = (base < first_key && base + 64 >= kept) ? first_key : base + 64) {
    const int lim = base < first_key ? kept - 1 : pos;   // last key of this stretch
    const int j = base + lane;
    float s = -INFINITY;
    int row = 0;
    if (j <= lim) {
      row = table[j];
      const int64_t kb = (int64_t)row * k_stride + (int64_t)g * dk;
      s = dot_row<DT>(sq, k_cache, kb, dk, vec) * scale;
    }
    const float tile_max = wave_max(s);
    const float m_new = fmaxf(m, tile_max);
    const float p = j <= lim ? expf(s - m_new) : 0.f;
    const float corr = m == -INFINITY ? 0.f : expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
    sp[lane] = p;
    sr[lane] = row;
    __builtin_amdgcn_wave_barrier();
    const int cnt = lim - base + 1 < 64 ? lim - base + 1 : 64;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int c = lane + 64 * i;
      float a = acc[i] * corr;
      if (c < dv) {
        for (int jj = 0; jj < cnt; ++jj) a += sp[jj] * ldv<DT>(v_cache, (int64_t)sr[jj] * v_stride + (int64_t)g * dv + c);
      }
      acc[i] = a;
    }
    __builtin_amdgcn_wave_barrier();
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = lane + 64 * i;
    if (c < dv) stv<DT>(out, t * out_stride + (int64_t)h * dv + c, acc[i] * inv);
  }
}

}  // namespace

#define LL_BY_DTYPE(dtype, CALL)             \
  do {                                       \
    if (dtype == LL_F16) { CALL(LL_F16); }   \
    else if (dtype == LL_BF16) { CALL(LL_BF16); } \
    else { CALL(LL_F32); }                   \
  } while (0)

extern "C" int ll_qk_norm_cache(const void* qkv, int64_t ld, const void* q_w, const void* k_w, float eps, float temp_coef,
                                int64_t temp_every, const int32_t* tok_pos, const int32_t* select, void* q_out, void* k_cache,
                                void* v_cache, int64_t n, int64_t heads, int64_t kv_heads, int64_t dk, int64_t dv, int dtype,
                                void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || heads < 1 || kv_heads < 1 || heads % kv_heads || dk < 1 || dv < 1 || temp_every < 1 ||
      ld < (heads + kv_heads) * dk + kv_heads * dv)
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!qkv || !tok_pos || !select || !q_out || !k_cache || !v_cache) return LL_ERR_ARG;
  const int64_t waves = n * (heads + 2 * kv_heads);
  const int epc = dtype == LL_F32 ? 4 : 8;
  const bool vec = dk % epc == 0 && dv % epc == 0 && ld % epc == 0 && dk <= 64 * epc && dv <= 64 * epc && ll_aligned16(qkv) &&
                   ll_aligned16(q_out) && ll_aligned16(k_cache) && ll_aligned16(v_cache);
  const dim3 grid((unsigned)((waves + 3) / 4)), grid_v((unsigned)((waves + 15) / 16));
#define LL_QK_ARGS \
  qkv, ld, q_w, k_w, eps, temp_coef, (int)temp_every, tok_pos, select, q_out, k_cache, v_cache, n, (int)heads, (int)kv_heads, (int)dk, (int)dv
#define CALL(DT)                                                                                  \
  if (vec) qk_norm_cache_vec_kernel<DT><<<grid_v, 256, 0, (hipStream_t)stream>>>(LL_QK_ARGS);     \
  else qk_norm_cache_kernel<DT><<<grid, 256, 0, (hipStream_t)stream>>>(LL_QK_ARGS)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef LL_QK_ARGS
  return LL_LAUNCH_CHECK();
}

namespace {
// one thread per (token, pair): out[t][i] = (cos(pos * f_i) * amp, sin(pos * f_i) * amp); rows of rot_stride(pairs) floats
__global__ __launch_bounds__(256) void rotation_table_kernel(const int32_t* __restrict__ tok_pos, const float* __restrict__ freq,
                                                             int pairs, float amp, float* __restrict__ out, int64_t n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int padded = (int)(rot_stride(pairs) / 2);
  if (idx >= n * padded) return;
  const int64_t t = idx / padded;
  const int i = (int)(idx - t * padded);
  if (i >= pairs) {   // the padding reads as zeros
    out[t * rot_stride(pairs) + 2 * i] = 0.f;
    out[t * rot_stride(pairs) + 2 * i + 1] = 0.f;
    return;
  }
  float sn, cs;
  sincosf((float)tok_pos[t] * freq[i], &sn, &cs);   // (one argument reduction for both)
  out[t * rot_stride(pairs) + 2 * i] = cs * amp;
  out[t * rot_stride(pairs) + 2 * i + 1] = sn * amp;
}
}  // namespace

extern "C" int ll_rotation_table(const int32_t* tok_pos, const float* freq, int64_t pairs, float amp, float* out, int64_t n,
                                 void* stream) {
  if (n < 0 || pairs < 1 || pairs > 4096) return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!tok_pos || !freq || !out) return LL_ERR_ARG;
  rotation_table_kernel<<<dim3((unsigned)((n * (rot_stride(pairs) / 2) + 255) / 256)), 256, 0, (hipStream_t)stream>>>(tok_pos, freq, (int)pairs,
                                                                                                                 amp, out, n);
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_conv_rope_cache(const void* qkv, int64_t ld, const void* bias, const void* conv_w, int64_t taps, void* conv_state,
                                  int64_t state_half, const float* freq, int64_t pairs, float amp, const float* rot_table,
                                  int unit_norm, float eps,
                                  const void* v_src, int64_t v_src_stride, const void* v_lam, const int32_t* tok_seq,
                                  const int32_t* tok_pos, const int32_t* select, const int32_t* seq_start,
                                  const int32_t* seq_first_pos, const int32_t* seq_slot, const int32_t* seq_parity, void* q_out,
                                  void* k_cache, void* v_cache, int64_t n, int64_t heads, int64_t kv_heads, int64_t dk, int64_t dv,
                                  int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || heads < 1 || kv_heads < 1 || heads % kv_heads || dk < 1 || dk > 1024 || dv < 1 || dv > 1024 || taps < 0 || taps > 64 ||
      pairs < 0 || 2 * pairs > dk || ld < (heads + kv_heads) * dk + kv_heads * dv || (v_src && v_src_stride < kv_heads * dv))
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!qkv || !tok_seq || !tok_pos || !select || !seq_start || !seq_first_pos || !seq_slot || !seq_parity || !q_out || !k_cache ||
      !v_cache || (taps > 0 && !conv_w) || (taps > 1 && !conv_state) || (pairs > 0 && !freq && !rot_table) || (v_src && !v_lam))
    return LL_ERR_ARG;
  const int64_t waves = n * (heads + 2 * kv_heads);
  const dim3 grid((unsigned)((waves + 3) / 4));
  const int64_t widest = dk > dv ? dk : dv;
  hipStream_t st = (hipStream_t)stream;
#define LL_CR_ARGS                                                                                                              \
  qkv, ld, bias, conv_w, (int)taps, conv_state, state_half, freq, (int)pairs, amp, rot_table, unit_norm, eps, v_src, v_src_stride, v_lam, tok_seq, \
      tok_pos, select, seq_start, seq_first_pos, seq_slot, seq_parity, q_out, k_cache, v_cache, n, (int)heads, (int)kv_heads, (int)dk, \
      (int)dv
  const int epc = dtype == LL_F32 ? 4 : 8;
  const bool vec = (pairs == 0 || (rot_table && ll_aligned16(rot_table))) && taps <= 4 && dk % epc == 0 && dv % epc == 0 && ld % epc == 0 && widest <= 64 * epc && ll_aligned16(qkv) &&
                   ll_aligned16(q_out) && ll_aligned16(k_cache) && ll_aligned16(v_cache) && (!bias || ll_aligned16(bias)) &&
                   (!conv_w || ll_aligned16(conv_w)) && (taps <= 1 || ll_aligned16(conv_state)) &&
                   (!v_src || (ll_aligned16(v_src) && v_src_stride % epc == 0));
  if (vec) {
    // 16 tokens per workgroup; the items of a token in groups of 4 when that still fills the chip, else one item each
    const int64_t tiles = (n + 15) / 16, items = heads + 2 * kv_heads;
    const int ipw = tiles * ((items + 3) / 4) >= 1024 ? 4 : 1;
    const dim3 grid_v((unsigned)tiles, (unsigned)((items + ipw - 1) / ipw));
    const size_t lds_v = 0;
#define LL_CRV_ARGS                                                                                                              \
  qkv, ld, bias, conv_w, conv_state, state_half, rot_table, (int)pairs, unit_norm, eps, v_src, v_src_stride, v_lam, tok_seq, tok_pos, \
      select, seq_start, seq_first_pos, seq_slot, seq_parity, q_out, k_cache, v_cache, n, (int)heads, (int)kv_heads, (int)dk, (int)dv, ipw
    const int npc = widest <= 16 * epc ? 1 : widest <= 32 * epc ? 2 : 4;
#define CALL_N(DT, T)                                                                                            \
  if (npc == 1) conv_rope_cache_vec_kernel<DT, T, 1><<<grid_v, 256, lds_v, st>>>(LL_CRV_ARGS);                   \
  else if (npc == 2) conv_rope_cache_vec_kernel<DT, T, 2><<<grid_v, 256, lds_v, st>>>(LL_CRV_ARGS);              \
  else conv_rope_cache_vec_kernel<DT, T, 4><<<grid_v, 256, lds_v, st>>>(LL_CRV_ARGS)
#define CALL(DT)                              \
  if (taps == 0) { CALL_N(DT, 0); }           \
  else if (taps == 1) { CALL_N(DT, 1); }      \
  else if (taps == 2) { CALL_N(DT, 2); }      \
  else if (taps == 3) { CALL_N(DT, 3); }      \
  else { CALL_N(DT, 4); }
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef CALL_N
#undef LL_CRV_ARGS
    return LL_LAUNCH_CHECK();
  }
#define CALL(DT)                                                                               \
  if (widest <= 128) conv_rope_cache_kernel<DT, 1><<<grid, 256, 0, st>>>(LL_CR_ARGS);          \
  else if (widest <= 256) conv_rope_cache_kernel<DT, 2><<<grid, 256, 0, st>>>(LL_CR_ARGS);     \
  else if (widest <= 512) conv_rope_cache_kernel<DT, 4><<<grid, 256, 0, st>>>(LL_CR_ARGS);     \
  else conv_rope_cache_kernel<DT, 8><<<grid, 256, 0, st>>>(LL_CR_ARGS)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef LL_CR_ARGS
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_ragged_attention(const void* q, const void* k_cache, const void* v_cache, const int32_t* token_table,
                                   int64_t tt_stride, const int32_t* seq_req, const int32_t* tok_seq, const int32_t* tok_pos,
                                   const void* sink, float scale, void* out, int64_t n, int64_t heads, int64_t kv_heads, int64_t dk,
                                   int64_t dv, int64_t k_stride, int64_t v_stride, int64_t window, int64_t keep_first,
                                   int64_t out_stride, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || heads < 1 || kv_heads < 1 || heads % kv_heads || dk < 1 || dk > 1024 || dv < 1 || dv > 1024 || window < 0 ||
      window > 0x7fffffff || keep_first < 0 || keep_first > 0x7fffffff || k_stride < kv_heads * dk || v_stride < kv_heads * dv ||
      out_stride < heads * dv)
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!q || !k_cache || !v_cache || !token_table || !seq_req || !tok_seq || !tok_pos || !out) return LL_ERR_ARG;
  const int64_t waves = n * heads;
  const dim3 grid((unsigned)((waves + 3) / 4));
  const size_t lds = sizeof(float) * 4 * (size_t)(dk + 128);
  const int vpl = (int)((dv + 63) / 64);
  hipStream_t st = (hipStream_t)stream;
#define CALL_V(DT, V)                                                                                                        \
  ragged_attention_kernel<DT, V><<<grid, 256, lds, st>>>(q, k_cache, v_cache, token_table, tt_stride, seq_req, tok_seq, tok_pos, \
                                                         sink, scale, out, n, (int)heads, (int)kv_heads, (int)dk, (int)dv, k_stride, \
                                                         v_stride, (int)window, (int)keep_first, out_stride)
#define CALL(DT)                     \
  if (vpl == 1) CALL_V(DT, 1);       \
  else if (vpl == 2) CALL_V(DT, 2);  \
  else if (vpl <= 4) CALL_V(DT, 4);  \
  else if (vpl <= 8) CALL_V(DT, 8);  \
  else CALL_V(DT, 16)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
#undef CALL_V
  return LL_LAUNCH_CHECK();
}
