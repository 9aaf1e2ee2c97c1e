// MFMA forms of the ragged attention with a sink (16-bit storage dtypes; the fp32 storage dtype keeps the VALU form of
// ragged_attn.hip).  A wave owns 16 QUERY COLUMNS and walks its key range in tiles of 32:
//
//   prompt portions   (and steps that mix them with decoded tokens) four waves = 64 consecutive tokens of one (sequence, head);
//                     a tile's K and V rows are fetched once per workgroup and shared through LDS
//   decoded tokens    one wave whose columns are (up to) 16 query heads of ONE token that share a key/value head, so K and V
//                     are read once for the whole group; the context is cut into partitions of kPart keys, one wave each,
//                     whose (max, sum, output) triples a merge kernel combines
//
// S^T = K Q^T puts keys in MFMA rows and queries in columns (the running softmax of a query is lane-local up to two row
// swaps), and the S^T accumulators are directly the P^T operand of O^T = V^T P^T.  Scores, weights and sums are fp32; for the
// second product the fp32 weight is split into two 16-bit parts (p = hi + lo, two MFMAs) so that it enters with ~16 mantissa
// bits instead of 8.  The sink starts the running softmax (max = sink, sum = 1) of a sequence's FIRST partition.
// Widths that are not multiples of 32 (keys) / 16 (values) are zero-padded; both must be multiples of 8.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

namespace {

constexpr int kPart = 256;  // keys per partition (decoded tokens)
constexpr float kLog2e = 1.4426950408889634f;

struct alignas(16) Q4 {
  uint32_t x, y, z, w;
};

template <int DT>
__device__ __forceinline__ f32x4 mfma16(const Q4& a, const Q4& b, f32x4 c) {
  if constexpr (DT == LL_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// fp32 -> (hi, lo) in the storage dtype with hi + lo = p up to ~2^-17 relative
template <int DT>
__device__ __forceinline__ void split2(float p, uint16_t& hi, uint16_t& lo) {
  hi = from_f32<DT>(p);
  const float rest = p - to_f32<DT>(hi);   // exact; |rest| <= half an ulp of hi
  if constexpr (DT == LL_BF16) lo = (uint16_t)(__float_as_uint(rest) >> 16);  // truncated: 2^-8 of 2^-9 of p
  else lo = from_f32<DT>(rest);
}

// Decoded tokens.  grid = (partitions of the longest context, kv_heads * column tiles per group, sequences)
template <int DT, int NSM, int NTM>
__global__ __launch_bounds__(64) void ragged_attention_mfma_decode_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const int32_t* __restrict__ token_table, int64_t tt_stride, const int32_t* __restrict__ seq_req,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const uint16_t* __restrict__ sink,
    float scale_log2, uint16_t* __restrict__ out, float* __restrict__ partials, int max_parts, int heads, int kv_heads, int dk,
    int dv, int64_t k_stride, int64_t v_stride, int window, int shared_kv, int keep_first, int64_t out_stride) {
  static_assert(NTM / 2 == NSM, "value fragments of shared rows are the key fragments");
  constexpr int QB = 1;
  constexpr bool DECODE = true;
  constexpr int VSTR = NTM * 16 + 8;
  __shared__ __attribute__((aligned(16))) uint16_t lds_v[32 * VSTR];
  const int lane = threadIdx.x, t = lane & 15, c = lane >> 4;
  const int b = blockIdx.z;
  const int start = seq_start[b], first = seq_first_pos[b];
  const int group = heads / kv_heads;
  int g, k_lo, k_hi, k_begin;   // k_begin: the first key a window still keeps (0 without one)
  int kept = 0;                 // the sequence's first keys that stay visible in front of the window
  int jump_from = -1, jump_to = 0;   // the tile walk leaves out what lies between the kept keys and the window
  int head[QB], token[QB], qpos[QB];
  bool valid[QB];
  {
    const int tiles = (group + 15) / 16;
    g = blockIdx.y / tiles;
    const int h0 = (blockIdx.y - g * tiles) * 16;
    valid[0] = h0 + t < group;
    head[0] = g * group + (valid[0] ? h0 + t : h0);
    token[0] = start;
    qpos[0] = first;  // (a decoded token: the sequence brings one)
    k_begin = window > 0 && first - window + 1 > 0 ? first - window + 1 : 0;
    kept = keep_first < k_begin ? keep_first : k_begin;
    k_lo = blockIdx.x * kPart;
    const bool in_window = !(k_lo > first || k_lo + kPart <= k_begin), in_kept = k_lo < kept;
    if (!in_window && !in_kept) return;   // (a partition past the token, or in front of the window with no kept key)
    k_hi = k_lo + kPart < first + 1 ? k_lo + kPart : first + 1;
    if (!in_window) k_hi = k_hi < kept ? k_hi : kept;
    if (k_lo < k_begin) {                 // the window's first partition starts at the tile that holds k_begin ...
      const int w_lo = (k_begin / 32) * 32;
      if (!in_kept) {
        k_lo = w_lo;
      } else if (in_window) {             // ... behind the tiles of the kept keys, when the partition holds both
        const int kept_end = ((kept < k_hi ? kept : k_hi) + 31) / 32 * 32;
        if (kept_end < w_lo) {
          jump_from = kept_end;
          jump_to = w_lo;
        }
      }
    }
  }
  auto next_tile = [&](int p) { return p + 32 == jump_from ? jump_to : p + 32; };
  const int32_t* table = token_table + (int64_t)seq_req[b] * tt_stride;
  const uint16_t* vtr = lds_v + (4 * c + (t >> 2)) * VSTR + (t & 3) * 4;
  const int ns = (dk + 31) / 32, nt = (dv + 15) / 16, nsv = (dv + 31) / 32;

  // Q^T fragments: column t, contraction chunk j = 4 s + c (8 channels at 8 j); chunks past dk are zero
  Q4 qf[QB][NSM];
  float m_i[QB], d_i[QB];
  f32x4 ot[QB][NTM];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
    for (int s = 0; s < NSM; ++s) {
      const int ch = 8 * (4 * s + c);
      qf[qb][s] = (s < ns && ch < dk) ? *reinterpret_cast<const Q4*>(q + ((int64_t)token[qb] * heads + head[qb]) * dk + ch)
                                      : Q4{0, 0, 0, 0};
    }
    m_i[qb] = -INFINITY;
    d_i[qb] = 0.f;
    if (sink && (int)blockIdx.x == (kept > 0 ? 0 : k_begin / kPart)) {
      m_i[qb] = to_f32<DT>(sink[head[qb]]) * kLog2e;
      d_i[qb] = 1.0f;
    }
#pragma unroll
    for (int i = 0; i < NTM; ++i) ot[qb][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // K / V fragments of a tile are requested one tile ahead (and its cache rows two tiles ahead): the loads of tile i + 1 are in
  // flight under the products and the softmax of tile i
  #define zero4 (Q4{0, 0, 0, 0})
  auto rows_of = [&](int p, int64_t& ra, int64_t& rb) {
    ra = p + t < k_hi ? table[p + t] : 0;
    rb = p + 16 + t < k_hi ? table[p + 16 + t] : 0;
  };
  auto fetch = [&](int p, int64_t ra, int64_t rb, Q4 (&fa)[NSM], Q4 (&fb)[NSM], Q4 (&ga)[NTM / 2], Q4 (&gb)[NTM / 2]) {
    const bool okA = p + t < k_hi, okB = p + 16 + t < k_hi;
    const uint16_t* kA = k_cache + ra * k_stride + (int64_t)g * dk;
    const uint16_t* kB = k_cache + rb * k_stride + (int64_t)g * dk;
    const uint16_t* vA = v_cache + ra * v_stride + (int64_t)g * dv;
    const uint16_t* vB = v_cache + rb * v_stride + (int64_t)g * dv;
#pragma unroll
    for (int s = 0; s < NSM; ++s) {
      const int ch = 8 * (4 * s + c);
      const bool in = s < ns && ch < dk;
      fa[s] = (in && okA) ? *reinterpret_cast<const Q4*>(kA + ch) : zero4;
      fb[s] = (in && okB) ? *reinterpret_cast<const Q4*>(kB + ch) : zero4;
    }
#pragma unroll
    for (int s = 0; s < NTM / 2; ++s) {
      const int ch = 8 * (4 * s + c);
      const bool in = s < nsv && ch < dv;
      // shared_kv: the value rows ARE the key rows (a latent cache): the key fragments just loaded are the value fragments
      // (channels past dv ride along into output columns that are never stored)
      ga[s] = shared_kv ? fa[s] : (in && okA) ? *reinterpret_cast<const Q4*>(vA + ch) : zero4;
      gb[s] = shared_kv ? fb[s] : (in && okB) ? *reinterpret_cast<const Q4*>(vB + ch) : zero4;
    }
  };
  Q4 ka[NSM], kb[NSM], va[NTM / 2], vb[NTM / 2];
  int64_t nra, nrb;
  {
    int64_t ra, rb;
    rows_of(k_lo, ra, rb);
    rows_of(next_tile(k_lo), nra, nrb);
    fetch(k_lo, ra, rb, ka, kb, va, vb);
  }
  for (int p0 = k_lo, p1; p0 < k_hi; p0 = p1) {
    p1 = next_tile(p0);
    Q4 nka[NSM], nkb[NSM], nva[NTM / 2], nvb[NTM / 2];
    fetch(p1, nra, nrb, nka, nkb, nva, nvb);   // (past the range: nothing is read)
    rows_of(next_tile(p1), nra, nrb);
    Q4 pf_hi[QB], pf_lo[QB];
    float alpha[QB];
    bool moved[QB];   // some column's running maximum moved (wave-uniform): only then the outputs are rescaled
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < NSM; ++s)
        if (s < ns) sa = mfma16<DT>(ka[s], qf[qb][s], sa);
#pragma unroll
      for (int s = 0; s < NSM; ++s)
        if (s < ns) sb = mfma16<DT>(kb[s], qf[qb][s], sb);
      // rows = keys p0 + 4 c + r (+ 16), column = query t
      float sc[8];
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int k0i = p0 + 4 * c + r, k1i = k0i + 16;
        sc[r] = (k0i <= qpos[qb] && k0i < k_hi && (k0i >= k_begin || k0i < kept)) ? sa[r] * scale_log2 : -INFINITY;
        sc[4 + r] = (k1i <= qpos[qb] && k1i < k_hi && (k1i >= k_begin || k1i < kept)) ? sb[r] * scale_log2 : -INFINITY;
        mx = fmaxf(mx, fmaxf(sc[r], sc[4 + r]));
      }
      mx = rows_max(mx);
      float m_new = fmaxf(m_i[qb], mx);
      if (m_new == -INFINITY) m_new = 0.f;      // nothing seen yet and nothing visible in this tile: every weight is exp2(-inf) = 0
      alpha[qb] = m_i[qb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_i[qb] - m_new);
      float p[8];
      float ps = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        p[j] = __builtin_amdgcn_exp2f(sc[j] - m_new);   // (v_exp_f32: 1 ulp; masked keys: exp2(-inf) = 0)
        ps += p[j];
      }
      ps = rows_sum(ps);
      d_i[qb] = d_i[qb] * alpha[qb] + ps;
      m_i[qb] = fmaxf(m_i[qb], mx);
      moved[qb] = __builtin_amdgcn_ballot_w64(alpha[qb] != 1.0f) != 0;
      uint16_t hi[8], lo[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) split2<DT>(p[j], hi[j], lo[j]);
      pf_hi[qb] = Q4{(uint32_t)hi[0] | ((uint32_t)hi[1] << 16), (uint32_t)hi[2] | ((uint32_t)hi[3] << 16),
                     (uint32_t)hi[4] | ((uint32_t)hi[5] << 16), (uint32_t)hi[6] | ((uint32_t)hi[7] << 16)};
      pf_lo[qb] = Q4{(uint32_t)lo[0] | ((uint32_t)lo[1] << 16), (uint32_t)lo[2] | ((uint32_t)lo[3] << 16),
                     (uint32_t)lo[4] | ((uint32_t)lo[5] << 16), (uint32_t)lo[6] | ((uint32_t)lo[7] << 16)};
    }

    __syncthreads();
#pragma unroll
    for (int s = 0; s < NTM / 2; ++s) {
      const int ch = 8 * (4 * s + c);
      if (s < nsv && ch < NTM * 16) {
        *reinterpret_cast<Q4*>(&lds_v[t * VSTR + ch]) = va[s];
        *reinterpret_cast<Q4*>(&lds_v[(16 + t) * VSTR + ch]) = vb[s];
      }
    }
    __syncthreads();
#pragma unroll
    for (int dt = 0; dt < NTM; ++dt) {
      if (dt < nt) {
        // V^T fragment by two transposing LDS reads: lane (t, c) ends with keys 4 c .. 4 c + 3 (and + 16) of channel dt * 16 + t
        const s16x4 tlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vtr + dt * 16));
        const s16x4 thi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vtr + 16 * VSTR + dt * 16));
        Q4 vf;
        vf.x = (uint32_t)(uint16_t)tlo.x | ((uint32_t)(uint16_t)tlo.y << 16);
        vf.y = (uint32_t)(uint16_t)tlo.z | ((uint32_t)(uint16_t)tlo.w << 16);
        vf.z = (uint32_t)(uint16_t)thi.x | ((uint32_t)(uint16_t)thi.y << 16);
        vf.w = (uint32_t)(uint16_t)thi.z | ((uint32_t)(uint16_t)thi.w << 16);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          f32x4 acc = ot[qb][dt];
          if (moved[qb]) {
            acc[0] *= alpha[qb]; acc[1] *= alpha[qb]; acc[2] *= alpha[qb]; acc[3] *= alpha[qb];
          }
          acc = mfma16<DT>(vf, pf_hi[qb], acc);
          ot[qb][dt] = mfma16<DT>(vf, pf_lo[qb], acc);
        }
      }
    }
#pragma unroll
    for (int s = 0; s < NSM; ++s) {
      ka[s] = nka[s];
      kb[s] = nkb[s];
    }
#pragma unroll
    for (int s = 0; s < NTM / 2; ++s) {
      va[s] = nva[s];
      vb[s] = nvb[s];
    }
  }

#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    if (!valid[qb]) continue;
    if (!DECODE || max_parts == 1) {
      const float inv = 1.0f / d_i[qb];
      uint16_t* o = out + (int64_t)token[qb] * out_stride + (int64_t)head[qb] * dv;
#pragma unroll
      for (int dt = 0; dt < NTM; ++dt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int ch = dt * 16 + 4 * c + r;
          if (dt < nt && ch < dv) o[ch] = from_f32<DT>(ot[qb][dt][r] * inv);
        }
      }
    } else {
      // partial triple of (token, head, partition): [max, sum, output[dv]]
      float* dst = partials + (((int64_t)token[qb] * heads + head[qb]) * max_parts + blockIdx.x) * (2 + dv);
      if (c == 0) {
        dst[0] = m_i[qb];
        dst[1] = d_i[qb];
      }
#pragma unroll
      for (int dt = 0; dt < NTM; ++dt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int ch = dt * 16 + 4 * c + r;
          if (dt < nt && ch < dv) dst[2 + ch] = ot[qb][dt][r];
        }
      }
    }
  }
}

// Prompt portions, four-wave form: a workgroup owns 64 consecutive tokens of one (sequence, head) -- wave w the 16 columns
// q0 + 16 w .. -- and walks the keys in tiles of 32 that are fetched ONCE per workgroup (global -> registers -> LDS, the next
// tile's loads in flight under the current tile's products): 64 queries per byte of K / V instead of 16.  K fragments are
// 16-byte LDS reads, V^T fragments transposing LDS reads.  A wave whose columns end before the tile (causality) or lie past
// the run's end only helps to load.
template <int DT, int NSM, int NTM>
__global__ __launch_bounds__(256) void ragged_attention_mfma_prefill4_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const int32_t* __restrict__ token_table, int64_t tt_stride, const int32_t* __restrict__ seq_req,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_first_pos, const uint16_t* __restrict__ sink,
    float scale_log2, uint16_t* __restrict__ out, int heads, int kv_heads, int dk, int dv, int64_t k_stride, int64_t v_stride,
    int window, int shared_kv, int keep_first, int64_t out_stride) {
  constexpr int KSTR = NSM * 32 + 8, VSTR = NTM * 16 + 8;
  constexpr int KPASS = (32 * NSM * 4 + 255) / 256, VPASS = (32 * NTM * 2 + 255) / 256;  // 16-byte pieces per thread
  __shared__ __attribute__((aligned(16))) uint16_t lds_k[32 * KSTR];
  __shared__ __attribute__((aligned(16))) uint16_t lds_v[32 * VSTR];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, t = lane & 15, c = lane >> 4;
  const int b = blockIdx.z;
  const int start = seq_start[b], count = seq_start[b + 1] - start, first = seq_first_pos[b];
  const int q0 = blockIdx.x * 64;
  if (q0 >= count) return;
  const int head = blockIdx.y, g = head / (heads / kv_heads);
  const int qw = q0 + 16 * wave;
  const bool wave_on = qw < count;
  const bool valid = qw + t < count;
  const int qi = valid ? qw + t : count - 1;   // columns past the run's end repeat its last token, never stored
  const int token = start + qi, qpos = first + qi;
  const int k_hi = first + (q0 + 64 < count ? q0 + 64 : count);            // the workgroup's key range
  const int k_hi_w = first + (qw + 16 < count ? qw + 16 : count);         // this wave's
  // with a window a column at position p sees keys p - window + 1 .. p: the workgroup starts at the tile that holds the first
  // key of its first column, a wave skips tiles in front of its own first column's window
  const int k_lo_wg = window > 0 && first + q0 - window + 1 > 0 ? ((first + q0 - window + 1) / 32) * 32 : 0;
  const int k_lo_w = window > 0 && first + qw - window + 1 > 0 ? first + qw - window + 1 : 0;
  const int wlo = window > 0 ? qpos - window + 1 : 0;
  // the sequence's first `keep_first` keys stay visible in front of a window: their tiles are walked first, then the walk jumps
  // to the window's first tile (keys in position order, whatever the step looks like)
  const int kept_wg = keep_first < k_lo_wg ? keep_first : k_lo_wg;
  const int kept_end = (kept_wg + 31) / 32 * 32;
  const int k_first_wg = kept_wg > 0 ? 0 : k_lo_wg;
  const int jump_from = kept_wg > 0 && kept_end < k_lo_wg ? kept_end : -1;
  auto next_tile = [&](int p) { return p + 32 == jump_from ? k_lo_wg : p + 32; };
  const int32_t* table = token_table + (int64_t)seq_req[b] * tt_stride;
  const int ns = (dk + 31) / 32, nt = (dv + 15) / 16;
  const int kcpr = dk / 8, vcpr = dv / 8;                                  // 16-byte pieces per cache row
  static_assert(KSTR == VSTR, "value tiles of shared rows are read from the key tile");
  // shared_kv: the value rows ARE the key rows (a latent cache): nothing is fetched or staged for V, the transposing reads go
  // to the key tile (channels past dv land in output columns that are never stored)
  const uint16_t* vtr = (shared_kv ? lds_k : lds_v) + (4 * c + (t >> 2)) * VSTR + (t & 3) * 4;

  for (int i = tid; i < 32 * KSTR / 8; i += 256) reinterpret_cast<Q4*>(lds_k)[i] = Q4{0, 0, 0, 0};   // (pad columns stay zero)
  for (int i = tid; i < 32 * VSTR / 8; i += 256) reinterpret_cast<Q4*>(lds_v)[i] = Q4{0, 0, 0, 0};

  Q4 qf[NSM];
#pragma unroll
  for (int s = 0; s < NSM; ++s) {
    const int ch = 8 * (4 * s + c);
    qf[s] = (s < ns && ch < dk) ? *reinterpret_cast<const Q4*>(q + ((int64_t)token * heads + head) * dk + ch) : Q4{0, 0, 0, 0};
  }
  float m_i = -INFINITY, d_i = 0.f;
  if (sink) {
    m_i = to_f32<DT>(sink[head]) * kLog2e;
    d_i = 1.0f;
  }
  f32x4 ot[NTM];
#pragma unroll
  for (int i = 0; i < NTM; ++i) ot[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  Q4 kr[KPASS], vr[VPASS];
  int rk[KPASS], rv[VPASS];   // cache rows of the pieces this thread fetches next: read one tile ahead of the pieces themselves
  // piece i of a tile: key i / pieces-per-row, channels 8 (i % pieces-per-row); keys past the range load zeros
#define LL_ROWS(P)                                                                                                 \
  _Pragma("unroll") for (int u = 0; u < KPASS; ++u) {                                                              \
    const int key = (tid + 256 * u) / kcpr;                                                                        \
    rk[u] = (key < 32 && (P) + key < k_hi) ? table[(P) + key] : 0;                                                 \
  }                                                                                                                \
  if (!shared_kv) _Pragma("unroll") for (int u = 0; u < VPASS; ++u) {                                              \
    const int key = (tid + 256 * u) / vcpr;                                                                        \
    rv[u] = (key < 32 && (P) + key < k_hi) ? table[(P) + key] : 0;                                                 \
  }
#define LL_FETCH(P)                                                                                                \
  _Pragma("unroll") for (int u = 0; u < KPASS; ++u) {                                                              \
    const int i = tid + 256 * u, key = i / kcpr, piece = i - key * kcpr;                                           \
    kr[u] = (key < 32 && (P) + key < k_hi)                                                                         \
                ? *reinterpret_cast<const Q4*>(k_cache + (int64_t)rk[u] * k_stride + (int64_t)g * dk + 8 * piece)  \
                : Q4{0, 0, 0, 0};                                                                                  \
  }                                                                                                                \
  if (!shared_kv) _Pragma("unroll") for (int u = 0; u < VPASS; ++u) {                                              \
    const int i = tid + 256 * u, key = i / vcpr, piece = i - key * vcpr;                                           \
    vr[u] = (key < 32 && (P) + key < k_hi)                                                                         \
                ? *reinterpret_cast<const Q4*>(v_cache + (int64_t)rv[u] * v_stride + (int64_t)g * dv + 8 * piece)  \
                : Q4{0, 0, 0, 0};                                                                                  \
  }
#define LL_STAGE()                                                                           \
  _Pragma("unroll") for (int u = 0; u < KPASS; ++u) {                                        \
    const int i = tid + 256 * u, key = i / kcpr, piece = i - key * kcpr;                     \
    if (key < 32) *reinterpret_cast<Q4*>(&lds_k[key * KSTR + 8 * piece]) = kr[u];            \
  }                                                                                          \
  if (!shared_kv) _Pragma("unroll") for (int u = 0; u < VPASS; ++u) {                        \
    const int i = tid + 256 * u, key = i / vcpr, piece = i - key * vcpr;                     \
    if (key < 32) *reinterpret_cast<Q4*>(&lds_v[key * VSTR + 8 * piece]) = vr[u];            \
  }
  LL_ROWS(k_first_wg)
  LL_FETCH(k_first_wg)
  LL_ROWS(next_tile(k_first_wg))   // (past the range: nothing is read)
  __syncthreads();   // the zero fill is complete
  LL_STAGE()
  __syncthreads();
  for (int p0 = k_first_wg, p1; p0 < k_hi; p0 = p1) {
    p1 = next_tile(p0);
    if (p1 < k_hi) {
      LL_FETCH(p1)
      LL_ROWS(next_tile(p1))
    }
    if (wave_on && p0 < k_hi_w && (p0 + 32 > k_lo_w || p0 < keep_first)) {
      f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < NSM; ++s) {
        if (s < ns) {
          const Q4 ka = *reinterpret_cast<const Q4*>(&lds_k[t * KSTR + 8 * (4 * s + c)]);
          const Q4 kb = *reinterpret_cast<const Q4*>(&lds_k[(16 + t) * KSTR + 8 * (4 * s + c)]);
          sa = mfma16<DT>(ka, qf[s], sa);
          sb = mfma16<DT>(kb, qf[s], sb);
        }
      }
      float sc[8];
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int k0i = p0 + 4 * c + r, k1i = k0i + 16;
        sc[r] = (k0i <= qpos && (k0i >= wlo || k0i < keep_first)) ? sa[r] * scale_log2 : -INFINITY;
        sc[4 + r] = (k1i <= qpos && (k1i >= wlo || k1i < keep_first)) ? sb[r] * scale_log2 : -INFINITY;
        mx = fmaxf(mx, fmaxf(sc[r], sc[4 + r]));
      }
      mx = rows_max(mx);
      float m_new = fmaxf(m_i, mx);
      if (m_new == -INFINITY) m_new = 0.f;  // a column whose window starts behind this tile and that has seen nothing yet
      const float alpha = m_i == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_i - m_new);
      float ps = 0.f;
      uint16_t hi[8], lo[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float pj = __builtin_amdgcn_exp2f(sc[j] - m_new);
        ps += pj;
        split2<DT>(pj, hi[j], lo[j]);
      }
      ps = rows_sum(ps);
      d_i = d_i * alpha + ps;
      m_i = fmaxf(m_i, mx);
      const Q4 pf_hi = {(uint32_t)hi[0] | ((uint32_t)hi[1] << 16), (uint32_t)hi[2] | ((uint32_t)hi[3] << 16),
                        (uint32_t)hi[4] | ((uint32_t)hi[5] << 16), (uint32_t)hi[6] | ((uint32_t)hi[7] << 16)};
      const Q4 pf_lo = {(uint32_t)lo[0] | ((uint32_t)lo[1] << 16), (uint32_t)lo[2] | ((uint32_t)lo[3] << 16),
                        (uint32_t)lo[4] | ((uint32_t)lo[5] << 16), (uint32_t)lo[6] | ((uint32_t)lo[7] << 16)};
      const bool moved = __builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0;
#pragma unroll
      for (int dt = 0; dt < NTM; ++dt) {
        if (dt < nt) {
          const s16x4 tlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vtr + dt * 16));
          const s16x4 thi =
              __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vtr + 16 * VSTR + dt * 16));
          Q4 vf;
          vf.x = (uint32_t)(uint16_t)tlo.x | ((uint32_t)(uint16_t)tlo.y << 16);
          vf.y = (uint32_t)(uint16_t)tlo.z | ((uint32_t)(uint16_t)tlo.w << 16);
          vf.z = (uint32_t)(uint16_t)thi.x | ((uint32_t)(uint16_t)thi.y << 16);
          vf.w = (uint32_t)(uint16_t)thi.z | ((uint32_t)(uint16_t)thi.w << 16);
          f32x4 acc = ot[dt];
          if (moved) {
            acc[0] *= alpha; acc[1] *= alpha; acc[2] *= alpha; acc[3] *= alpha;
          }
          acc = mfma16<DT>(vf, pf_hi, acc);
          ot[dt] = mfma16<DT>(vf, pf_lo, acc);
        }
      }
    }
    __syncthreads();   // everybody has read this tile
    if (p1 < k_hi) { LL_STAGE() }
    __syncthreads();
  }
#undef LL_ROWS
#undef LL_FETCH
#undef LL_STAGE
  if (!valid) return;
  const float inv = 1.0f / d_i;
  uint16_t* o = out + (int64_t)token * out_stride + (int64_t)head * dv;
#pragma unroll
  for (int dt = 0; dt < NTM; ++dt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ch = dt * 16 + 4 * c + r;
      if (dt < nt && ch < dv) o[ch] = from_f32<DT>(ot[dt][r] * inv);
    }
  }
}

// one wave per (token, head): combine the partitions of a decoded token in partition order
template <int DT>
__global__ __launch_bounds__(256) void ragged_attention_merge_kernel(const float* __restrict__ partials, int max_parts,
                                                                     const int32_t* __restrict__ seq_first_pos,
                                                                     uint16_t* __restrict__ out, int64_t n, int heads, int dv,
                                                                     int window, int keep_first, int64_t out_stride) {
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= n * heads) return;
  const int lane = threadIdx.x & 63;
  const int64_t token = w / heads;
  const int pos = seq_first_pos[token];                // (decoded tokens: token index == sequence index)
  const int parts = pos / kPart + 1;
  const int k_begin = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
  const int p_lo = k_begin / kPart;   // partitions in front of it wrote nothing, but for those that hold kept first keys
  const int kept = keep_first < k_begin ? keep_first : k_begin;
  const int p_kept = (kept + kPart - 1) / kPart;
  const float* src = partials + w * max_parts * (2 + dv);
  float m = -INFINITY;
  for (int p = 0; p < parts; ++p)
    if (p >= p_lo || p < p_kept) m = fmaxf(m, src[p * (2 + dv)]);
  float d = 0.f;
  for (int p = 0; p < parts; ++p)
    if (p >= p_lo || p < p_kept) d += src[p * (2 + dv) + 1] * exp2f(src[p * (2 + dv)] - m);
  const int h = (int)(w - token * heads);
  for (int ch = lane; ch < dv; ch += 64) {
    float o = 0.f;
    for (int p = 0; p < parts; ++p)
      if (p >= p_lo || p < p_kept) o += src[p * (2 + dv) + 2 + ch] * exp2f(src[p * (2 + dv)] - m);
    out[token * out_stride + (int64_t)h * dv + ch] = from_f32<DT>(o / d);
  }
}

}  // namespace

extern "C" int ll_ragged_attention_mfma_supported(int64_t dk, int64_t dv, int dtype) {
  return (dtype == LL_F16 || dtype == LL_BF16) && dk >= 8 && dv >= 8 && dk % 8 == 0 && dv % 8 == 0 && dk <= 256 && dv <= 256;
}

extern "C" int64_t ll_ragged_attention_partition(void) { return kPart; }

// decode != 0: every sequence brings ONE token (n == batch); partials = fp32 scratch of n * heads * max_parts * (2 + dv)
// floats when max_parts = ceil((longest context) / partition) > 1, else unused.  decode == 0: longest_run = most tokens a
// sequence brings.
extern "C" int ll_ragged_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const int32_t* token_table,
                                        int64_t tt_stride, const int32_t* seq_req, const int32_t* seq_start,
                                        const int32_t* seq_first_pos, const void* sink, float scale, void* out, int64_t n,
                                        int64_t batch, int64_t longest_run, int64_t longest_context, int decode, float* partials,
                                        int64_t heads, int64_t kv_heads, int64_t dk, int64_t dv, int64_t k_stride, int64_t v_stride,
                                        int64_t window, int64_t keep_first, int64_t out_stride, int dtype, void* stream) {
  if (!ll_ragged_attention_mfma_supported(dk, dv, dtype)) return dtype == LL_F32 ? LL_ERR_DTYPE : LL_ERR_SHAPE;
  if (k_stride < kv_heads * dk || v_stride < kv_heads * dv || k_stride % 8 || v_stride % 8 || window < 0 || window > 0x7fffffff ||
      keep_first < 0 || keep_first > 0x7fffffff || out_stride < heads * dv ||
      !ll_aligned16(k_cache) || !ll_aligned16(v_cache) || !ll_aligned16(q))
    return LL_ERR_SHAPE;
  if (n < 0 || batch < 0 || heads < 1 || kv_heads < 1 || heads % kv_heads || heads > 65535 || batch > 65535 || longest_run < 1 ||
      longest_context < 1 || (decode && n != batch))
    return LL_ERR_SHAPE;
  if (n == 0 || batch == 0) return LL_OK;
  if (!q || !k_cache || !v_cache || !token_table || !seq_req || !seq_start || !seq_first_pos || !out) return LL_ERR_ARG;
  const int max_parts = decode ? (int)((longest_context + kPart - 1) / kPart) : 1;
  if (decode && max_parts > 1 && !partials) return LL_ERR_ARG;
  const int group = (int)(heads / kv_heads);
  const int shared_kv = (v_cache == k_cache && v_stride == k_stride && kv_heads == 1) ? 1 : 0;   // a latent cache: values = leading key columns
  const dim3 grid((unsigned)max_parts, (unsigned)(kv_heads * ((group + 15) / 16)), (unsigned)batch);
  hipStream_t st = (hipStream_t)stream;
  const float scale_log2 = scale * kLog2e;
#define CALL_D(DT, NS, NT)                                                                                                   \
  ragged_attention_mfma_decode_kernel<DT, NS, NT><<<grid, 64, 0, st>>>(                                                      \
      (const uint16_t*)q, (const uint16_t*)k_cache, (const uint16_t*)v_cache, token_table, tt_stride, seq_req, seq_start,    \
      seq_first_pos, (const uint16_t*)sink, scale_log2, (uint16_t*)out, partials, max_parts, (int)heads, (int)kv_heads, (int)dk, \
      (int)dv, k_stride, v_stride, (int)window, shared_kv, (int)keep_first, out_stride)
#define CALL(DT)                                         \
  if (dk <= 64 && dv <= 64) { CALL_D(DT, 2, 4); }        \
  else if (dk <= 128 && dv <= 128) { CALL_D(DT, 4, 8); } \
  else { CALL_D(DT, 8, 16); }
  if (!decode) {
    const dim3 grid4((unsigned)((longest_run + 63) / 64), (unsigned)heads, (unsigned)batch);
#define CALL_4(DT, NS, NT)                                                                                                  \
  ragged_attention_mfma_prefill4_kernel<DT, NS, NT><<<grid4, 256, 0, st>>>(                                                 \
      (const uint16_t*)q, (const uint16_t*)k_cache, (const uint16_t*)v_cache, token_table, tt_stride, seq_req, seq_start,   \
      seq_first_pos, (const uint16_t*)sink, scale_log2, (uint16_t*)out, (int)heads, (int)kv_heads, (int)dk, (int)dv, k_stride,   \
      v_stride, (int)window, shared_kv, (int)keep_first, out_stride)
#define CALL_P(DT)                                       \
  if (dk <= 64 && dv <= 64) { CALL_4(DT, 2, 4); }        \
  else if (dk <= 128 && dv <= 128) { CALL_4(DT, 4, 8); } \
  else { CALL_4(DT, 8, 16); }
    if (dtype == LL_F16) { CALL_P(LL_F16) } else { CALL_P(LL_BF16) }
#undef CALL_P
#undef CALL_4
    return LL_LAUNCH_CHECK();
  }
  if (dtype == LL_F16) { CALL(LL_F16) } else { CALL(LL_BF16) }
#undef CALL
#undef CALL_D
  if (decode && max_parts > 1) {
    const int64_t waves = n * heads;
    if (dtype == LL_F16)
      ragged_attention_merge_kernel<LL_F16><<<dim3((unsigned)((waves + 3) / 4)), 256, 0, st>>>(partials, max_parts, seq_first_pos,
                                                                                            (uint16_t*)out, n, (int)heads, (int)dv, (int)window, (int)keep_first, out_stride);
    else
      ragged_attention_merge_kernel<LL_BF16><<<dim3((unsigned)((waves + 3) / 4)), 256, 0, st>>>(partials, max_parts, seq_first_pos,
                                                                                             (uint16_t*)out, n, (int)heads, (int)dv, (int)window, (int)keep_first, out_stride);
  }
  return LL_LAUNCH_CHECK();
}
