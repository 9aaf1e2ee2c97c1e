// Mixture of experts with a SIGMOID router over expert groups, for 16-bit and 32-bit storage dtypes (the softmax-router fp16
// path of moe.hip stays as it is):
//
//   ll_group_router   logits = W_router h in fp32, scores = sigmoid(logits); the experts form `group_count` equal groups of
//                     neighbours, a group's score is the sum of its two best scores, only the best `group_keep` groups stay
//                     eligible; the `top` best eligible experts are chosen, their scores divided by their sum (+ 1e-20) and
//                     multiplied by `route_scale`.  One more row of weights may give a per-token sigmoid scale (for a shared
//                     expert).  Two launches: the logits as an 8 x 8 register-tiled product per wave, then one wave per token
//                     that selects by ranks (ties: the lower index first), so slot k of a token holds its k-th best expert.
//   ll_moe_sort       slots (token, k) sorted by expert, every expert's run padded to the row-block size with a sentinel:
//                     sorted_ids / block_expert / num_post as in moe_align_block_size.  Deterministic: no atomics.
//   ll_moe_rows_gemm  the grouped products over sorted row blocks: either act = silu(a Wg_e^T) * (a Wu_e^T) (gate and up rows
//                     stacked in one matrix per expert) or out = (a W_e^T) * slot weight, fp32 accumulation.  MFMA form for
//                     16-bit storage with contraction widths that are multiples of 8, a plain tiled form otherwise.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

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

__device__ __forceinline__ float sigmoid_exact(float v) { return 1.0f / (1.0f + expf(-v)); }

// the gated pair of an expert's first product.  limit < 0: silu(g) u; else the clamped form g' sigmoid(1.702 g') (u' + 1) with
// g' = min(g, limit), u' = clamp(u, -limit, limit)
template <int DT>
__device__ __forceinline__ float glu_pair(float g, float u, float limit) {
  if (limit >= 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit) + 1.0f;
    return g * (DT == LL_F32 ? sigmoid_exact(1.702f * g) : ll_sigmoidf(1.702f * g)) * u;
  }
  return g * (DT == LL_F32 ? sigmoid_exact(g) : ll_sigmoidf(g)) * u;
}

// ------------------------------------------------------------------------------------------------------------------------
// router, first launch: logits [n][experts (+ 1)] = h W^T in fp32.  A wave owns 8 tokens x 8 weight rows (x 2 rows for steps of
// a few tokens, where more and shorter waves matter more than reuse) and walks the width
// in pieces (16 bytes where rows are aligned): 16 piece loads feed 64 x VEC fused multiply-adds, so a weight row is fetched
// once per 8 tokens and a token row once per 8 experts.  A token's logit does not depend on which other tokens ride along:
// every lane sums ITS pieces in order, then the lanes are added in a fixed order.
// ------------------------------------------------------------------------------------------------------------------------
template <int DT, int VEC>
__device__ __forceinline__ void load_piece(const void* p, int64_t at, float (&o)[VEC]) {
  if constexpr (VEC == 1) {
    o[0] = ldv<DT>(p, at);
  } else if constexpr (DT == LL_F32) {
    const f32x4 v = *reinterpret_cast<const f32x4*>((const float*)p + at);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = v[i];
  } else {
    const U16x8 v = *reinterpret_cast<const U16x8*>((const uint16_t*)p + at);
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = to_f32<DT>(v.v[i]);
  }
}

template <int DT, int VEC, int EW>
__global__ __launch_bounds__(256) void router_logits_kernel(const void* __restrict__ h, int64_t h_ld, const void* __restrict__ w_router,
                                                            const void* __restrict__ w_extra, int width, int experts, int rows,
                                                            float* __restrict__ logits, int64_t n) {
  constexpr int TW = 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t0 = (int64_t)blockIdx.x * TW;
  const int e0 = (blockIdx.y * 4 + wave) * EW;
  if (e0 >= rows) return;   // (wave-uniform; no workgroup barrier below)
  int64_t hat[TW];
  const void* wp[EW];
  int64_t wat[EW];
#pragma unroll
  for (int i = 0; i < TW; ++i) hat[i] = (t0 + i < n ? t0 + i : n - 1) * h_ld;
#pragma unroll
  for (int j = 0; j < EW; ++j) {
    const int e = e0 + j < rows ? e0 + j : rows - 1;
    wp[j] = e < experts ? w_router : w_extra;
    wat[j] = e < experts ? (int64_t)e * width : 0;
  }
  float acc[TW][EW];
#pragma unroll
  for (int i = 0; i < TW; ++i)
#pragma unroll
    for (int j = 0; j < EW; ++j) acc[i][j] = 0.f;
  for (int p = lane * VEC; p < width; p += 64 * VEC) {
    float hv[TW][VEC];
#pragma unroll
    for (int i = 0; i < TW; ++i) load_piece<DT, VEC>(h, hat[i] + p, hv[i]);
#pragma unroll
    for (int j = 0; j < EW; ++j) {
      float wv[VEC];
      load_piece<DT, VEC>(wp[j], wat[j] + p, wv);
#pragma unroll
      for (int i = 0; i < TW; ++i)
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[i][j] += hv[i][k] * wv[k];
    }
  }
#pragma unroll
  for (int i = 0; i < TW; ++i)
#pragma unroll
    for (int j = 0; j < EW; ++j) {
      const float v = wave_sum(acc[i][j]);
      if (lane == 0 && t0 + i < n && e0 + j < rows) logits[(t0 + i) * rows + e0 + j] = v;
    }
}

// router, second launch: one 64-thread workgroup per token over its logits.  LDS: scores [E], group score [G], group kept
// [G], chosen scores [top].  SCORING 0: sigmoid scores, weights = chosen / sum; 1: the logits themselves rank the experts (no
// groups) and the weights are the softmax over the chosen logits alone; 2: scores = softmax over ALL logits (no groups), the
// experts are ranked by score + correction[e], the weights are the chosen scores themselves (not renormalised); the last
// `identity` experts have no weights of their own -- a slot that chose one keeps its id (>= experts - identity, which the sort
// by expert never places) and its score is added to extra_scale[t], the factor of the token's own input row
template <int SCORING, int DT = LL_F32>
__global__ __launch_bounds__(64) void group_select_kernel(const float* __restrict__ logits, int rows, int experts, int top,
                                                          int group_count, int group_keep, float route_scale,
                                                          int32_t* __restrict__ ids, float* __restrict__ weights,
                                                          float* __restrict__ extra_scale, const void* __restrict__ correction = nullptr,
                                                          int identity = 0) {
  extern __shared__ float lds[];
  float* score = lds;                       // [experts]
  float* gscore = score + experts;          // [group_count]
  float* gkeep = gscore + group_count;      // [group_count]
  float* chosen = gkeep + group_count;      // [top]
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  if constexpr (SCORING == 2) {
    // softmax over all experts: every lane adds the exponentials in index order (one value for the whole wave); the ranking
    // below sees score + correction, the weights the score alone
    float top_z = -INFINITY;
    for (int e = 0; e < experts; ++e) top_z = fmaxf(top_z, logits[t * rows + e]);
    float total = 0.f;
    for (int e = 0; e < experts; ++e) total += expf(logits[t * rows + e] - top_z);
    float* plain = chosen + top;            // [experts] scores without the correction
    for (int e = lane; e < experts; e += 64) {
      const float sc = expf(logits[t * rows + e] - top_z) / total;
      plain[e] = sc;
      score[e] = correction ? sc + ldv<DT>(correction, e) : sc;
    }
    __syncthreads();
    for (int e = lane; e < experts; e += 64) {
      const float mine = score[e];
      int rank = 0;
      for (int o = 0; o < experts; ++o) {
        const float sc = score[o];
        rank += (sc > mine || (sc == mine && o < e)) ? 1 : 0;
      }
      if (rank < top) {
        ids[t * top + rank] = e;
        chosen[rank] = plain[e];
        weights[t * top + rank] = plain[e] * route_scale;
      }
    }
    __syncthreads();
    if (extra_scale && lane == 0) {         // slots in rank order: the same sum whatever lane found which slot
      float own = 0.f;
      for (int k = 0; k < top; ++k)
        if (ids[t * top + k] >= experts - identity) own += chosen[k];
      extra_scale[t] = own * route_scale;
    }
    return;
  }
  for (int e = lane; e < rows; e += 64) {
    const float z = logits[t * rows + e];
    if (e < experts) score[e] = SCORING == 1 ? z : sigmoid_exact(z);
    else extra_scale[t] = sigmoid_exact(z);
  }
  __syncthreads();
  const int per = experts / group_count;
  for (int g = lane; g < group_count; g += 64) {
    float b1 = -INFINITY, b2 = -INFINITY;   // the two largest of the group
    for (int j = 0; j < per; ++j) {
      const float s = score[g * per + j];
      if (s > b1) { b2 = b1; b1 = s; }
      else if (s > b2) b2 = s;
    }
    gscore[g] = per > 1 ? b1 + b2 : b1;
  }
  __syncthreads();
  for (int g = lane; g < group_count; g += 64) {
    const float mine = gscore[g];
    int rank = 0;
    for (int o = 0; o < group_count; ++o) {
      const float s = gscore[o];
      rank += (s > mine || (s == mine && o < g)) ? 1 : 0;
    }
    gkeep[g] = rank < group_keep ? 1.0f : 0.0f;
  }
  __syncthreads();
  for (int e = lane; e < experts; e += 64) {
    if (gkeep[e / per] == 0.0f) continue;
    const float mine = score[e];
    int rank = 0;
    for (int o = 0; o < experts; ++o) {
      const float s = score[o];
      rank += (gkeep[o / per] != 0.0f && (s > mine || (s == mine && o < e))) ? 1 : 0;
    }
    if (rank < top) {
      ids[t * top + rank] = e;
      chosen[rank] = mine;
    }
  }
  __syncthreads();
  float sum = 0.f;
  if constexpr (SCORING == 1) {   // chosen[0] is the largest: exp(z - z_max) summed in slot order by every lane
    for (int k = 0; k < top; ++k) sum += expf(chosen[k] - chosen[0]);
    for (int k = lane; k < top; k += 64) weights[t * top + k] = expf(chosen[k] - chosen[0]) / sum * route_scale;
  } else {
    for (int k = 0; k < top; ++k) sum += chosen[k];
    for (int k = lane; k < top; k += 64) weights[t * top + k] = chosen[k] / (sum + 1e-20f) * route_scale;
  }
}

// ------------------------------------------------------------------------------------------------------------------------
// sort by expert: one workgroup per expert, twice (count, then place)
// ------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_count_kernel(const int32_t* __restrict__ ids, int num_slots, int32_t* __restrict__ counts) {
  __shared__ int part[4];
  const int e = blockIdx.x, tid = threadIdx.x;
  int c = 0;
  for (int i = tid; i < num_slots; i += 256) c += ids[i] == e ? 1 : 0;
  for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
  if ((tid & 63) == 0) part[tid >> 6] = c;
  __syncthreads();
  if (tid == 0) counts[e] = part[0] + part[1] + part[2] + part[3];
}

__global__ __launch_bounds__(256) void moe_place_kernel(const int32_t* __restrict__ ids, int num_slots, int experts, int block_m,
                                                        const int32_t* __restrict__ counts, int32_t* __restrict__ sorted,
                                                        int32_t* __restrict__ block_expert, int32_t* __restrict__ num_post) {
  __shared__ int wtot[4];
  const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int base = 0;
  for (int o = 0; o < e; ++o) base += (counts[o] + block_m - 1) / block_m * block_m;
  const int mine = counts[e];
  const int padded = (mine + block_m - 1) / block_m * block_m;
  int running = 0;
  for (int at = 0; at < num_slots; at += 256) {
    const int i = at + tid;
    const bool hit = i < num_slots && ids[i] == e;
    const unsigned long long mask = __ballot(hit);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    __syncthreads();   // (the previous round's totals have been read)
    if (lane == 0) wtot[wave] = __popcll(mask);
    __syncthreads();
    int off = running;
    for (int w = 0; w < wave; ++w) off += wtot[w];
    if (hit) sorted[base + off + before] = i;
    running += wtot[0] + wtot[1] + wtot[2] + wtot[3];
  }
  for (int i = mine + tid; i < padded; i += 256) sorted[base + i] = num_slots;
  for (int b = tid; b < padded / block_m; b += 256) block_expert[base / block_m + b] = e;
  if (e == experts - 1 && tid == 0) num_post[0] = base + padded;
}

// ------------------------------------------------------------------------------------------------------------------------
// grouped products, plain tiled form: 32 sorted rows x 64 columns per workgroup, 32 contraction entries per pass
// ------------------------------------------------------------------------------------------------------------------------
template <int DT, bool GLU>
__global__ __launch_bounds__(256) void moe_rows_gemm_kernel(const void* __restrict__ a, int64_t a_ld, int a_div,
                                                            const void* __restrict__ w, int64_t w_stride_e, int K, int N,
                                                            const float* __restrict__ slot_weight, void* __restrict__ out,
                                                            int64_t out_ld, const int32_t* __restrict__ sorted,
                                                            const int32_t* __restrict__ block_expert,
                                                            const int32_t* __restrict__ num_post, int num_slots, float glu_limit) {
  constexpr int BM = 32, BN = 64, BK = 32;
  __shared__ float As[BM][BK + 1];
  __shared__ int rows[BM];
  const int block = blockIdx.x;
  if (block * BM >= num_post[0]) return;
  const int e = block_expert[block];
  const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
  if (tid < BM) rows[tid] = sorted[block * BM + tid];
  const int col = blockIdx.y * BN + tx;
  const bool colok = col < N;
  const int64_t wg_at = (int64_t)e * w_stride_e + (int64_t)col * K;
  const int64_t wu_at = (int64_t)e * w_stride_e + (int64_t)(N + col) * K;
  float acc_g[8], acc_u[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) acc_g[r] = acc_u[r] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < BM * BK / 256; ++u) {
      const int idx = tid + 256 * u, r = idx / BK, kk = idx - r * BK;
      const int slot = rows[r];
      As[r][kk] = (slot < num_slots && k0 + kk < K) ? ldv<DT>(a, (int64_t)(slot / a_div) * a_ld + k0 + kk) : 0.f;
    }
    __syncthreads();
    if (colok) {
      const int kn = K - k0 < BK ? K - k0 : BK;
      for (int kk = 0; kk < kn; ++kk) {
        const float wg = ldv<DT>(w, wg_at + k0 + kk);
        const float wu = GLU ? ldv<DT>(w, wu_at + k0 + kk) : 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const float av = As[ty * 8 + r][kk];
          acc_g[r] += av * wg;
          if (GLU) acc_u[r] += av * wu;
        }
      }
    }
  }
  if (!colok) return;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int slot = rows[ty * 8 + r];
    if (slot >= num_slots) continue;
    float v;
    if (GLU) {
      v = glu_pair<DT>(acc_g[r], acc_u[r], glu_limit);
    } else {
      v = slot_weight ? acc_g[r] * slot_weight[slot] : acc_g[r];
    }
    stv<DT>(out, (int64_t)slot * out_ld + col, v);
  }
}

// ------------------------------------------------------------------------------------------------------------------------
// grouped products, MFMA form (16-bit storage, K a multiple of 8, 16-byte aligned rows): one wave per 32 sorted rows x 32
// columns (gate and up: 32 + 32).  Both operands are contraction-contiguous, so a lane's fragment is ONE 16-byte load: lane
// (t, c) holds entries 8 c .. 8 c + 7 (+ 32 per pass) of row / column t.  Rows = columns of the MFMA (B operand), weight rows
// = MFMA rows (A operand): the accumulator of lane (t, c) holds weight rows 4 c .. 4 c + 3 of sorted row t.
// ------------------------------------------------------------------------------------------------------------------------
struct alignas(16) Q4 {
  uint32_t x, y, z, w;
};
template <int DT>
__device__ __forceinline__ f32x4 mfma16(const Q4& a, const Q4& b, f32x4 c) {
  if constexpr (DT == LL_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

template <int DT, bool GLU>
__global__ __launch_bounds__(64) void moe_rows_gemm_mfma_kernel(const uint16_t* __restrict__ a, int64_t a_ld, int a_div,
                                                                const uint16_t* __restrict__ w, int64_t w_stride_e, int K, int N,
                                                                const float* __restrict__ slot_weight, uint16_t* __restrict__ out,
                                                                int64_t out_ld, const int32_t* __restrict__ sorted,
                                                                const int32_t* __restrict__ block_expert,
                                                                const int32_t* __restrict__ num_post, int num_slots, float glu_limit) {
  constexpr int BM = 32, BN = 32;
  constexpr int NW = GLU ? 4 : 2;   // weight-row tiles of 16: gate 0..1, up 2..3
  const int block = blockIdx.x;
  if (block * BM >= num_post[0]) return;
  const int e = block_expert[block];
  const int lane = threadIdx.x, t = lane & 15, c = lane >> 4;
  const int n0 = blockIdx.y * BN;
  int slot[2];
  const uint16_t* arow[2];
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    slot[m] = sorted[block * BM + 16 * m + t];
    arow[m] = slot[m] < num_slots ? a + (int64_t)(slot[m] / a_div) * a_ld : nullptr;
  }
  const uint16_t* wrow[NW];
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    const int col = n0 + 16 * (j & 1) + t;
    const int64_t r = (GLU && j >= 2) ? (int64_t)N + col : col;
    wrow[j] = col < N ? w + (int64_t)e * w_stride_e + r * K : nullptr;
  }
  f32x4 acc[NW][2];
#pragma unroll
  for (int j = 0; j < NW; ++j) acc[j][0] = acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the fragments of the next two contraction steps are requested before the products of the current one: with a handful of
  // rows per expert (decoding) the launch streams every weight row once, and only loads in flight hide that latency
  constexpr int AHEAD = 2;
  Q4 af[AHEAD + 1][2], wf[AHEAD + 1][NW];
  auto fetch = [&](int k0, Q4 (&fa)[2], Q4 (&fw)[NW]) {
    const int ch = k0 + 8 * c;
    const bool in = ch < K;
#pragma unroll
    for (int m = 0; m < 2; ++m) fa[m] = (in && arow[m]) ? *reinterpret_cast<const Q4*>(arow[m] + ch) : Q4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < NW; ++j) fw[j] = (in && wrow[j]) ? *reinterpret_cast<const Q4*>(wrow[j] + ch) : Q4{0, 0, 0, 0};
  };
#pragma unroll
  for (int a2 = 0; a2 < AHEAD; ++a2) fetch(32 * a2, af[a2], wf[a2]);
  for (int k0 = 0; k0 < K; k0 += 32 * (AHEAD + 1)) {
#pragma unroll
    for (int u = 0; u <= AHEAD; ++u) {   // (slot u holds step k0 + 32 u; the slot just freed receives step + AHEAD)
      fetch(k0 + 32 * (u + AHEAD), af[(u + AHEAD) % (AHEAD + 1)], wf[(u + AHEAD) % (AHEAD + 1)]);
#pragma unroll
      for (int j = 0; j < NW; ++j) {
        acc[j][0] = mfma16<DT>(wf[u][j], af[u][0], acc[j][0]);
        acc[j][1] = mfma16<DT>(wf[u][j], af[u][1], acc[j][1]);
      }
    }
  }
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    if (slot[m] >= num_slots) continue;
    const float sw = (!GLU && slot_weight) ? slot_weight[slot[m]] : 1.0f;
    uint16_t* orow = out + (int64_t)slot[m] * out_ld;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = n0 + 16 * j + 4 * c + r;
        if (col >= N) continue;
        float v;
        if (GLU) {
          const float g = acc[j][m][r];
          v = glu_pair<DT>(g, acc[j + 2][m][r], glu_limit);
        } else {
          v = acc[j][m][r] * sw;
        }
        orow[col] = from_f32<DT>(v);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------------
// grouped products, LDS-tiled MFMA form for prompt-sized inputs: a workgroup of four waves owns 128 sorted rows x 128 weight
// rows (gate|up: 64 output columns, gate rows and up rows of the same columns side by side) and walks the contraction in steps
// of 64.  Both tiles are fetched ONCE per workgroup (global -> registers -> LDS, the next step's loads in flight under the
// products); a wave multiplies all eight row tiles with two weight tiles (its gate and its up tile), so every A fragment read
// from LDS feeds two MFMAs and every weight fragment eight.
// ------------------------------------------------------------------------------------------------------------------------
template <int DT, bool GLU>
__global__ __launch_bounds__(256) void moe_rows_gemm_tiled_kernel(const uint16_t* __restrict__ a, int64_t a_ld, int a_div,
                                                                  const uint16_t* __restrict__ w, int64_t w_stride_e, int K, int N,
                                                                  const float* __restrict__ slot_weight, uint16_t* __restrict__ out,
                                                                  int64_t out_ld, const int32_t* __restrict__ sorted,
                                                                  const int32_t* __restrict__ block_expert,
                                                                  const int32_t* __restrict__ num_post, int num_slots, float glu_limit) {
  constexpr int BM = 128, WN = 128, BK = 64, STR = BK + 8, CW = GLU ? 64 : 128;
  __shared__ __attribute__((aligned(16))) uint16_t lds_a[BM * STR];
  __shared__ __attribute__((aligned(16))) uint16_t lds_w[WN * STR];
  __shared__ int rows_s[BM];
  const int block = blockIdx.x;
  if (block * BM >= num_post[0]) return;
  const int e = block_expert[block];
  const int n0 = blockIdx.y * CW;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, t = lane & 15, c = lane >> 4;
  if (tid < BM) rows_s[tid] = sorted[block * BM + tid];
  __syncthreads();
  const uint16_t* aptr[4];
  const uint16_t* wptr[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int i = tid + 256 * u, row = i >> 3, pc = i & 7;
    const int slot = rows_s[row];
    aptr[u] = slot < num_slots ? a + (int64_t)(slot / a_div) * a_ld + 8 * pc : nullptr;
    const int col = GLU ? n0 + (row & 63) : n0 + row;
    const int64_t grow = (GLU && row >= 64) ? (int64_t)N + col : col;
    wptr[u] = col < N ? w + (int64_t)e * w_stride_e + grow * K + 8 * pc : nullptr;
  }
  Q4 ra[4], rw[4];
#define LL_FETCH(K0)                                                                                        \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) {                                                           \
    const bool in = (K0) + 8 * ((tid + 256 * u) & 7) < K;                                                   \
    ra[u] = (in && aptr[u]) ? *reinterpret_cast<const Q4*>(aptr[u] + (K0)) : Q4{0, 0, 0, 0};                \
    rw[u] = (in && wptr[u]) ? *reinterpret_cast<const Q4*>(wptr[u] + (K0)) : Q4{0, 0, 0, 0};                \
  }
#define LL_STAGE()                                                                                          \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) {                                                           \
    const int i = tid + 256 * u, row = i >> 3, pc = i & 7;                                                  \
    *reinterpret_cast<Q4*>(&lds_a[row * STR + 8 * pc]) = ra[u];                                             \
    *reinterpret_cast<Q4*>(&lds_w[row * STR + 8 * pc]) = rw[u];                                             \
  }
  const int tile0 = GLU ? wave : 2 * wave, tile1 = GLU ? 4 + wave : 2 * wave + 1;
  f32x4 acc[2][8];
#pragma unroll
  for (int m = 0; m < 8; ++m) acc[0][m] = acc[1][m] = f32x4{0.f, 0.f, 0.f, 0.f};
  LL_FETCH(0)
  LL_STAGE()
  __syncthreads();
  for (int k0 = 0; k0 < K; k0 += BK) {
    if (k0 + BK < K) { LL_FETCH(k0 + BK) }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const Q4 w0 = *reinterpret_cast<const Q4*>(&lds_w[(16 * tile0 + t) * STR + 32 * ks + 8 * c]);
      const Q4 w1 = *reinterpret_cast<const Q4*>(&lds_w[(16 * tile1 + t) * STR + 32 * ks + 8 * c]);
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        const Q4 af = *reinterpret_cast<const Q4*>(&lds_a[(16 * m + t) * STR + 32 * ks + 8 * c]);
        acc[0][m] = mfma16<DT>(w0, af, acc[0][m]);
        acc[1][m] = mfma16<DT>(w1, af, acc[1][m]);
      }
    }
    __syncthreads();   // everybody has read this step's tiles
    if (k0 + BK < K) { LL_STAGE() }
    __syncthreads();
  }
#undef LL_FETCH
#undef LL_STAGE
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const int slot = rows_s[16 * m + t];
    if (slot >= num_slots) continue;
    uint16_t* orow = out + (int64_t)slot * out_ld;
    if (GLU) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = n0 + 16 * wave + 4 * c + r;
        const float g = acc[0][m][r];
        if (col < N) orow[col] = from_f32<DT>(glu_pair<DT>(g, acc[1][m][r], glu_limit));
      }
    } else {
      const float sw = slot_weight ? slot_weight[slot] : 1.0f;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int col = n0 + 16 * (2 * wave + j) + 4 * c + r;
          if (col < N) orow[col] = from_f32<DT>(acc[j][m][r] * sw);
        }
    }
  }
}

}  // namespace

#define LL_BY_DTYPE(dtype, CALL)             \
  do {                                       \
    if (dtype == LL_F16) { CALL(LL_F16); }   \
    else if (dtype == LL_BF16) { CALL(LL_BF16); } \
    else { CALL(LL_F32); }                   \
  } while (0)

// logits: fp32 scratch [n][experts + (w_extra ? 1 : 0)]
extern "C" int ll_group_router(const void* h, int64_t h_ld, const void* w_router, const void* w_extra, int64_t n, int64_t width,
                               int64_t experts, int64_t top, int64_t group_count, int64_t group_keep, float route_scale, int scoring,
                               int32_t* ids, float* weights, float* extra_scale, float* logits, const void* correction, int64_t identity,
                               int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (scoring == 2 && (group_count != 1 || w_extra || identity < 0 || identity > experts || (identity > 0 && !extra_scale)))
    return LL_ERR_SHAPE;
  if (scoring != 2 && (correction || identity)) return LL_ERR_SHAPE;
  if (n < 0 || width < 1 || h_ld < width || experts < 1 || experts > 4096 || top < 1 || top > experts || top > 64 || group_count < 1 ||
      experts % group_count || group_keep < 1 || group_keep > group_count || group_keep * (experts / group_count) < top ||
      scoring < 0 || scoring > 2 || (scoring == 1 && group_count != 1))
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!h || !w_router || !ids || !weights || !logits || (w_extra && !extra_scale)) return LL_ERR_ARG;
  const int rows = (int)experts + (w_extra ? 1 : 0);
  const int vec = dtype == LL_F32 ? 4 : 8;
  const bool aligned = width % vec == 0 && h_ld % vec == 0 && ll_aligned16(h) && ll_aligned16(w_router) && (!w_extra || ll_aligned16(w_extra));
  const int ew = n >= 512 ? 8 : 2;   // weight rows per wave
  const dim3 grid((unsigned)((n + 7) / 8), (unsigned)((rows + 4 * ew - 1) / (4 * ew)));
  hipStream_t st = (hipStream_t)stream;
#define LL_RL_ARGS h, h_ld, w_router, w_extra, (int)width, (int)experts, rows, logits, n
#define LL_RL(DT, V)                                                                         \
  if (ew == 8) router_logits_kernel<DT, V, 8><<<grid, 256, 0, st>>>(LL_RL_ARGS);             \
  else router_logits_kernel<DT, V, 2><<<grid, 256, 0, st>>>(LL_RL_ARGS)
  if (!aligned) {
#define CALL(DT) LL_RL(DT, 1)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
  } else if (dtype == LL_F32) {
    LL_RL(LL_F32, 4);
  } else if (dtype == LL_F16) {
    LL_RL(LL_F16, 8);
  } else {
    LL_RL(LL_BF16, 8);
  }
#undef LL_RL
#undef LL_RL_ARGS
  const size_t lds = sizeof(float) * (size_t)(experts + 2 * group_count + top + (scoring == 2 ? experts : 0));
  if (scoring == 2) {
#define CALL(DT)                                                                                                                    \
  group_select_kernel<2, DT><<<dim3((unsigned)n), 64, lds, st>>>(logits, rows, (int)experts, (int)top, 1, 1, route_scale, ids, weights, \
                                                                 extra_scale, correction, (int)identity)
    LL_BY_DTYPE(dtype, CALL);
#undef CALL
  } else if (scoring == 1)
    group_select_kernel<1><<<dim3((unsigned)n), 64, lds, st>>>(logits, rows, (int)experts, (int)top, (int)group_count, (int)group_keep,
                                                               route_scale, ids, weights, extra_scale);
  else
    group_select_kernel<0><<<dim3((unsigned)n), 64, lds, st>>>(logits, rows, (int)experts, (int)top, (int)group_count, (int)group_keep,
                                                               route_scale, ids, weights, extra_scale);
  return LL_LAUNCH_CHECK();
}

// rows per sorted block: 128 (the LDS-tiled form) when the experts average at least 128 slots each and the 16-bit matrix-core
// forms apply, else 32
extern "C" int64_t ll_moe_rows_block(int64_t num_slots, int64_t experts, int64_t width, int64_t ff, int dtype) {
  static const bool small = getenv("LL_MOE_ROWS_SMALL") != nullptr;   // A/B knob, read once
  return (!small && dtype != LL_F32 && width % 8 == 0 && ff % 8 == 0 && num_slots >= 128 * experts) ? 128 : 32;
}

// counts: int32 scratch [experts].  sorted [num_slots + experts * (block - 1)], block_expert [ceil(that / block)], num_post [1]
extern "C" int ll_moe_sort(const int32_t* ids, int64_t num_slots, int64_t experts, int64_t block, int32_t* counts, int32_t* sorted,
                           int32_t* block_expert, int32_t* num_post, void* stream) {
  if (num_slots < 0 || experts < 1 || experts > 65535 || (block != 32 && block != 128) || num_slots + experts * block >= (1ll << 31))
    return LL_ERR_SHAPE;
  if (!ids || !counts || !sorted || !block_expert || !num_post) return LL_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  moe_count_kernel<<<dim3((unsigned)experts), 256, 0, st>>>(ids, (int)num_slots, counts);
  moe_place_kernel<<<dim3((unsigned)experts), 256, 0, st>>>(ids, (int)num_slots, (int)experts, (int)block, counts, sorted,
                                                            block_expert, num_post);
  return LL_LAUNCH_CHECK();
}

// glu != 0: w [experts][2 N][K] (gate rows, then up rows), out[slot][N] = silu(a_row Wg^T) * (a_row Wu^T) with a_row =
// a[slot / a_div] (glu == 2: the clamped pair g' sigmoid(1.702 g') (u' + 1), g' = min(g, limit), u' = clamp(u, +-limit)); glu == 0: w [experts][N][K], out[slot][N] = (a[slot / a_div] W^T) * slot_weight[slot] (NULL: 1).
extern "C" int ll_moe_rows_gemm(const void* a, int64_t a_ld, int64_t a_div, const void* w, int64_t w_stride_e, int64_t K, int64_t N,
                                int glu, const float* slot_weight, void* out, int64_t out_ld, const int32_t* sorted,
                                const int32_t* block_expert, const int32_t* num_post, int64_t num_slots, int64_t experts,
                                int64_t block, float limit, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (glu < 0 || glu > 2 || (glu == 2 && !(limit >= 0.f))) return LL_ERR_SHAPE;
  const float glu_limit = glu == 2 ? limit : -1.0f;
  if (num_slots < 0 || K < 1 || N < 1 || a_div < 1 || a_ld < K || out_ld < N || w_stride_e < (glu ? 2 : 1) * N * K || experts < 1 ||
      (block != 32 && block != 128))
    return LL_ERR_SHAPE;
  if (num_slots == 0) return LL_OK;
  if (!a || !w || !out || !sorted || !block_expert || !num_post) return LL_ERR_ARG;
  const int64_t max_blocks = (num_slots + experts * (block - 1) + block - 1) / block;
  hipStream_t st = (hipStream_t)stream;
  static const bool no_mfma = getenv("LL_MOE_ROWS_VALU") != nullptr;   // A/B knob, read once
  const bool mfma = !no_mfma && dtype != LL_F32 && K % 8 == 0 && a_ld % 8 == 0 && w_stride_e % 8 == 0 && ll_aligned16(a) && ll_aligned16(w);
  if (block == 128) {
    if (!mfma) return LL_ERR_SHAPE;   // (blocks of 128 rows are only sorted for the tiled matrix-core form)
    const dim3 grid((unsigned)max_blocks, (unsigned)((N + (glu ? 63 : 127)) / (glu ? 64 : 128)));
#define CALL_T(DT, G)                                                                                                          \
  moe_rows_gemm_tiled_kernel<DT, G><<<grid, 256, 0, st>>>((const uint16_t*)a, a_ld, (int)a_div, (const uint16_t*)w, w_stride_e, \
                                                          (int)K, (int)N, slot_weight, (uint16_t*)out, out_ld, sorted, block_expert, \
                                                          num_post, (int)num_slots, glu_limit)
    if (dtype == LL_F16) { if (glu) CALL_T(LL_F16, true); else CALL_T(LL_F16, false); }
    else { if (glu) CALL_T(LL_BF16, true); else CALL_T(LL_BF16, false); }
#undef CALL_T
    return LL_LAUNCH_CHECK();
  }
  if (mfma) {
    const dim3 grid((unsigned)max_blocks, (unsigned)((N + 31) / 32));
#define CALL_M(DT, G)                                                                                                         \
  moe_rows_gemm_mfma_kernel<DT, G><<<grid, 64, 0, st>>>((const uint16_t*)a, a_ld, (int)a_div, (const uint16_t*)w, w_stride_e, \
                                                        (int)K, (int)N, slot_weight, (uint16_t*)out, out_ld, sorted, block_expert, \
                                                        num_post, (int)num_slots, glu_limit)
    if (dtype == LL_F16) { if (glu) CALL_M(LL_F16, true); else CALL_M(LL_F16, false); }
    else { if (glu) CALL_M(LL_BF16, true); else CALL_M(LL_BF16, false); }
#undef CALL_M
    return LL_LAUNCH_CHECK();
  }
  const dim3 grid((unsigned)max_blocks, (unsigned)((N + 63) / 64));
#define CALL(DT)                                                                                                             \
  if (glu) moe_rows_gemm_kernel<DT, true><<<grid, 256, 0, st>>>(a, a_ld, (int)a_div, w, w_stride_e, (int)K, (int)N, slot_weight, \
                                                                out, out_ld, sorted, block_expert, num_post, (int)num_slots, glu_limit);    \
  else moe_rows_gemm_kernel<DT, false><<<grid, 256, 0, st>>>(a, a_ld, (int)a_div, w, w_stride_e, (int)K, (int)N, slot_weight,   \
                                                             out, out_ld, sorted, block_expert, num_post, (int)num_slots, glu_limit)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}
