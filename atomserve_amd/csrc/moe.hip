// Feed-forward layers made of several small experts, of which every token uses a few.
//
// Which experts a token uses is decided on the GPU (a table indexed by the token id here), so a step
// never waits for the host and can be replayed as a graph.  A (token, chosen expert) is a "pair":
// pair p = token * top + choice.  `moe_route` sorts the pairs by expert and cuts every expert's run
// into tiles of up to 64; the two grouped products then take one workgroup per (tile, 64 outputs): the first
// applies act(gate) * up on the way out, the second writes every pair's output where the pair stands
// (so the outputs of a token's experts lie side by side), and `moe_combine` adds them up with their
// weights.  A pair's result does not depend on what else is in the step: every output is a dot product
// over the whole width in a fixed order.
#include "common.h"
#include <type_traits>

#define MOE_TILE 64      // pairs of one expert that a workgroup takes (four column tiles of 16)
#define MOE_KC 128       // inputs per round: the tile's activations of a round meet in LDS
#define MOE_STRIP 64     // outputs that a workgroup takes: four waves of 16
#define MOE_MAX_EXPERTS 1024

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // 16 bytes as they are moved, whatever they hold

// ---- routing ------------------------------------------------------------------------------------
// table [vocab, top] int32: the experts of every token id.  order [P]: the pairs sorted by expert;
// tiles [max_tiles, 3]: (expert, first place in `order`, count <= 64); counts[0] = number of tiles.
// One workgroup; the order of pairs within an expert is whatever the atomics make it, which no
// result depends on.
// With token_ids null, `table` is [P]: the expert of every pair as a router's kernel left it.
__device__ __forceinline__ int expert_of_pair(const int* token_ids, const int* table, int vocab, int top, int experts,
                                              int p) {
  int e;
  if (token_ids) {
    int id = token_ids[p / top];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    e = table[(size_t)id * top + p % top];
  } else {
    e = table[p];
  }
  return e < 0 ? 0 : (e >= experts ? experts - 1 : e);
}

__global__ __launch_bounds__(1024) void moe_route_table_kernel(const int* __restrict__ token_ids,
                                                               const int* __restrict__ table, int vocab, int top,
                                                               int experts, int num_tokens, int* __restrict__ order,
                                                               int* __restrict__ tiles, int* __restrict__ counts,
                                                               int max_tiles) {
  __shared__ int hist[MOE_MAX_EXPERTS];
  __shared__ int cursor[MOE_MAX_EXPERTS];
  const int P = num_tokens * top;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) hist[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = expert_of_pair(token_ids, table, vocab, top, experts, p);
    atomicAdd(&hist[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, n = 0;
    for (int e = 0; e < experts; ++e) {
      cursor[e] = at;
      for (int s = 0; s < hist[e] && n < max_tiles; s += MOE_TILE, ++n) {
        tiles[3 * n] = e;
        tiles[3 * n + 1] = at + s;
        tiles[3 * n + 2] = min(MOE_TILE, hist[e] - s);
      }
      at += hist[e];
    }
    counts[0] = n;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = expert_of_pair(token_ids, table, vocab, top, experts, p);
    order[atomicAdd(&cursor[e], 1)] = p;
  }
}

// ---- a router that scores every expert ---------------------------------------------------------------
// z = router h (+ bias [experts] fp32) in fp32 (router [experts, K], h [T, K], both T-typed).  mode 0: s = sigmoid(z); a
// token's `top` experts are those with the largest s (of equal ones the lower number first); their weights are
// s / (sum of the chosen + 1e-20).  mode 1: the experts with the largest z, weighing the softmax over the chosen z alone.
// mode 2: s = softmax(z) over all experts; the experts form `groups` equal groups of neighbours, a group scores its
// largest s, and only experts of the `keep` best groups (of equal ones the lower number first) can be chosen; the `top`
// largest s among them weigh s * scale, not renormalised.
// pair_expert, pair_weight [T * top].  A workgroup per token: its waves take the experts four at a time, a lane 16 bytes
// of the token's row and of the four router rows at a time (the rows stream once, coalesced), the sums meet by lane swaps
// and the scores in LDS, where the first wave makes the choice.
template <typename T> struct RoutePiece;
template <> struct RoutePiece<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
};
template <> struct RoutePiece<bf16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16* p, float* v) {
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)x[i];
  }
};

template <typename T>
__global__ __launch_bounds__(256) void moe_route_scores_kernel(const T* __restrict__ h, const T* __restrict__ router,
                                                                const float* __restrict__ bias, int mode,
                                                                int groups, int keep, float scale,
                                                                int K, int experts, int top, int num_tokens,
                                                                int* __restrict__ pair_expert,
                                                                float* __restrict__ pair_weight) {
  extern __shared__ float scores[];  // [experts], then [groups] group scores and [groups] marks of the kept ones
  constexpr int N = RoutePiece<T>::N;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int t = blockIdx.x;
  const T* row = h + (size_t)t * K;
  const bool whole = K % N == 0;  // rows start on 16 bytes
  // a wave takes four experts at a time: the token's piece is loaded once for the four rows' pieces, and four
  // rows' loads are in flight together
  for (int e0 = wave * 4; e0 < experts; e0 += 16) {
    float z[4] = {0.f, 0.f, 0.f, 0.f};
    if (whole) {
      for (int k = lane * N; k < K; k += WAVE * N) {
        float hv[N], wv[4][N];
        RoutePiece<T>::load(row + k, hv);
#pragma unroll
        for (int j = 0; j < 4; ++j) RoutePiece<T>::load(router + (size_t)min(e0 + j, experts - 1) * K + k, wv[j]);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < N; ++i) z[j] = fmaf(hv[i], wv[j][i], z[j]);
      }
    } else {
      for (int k = lane; k < K; k += WAVE) {
        const float hv = to_f32(row[k]);
#pragma unroll
        for (int j = 0; j < 4; ++j) z[j] = fmaf(hv, to_f32(router[(size_t)min(e0 + j, experts - 1) * K + k]), z[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float zs = wave_sum(z[j]);
      if (lane == 0 && e0 + j < experts) {
        if (bias) zs += bias[e0 + j];
        scores[e0 + j] = mode >= 1 ? zs : 1.0f / (1.0f + expf(-zs));
      }
    }
  }
  __syncthreads();
  if (wave) return;
  float* mine = scores;
  if (mode == 2) {
    float mx = -INFINITY, sum = 0.f;
    for (int e = lane; e < experts; e += WAVE) mx = fmaxf(mx, mine[e]);
    mx = wave_max(mx);
    for (int e = lane; e < experts; e += WAVE) sum += expf(mine[e] - mx);
    sum = wave_sum(sum);
    for (int e = lane; e < experts; e += WAVE) mine[e] = expf(mine[e] - mx) / sum;
    __builtin_amdgcn_wave_barrier();
    if (groups > 1 && keep < groups) {
      float* gscore = scores + experts;
      float* gkept = gscore + groups;
      const int per = experts / groups;
      for (int g = lane; g < groups; g += WAVE) {
        float m = -INFINITY;
        for (int e = g * per; e < (g + 1) * per; ++e) m = fmaxf(m, mine[e]);
        gscore[g] = m;
        gkept[g] = 0.f;
      }
      __builtin_amdgcn_wave_barrier();
      for (int j = 0; j < keep; ++j) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int g = lane; g < groups; g += WAVE) {
          const float v = gscore[g];
          if (gkept[g] == 0.f && (v > best || at == 0x7fffffff)) { best = v; at = g; }
        }
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1) {
          const float ob = __shfl_xor(best, off, WAVE);
          const int oa = __shfl_xor(at, off, WAVE);
          if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
        }
        if (lane == 0 && at < groups) gkept[at] = 1.f;
        __builtin_amdgcn_wave_barrier();
      }
      for (int e = lane; e < experts; e += WAVE)
        if (gkept[e / per] == 0.f) mine[e] = -INFINITY;
      __builtin_amdgcn_wave_barrier();
    }
  }
  float total = 0.f, my_score = 0.f, largest = 0.f;
  int my_expert = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < experts; e += WAVE) {
      const float v = mine[e];
      if (v > best) { best = v; at = e; }
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE);
      const int oa = __shfl_xor(at, off, WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= experts) { at = 0; best = 0.f; }  // nothing left to choose (scores that are not numbers)
    if (mode == 1) {  // the first found is the largest: weights are exponentials of the distance to it
      if (j == 0) largest = best;
      best = expf(best - largest);
    }
    if (lane == j % WAVE && j / WAVE == 0) { my_score = best; my_expert = at; }
    if (j >= WAVE && lane == 0) {  // more than 64 experts a token: written as they are found, weighed below
      pair_expert[(size_t)t * top + j] = at;
      pair_weight[(size_t)t * top + j] = best;
    }
    total += best;
    if (lane == 0) mine[at] = -INFINITY;
    __builtin_amdgcn_wave_barrier();
  }
  const float inv = mode == 2 ? scale : 1.0f / (total + (mode == 1 ? 0.f : 1e-20f));
  if (lane < top && lane < WAVE) {
    pair_expert[(size_t)t * top + lane] = my_expert;
    pair_weight[(size_t)t * top + lane] = my_score * inv;
  }
  if (lane == 0)
    for (int j = WAVE; j < top; ++j) pair_weight[(size_t)t * top + j] *= inv;
}

extern "C" int as_moe_route_scores(const void* h, const void* router, const float* bias, int mode, int groups, int keep,
                                   float scale, int dtype, int K,
                                   int experts, int top, int num_tokens, int* pair_expert, float* pair_weight,
                                   hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (K <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS || top <= 0 || top > experts || mode < 0 || mode > 2) return AS_BAD_SHAPE;
  if (mode == 2 && (groups < 1 || experts % groups || keep < 1 || keep > groups || keep * (experts / groups) < top)) return AS_BAD_SHAPE;
  const int blocks = num_tokens;
  const size_t lds = (size_t)(experts + 2 * (groups > 0 ? groups : 0)) * sizeof(float);
  if (dtype == DT_F32)
    moe_route_scores_kernel<float><<<blocks, 256, lds, stream>>>((const float*)h, (const float*)router, bias, mode, groups, keep, scale, K, experts, top,
                                                                  num_tokens, pair_expert, pair_weight);
  else if (dtype == DT_BF16)
    moe_route_scores_kernel<bf16><<<blocks, 256, lds, stream>>>((const bf16*)h, (const bf16*)router, bias, mode, groups, keep, scale, K, experts, top,
                                                                 num_tokens, pair_expert, pair_weight);
  else return AS_BAD_DTYPE;
  return launch_status();
}

extern "C" int as_moe_route_table(const int* token_ids, const int* table, int vocab, int top, int experts,
                                  int num_tokens, int* order, int* tiles, int* counts, int max_tiles,
                                  hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (top <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS || (token_ids && vocab <= 0)) return AS_BAD_SHAPE;
  if (max_tiles < (num_tokens * top + MOE_TILE - 1) / MOE_TILE + experts) return AS_BAD_SHAPE;
  moe_route_table_kernel<<<1, 1024, 0, stream>>>(token_ids, table, vocab, top, experts, num_tokens, order, tiles,
                                                 counts, max_tiles);
  return launch_status();
}

// ---- the grouped products -------------------------------------------------------------------------
// a: the inputs, a row per token (pair p reads row p / a_div: a_div = top for the first product, 1 for
// the second, whose inputs are the first one's outputs, a row per pair).  w [experts, N_w, K].
// GATED: N_w = 2 N, rows 0..N-1 the gate, N..2N-1 the up projection; out[p, n] = silu(gate) * up.
// else:  out[p, n] = the product.  out has a row per pair.
//
// bf16: v_mfma_f32_16x16x32_bf16 with the weights as the A operand (16 rows of w) and 16 of the tile's
// pairs as the B operand.  A wave owns 16 outputs (and their up rows) for all of the tile's pairs (up to
// four column tiles of 16).  Per round of 128 inputs the workgroup brings the tile's activations and its 64
// (gated: 128) weight rows into LDS, whole 256-byte runs of a row per 16 lanes, rows padded by 16 bytes
// against bank conflicts; the next round's loads are in flight while this round is multiplied.  Few pairs
// (a decode step) cost few products: column tiles beyond the tile's count are skipped.  Rows of any width (16-byte loads where K % 8 == 0, single values else).
// Eight inputs of a row from column k on, one by one, zeros beyond the row's end (rows that do not start on
// 16 bytes, and a round that reaches beyond K).
__device__ __forceinline__ bf16x8 row_piece(const bf16* row, int k, int K) {
  bf16x8 v;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = k + i < K ? row[k + i] : (bf16)0.f;
  return v;
}

// silu(g) * u, or with limits (limit > 0): g = min(g, limit), u = clamp(u, -limit, limit): g sigmoid(1.702 g) (u + 1)
#define CLAMPED_GATE_ALPHA 1.702f
__device__ __forceinline__ float gate_times_up(float g, float u, float limit) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-CLAMPED_GATE_ALPHA * g)) * (u + 1.0f);
  }
  return g / (1.0f + expf(-g)) * u;
}

template <bool GATED, typename OutT, bool RELU2 = false>
__global__ __launch_bounds__(256) void moe_gemm_bf16_kernel(const bf16* __restrict__ a, int a_div,
                                                            const bf16* __restrict__ w, int N, int K,
                                                            const int* __restrict__ order,
                                                            const int* __restrict__ tiles,
                                                            const int* __restrict__ counts, OutT* __restrict__ out,
                                                            float limit) {
  constexpr int WROWS = GATED ? 2 * MOE_STRIP : MOE_STRIP;  // weight rows of a round: the strip's, then their up rows
  constexpr int WLOADS = WROWS * (MOE_KC / 8) / 256;        // 16-byte pieces of them per thread
  __shared__ __attribute__((aligned(16))) bf16 acts[MOE_TILE][MOE_KC + 8];
  __shared__ __attribute__((aligned(16))) bf16 wts[WROWS][MOE_KC + 8];
  __shared__ int pair_of[MOE_TILE];
  const int tile = blockIdx.y;
  if (tile >= counts[0]) return;
  const int e = tiles[3 * tile], at = tiles[3 * tile + 1], cnt = tiles[3 * tile + 2];
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int lr = lane & 15, lg = lane >> 4;
  const int nb = blockIdx.x * MOE_STRIP, n0 = nb + wave * 16;
  const int col_tiles = (cnt + 15) >> 4;
  if (threadIdx.x < MOE_TILE) pair_of[threadIdx.x] = threadIdx.x < cnt ? order[at + threadIdx.x] : -1;
  __syncthreads();
  const int NW = GATED ? 2 * N : N;
  const bf16* wbase = w + (size_t)e * NW * K;
  floatx4 acc[4], acc_up[4];
#pragma unroll
  for (int ct = 0; ct < 4; ++ct) { acc[ct] = floatx4{0.f, 0.f, 0.f, 0.f}; acc_up[ct] = floatx4{0.f, 0.f, 0.f, 0.f}; }
  const bool whole = (K & 7) == 0;
  // thread -> (row, 16-byte piece of the round): 16 pieces a row, so 16 lanes read 256 bytes of a row in a run.
  // Rows that stand for no pair or no output read a row that exists (their products are never stored); only a
  // round that reaches beyond K, or rows that do not start on 16 bytes, take the careful way.
  const int piece_k = (threadIdx.x & 15) * 8, piece_row = threadIdx.x >> 4;  // rows piece_row + 16 i
  const bf16* arow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = piece_row + 16 * i;
    const int pair = row < col_tiles * 16 ? pair_of[row] : -1;
    arow[i] = a + (size_t)(pair >= 0 ? pair / a_div : 0) * K;
  }
  const bf16* wrow[WLOADS];
#pragma unroll
  for (int i = 0; i < WLOADS; ++i) {
    const int row = piece_row + 16 * i;                                        // of the round's weight rows
    const int n = min(nb + (row & (MOE_STRIP - 1)), N - 1);                    // the output it belongs to
    wrow[i] = wbase + (size_t)((GATED && row >= MOE_STRIP) ? N + n : n) * K;
  }
  u32x4 staged[4], wstaged[WLOADS];
  auto fetch = [&](int k0) {
    const int k = k0 + piece_k;
    if (whole && k0 + MOE_KC <= K) {
#pragma unroll
      for (int i = 0; i < 4; ++i) staged[i] = *reinterpret_cast<const u32x4*>(arow[i] + k);
#pragma unroll
      for (int i = 0; i < WLOADS; ++i) wstaged[i] = *reinterpret_cast<const u32x4*>(wrow[i] + k);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) staged[i] = __builtin_bit_cast(u32x4, row_piece(arow[i], k, K));
#pragma unroll
      for (int i = 0; i < WLOADS; ++i) wstaged[i] = __builtin_bit_cast(u32x4, row_piece(wrow[i], k, K));
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += MOE_KC) {
    __syncthreads();  // the round before has been read
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (piece_row + 16 * i < col_tiles * 16) *reinterpret_cast<u32x4*>(&acts[piece_row + 16 * i][piece_k]) = staged[i];
#pragma unroll
    for (int i = 0; i < WLOADS; ++i) *reinterpret_cast<u32x4*>(&wts[piece_row + 16 * i][piece_k]) = wstaged[i];
    __syncthreads();
    if (k0 + MOE_KC < K) fetch(k0 + MOE_KC);  // in flight while this round is multiplied
    // the round's products in a straight line for the tile's number of column tiles (a test between the
    // products makes the compiler move the accumulators about: three times the kernel's time)
    auto multiply = [&](auto count) {
      constexpr int CT = decltype(count)::value;
#pragma unroll
      for (int s = 0; s < MOE_KC / 32; ++s) {
        const bf16x8 wv = *reinterpret_cast<const bf16x8*>(&wts[wave * 16 + lr][s * 32 + lg * 8]);
        bf16x8 uv = wv;
        if (GATED) uv = *reinterpret_cast<const bf16x8*>(&wts[MOE_STRIP + wave * 16 + lr][s * 32 + lg * 8]);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const bf16x8 av = *reinterpret_cast<const bf16x8*>(&acts[ct * 16 + lr][s * 32 + lg * 8]);
          acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, av, acc[ct], 0, 0, 0);
          if (GATED) acc_up[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uv, av, acc_up[ct], 0, 0, 0);
        }
      }
    };
    if (n0 < N) {
      if (col_tiles == 4) multiply(std::integral_constant<int, 4>{});
      else if (col_tiles == 3) multiply(std::integral_constant<int, 3>{});
      else if (col_tiles == 2) multiply(std::integral_constant<int, 2>{});
      else multiply(std::integral_constant<int, 1>{});
    }
  }
  // a lane holds outputs n0 + 4 lg + i (i < 4) of the pair in column lr of each column tile
  if (n0 >= N) return;
#pragma unroll
  for (int ct = 0; ct < 4; ++ct) {
    if (ct >= col_tiles) continue;
    const int pair = pair_of[ct * 16 + lr];
    if (pair < 0) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * lg + i;
      if (n >= N) continue;
      float v = acc[ct][i];
      if (GATED) {
        const float g = to_f32((bf16)acc[ct][i]), u = to_f32((bf16)acc_up[ct][i]);  // the two products rounded as if stored
        v = gate_times_up(g, u, limit);
      }
      if (RELU2) {
        const float u = fmaxf(to_f32((bf16)v), 0.f);  // the product rounded as if stored
        v = u * u;
      }
      out[(size_t)pair * N + n] = from_f32<OutT>(v);
    }
  }
}

// fp32: plain multiply-add, every output one chain over k in order.  A thread owns an output and, of every
// sixteen of the tile's pairs in turn, four.
template <bool GATED, bool RELU2 = false>
__global__ __launch_bounds__(256) void moe_gemm_f32_kernel(const float* __restrict__ a, int a_div,
                                                           const float* __restrict__ w, int N, int K,
                                                           const int* __restrict__ order,
                                                           const int* __restrict__ tiles,
                                                           const int* __restrict__ counts, float* __restrict__ out,
                                                           float limit) {
  const int tile = blockIdx.y;
  if (tile >= counts[0]) return;
  const int e = tiles[3 * tile], at = tiles[3 * tile + 1], cnt = tiles[3 * tile + 2];
  const int n = blockIdx.x * MOE_STRIP + (threadIdx.x & 63), quarter = threadIdx.x >> 6;
  if (n >= N) return;
  const int NW = GATED ? 2 * N : N;
  const float* wrow = w + ((size_t)e * NW + n) * K;
  const float* urow = w + ((size_t)e * NW + N + n) * K;
  for (int base = 0; base < cnt; base += 16) {
    int pairs[4];
    const float* arow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int place = base + quarter * 4 + i;
      pairs[i] = place < cnt ? order[at + place] : -1;
      arow[i] = a + (size_t)(pairs[i] < 0 ? 0 : pairs[i] / a_div) * K;
    }
    if (pairs[0] < 0) continue;
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, acc_up[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < K; ++k) {
      const float wv = wrow[k], uv = GATED ? urow[k] : 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float av = arow[i][k];
        acc[i] = fmaf(wv, av, acc[i]);
        if (GATED) acc_up[i] = fmaf(uv, av, acc_up[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (pairs[i] < 0) continue;
      float v = acc[i];
      if (GATED) v = gate_times_up(v, acc_up[i], limit);
      if (RELU2) v = fmaxf(v, 0.f) * fmaxf(v, 0.f);
      out[(size_t)pairs[i] * N + n] = v;
    }
  }
}

// out_dtype: DT_BF16 or DT_F32 for the bf16 product's results (fp32 where several experts' outputs
// are still to be added up); the fp32 product writes fp32.
// gated: 0: the product; 1: act(gate) * up (limit 0: silu(gate) * up; > 0: the gated activation with limits);
// 2: relu(product)^2 (an expert without a gate).
extern "C" int as_moe_gemm(const void* a, int dtype, int a_div, const void* w, int N, int K, int gated, const int* order,
                           const int* tiles, const int* counts, int max_tiles, void* out, int out_dtype, float limit,
                           hipStream_t stream) {
  if (max_tiles <= 0) return AS_OK;
  if (N <= 0 || K <= 0 || a_div <= 0 || max_tiles > 65535) return AS_BAD_SHAPE;
  dim3 grid((N + MOE_STRIP - 1) / MOE_STRIP, max_tiles);
  if (dtype == DT_F32) {
    if (out_dtype != DT_F32) return AS_BAD_DTYPE;
    if (gated == 2) moe_gemm_f32_kernel<false, true><<<grid, 256, 0, stream>>>((const float*)a, a_div, (const float*)w, N, K, order, tiles, counts, (float*)out, limit);
    else if (gated) moe_gemm_f32_kernel<true><<<grid, 256, 0, stream>>>((const float*)a, a_div, (const float*)w, N, K, order, tiles, counts, (float*)out, limit);
    else moe_gemm_f32_kernel<false><<<grid, 256, 0, stream>>>((const float*)a, a_div, (const float*)w, N, K, order, tiles, counts, (float*)out, limit);
    return launch_status();
  }
  if (dtype != DT_BF16) return AS_BAD_DTYPE;
  if (gated == 2) {
    if (out_dtype != DT_BF16) return AS_BAD_DTYPE;
    moe_gemm_bf16_kernel<false, bf16, true><<<grid, 256, 0, stream>>>((const bf16*)a, a_div, (const bf16*)w, N, K, order, tiles, counts, (bf16*)out, limit);
  } else if (gated) {
    if (out_dtype != DT_BF16) return AS_BAD_DTYPE;
    moe_gemm_bf16_kernel<true, bf16><<<grid, 256, 0, stream>>>((const bf16*)a, a_div, (const bf16*)w, N, K, order, tiles, counts, (bf16*)out, limit);
  } else if (out_dtype == DT_BF16) {
    moe_gemm_bf16_kernel<false, bf16><<<grid, 256, 0, stream>>>((const bf16*)a, a_div, (const bf16*)w, N, K, order, tiles, counts, (bf16*)out, limit);
  } else if (out_dtype == DT_F32) {
    moe_gemm_bf16_kernel<false, float><<<grid, 256, 0, stream>>>((const bf16*)a, a_div, (const bf16*)w, N, K, order, tiles, counts, (float*)out, limit);
  } else {
    return AS_BAD_DTYPE;
  }
  return launch_status();
}

// out[t, n] = sum over a token's `top` pairs of weight * pair_weight[t * top + j] * pair_out[t * top + j, n]
// (+ add[t, n]); fp32 in, T out.  pair_weight null: every pair weighs `weight`; add (T) null: nothing is added.
template <typename T>
__global__ void moe_combine_kernel(const float* __restrict__ pair_out, int top, float weight, int N,
                                   T* __restrict__ out, size_t total, const float* __restrict__ pair_weight,
                                   const T* __restrict__ add) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const size_t t = idx / N;
    const int n = (int)(idx % N);
    float s = 0.f;
    for (int j = 0; j < top; ++j)
      s += weight * (pair_weight ? pair_weight[t * top + j] : 1.f) * pair_out[(t * top + j) * N + n];
    if (add) s += to_f32(add[idx]);
    out[idx] = from_f32<T>(s);
  }
}

extern "C" int as_moe_combine(const float* pair_out, int top, float weight, int N, void* out, int out_dtype,
                              int num_tokens, const float* pair_weight, const void* add, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (top <= 0 || N <= 0) return AS_BAD_SHAPE;
  const size_t total = (size_t)num_tokens * N, want = (total + 255) / 256;
  const int blocks = (int)(want > 8192 ? 8192 : want);
  if (out_dtype == DT_F32) moe_combine_kernel<float><<<blocks, 256, 0, stream>>>(pair_out, top, weight, N, (float*)out, total, pair_weight, (const float*)add);
  else if (out_dtype == DT_BF16) moe_combine_kernel<bf16><<<blocks, 256, 0, stream>>>(pair_out, top, weight, N, (bf16*)out, total, pair_weight, (const bf16*)add);
  else return AS_BAD_DTYPE;
  return launch_status();
}
