// Attention through a latent: keys and values of all heads are matrices times one cached vector c [kv_rank] per
// token, beside one rotated key part k_r [rot_dim] that all heads share.  With k_h = U_h c and v_h = V_h c,
//
//   q_h . k_h = (U_h^T q_h) . c          and          sum_j p_j v_h(j) = V_h (sum_j p_j c_j),
//
// so the attention itself runs over one kv head whose keys are [c | k_r] and whose values are c, with queries
// [U_h^T q_h | rotated part of q_h]: the paged attention kernels of this package as they are.  Here are the steps
// around them:
//
//   rows_rms_norm     a plain RMS norm of columns of a product's result (the latent of the queries)
//   latent_kv_store   norm of c, rotation of k_r, [c | k_r] into the key pages and c into the value pages
//   latent_q_absorb   q [T, H, D + R] -> [U_h^T q_h | rotate(q_h[D:])], zeros up to the pages' width
//   latent_v_expand   heads [T, H, width] (their first kv_rank coordinates) -> V_h heads, times sigmoid(gate)
//   wide_attend       the attention itself for latents wider than the paged attention kernels' heads
//
// Norms, the rotation and every sum are fp32, taken in an order that does not depend on what else is in the step.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void rows_rms_norm_kernel(const T* __restrict__ proj, int ld, int off, int n,
                                                            const float* __restrict__ gain, float eps,
                                                            T* __restrict__ out) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * ld + off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) { const float v = to_f32(row[i]); ss = fmaf(v, v, ss); }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) out[(size_t)t * n + i] = from_f32<T>(to_f32(row[i]) * inv * gain[i]);
}

extern "C" int as_rows_rms_norm(const void* proj, int dtype, int ld, int off, int n, const float* gain, float eps,
                                void* out, int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (n <= 0 || off < 0 || off + n > ld) return AS_BAD_SHAPE;
  if (dtype == DT_F32) rows_rms_norm_kernel<float><<<num_tokens, 256, 0, stream>>>((const float*)proj, ld, off, n, gain, eps, (float*)out);
  else if (dtype == DT_BF16) rows_rms_norm_kernel<bf16><<<num_tokens, 256, 0, stream>>>((const bf16*)proj, ld, off, n, gain, eps, (bf16*)out);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// proj[t, off .. off + rank) is the latent before its norm, the next `rot` columns the shared key part before its
// rotation; cos_sin [T, rot/2, 2] fp32.  k_pages [pages, 1, bs, width], v_pages [pages, 1, width, bs]; slots[t] < 0:
// nothing is stored.  What is not finite is stored as zero; the pages' columns beyond what is stored get zeros.
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_store_kernel(const T* __restrict__ proj, int ld, int off, int rank,
                                                              int rot, const float* __restrict__ gain, float eps,
                                                              const float* __restrict__ cos_sin,
                                                              const int* __restrict__ slots, T* __restrict__ k_pages,
                                                              T* __restrict__ v_pages, int bs, int width) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  const int slot = slots[t];
  if (slot < 0) return;
  const T* row = proj + (size_t)t * ld + off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) { const float v = to_f32(row[i]); ss = fmaf(v, v, ss); }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  const int page = slot / bs, in_page = slot % bs;
  T* kd = k_pages + ((size_t)page * bs + in_page) * width;
  T* vd = v_pages + (size_t)page * width * bs + in_page;
  const int half = rot / 2;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float key = 0.f, value = 0.f;
    if (i < rank) {
      key = value = to_f32(row[i]) * inv * gain[i];
    } else if (i < rank + rot) {
      const int j = i - rank, p = j < half ? j : j - half;
      const float c = cos_sin[((size_t)t * half + p) * 2], s = cos_sin[((size_t)t * half + p) * 2 + 1];
      const float u = to_f32(row[rank + p]), v = to_f32(row[rank + half + p]);
      key = j < half ? u * c - v * s : v * c + u * s;
    }
    kd[i] = finite_or_zero(from_f32<T>(key));
    vd[(size_t)i * bs] = finite_or_zero(from_f32<T>(value));
  }
}

extern "C" int as_latent_kv_store(const void* proj, int dtype, int ld, int off, int rank, int rot, const float* gain,
                                  float eps, const float* cos_sin, const int* slots, void* k_pages, void* v_pages,
                                  int bs, int width, int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (rank <= 0 || rot < 0 || rot % 2 || rank + rot > width || off < 0 || off + rank + rot > ld || bs <= 0) return AS_BAD_SHAPE;
  if (rot > 0 && !cos_sin) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    latent_kv_store_kernel<float><<<num_tokens, 256, 0, stream>>>((const float*)proj, ld, off, rank, rot, gain, eps, cos_sin, slots,
                                                                 (float*)k_pages, (float*)v_pages, bs, width);
  else if (dtype == DT_BF16)
    latent_kv_store_kernel<bf16><<<num_tokens, 256, 0, stream>>>((const bf16*)proj, ld, off, rank, rot, gain, eps, cos_sin, slots,
                                                                (bf16*)k_pages, (bf16*)v_pages, bs, width);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- products with a matrix per head --------------------------------------------------------------------------
// out[t, h, n] = sum_k x[t, h, k] W_h[k, n] for two uses: the queries' plain part through U_h (k a coordinate of the
// head, n one of the latent) and the attention's result through V_h (k a coordinate of the latent, n one of the
// value).  Few tokens: `head_product_kernel`, any dtype, W_h stored [k][n]; a workgroup owns 64 outputs of a head for
// up to 8 tokens, its four waves a quarter of k each, and the four partial sums are added in the waves' order.
// Prompts in bfloat16: `head_product_mfma_kernel`, W_h stored [n][k], on the matrix cores (weights as the first
// operand, 16 tokens as the second: a lane then holds four consecutive outputs of one token).
#define ABSORB_TOKENS 8
#define HEAD_STRIP 64  // outputs a workgroup owns

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// What follows the product.  TAIL (the queries): out[t, h, N .. N + R) = the R coordinates after the K plain ones
// of x[t, h], turned by cos_sin [T, R/2, 2], then zeros up to `os`.  GATE (the values): the product rounded as it
// would be stored, times sigmoid(gate[t, g_off + h N + n]) (gate null: none).
struct HeadEpilogue {
  int R;
  const float* cos_sin;
  const void* gate;
  int ld, g_off;
};

template <typename T, bool GATE>
__device__ __forceinline__ void head_store(float v, size_t t, int h, int n, int N, int H, T* __restrict__ out, int os,
                                           const HeadEpilogue& ep) {
  if (GATE) {
    if (ep.gate) {
      v = to_f32(from_f32<T>(v));
      v *= 1.0f / (1.0f + expf(-to_f32(((const T*)ep.gate)[t * ep.ld + ep.g_off + h * N + n])));
    }
  }
  out[(t * H + h) * os + n] = from_f32<T>(v);
}

template <typename T>
__device__ __forceinline__ void head_tail(const T* __restrict__ x, int xs, int K, int N, int H, int h, int t0, int nt,
                                          T* __restrict__ out, int os, const HeadEpilogue& ep) {
  const int half = ep.R / 2, tail = os - N;
  for (int i = threadIdx.x; i < nt * tail; i += blockDim.x) {
    const int tq = i / tail, j = i % tail;
    const size_t t = t0 + tq;
    float v = 0.f;
    if (j < ep.R) {
      const int p = j < half ? j : j - half;
      const T* xr = x + (t * H + h) * xs + K;
      const float c = ep.cos_sin[(t * half + p) * 2], s = ep.cos_sin[(t * half + p) * 2 + 1];
      const float a = to_f32(xr[p]), b = to_f32(xr[half + p]);
      v = j < half ? a * c - b * s : b * c + a * s;
    }
    out[(t * H + h) * os + N + j] = from_f32<T>(v);
  }
}

// x [T, H, xs] (the first K of a row count), w [H, K, N], out [T, H, os].  grid (token tiles of ABSORB_TOKENS, heads,
// strips of HEAD_STRIP outputs).
template <typename T, bool GATE>
__global__ __launch_bounds__(256) void head_product_kernel(const T* __restrict__ x, int xs, const T* __restrict__ w,
                                                           int K, int N, int H, int num_tokens, T* __restrict__ out,
                                                           int os, HeadEpilogue ep) {
  extern __shared__ float lds[];  // [ABSORB_TOKENS][K] the inputs, [4][ABSORB_TOKENS][HEAD_STRIP] the waves' sums
  float* xl = lds;
  float* part = lds + ABSORB_TOKENS * K;
  const int t0 = blockIdx.x * ABSORB_TOKENS, h = blockIdx.y, n0 = blockIdx.z * HEAD_STRIP;
  const int nt = min(ABSORB_TOKENS, num_tokens - t0);
  for (int i = threadIdx.x; i < ABSORB_TOKENS * K; i += blockDim.x) {
    const int tq = i / K, k = i % K;
    xl[i] = tq < nt ? to_f32(x[((size_t)(t0 + tq) * H + h) * xs + k]) : 0.f;
  }
  __syncthreads();
  const int nl = threadIdx.x & 63, slice = threadIdx.x >> 6, n = n0 + nl;
  const int per = (K + 3) / 4, k_lo = slice * per, k_hi = min(K, k_lo + per);
  float acc[ABSORB_TOKENS];
#pragma unroll
  for (int tq = 0; tq < ABSORB_TOKENS; ++tq) acc[tq] = 0.f;
  if (n < N) {
    const T* wh = w + (size_t)h * K * N + n;
#pragma unroll 4
    for (int k = k_lo; k < k_hi; ++k) {
      const float wv = to_f32(wh[(size_t)k * N]);
#pragma unroll
      for (int tq = 0; tq < ABSORB_TOKENS; ++tq) acc[tq] = fmaf(xl[tq * K + k], wv, acc[tq]);
    }
  }
#pragma unroll
  for (int tq = 0; tq < ABSORB_TOKENS; ++tq) part[(slice * ABSORB_TOKENS + tq) * HEAD_STRIP + nl] = acc[tq];
  __syncthreads();
  for (int i = threadIdx.x; i < nt * HEAD_STRIP; i += blockDim.x) {
    const int tq = i / HEAD_STRIP, c = i % HEAD_STRIP;
    if (n0 + c >= N) continue;
    const float v = ((part[(0 * ABSORB_TOKENS + tq) * HEAD_STRIP + c] + part[(1 * ABSORB_TOKENS + tq) * HEAD_STRIP + c]) +
                     part[(2 * ABSORB_TOKENS + tq) * HEAD_STRIP + c]) + part[(3 * ABSORB_TOKENS + tq) * HEAD_STRIP + c];
    head_store<T, GATE>(v, t0 + tq, h, n0 + c, N, H, out, os, ep);
  }
  if (!GATE && blockIdx.z == 0) head_tail<T>(x, xs, K, N, H, h, t0, nt, out, os, ep);
}

// bfloat16, K % 32 == 0, xs % 8 == 0: w [H, N, K].  grid (token tiles of 128, heads, strips of HEAD_STRIP outputs); a
// wave owns 32 tokens.
#define MFMA_TOKENS 128
template <bool GATE>
__global__ __launch_bounds__(256) void head_product_mfma_kernel(const bf16* __restrict__ x, int xs,
                                                                const bf16* __restrict__ w, int K, int N, int H,
                                                                int num_tokens, bf16* __restrict__ out, int os,
                                                                HeadEpilogue ep) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lr = lane & 15, lg = lane >> 4;
  const int t0 = blockIdx.x * MFMA_TOKENS, h = blockIdx.y, n0 = blockIdx.z * HEAD_STRIP;
  const int tw = t0 + wave * 32;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  floatx4 acc[2][4];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) acc[tt][nt] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    bf16x8 b[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const int t = tw + tt * 16 + lr;
      b[tt] = t < num_tokens ? *reinterpret_cast<const bf16x8*>(x + ((size_t)t * H + h) * xs + k0 + lg * 8) : zero;
    }
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int n = n0 + nt * 16 + lr;
      const bf16x8 a = n < N ? *reinterpret_cast<const bf16x8*>(w + ((size_t)h * N + n) * K + k0 + lg * 8) : zero;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) acc[tt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[tt], acc[tt][nt], 0, 0, 0);
    }
  }
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    const int t = tw + tt * 16 + lr;
    if (t >= num_tokens) continue;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + nt * 16 + 4 * lg + i;
        if (n < N) head_store<bf16, GATE>(acc[tt][nt][i], (size_t)t, h, n, N, H, out, os, ep);
      }
  }
  if (!GATE && blockIdx.z == 0) head_tail<bf16>(x, xs, K, N, H, h, t0, min(MFMA_TOKENS, num_tokens - t0), out, os, ep);
}

template <bool GATE>
static int launch_head_product(const void* x, int xs, const void* w, const void* w_nk, int dtype, int K, int N, int H,
                               int num_tokens, void* out, int os, const HeadEpilogue& ep, hipStream_t stream) {
  const int strips = (N + HEAD_STRIP - 1) / HEAD_STRIP;
  if (dtype == DT_BF16 && w_nk && num_tokens >= 32 && K % 32 == 0 && xs % 8 == 0) {
    dim3 grid((num_tokens + MFMA_TOKENS - 1) / MFMA_TOKENS, H, strips);
    head_product_mfma_kernel<GATE><<<grid, 256, 0, stream>>>((const bf16*)x, xs, (const bf16*)w_nk, K, N, H, num_tokens, (bf16*)out, os, ep);
    return launch_status();
  }
  dim3 grid((num_tokens + ABSORB_TOKENS - 1) / ABSORB_TOKENS, H, strips);
  const size_t lds = (size_t)ABSORB_TOKENS * (K + 4 * HEAD_STRIP) * sizeof(float);
  if (lds > (64u << 10)) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    head_product_kernel<float, GATE><<<grid, 256, lds, stream>>>((const float*)x, xs, (const float*)w, K, N, H, num_tokens, (float*)out, os, ep);
  else if (dtype == DT_BF16)
    head_product_kernel<bf16, GATE><<<grid, 256, lds, stream>>>((const bf16*)x, xs, (const bf16*)w, K, N, H, num_tokens, (bf16*)out, os, ep);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// q [T, H, D + R]; uk [H * D, rank] (row h D + d: what coordinate d of head h's keys reads of the latent), uk_t
// [H, rank, D] the same transposed (null: none; bfloat16 prompts then run the general kernel).
// out [T, H, width]: out[t, h, r] = sum_d q[t, h, d] uk[h D + d, r] for r < rank, then the R rotated coordinates
// of q, then zeros.
extern "C" int as_latent_q_absorb(const void* q, const void* uk, const void* uk_t, int dtype, int H, int D, int R,
                                  int rank, const float* cos_sin, void* out, int width, int num_tokens,
                                  hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || H > 65535 || D <= 0 || R < 0 || R % 2 || rank <= 0 || rank + R > width || D > 1024) return AS_BAD_SHAPE;
  if (R > 0 && !cos_sin) return AS_BAD_SHAPE;
  const HeadEpilogue ep = {R, cos_sin, nullptr, 0, 0};
  return launch_head_product<false>(q, D + R, uk, uk_t, dtype, D, rank, H, num_tokens, out, width, ep, stream);
}

// heads [T, H, width]: what the attention over the latent left per head (its first `rank` coordinates count).
// uv_t [H, rank, E]: head h's value matrix, transposed; uv [H * E, rank] as the checkpoint holds it (null: none).
// out[t, h E + e] = (sum_r heads[t, h, r] uv_t[h, r, e]) * sigmoid(gate[t, g_off + h E + e]) (gate null: no gate).
extern "C" int as_latent_v_expand(const void* heads, const void* uv_t, const void* uv, int dtype, int H, int E,
                                  int rank, int width, const void* gate, int ld, int g_off, void* out,
                                  int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || H > 65535 || E <= 0 || rank <= 0 || rank > width || rank > 1536) return AS_BAD_SHAPE;
  const HeadEpilogue ep = {0, nullptr, gate, ld, g_off};
  return launch_head_product<true>(heads, width, uv_t, uv, dtype, rank, E, H, num_tokens, out, E, ep, stream);
}

// ---- attention over one kv head of any width ------------------------------------------------------------------
// For pages whose one head is wider than the paged attention kernels take.  q, out [T, H, width]; k_pages
// [pages, 1, bs, width], v_pages [pages, 1, width, bs]; a token at position p of row r sees keys 0 .. p of the row's
// block table.  grid (tokens, heads), 256 threads: the keys come 256 at a time from position 0 (a thread a key, its
// score one chain of multiply-adds), the softmax's maximum and sum move on from block to block, and a thread owns
// every 256th coordinate of the output.  All sums are fp32 and taken in an order that only positions decide.
#define WIDE_MAX_COLS 8  // coordinates of the output a thread owns: widths up to 2,048

template <typename T>
__global__ __launch_bounds__(256) void wide_attend_kernel(const T* __restrict__ q, const T* __restrict__ k_pages,
                                                          const T* __restrict__ v_pages,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ tok_row,
                                                          const int* __restrict__ block_tables, int table_width,
                                                          T* __restrict__ out, int H, int width, int bs, float scale) {
  extern __shared__ float lds[];  // [width] the query, [256] the block's weights
  __shared__ float red[17];
  float* qs = lds;
  float* ps = lds + width;
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int ctx = positions[t] + 1;
  const int* table = block_tables + (size_t)(tok_row ? tok_row[t] : t) * table_width;
  for (int i = tid; i < width; i += 256) qs[i] = to_f32(q[((size_t)t * H + h) * width + i]) * scale;
  float acc[WIDE_MAX_COLS];
#pragma unroll
  for (int c = 0; c < WIDE_MAX_COLS; ++c) acc[c] = 0.f;
  float m = -__builtin_inff(), l = 0.f;
  __syncthreads();
  for (int k0 = 0; k0 < ctx; k0 += 256) {
    const int j = k0 + tid;
    float sc = -__builtin_inff();
    if (j < ctx) {
      const T* key = k_pages + ((size_t)table[j / bs] * bs + j % bs) * width;
      sc = 0.f;
      for (int i = 0; i < width; ++i) sc = fmaf(qs[i], to_f32(key[i]), sc);
    }
    float top = sc;
    for (int off = 32; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, WAVE));
    if ((tid & 63) == 0) red[tid >> 6] = top;
    __syncthreads();
    const float mn = fmaxf(m, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
    __syncthreads();
    const float p = j < ctx ? expf(sc - mn) : 0.f;
    const float a = expf(m - mn);  // m = -inf in the first block: 0
    ps[tid] = p;
    const float sum = block_sum(p, red);  // synchronises: ps is written
    l = l * a + sum;
    m = mn;
    const int here = min(256, ctx - k0);
#pragma unroll
    for (int c = 0; c < WIDE_MAX_COLS; ++c) {
      const int d = tid + 256 * c;
      if (d < width) {
        float s = 0.f;
        for (int jj = 0; jj < here; ++jj) {
          const int key = k0 + jj;
          s = fmaf(ps[jj], to_f32(v_pages[((size_t)table[key / bs] * width + d) * bs + key % bs]), s);
        }
        acc[c] = acc[c] * a + s;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int c = 0; c < WIDE_MAX_COLS; ++c) {
    const int d = tid + 256 * c;
    if (d < width) out[((size_t)t * H + h) * width + d] = from_f32<T>(acc[c] / l);
  }
}

extern "C" int as_wide_attend(const void* q, const void* k_pages, const void* v_pages, int dtype, const int* positions,
                              const int* tok_row, const int* block_tables, int table_width, void* out, int H, int width,
                              int bs, float scale, int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || H > 65535 || width <= 0 || width > 256 * WIDE_MAX_COLS || bs <= 0 || table_width <= 0) return AS_BAD_SHAPE;
  dim3 grid(num_tokens, H);
  const size_t lds = (size_t)(width + 256) * sizeof(float);
  if (dtype == DT_F32)
    wide_attend_kernel<float><<<grid, 256, lds, stream>>>((const float*)q, (const float*)k_pages, (const float*)v_pages, positions,
                                                         tok_row, block_tables, table_width, (float*)out, H, width, bs, scale);
  else if (dtype == DT_BF16)
    wide_attend_kernel<bf16><<<grid, 256, lds, stream>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, positions,
                                                        tok_row, block_tables, table_width, (bf16*)out, H, width, bs, scale);
  else return AS_BAD_DTYPE;
  return launch_status();
}
