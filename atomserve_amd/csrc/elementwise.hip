// Row-wise kernels of the decoder: embedding lookup, RMSNorm with the residual sum
// fused in, the rotary table, per-head q/k norm + rotation + cache store, and the
// gated activation.  All arithmetic is fp32; storage is fp32 or bf16.
#include "common.h"

// ---- embedding --------------------------------------------------------------------
// out[t, :] = scale * table[ids[t], :] as fp32 (the residual stream is always fp32; the scale is 1
// for models that do not multiply their embeddings).
// Plain reference: reference atomserve/model.py:373.
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int width, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // ids are validated on the host; never read outside
  const T* src = table + (size_t)id * width;
  float* dst = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_f32(src[i]) * scale;
}

extern "C" int as_embed_gather(const void* table, int table_dtype, const int* ids, float* out,
                               int num_tokens, int width, int vocab, float scale, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (width <= 0 || vocab <= 0) return AS_BAD_SHAPE;
  const int threads = width >= 1024 ? 256 : 64;
  if (table_dtype == DT_F32)
    embed_gather_kernel<float><<<num_tokens, threads, 0, stream>>>((const float*)table, ids, out, width, vocab, scale);
  else if (table_dtype == DT_BF16)
    embed_gather_kernel<bf16><<<num_tokens, threads, 0, stream>>>((const bf16*)table, ids, out, width, vocab, scale);
  else
    return AS_BAD_DTYPE;
  return launch_status();
}

// ---- what a head may still do to its logits ------------------------------------------
// logits = cap * tanh(scale * logits / cap) (cap 0: only the scale), in place, fp32.  Qwen3 does
// neither (reference atomserve/model.py:405-415); the decoder launches this only for a plan that
// names a scale or a cap.
__global__ void logits_finish_kernel(float* __restrict__ logits, size_t count, float scale, float cap) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
    const float v = logits[i] * scale;
    logits[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

extern "C" int as_logits_finish(float* logits, long long count, float scale, float cap, hipStream_t stream) {
  if (count <= 0) return AS_OK;
  if (cap < 0.f) return AS_BAD_SHAPE;
  const long long blocks = (count + 255) / 256;
  logits_finish_kernel<<<(int)(blocks < 2048 ? blocks : 2048), 256, 0, stream>>>(logits, (size_t)count, scale, cap);
  return launch_status();
}

// ---- RMSNorm with fused residual sum and row selection --------------------------
// For output row r (source row s = rows ? rows[r] : r):
//   v = x[s] + (delta ? delta[s] : 0)          in fp32; written back to x[s] if update_x
//   out[r] = v / sqrt(mean(v^2) + eps) * w     rounded once
// Plain reference: reference atomserve/model.py:125-139 (weight multiplies directly).
//
// The pending sum may also arrive as the partial sums of a matrix product whose K was cut into
// `splits` ranges (SplitDelta: fp32 [splits, rows, n]): they are added in the order of the ranges
// and rounded to O once, which is what the product alone would have stored.
struct SplitDelta {
  const float* sums;  // null: none
  int splits;
  size_t stride;  // elements from one range's sums to the next: rows * n
};

template <typename O>
__device__ __forceinline__ float split_delta(const SplitDelta& sd, size_t at) {
  float d = sd.sums[at];
  for (int k = 1; k < sd.splits; ++k) d += sd.sums[(size_t)k * sd.stride + at];
  return to_f32(from_f32<O>(d));
}

template <typename O, typename W>
__global__ void rmsnorm_kernel(float* __restrict__ x, const O* __restrict__ delta,
                               const int* __restrict__ rows, const W* __restrict__ w, float eps,
                               O* __restrict__ out, int n, int update_x, SplitDelta sd) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + s * n;
  const O* dr = delta ? delta + s * n : nullptr;
  const bool pending = dr || sd.sums;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];
    if (pending) {
      v += dr ? to_f32(dr[i]) : split_delta<O>(sd, s * n + i);
      if (update_x) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  O* o = out + (size_t)r * n;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];  // the thread's own earlier store, if any, is what it reads back
    if (pending && !update_x) v += dr ? to_f32(dr[i]) : split_delta<O>(sd, s * n + i);
    o[i] = from_f32<O>(v * inv * to_f32(w[i]));
  }
}

// The same with 16-byte accesses and the row kept in registers between the two passes:
// every load of a row is in flight at once, which is what a decode step (few rows) needs.
// Requires n % 4 == 0 and n <= 4 * blockDim.x * RN_CHUNKS.
#define RN_CHUNKS 4
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ __forceinline__ void store(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Vec4<bf16> {
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ float4 load(const bf16* p) {
    const bf16x4 r = *reinterpret_cast<const bf16x4*>(p);
    return make_float4((float)r[0], (float)r[1], (float)r[2], (float)r[3]);
  }
  static __device__ __forceinline__ void store(bf16* p, float4 v) {
    const bf16x4 r = {(bf16)v.x, (bf16)v.y, (bf16)v.z, (bf16)v.w};
    *reinterpret_cast<bf16x4*>(p) = r;
  }
};

template <typename O, typename W>
__global__ __launch_bounds__(1024) void rmsnorm_vec_kernel(float* __restrict__ x, const O* __restrict__ delta,
                                                           const int* __restrict__ rows,
                                                           const W* __restrict__ w, float eps,
                                                           O* __restrict__ out, int n, int update_x,
                                                           SplitDelta sd) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + s * n;
  const O* dr = delta ? delta + s * n : nullptr;
  const int chunks = n >> 2;
  float4 v[RN_CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < RN_CHUNKS; ++j) {
    const int c = threadIdx.x + j * blockDim.x;
    if (c < chunks) {
      v[j] = Vec4<float>::load(xr + 4 * c);
      if (dr || sd.sums) {
        float4 d;
        if (dr) {
          d = Vec4<O>::load(dr + 4 * c);
        } else {
          const float* p = sd.sums + s * n + 4 * c;
          d = Vec4<float>::load(p);
          for (int k = 1; k < sd.splits; ++k) {
            const float4 e = Vec4<float>::load(p + (size_t)k * sd.stride);
            d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
          }
          d = make_float4(to_f32(from_f32<O>(d.x)), to_f32(from_f32<O>(d.y)), to_f32(from_f32<O>(d.z)),
                          to_f32(from_f32<O>(d.w)));
        }
        v[j].x += d.x; v[j].y += d.y; v[j].z += d.z; v[j].w += d.w;
        if (update_x) Vec4<float>::store(xr + 4 * c, v[j]);
      }
      ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  O* o = out + (size_t)r * n;
#pragma unroll
  for (int j = 0; j < RN_CHUNKS; ++j) {
    const int c = threadIdx.x + j * blockDim.x;
    if (c < chunks) {
      const float4 g = Vec4<W>::load(w + 4 * c);
      Vec4<O>::store(o + 4 * c, make_float4(v[j].x * inv * g.x, v[j].y * inv * g.y, v[j].z * inv * g.z, v[j].w * inv * g.w));
    }
  }
}

static int launch_rmsnorm(float* x, const void* delta, const SplitDelta& sd, const int* rows, const void* w,
                          int w_dtype, float eps, void* out, int out_dtype, int num_out_rows, int n, int update_x,
                          hipStream_t stream) {
  if (num_out_rows <= 0) return AS_OK;
  if (n <= 0) return AS_BAD_SHAPE;
  const bool vec = (n & 3) == 0 && n <= 4 * 1024 * RN_CHUNKS;
  int threads = n >= 2048 ? 256 : (n >= 512 ? 128 : 64);
  if (vec) {
    // few rows: one chunk per thread, all loads in flight; many rows: fewer, fuller threads
    const int chunks = n >> 2, per_thread = num_out_rows >= 512 ? RN_CHUNKS : 1;
    threads = (chunks + per_thread - 1) / per_thread;
    threads = ((threads + 63) / 64) * 64;
    if (threads > 1024) threads = 1024;
  }
#define LAUNCH(O, W)                                                                               \
  do {                                                                                             \
    if (vec)                                                                                       \
      rmsnorm_vec_kernel<O, W><<<num_out_rows, threads, 0, stream>>>(x, (const O*)delta, rows, (const W*)w, eps, \
                                                                     (O*)out, n, update_x, sd);    \
    else                                                                                           \
      rmsnorm_kernel<O, W><<<num_out_rows, threads, 0, stream>>>(x, (const O*)delta, rows, (const W*)w, eps,     \
                                                                 (O*)out, n, update_x, sd);        \
  } while (0)
  if (out_dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (out_dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (out_dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

extern "C" int as_rmsnorm(float* x, const void* delta, const int* rows, const void* w, int w_dtype,
                          float eps, void* out, int out_dtype, int num_out_rows, int n, int update_x,
                          hipStream_t stream) {
  return launch_rmsnorm(x, delta, SplitDelta{nullptr, 0, 0}, rows, w, w_dtype, eps, out, out_dtype, num_out_rows, n,
                        update_x, stream);
}

// The same with the pending sum given as the partial sums [splits, num_rows, n] (fp32) of a product
// whose K was cut into ranges; num_rows counts the rows of x.
extern "C" int as_rmsnorm_split(float* x, const float* sums, int splits, int num_rows, const int* rows, const void* w,
                                int w_dtype, float eps, void* out, int out_dtype, int num_out_rows, int n,
                                int update_x, hipStream_t stream) {
  if (!sums || splits <= 0 || num_rows <= 0) return AS_BAD_SHAPE;
  return launch_rmsnorm(x, nullptr, SplitDelta{sums, splits, (size_t)num_rows * n}, rows, w, w_dtype, eps, out,
                        out_dtype, num_out_rows, n, update_x, stream);
}

// ---- rotary table -------------------------------------------------------------------
// cs[t, i] = (cos, sin)(positions[t] * inv_freq[i]), i < half.  The product and the
// range reduction are done in fp64 so that large positions keep fp32-exact angles;
// the rotation itself is fp32.  Plain reference: reference atomserve/model.py:142-169.
__global__ void rope_table_kernel(const int* __restrict__ positions, const double* __restrict__ inv_freq,
                                  float2* __restrict__ cs, int num_tokens, int half, float magnitude) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= num_tokens * half) return;
  const int t = idx / half, i = idx % half;
  const double a = (double)positions[t] * inv_freq[i];
  double s, c;
  sincos(a, &s, &c);
  cs[idx] = make_float2((float)c * magnitude, (float)s * magnitude);
}

extern "C" int as_rope_table(const int* positions, const double* inv_freq, float* cs, int num_tokens,
                             int half, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (half <= 0) return AS_BAD_SHAPE;
  const int total = num_tokens * half;
  rope_table_kernel<<<(total + 255) / 256, 256, 0, stream>>>(positions, inv_freq, (float2*)cs, num_tokens, half, 1.0f);
  return launch_status();
}

// The same with cosines and sines multiplied by `magnitude` (rotations stretched for long contexts).
extern "C" int as_rope_table_scaled(const int* positions, const double* inv_freq, float* cs, int num_tokens,
                                    int half, float magnitude, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (half <= 0) return AS_BAD_SHAPE;
  const int total = num_tokens * half;
  rope_table_kernel<<<(total + 255) / 256, 256, 0, stream>>>(positions, inv_freq, (float2*)cs, num_tokens, half, magnitude);
  return launch_status();
}

// ---- per-head q/k norm + rotation + cache store -----------------------------------
// One wave per (token, head slot) of qkv [T, H + 2 KV, D].  q and k heads: optional
// RMSNorm over the head's D values with gains qw / kw, then rotation of the pairs
// (i, i + R/2), i < R/2, by the token's angle; coordinates >= R pass unrotated.
// q goes to q_out [T, H, D]; k goes to k_pages [num_pages, KV, bs, D] and v, copied as it
// is, to v_pages [num_pages, KV, D, bs] (each page of values is stored transposed, so that
// the keys of one coordinate are contiguous), at slot = page * bs + offset.
// store_kv = 0 computes q only.
// Plain reference: reference atomserve/kernels.py:74-145, atomserve/model.py:326-333.
template <typename O, typename W>
__global__ void qk_norm_rope_store_kernel(const O* __restrict__ qkv, const W* __restrict__ qw,
                                          const W* __restrict__ kw, const float2* __restrict__ cs,
                                          const int* __restrict__ slots, O* __restrict__ q_out,
                                          O* __restrict__ k_pages, O* __restrict__ v_pages, int H, int KV,
                                          int D, int R, float eps, int block_size) {
  const int t = blockIdx.x, hs = blockIdx.y, lane = threadIdx.x;
  const O* src = qkv + ((size_t)t * (H + 2 * KV) + hs) * D;
  const bool is_q = hs < H, is_k = !is_q && hs < H + KV;
  O* dst;
  if (is_q) {
    dst = q_out + ((size_t)t * H + hs) * D;
  } else {
    const int slot = slots[t];
    if (slot < 0) return;  // this token's keys are not stored (whole wave returns)
    const int kvh = is_k ? hs - H : hs - H - KV;
    const size_t head = (size_t)(slot / block_size) * KV + kvh;
    if (!is_k) {  // values: transposed within the page
      O* vt = v_pages + head * block_size * D + slot % block_size;
      for (int i = lane; i < D; i += WAVE) vt[(size_t)i * block_size] = finite_or_zero(src[i]);
      return;
    }
    dst = k_pages + (head * block_size + slot % block_size) * D;
  }
  const W* w = is_q ? qw : kw;
  float inv = 1.0f;
  if (w) {
    float ss = 0.f;
    for (int i = lane; i < D; i += WAVE) { const float v = to_f32(src[i]); ss += v * v; }
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)D + eps);
  }
  const int half = R / 2;
  for (int i = lane; i < half; i += WAVE) {
    float a = to_f32(src[i]) * inv, b = to_f32(src[i + half]) * inv;
    if (w) { a *= to_f32(w[i]); b *= to_f32(w[i + half]); }
    float c = 1.f, s = 0.f;
    if (cs) { const float2 v = cs[(size_t)t * half + i]; c = v.x; s = v.y; }
    const O ra = from_f32<O>(a * c - b * s), rb = from_f32<O>(b * c + a * s);
    dst[i] = is_k ? finite_or_zero(ra) : ra;
    dst[i + half] = is_k ? finite_or_zero(rb) : rb;
  }
  for (int i = R + lane; i < D; i += WAVE) {
    float a = to_f32(src[i]) * inv;
    if (w) a *= to_f32(w[i]);
    const O ra = from_f32<O>(a);
    dst[i] = is_k ? finite_or_zero(ra) : ra;
  }
}

// The same for bf16 heads that are rotated whole (R == D) and whose width is 16 times a power
// of two: a group of D / 16 lanes owns one (token, head) and every lane moves 16-byte pieces
// (coordinates 8l .. 8l+7 and their partners in the other half), so a wave serves several
// heads at once and a prompt's rows move at memory speed.  Same arithmetic, same order.
template <typename W> struct Gain8;
template <> struct Gain8<bf16> {
  static __device__ __forceinline__ void load(const bf16* p, float* g) {
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) g[j] = (float)v[j];
  }
};
template <> struct Gain8<float> {
  static __device__ __forceinline__ void load(const float* p, float* g) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    g[0] = a.x; g[1] = a.y; g[2] = a.z; g[3] = a.w; g[4] = b.x; g[5] = b.y; g[6] = b.z; g[7] = b.w;
  }
};

template <typename W>
__global__ __launch_bounds__(256) void qk_norm_rope_store_bf16x8_kernel(
    const bf16* __restrict__ qkv, const W* __restrict__ qw, const W* __restrict__ kw,
    const float2* __restrict__ cs, const int* __restrict__ slots, bf16* __restrict__ q_out,
    bf16* __restrict__ k_pages, bf16* __restrict__ v_pages, int H, int KV, int D, float eps, int block_size,
    int heads, size_t units) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  const int lpu = D >> 4, half = D >> 1;  // lanes per (token, head)
  const size_t unit = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) / lpu;
  const int l = threadIdx.x & (lpu - 1);
  if (unit >= units) return;  // whole groups leave: the shuffles below stay inside a group
  const size_t t = unit / heads;
  const int hs = (int)(unit % heads);
  const bf16* src = qkv + (t * (H + 2 * KV) + hs) * D;
  const bool is_q = hs < H, is_k = !is_q && hs < H + KV;
  bf16* dst;
  if (!is_q && !is_k) {  // values: transposed within the page
    const int slot = slots[t];
    if (slot < 0) return;  // uniform over the group
    const size_t head = (size_t)(slot / block_size) * KV + (hs - H - KV);
    // A prompt's tokens fill a page slot after slot.  Where eight tokens in a row go to eight
    // slots in a row that start at a multiple of eight, a coordinate's eight values are 16
    // contiguous bytes of the transposed page, where token by token they would be eight stores
    // of two bytes, 2 * block_size bytes apart.  The eight tokens' lane groups share that work:
    // each takes an eighth of the coordinates, two per lane, reads them from all eight tokens'
    // rows and stores two 16-byte pieces.
    const int nth = slot & 7;
    const long lead = (long)t - nth;
    bool run = (block_size & 7) == 0 && lead >= 0 && lead + 8 <= (long)(units / heads);
    if (run) {
#pragma unroll
      for (int i = 0; i < 8; ++i) run = run && slots[lead + i] == slot - nth + i;
    }
    if (run) {  // uniform over the lanes of this (token, head), and the same for all eight tokens
      typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
      const int d0 = nth * (D >> 3) + 2 * l;
      const bf16* first = qkv + ((size_t)lead * (H + 2 * KV) + hs) * D + d0;
      bf16x2 pair[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) pair[i] = *reinterpret_cast<const bf16x2*>(first + (size_t)i * (H + 2 * KV) * D);
      bf16x8 oa, ob;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        oa[i] = finite_or_zero((bf16)pair[i][0]);
        ob[i] = finite_or_zero((bf16)pair[i][1]);
      }
      bf16* vt = v_pages + head * block_size * D + (slot - nth) % block_size;
      *reinterpret_cast<bf16x8*>(vt + (size_t)d0 * block_size) = oa;
      *reinterpret_cast<bf16x8*>(vt + (size_t)(d0 + 1) * block_size) = ob;
      return;
    }
    const bf16x8 a8 = *reinterpret_cast<const bf16x8*>(src + 8 * l);
    const bf16x8 b8 = *reinterpret_cast<const bf16x8*>(src + half + 8 * l);
    bf16* vt = v_pages + head * block_size * D + slot % block_size;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      vt[(size_t)(8 * l + j) * block_size] = finite_or_zero((bf16)a8[j]);
      vt[(size_t)(half + 8 * l + j) * block_size] = finite_or_zero((bf16)b8[j]);
    }
    return;
  }
  const bf16x8 a8 = *reinterpret_cast<const bf16x8*>(src + 8 * l);
  const bf16x8 b8 = *reinterpret_cast<const bf16x8*>(src + half + 8 * l);
  if (is_q) {
    dst = q_out + (t * H + hs) * D;
  } else {
    const int slot = slots[t];
    if (slot < 0) return;  // uniform over the group
    const size_t head = (size_t)(slot / block_size) * KV + (hs - H);
    dst = k_pages + (head * block_size + slot % block_size) * D;
  }
  const W* w = is_q ? qw : kw;
  float inv = 1.0f;
  if (w) {
    float ss = 0.f;
    // the generic kernel's order within a lane differs; the sum over D squares is the same up to rounding
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += (float)a8[j] * (float)a8[j];
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += (float)b8[j] * (float)b8[j];
    for (int off = 1; off < lpu; off <<= 1) ss += __shfl_xor(ss, off, WAVE);
    inv = 1.0f / sqrtf(ss / (float)D + eps);
  }
  float ga[8], gb[8];
  if (w) {
    Gain8<W>::load(w + 8 * l, ga);
    Gain8<W>::load(w + half + 8 * l, gb);
  }
  // the angles of this lane's eight pairs: 64 contiguous bytes, four loads
  float4 turn[4];
  if (cs) {
    const float4* cs4 = reinterpret_cast<const float4*>(cs + t * half + 8 * l);
#pragma unroll
    for (int j = 0; j < 4; ++j) turn[j] = cs4[j];
  }
  bf16x8 oa, ob;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float a = (float)a8[j] * inv, b = (float)b8[j] * inv;
    if (w) { a *= ga[j]; b *= gb[j]; }
    float c = 1.f, sn = 0.f;
    if (cs) { c = (j & 1) ? turn[j >> 1].z : turn[j >> 1].x; sn = (j & 1) ? turn[j >> 1].w : turn[j >> 1].y; }
    oa[j] = (bf16)(a * c - b * sn);
    ob[j] = (bf16)(b * c + a * sn);
    if (is_k) { oa[j] = finite_or_zero((bf16)oa[j]); ob[j] = finite_or_zero((bf16)ob[j]); }
  }
  *reinterpret_cast<bf16x8*>(dst + 8 * l) = oa;
  *reinterpret_cast<bf16x8*>(dst + half + 8 * l) = ob;
}

extern "C" int as_qk_norm_rope_store(const void* qkv, int dtype, const void* qw, const void* kw, int w_dtype,
                                     const float* cs, const int* slots, void* q_out, void* k_pages,
                                     void* v_pages, int num_tokens, int H, int KV, int D, int R, float eps,
                                     int block_size, int store_kv, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || D <= 0 || R < 0 || R > D || (R & 1) || block_size <= 0) return AS_BAD_SHAPE;
  if ((qw == nullptr) != (kw == nullptr)) return AS_BAD_SHAPE;
  const int lpu = D >> 4;
  if (dtype == DT_BF16 && R == D && (D & 15) == 0 && lpu <= WAVE && (lpu & (lpu - 1)) == 0) {
    const int heads = store_kv ? H + 2 * KV : H;
    const size_t units = (size_t)num_tokens * heads;
    const size_t blocks = (units * lpu + 255) / 256;
    if (blocks > 0x7fffffff) return AS_BAD_SHAPE;
#define LAUNCH8(W)                                                                                   \
  qk_norm_rope_store_bf16x8_kernel<W><<<(int)blocks, 256, 0, stream>>>(                              \
      (const bf16*)qkv, (const W*)qw, (const W*)kw, (const float2*)cs, slots, (bf16*)q_out,          \
      (bf16*)k_pages, (bf16*)v_pages, H, KV, D, eps, block_size, heads, units)
    if (w_dtype == DT_BF16) LAUNCH8(bf16);
    else if (w_dtype == DT_F32) LAUNCH8(float);
    else return AS_BAD_DTYPE;
#undef LAUNCH8
    return launch_status();
  }
  dim3 grid(num_tokens, store_kv ? H + 2 * KV : H);
#define LAUNCH(O, W)                                                                                   \
  qk_norm_rope_store_kernel<O, W><<<grid, WAVE, 0, stream>>>(                                          \
      (const O*)qkv, (const W*)qw, (const W*)kw, (const float2*)cs, slots, (O*)q_out, (O*)k_pages,    \
      (O*)v_pages, H, KV, D, R, eps, block_size)
  if (dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ---- gated activation -----------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(g) = g / (1 + exp(-g)).
// Plain reference: reference atomserve/kernels.py:439-449, atomserve/model.py:358-359.
template <typename O>
__global__ void silu_mul_kernel(const O* __restrict__ gu, O* __restrict__ out, int inter, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inter;
    const int i = (int)(idx % inter);
    const float g = to_f32(gu[t * 2 * inter + i]);
    const float u = to_f32(gu[t * 2 * inter + inter + i]);
    out[idx] = from_f32<O>(g / (1.0f + expf(-g)) * u);
  }
}

// The same for bf16 rows whose width is a multiple of 8: 16-byte loads and stores, which is
// what a prompt's thousands of rows need to move at memory speed.
__global__ __launch_bounds__(256) void silu_mul_bf16x8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out,
                                                              int inter, size_t chunks) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  const int per_row = inter >> 3;
  for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += (size_t)gridDim.x * blockDim.x) {
    const size_t t = c / per_row;
    const int i = (int)(c % per_row) * 8;
    const bf16x8 g8 = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + i);
    const bf16x8 u8 = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + inter + i);
    bf16x8 o8;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float g = (float)g8[j];
      o8[j] = (bf16)(g / (1.0f + expf(-g)) * (float)u8[j]);
    }
    *reinterpret_cast<bf16x8*>(out + t * inter + i) = o8;
  }
}

extern "C" int as_silu_mul(const void* gate_up, void* out, int dtype, int num_tokens, int inter,
                           hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (inter <= 0) return AS_BAD_SHAPE;
  const size_t total = (size_t)num_tokens * inter;
  const size_t want = (total + 255) / 256;
  const int blocks = (int)(want > 8192 ? 8192 : want);
  if (dtype == DT_BF16 && (inter & 7) == 0) {
    const size_t chunks = total >> 3, want8 = (chunks + 255) / 256;
    silu_mul_bf16x8_kernel<<<(int)(want8 > 16384 ? 16384 : want8), 256, 0, stream>>>((const bf16*)gate_up, (bf16*)out,
                                                                                    inter, chunks);
    return launch_status();
  }
  if (dtype == DT_F32) silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter, total);
  else if (dtype == DT_BF16) silu_mul_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)gate_up, (bf16*)out, inter, total);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- one sum, two norms ------------------------------------------------------------------
// A layer whose mixer and feed-forward read the same stream through a norm each:
//   v = x[s] + (d1[s] + d2[s])        fp32; written back to x[s] if update_x (either d may be absent)
//   out1[r] = v / sqrt(mean(v^2) + eps) * w1;   out2[r] = the same with w2 (absent: one output)
// with s = rows ? rows[r] : r.  The root mean square is computed once.
template <typename O, typename W>
__global__ void rmsnorm_multi_kernel(float* __restrict__ x, const O* __restrict__ d1, const O* __restrict__ d2,
                                     const int* __restrict__ rows, const W* __restrict__ w1,
                                     const W* __restrict__ w2, float eps, O* __restrict__ out1,
                                     O* __restrict__ out2, int n, int update_x) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + s * n;
  const O* a = d1 ? d1 + s * n : nullptr;
  const O* b = d2 ? d2 + s * n : nullptr;
  const bool pending = a || b;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];
    if (pending) {
      v += (a ? to_f32(a[i]) : 0.f) + (b ? to_f32(b[i]) : 0.f);
      if (update_x) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];
    if (pending && !update_x) v += (a ? to_f32(a[i]) : 0.f) + (b ? to_f32(b[i]) : 0.f);
    const float u = v * inv;
    out1[(size_t)r * n + i] = from_f32<O>(u * to_f32(w1[i]));
    if (out2) out2[(size_t)r * n + i] = from_f32<O>(u * to_f32(w2[i]));
  }
}

extern "C" int as_rmsnorm_multi(float* x, const void* d1, const void* d2, const int* rows, const void* w1,
                                const void* w2, int w_dtype, float eps, void* out1, void* out2, int out_dtype,
                                int num_out_rows, int n, int update_x, hipStream_t stream) {
  if (num_out_rows <= 0) return AS_OK;
  if (n <= 0 || !out1 || !w1 || (out2 && !w2)) return AS_BAD_SHAPE;
  // few rows (a decode step): two columns a thread, every load of a row in flight at once; many rows: fuller threads
  int threads = num_out_rows >= 512 ? (n + 7) / 8 : (n + 1) / 2;
  threads = ((threads + 63) / 64) * 64;
  if (threads > 1024) threads = 1024;
#define LAUNCH(O, W)                                                                                        \
  rmsnorm_multi_kernel<O, W><<<num_out_rows, threads, 0, stream>>>(x, (const O*)d1, (const O*)d2, rows,     \
                                                                   (const W*)w1, (const W*)w2, eps, (O*)out1, \
                                                                   (O*)out2, n, update_x)
  if (out_dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (out_dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (out_dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ---- heads out of a wider projection: per-head norm, padding, cache store ------------------
// proj [T, ld] holds, among other columns, H query heads and KV key heads of `dim` coordinates and KV
// value heads of `vdim`, starting at columns q_off, k_off, v_off.  Queries and keys are normed per head
// (x / sqrt(mean(x^2) + eps) * weight over dim; no weights: left as they are), then turned if a table of
// angles comes with them (cs [T, R/2] of (cos, sin): the pairs (i, i + R/2) of a head's first R coordinates, as
// in qk_norm_rope_store; values are never turned, so values read from the keys' columns are the keys unturned).
// The attention kernels take one head width for keys and values, so every head is laid out with
// Dp >= max(dim, vdim) coordinates, the ones a head does not have being zero: scores and outputs are
// unchanged.  q_out [T, H, Dp]; keys to k_pages [pages, KV, bs, Dp] and values transposed to v_pages
// [pages, KV, Dp, bs] at slots[t] (page * bs + offset; negative or store == 0: not stored).
template <typename T, typename W>
__global__ __launch_bounds__(64) void head_norm_store_kernel(const T* __restrict__ proj, int ld, int q_off, int k_off,
                                                             int v_off, int H, int KV, int dim, int vdim, int Dp,
                                                             const W* __restrict__ qw, const W* __restrict__ kw,
                                                             float eps, const int* __restrict__ slots,
                                                             T* __restrict__ q_out, T* __restrict__ k_pages,
                                                             T* __restrict__ v_pages, int bs, int store,
                                                             const float2* __restrict__ cs, int R) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const T* row = proj + (size_t)t * ld;
  if (head < H + KV) {  // a query or a key head
    const bool is_q = head < H;
    const int hh = is_q ? head : head - H;
    const T* src = row + (is_q ? q_off : k_off) + hh * dim;
    const W* w = is_q ? qw : kw;
    T* dst;
    if (is_q) {
      dst = q_out + ((size_t)t * H + hh) * Dp;
    } else {
      const int slot = (store && slots) ? slots[t] : -1;
      if (slot < 0) return;
      dst = k_pages + (((size_t)(slot / bs) * KV + hh) * bs + slot % bs) * Dp;
    }
    float inv = 1.f;
    if (w) {
      float ss = 0.f;
      for (int d = lane; d < dim; d += WAVE) { const float v = to_f32(src[d]); ss += v * v; }
      ss = wave_sum(ss);
      inv = 1.0f / sqrtf(ss / (float)dim + eps);
    }
    const int half = cs ? R / 2 : 0;
    for (int d = lane; d < Dp; d += WAVE) {
      float v = 0.f;
      if (d < dim) v = w ? to_f32(src[d]) * inv * to_f32(w[d]) : to_f32(src[d]);
      if (d < 2 * half) {  // the partner of coordinate d, and the turn by the token's angle
        const int i = d < half ? d : d - half, o = d < half ? d + half : d - half;
        const float u = w ? to_f32(src[o]) * inv * to_f32(w[o]) : to_f32(src[o]);
        const float2 a = cs[(size_t)t * half + i];
        v = d < half ? v * a.x - u * a.y : v * a.x + u * a.y;
      }
      dst[d] = from_f32<T>(finite_or_zero(v));
    }
    return;
  }
  const int g = head - H - KV;  // a value head
  const int slot = (store && slots) ? slots[t] : -1;
  if (slot < 0) return;
  const T* src = row + v_off + g * vdim;
  T* dst = v_pages + ((size_t)(slot / bs) * KV + g) * Dp * bs + slot % bs;
  for (int d = lane; d < Dp; d += WAVE) dst[(size_t)d * bs] = d < vdim ? finite_or_zero(src[d]) : from_f32<T>(0.f);
}

extern "C" int as_head_norm_store(const void* proj, int dtype, int ld, int q_off, int k_off, int v_off, int H, int KV,
                                  int dim, int vdim, int Dp, const void* qw, const void* kw, int w_dtype, float eps,
                                  const int* slots, void* q_out, void* k_pages, void* v_pages, int bs, int store,
                                  int num_tokens, const float* cs, int R, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (cs && (R <= 0 || (R & 1) || R > dim)) return AS_BAD_SHAPE;
  if (H <= 0 || KV <= 0 || dim <= 0 || vdim <= 0 || Dp < dim || Dp < vdim || bs <= 0 || ld <= 0 || (!qw) != (!kw))
    return AS_BAD_SHAPE;
  if (H + 2 * KV > 65535) return AS_BAD_SHAPE;
  dim3 grid(num_tokens, H + 2 * KV);
#define LAUNCH(T, W)                                                                                          \
  head_norm_store_kernel<T, W><<<grid, 64, 0, stream>>>((const T*)proj, ld, q_off, k_off, v_off, H, KV, dim,  \
                                                        vdim, Dp, (const W*)qw, (const W*)kw, eps, slots,     \
                                                        (T*)q_out, (T*)k_pages, (T*)v_pages, bs, store,       \
                                                        (const float2*)cs, R)
  if (dtype == DT_F32 && (w_dtype == DT_F32 || !qw)) LAUNCH(float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ---- heads out of a wider projection, normed over the whole projection ---------------------------------
// As head_norm_store, with three more things a design may ask for.  Biases q_bias [H dim], k_bias [KV dim], v_bias
// [KV vdim] (fp32, or none) are added to the projection's output first.  With gains qw [H dim] and kw [KV dim] (fp32)
// queries and keys are RMS-normed over ALL their heads at once: x / sqrt(mean over H dim (x^2) + eps) * gain.  The
// values may be mixed with those that an earlier layer kept for the same tokens: v_mode 1 writes this layer's values
// (bias added) into v_keep fp32 [T, KV vdim]; v_mode 2 stores (1 - lam) v + lam v_keep[t] instead of v.  The rotation
// (after the norm) and the layout of q_out and of the pages are head_norm_store's.  A workgroup per token.
template <typename T>
__global__ __launch_bounds__(256) void whole_norm_store_kernel(
    const T* __restrict__ proj, int ld, int q_off, int k_off, int v_off, int H, int KV, int dim, int vdim, int Dp,
    const float* __restrict__ q_bias, const float* __restrict__ k_bias, const float* __restrict__ v_bias,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps, const float2* __restrict__ cs, int R,
    float* __restrict__ v_keep, int v_mode, float lam, const int* __restrict__ slots, T* __restrict__ q_out,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int bs, int store) {
  // blockIdx.y: one of gridDim.y workgroups that share a token's heads (query, key and value heads in one list, dealt
  // out in turn); every one of them takes the root mean squares over the whole projections for itself.
  __shared__ float red[17];
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * ld;
  const int nq = H * dim, nk = KV * dim, nv = KV * vdim;
  float inv_q = 1.f, inv_k = 1.f;
  if (qw) {
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < nq; c += blockDim.x) {
      const float v = to_f32(row[q_off + c]) + (q_bias ? q_bias[c] : 0.f);
      sq = fmaf(v, v, sq);
    }
    for (int c = threadIdx.x; c < nk; c += blockDim.x) {
      const float v = to_f32(row[k_off + c]) + (k_bias ? k_bias[c] : 0.f);
      sk = fmaf(v, v, sk);
    }
    inv_q = 1.0f / sqrtf(block_sum(sq, red) / (float)nq + eps);
    inv_k = 1.0f / sqrtf(block_sum(sk, red) / (float)nk + eps);
  }
  const int half = cs ? R / 2 : 0;
  const int slot = (store && slots) ? slots[t] : -1;
  const int all = H + 2 * KV, share = (all - (int)blockIdx.y + (int)gridDim.y - 1) / (int)gridDim.y;  // heads of this workgroup
  for (int idx = threadIdx.x; idx < share * Dp; idx += blockDim.x) {
    const int head = blockIdx.y + (idx / Dp) * gridDim.y, d = idx % Dp;
    if (head < H + KV) {  // a query or a key head: coordinate d, with its partner if it turns
      const bool is_k = head >= H;
      const int hh = is_k ? head - H : head, off = is_k ? k_off : q_off;
      const float* bias = is_k ? k_bias : q_bias;
      const float* w = is_k ? kw : qw;
      const float inv = is_k ? inv_k : inv_q;
      if (is_k && slot < 0) continue;
      T* dst = is_k ? k_pages + (((size_t)(slot / bs) * KV + hh) * bs + slot % bs) * Dp : q_out + ((size_t)t * H + hh) * Dp;
      auto value = [&](int dd) {
        const int c = hh * dim + dd;
        float v = to_f32(row[off + c]) + (bias ? bias[c] : 0.f);
        if (w) v = v * inv * w[c];
        return v;
      };
      float v = d < dim ? value(d) : 0.f;
      if (d < 2 * half) {
        const int i = d < half ? d : d - half, o = d < half ? d + half : d - half;
        const float u = value(o);
        const float2 a = cs[(size_t)t * half + i];
        v = d < half ? v * a.x - u * a.y : v * a.x + u * a.y;
      }
      dst[d] = from_f32<T>(finite_or_zero(v));
    } else {  // a value head
      const int g = head - H - KV;
      float v = 0.f;
      if (d < vdim) {
        const int c = g * vdim + d;
        v = to_f32(row[v_off + c]) + (v_bias ? v_bias[c] : 0.f);
        if (v_mode == 1) v_keep[(size_t)t * nv + c] = v;
        else if (v_mode == 2) v = (1.0f - lam) * v + lam * v_keep[(size_t)t * nv + c];
      }
      if (slot >= 0) v_pages[((size_t)(slot / bs) * KV + g) * Dp * bs + (size_t)d * bs + slot % bs] = from_f32<T>(finite_or_zero(v));
    }
  }
}

extern "C" int as_whole_norm_store(const void* proj, int dtype, int ld, int q_off, int k_off, int v_off, int H, int KV,
                                   int dim, int vdim, int Dp, const float* q_bias, const float* k_bias,
                                   const float* v_bias, const float* qw, const float* kw, float eps, const float* cs,
                                   int R, float* v_keep, int v_mode, float lam, const int* slots, void* q_out,
                                   void* k_pages, void* v_pages, int bs, int store, int num_tokens,
                                   hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (cs && (R <= 0 || (R & 1) || R > dim)) return AS_BAD_SHAPE;
  if (H <= 0 || KV <= 0 || dim <= 0 || vdim <= 0 || Dp < dim || Dp < vdim || bs <= 0 || ld <= 0 || (!qw) != (!kw))
    return AS_BAD_SHAPE;
  if (v_mode < 0 || v_mode > 2 || (v_mode && !v_keep)) return AS_BAD_SHAPE;
  // few tokens (a decode step): a token's heads are dealt out over several workgroups; many: one takes them all
  int across = num_tokens >= 256 ? 1 : (H + 2 * KV < 32 ? H + 2 * KV : 32);
  const int threads = across > 1 && Dp <= 128 ? (Dp > 64 ? 128 : 64) : 256;
  dim3 grid(num_tokens, across);
  if (dtype == DT_F32)
    whole_norm_store_kernel<float><<<grid, threads, 0, stream>>>(
        (const float*)proj, ld, q_off, k_off, v_off, H, KV, dim, vdim, Dp, q_bias, k_bias, v_bias, qw, kw, eps,
        (const float2*)cs, R, v_keep, v_mode, lam, slots, (float*)q_out, (float*)k_pages, (float*)v_pages, bs, store);
  else if (dtype == DT_BF16)
    whole_norm_store_kernel<bf16><<<grid, threads, 0, stream>>>(
        (const bf16*)proj, ld, q_off, k_off, v_off, H, KV, dim, vdim, Dp, q_bias, k_bias, v_bias, qw, kw, eps,
        (const float2*)cs, R, v_keep, v_mode, lam, slots, (bf16*)q_out, (bf16*)k_pages, (bf16*)v_pages, bs, store);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- an output gate on attention heads --------------------------------------------------------
// out[t, out_off + h * vdim + j] = scale * sigmoid(gate[t, gate_off + h * vdim + j]) * heads[t, h, j]
// for j < vdim of the Dp coordinates a head is laid out with; gate [T, ld_gate], out [T, ld_out].
template <typename T>
__global__ void sigmoid_gate_heads_kernel(const T* __restrict__ heads, int H, int vdim, int Dp,
                                          const T* __restrict__ gate, int ld_gate, int gate_off, float scale,
                                          T* __restrict__ out, int ld_out, int out_off, size_t total) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const int per = H * vdim;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const size_t t = idx / per;
    const int c = (int)(idx % per), h = c / vdim, j = c % vdim;
    const float v = to_f32(heads[(t * H + h) * Dp + j]);
    // no gate: the heads, scaled
    out[t * ld_out + out_off + c] = from_f32<T>(gate ? scale * v / (1.0f + expf(-to_f32(gate[t * ld_gate + gate_off + c]))) : scale * v);
  }
}

extern "C" int as_sigmoid_gate_heads(const void* heads, int dtype, int H, int vdim, int Dp, const void* gate,
                                     int ld_gate, int gate_off, float scale, void* out, int ld_out, int out_off,
                                     int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || vdim <= 0 || Dp < vdim) return AS_BAD_SHAPE;
  const size_t total = (size_t)num_tokens * H * vdim;
  const size_t want = (total + 255) / 256;
  const int blocks = (int)(want > 8192 ? 8192 : want);
  if (dtype == DT_F32)
    sigmoid_gate_heads_kernel<float><<<blocks, 256, 0, stream>>>((const float*)heads, H, vdim, Dp, (const float*)gate,
                                                                 ld_gate, gate_off, scale, (float*)out, ld_out, out_off, total);
  else if (dtype == DT_BF16)
    sigmoid_gate_heads_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)heads, H, vdim, Dp, (const bf16*)gate,
                                                                ld_gate, gate_off, scale, (bf16*)out, ld_out, out_off, total);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- a gated, scaled residual sum, with the norm that follows it -------------------------------
// For source row s (= rows ? rows[r] : r) of the fp32 stream x [T, n]:
//   v = x[s] + mult * sigmoid(gate[s, gate_off + i] + bias[i]) * y[s, i]      (y null: v = x[s]); written back if update_x
//   out[r]  = v / sqrt(mean(v^2) + eps) * w, rounded once                     (w null: no norm is taken)
//   join[r] = [ v | other[s] ] rounded to O, 2n wide                           (join null: none)
// y and gate are a part's output and the logits of its output gate (columns of a wider product, ld_gate wide);
// the sum and the sigmoid are fp32.  `join` hands the stream, beside another fp32 stream, to a product that
// takes both.
template <typename O, typename W, typename NO>
__global__ void gated_add_norm_kernel(float* __restrict__ x, const O* __restrict__ y, const O* __restrict__ gate,
                                      int ld_gate, int gate_off, const W* __restrict__ bias, float mult,
                                      const int* __restrict__ rows, const W* __restrict__ w, float eps,
                                      NO* __restrict__ out, int n, int update_x, const float* __restrict__ other,
                                      O* __restrict__ join) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + s * n;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];
    if (y) {
      const float g = to_f32(gate[s * ld_gate + gate_off + i]) + (bias ? to_f32(bias[i]) : 0.f);
      v += mult * to_f32(y[s * n + i]) / (1.0f + expf(-g));
      if (update_x) xr[i] = v;
    }
    ss += v * v;
    if (join) {
      join[(size_t)r * 2 * n + i] = from_f32<O>(v);
      join[(size_t)r * 2 * n + n + i] = from_f32<O>(other[s * n + i]);
    }
  }
  if (!w) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  NO* o = out + (size_t)r * n;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];  // the thread's own earlier store, if any, is what it reads back
    if (y && !update_x) {
      const float g = to_f32(gate[s * ld_gate + gate_off + i]) + (bias ? to_f32(bias[i]) : 0.f);
      v += mult * to_f32(y[s * n + i]) / (1.0f + expf(-g));
    }
    o[i] = from_f32<NO>(v * inv * to_f32(w[i]));
  }
}

// dtype: of y, gate and join; w_dtype: of bias and w; out_dtype: of out (fp32 for a norm whose result is a stream).
extern "C" int as_gated_add_norm(float* x, const void* y, const void* gate, int dtype, int ld_gate, int gate_off,
                                 const void* bias, float mult, const int* rows, const void* w, int w_dtype, float eps,
                                 void* out, int out_dtype, int n_out, int n, int update_x, const float* other,
                                 void* join, hipStream_t stream) {
  if (n_out <= 0) return AS_OK;
  if (n <= 0 || (y && (!gate || ld_gate < n || gate_off < 0 || gate_off + n > ld_gate)) || (w && !out) ||
      (join && !other))
    return AS_BAD_SHAPE;
  // four values a thread where the row allows it: a decode step's few rows wait for memory, not for arithmetic
  const int threads = n >= 4096 ? 1024 : (n >= 2048 ? 512 : (n >= 512 ? 256 : 64));
#define LAUNCH(O, W, NO)                                                                                          \
  gated_add_norm_kernel<O, W, NO><<<n_out, threads, 0, stream>>>(x, (const O*)y, (const O*)gate, ld_gate, gate_off, \
                                                                 (const W*)bias, mult, rows, (const W*)w, eps,      \
                                                                 (NO*)out, n, update_x, other, (O*)join)
  if (dtype == DT_F32 && w_dtype == DT_F32 && out_dtype == DT_F32) LAUNCH(float, float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_BF16) LAUNCH(bf16, bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32 && out_dtype == DT_BF16) LAUNCH(bf16, float, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_F32) LAUNCH(bf16, bf16, float);
  else if (dtype == DT_BF16 && w_dtype == DT_F32 && out_dtype == DT_F32) LAUNCH(bf16, float, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ---- relu(x)^2 on the first columns of a wider product --------------------------------------------
// out[t, i] = max(a[t, off + i], 0)^2 for i < n; a [T, ld].
template <typename T>
__global__ void relu2_kernel(const T* __restrict__ a, int ld, int off, T* __restrict__ out, int n, size_t total) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const size_t t = idx / n;
    const float v = fmaxf(to_f32(a[t * ld + off + idx % n]), 0.f);
    out[idx] = from_f32<T>(v * v);
  }
}

extern "C" int as_relu2(const void* a, int dtype, int ld, int off, void* out, int n, int num_tokens,
                        hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (n <= 0 || off < 0 || off + n > ld) return AS_BAD_SHAPE;
  const size_t total = (size_t)num_tokens * n, want = (total + 255) / 256;
  const int blocks = (int)(want > 8192 ? 8192 : want);
  if (dtype == DT_F32) relu2_kernel<float><<<blocks, 256, 0, stream>>>((const float*)a, ld, off, (float*)out, n, total);
  else if (dtype == DT_BF16) relu2_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)a, ld, off, (bf16*)out, n, total);
  else return AS_BAD_DTYPE;
  return launch_status();
}
