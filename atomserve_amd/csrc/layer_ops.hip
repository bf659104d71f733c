// What a layer does to the stream around its parts, beyond a plain norm:
//
//   group_norm        an RMS norm in groups: a row is cut into `groups` equal consecutive parts, each divided by
//                     its own sqrt(mean(part^2) + eps), the whole times a gain; with the pending residual sum
//                     and the row selection of the plain norm's kernel
//   group_norm_shift  the same norm followed by a token shift: h_t + (h_(t-1) - h_t) * mu, h_(t-1) the normed
//                     row of the token before (zeros before a sequence's first token, a request's state slot
//                     before a row's first token)
//   depth_average     the layer's result X_n = x + delta is kept beside the results of all layers before it
//                     (and the embedding's), and the stream goes on as sum_j c[j] X_j
//   clamped_gate      g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha g) * (u + 1)
//
// Sums of squares, the norm, the shift, the residual sum and the depth average are fp32 in both precisions.
#include "common.h"

// Four consecutive values at once (the address a multiple of 16 bytes for fp32, of 8 for bfloat16).
__device__ __forceinline__ void load4(const float* p, float* v) {
  const float4 r = *reinterpret_cast<const float4*>(p);
  v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
}
__device__ __forceinline__ void load4(const bf16* p, float* v) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
  v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16* p, const float* v) {
  bf16 b[4] = {from_f32<bf16>(v[0]), from_f32<bf16>(v[1]), from_f32<bf16>(v[2]), from_f32<bf16>(v[3])};
  *reinterpret_cast<uint2*>(p) = *reinterpret_cast<const uint2*>(b);
}

// ---- the grouped norm of one row ------------------------------------------------------------------
// inv[g] = 1 / sqrt(mean over group g of (x + d)^2 + eps); the waves take the groups in turn, a group's sum meets
// by lane swaps.  The caller synchronises before reading `inv`.
template <typename O>
__device__ __forceinline__ void group_inverse_rms(const float* __restrict__ xr, const O* __restrict__ dr, int n,
                                                  int groups, float eps, float* inv) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
  const int gs = n / groups;
  for (int g = wave; g < groups; g += waves) {
    float ss = 0.f;
    if (gs % 4 == 0) {  // groups of a multiple of four: four values a load (rows start on 16 bytes)
      for (int i = 4 * lane; i < gs; i += 4 * WAVE) {
        float v[4], d[4];
        load4(xr + g * gs + i, v);
        if (dr) {
          load4(dr + g * gs + i, d);
#pragma unroll
          for (int c = 0; c < 4; ++c) v[c] += d[c];
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) ss = fmaf(v[c], v[c], ss);
      }
    } else {
      for (int i = lane; i < gs; i += WAVE) {
        float v = xr[g * gs + i];
        if (dr) v += to_f32(dr[g * gs + i]);
        ss = fmaf(v, v, ss);
      }
    }
    ss = wave_sum(ss);
    if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)gs + eps);
  }
}

#define MAX_NORM_GROUPS 256

// out[r] = group_norm(x[s] + d[s]) * w, s = rows ? rows[r] : r; x[s] receives the sum if update_x.
template <typename O>
__global__ __launch_bounds__(256) void group_norm_kernel(float* __restrict__ x, const O* __restrict__ d,
                                                         const int* __restrict__ rows, const float* __restrict__ w,
                                                         float eps, int groups, O* __restrict__ out, int n,
                                                         int update_x) {
  __shared__ float inv[MAX_NORM_GROUPS];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + s * n;
  const O* dr = d ? d + s * n : nullptr;
  group_inverse_rms<O>(xr, dr, n, groups, eps, inv);
  __syncthreads();
  const int gs = n / groups;
  if (gs % 4 == 0) {
    for (int i = 4 * threadIdx.x; i < n; i += 4 * blockDim.x) {
      float v[4], d[4], g[4];
      load4(xr + i, v);
      load4(w + i, g);
      if (dr) {
        load4(dr + i, d);
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] += d[c];
        if (update_x) store4(xr + i, v);
      }
      const float scale = inv[i / gs];
#pragma unroll
      for (int c = 0; c < 4; ++c) v[c] = v[c] * scale * g[c];
      store4(out + (size_t)r * n + i, v);
    }
    return;
  }
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i];
    if (dr) {
      v += to_f32(dr[i]);
      if (update_x) xr[i] = v;
    }
    out[(size_t)r * n + i] = from_f32<O>(v * inv[i / gs] * w[i]);
  }
}

// A workgroup per token t of row r = tok_row[t] (tok_row null: token t is row t).  h = group_norm(x[t]) * w;
// before = the same of x[t - 1], or, for a row's first token, the row's state slot (zeros if the row starts its
// sequence).  out[t] = h + (before - h) * mu.  The workgroup of a row's first token, which alone reads the slot,
// afterwards leaves there the normed row of the row's last token for the request's next row; nothing is kept for
// a row without a slot (slot < 0), and nothing is written where `writes` is 0.
template <typename O>
__global__ __launch_bounds__(256) void group_norm_shift_kernel(const float* __restrict__ x,
                                                               const float* __restrict__ w,
                                                               const float* __restrict__ mu, float eps, int groups,
                                                               const int* __restrict__ tok_row,
                                                               const int* __restrict__ row_first,
                                                               const int* __restrict__ row_len,
                                                               const int* __restrict__ row_start,
                                                               const int* __restrict__ row_slots,
                                                               float* __restrict__ state, O* __restrict__ out, int n,
                                                               int writes) {
  __shared__ float inv[MAX_NORM_GROUPS], inv_before[MAX_NORM_GROUPS], inv_last[MAX_NORM_GROUPS];
  const int t = blockIdx.x;
  const int r = tok_row ? tok_row[t] : t;
  const int first = row_first[r], len = row_len[r], slot = row_slots[r];
  const bool leads = t == first;
  const bool keeps = leads && writes && slot >= 0;
  const int last = first + len - 1;
  const float* xr = x + (size_t)t * n;
  const float* xb = x + (size_t)(leads ? t : t - 1) * n;
  const float* xl = x + (size_t)last * n;
  group_inverse_rms<O>(xr, nullptr, n, groups, eps, inv);
  if (!leads) group_inverse_rms<O>(xb, nullptr, n, groups, eps, inv_before);
  if (keeps && last != t) group_inverse_rms<O>(xl, nullptr, n, groups, eps, inv_last);
  __syncthreads();
  const int gs = n / groups;
  const bool from_slot = leads && row_start[r] > 0 && slot >= 0;
  float* kept = slot >= 0 ? state + (size_t)slot * n : nullptr;
  if (gs % 4 == 0) {
    for (int i = 4 * threadIdx.x; i < n; i += 4 * blockDim.x) {
      float h[4], g[4], m[4], before[4] = {0.f, 0.f, 0.f, 0.f}, o[4];
      load4(xr + i, h);
      load4(w + i, g);
      load4(mu + i, m);
      const float scale = inv[i / gs];
#pragma unroll
      for (int c = 0; c < 4; ++c) h[c] = h[c] * scale * g[c];
      if (!leads) {
        load4(xb + i, before);
        const float sb = inv_before[i / gs];
#pragma unroll
        for (int c = 0; c < 4; ++c) before[c] = before[c] * sb * g[c];
      } else if (from_slot) {
        load4(kept + i, before);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) o[c] = h[c] + (before[c] - h[c]) * m[c];
      store4(out + (size_t)t * n + i, o);
      if (keeps) {  // read above by this same thread
        if (last != t) {
          load4(xl + i, h);
          const float sl = inv_last[i / gs];
#pragma unroll
          for (int c = 0; c < 4; ++c) h[c] = h[c] * sl * g[c];
        }
        store4(kept + i, h);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float h = xr[i] * inv[i / gs] * w[i];
    float before = 0.f;
    if (!leads) before = xb[i] * inv_before[i / gs] * w[i];
    else if (from_slot) before = kept[i];
    out[(size_t)t * n + i] = from_f32<O>(h + (before - h) * mu[i]);
    if (keeps) kept[i] = last == t ? h : xl[i] * inv_last[i / gs] * w[i];  // read above by this same thread
  }
}

extern "C" int as_group_norm(float* x, const void* delta, const int* rows, const float* weight, float eps, int groups,
                             void* out, int dtype, int n_out, int n, int update_x, hipStream_t stream) {
  if (n_out <= 0) return AS_OK;
  if (n <= 0 || groups <= 0 || groups > MAX_NORM_GROUPS || n % groups) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    group_norm_kernel<float><<<n_out, 256, 0, stream>>>(x, (const float*)delta, rows, weight, eps, groups, (float*)out, n, update_x);
  else if (dtype == DT_BF16)
    group_norm_kernel<bf16><<<n_out, 256, 0, stream>>>(x, (const bf16*)delta, rows, weight, eps, groups, (bf16*)out, n, update_x);
  else return AS_BAD_DTYPE;
  return launch_status();
}

extern "C" int as_group_norm_shift(const float* x, const float* weight, const float* mu, float eps, int groups,
                                   const int* tok_row, const int* row_first, const int* row_len, const int* row_start,
                                   const int* row_slots, float* state, void* out, int dtype, int num_tokens, int n,
                                   int writes, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (n <= 0 || groups <= 0 || groups > MAX_NORM_GROUPS || n % groups) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    group_norm_shift_kernel<float><<<num_tokens, 256, 0, stream>>>(x, weight, mu, eps, groups, tok_row, row_first, row_len,
                                                                  row_start, row_slots, state, (float*)out, n, writes);
  else if (dtype == DT_BF16)
    group_norm_shift_kernel<bf16><<<num_tokens, 256, 0, stream>>>(x, weight, mu, eps, groups, tok_row, row_first, row_len,
                                                                 row_start, row_slots, state, (bf16*)out, n, writes);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- the depth average ------------------------------------------------------------------------------
// kept [slots, total] fp32: the results of the layers so far (kept[0]: what the embedding gave).  v = x + delta is
// this layer's result, kept as kept[n]; x = sum_(j < n) c[j] kept[j] + c[n] v.  Sums in the order of j.
template <typename O>
__global__ __launch_bounds__(256) void depth_average_kernel(float* __restrict__ x, const O* __restrict__ d,
                                                            float* __restrict__ kept, const float* __restrict__ c,
                                                            int n, size_t total) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    float v = x[i];
    if (d) v += to_f32(d[i]);
    kept[(size_t)n * total + i] = v;
    float s = 0.f;
    for (int j = 0; j < n; ++j) s = fmaf(c[j], kept[(size_t)j * total + i], s);
    x[i] = fmaf(c[n], v, s);
  }
}

extern "C" int as_depth_average(float* x, const void* delta, int dtype, float* kept, const float* coef, int n,
                                long long total, hipStream_t stream) {
  if (total <= 0) return AS_OK;
  if (n < 0) return AS_BAD_SHAPE;
  const size_t want = ((size_t)total + 255) / 256;
  const int blocks = (int)(want > 16384 ? 16384 : want);
  if (dtype == DT_F32) depth_average_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)delta, kept, coef, n, (size_t)total);
  else if (dtype == DT_BF16) depth_average_kernel<bf16><<<blocks, 256, 0, stream>>>(x, (const bf16*)delta, kept, coef, n, (size_t)total);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- a gated activation with limits -------------------------------------------------------------------
// gate_up [T, 2 I]: a row's gate values, then its up values.  out [T, I].
template <typename O>
__global__ void clamped_gate_kernel(const O* __restrict__ gu, O* __restrict__ out, int inter, float limit, float alpha,
                                    size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inter;
    const int i = (int)(idx % inter);
    const float g = fminf(to_f32(gu[t * 2 * inter + i]), limit);
    const float u = fminf(fmaxf(to_f32(gu[t * 2 * inter + inter + i]), -limit), limit);
    out[idx] = from_f32<O>(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

extern "C" int as_clamped_gate(const void* gate_up, void* out, int dtype, int num_tokens, int inter, float limit,
                               float alpha, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (inter <= 0) return AS_BAD_SHAPE;
  const size_t total = (size_t)num_tokens * inter, want = (total + 255) / 256;
  const int blocks = (int)(want > 16384 ? 16384 : want);
  if (dtype == DT_F32) clamped_gate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter, limit, alpha, total);
  else if (dtype == DT_BF16) clamped_gate_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)gate_up, (bf16*)out, inter, limit, alpha, total);
  else return AS_BAD_DTYPE;
  return launch_status();
}
