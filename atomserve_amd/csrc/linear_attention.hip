// Linear attention with a fixed decay per head: a state S [D, E] per head and request,
//
//   S_t = lam_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
//
// with q, k [D] and v [E] columns of one input product (an activation and a factor applied as they are read).
// The state is fp32 and lives in a slot per request; a row that starts its sequence starts from zero whatever its
// slot holds, a later row goes on from what the row before left.  Everything after the products is fp32.
//
//   decay_scan    token by token: a lane keeps a slice of one column of the state in registers for all of a row's tokens
//   decay_finish  o normed in groups (per head, or all heads together) with an optional gain, times act(gate)
#include "common.h"

#define ACT_NONE 0
#define ACT_SILU 1
#define ACT_SIGMOID 2

__device__ __forceinline__ float apply_act(float v, int act) {
  if (act == ACT_SILU) return v / (1.0f + expf(-v));
  if (act == ACT_SIGMOID) return 1.0f / (1.0f + expf(-v));
  return v;
}

// ---- token by token ------------------------------------------------------------------------------------
// grid (column groups, heads, rows), one wave a workgroup.  The wave owns 64 / SL columns e of a head's state; a
// column's D rows are cut into SL slices of DPER in neighbouring lanes, whose partial sums meet by lane swaps.
#define SCAN_DPER 32

template <typename T>
__global__ __launch_bounds__(64) void decay_scan_kernel(const T* __restrict__ proj, int ld, int q_off, int k_off,
                                                        int v_off, int H, int D, int E, int act, float k_scale,
                                                        const float* __restrict__ decay, float* __restrict__ state,
                                                        const int* __restrict__ row_first,
                                                        const int* __restrict__ row_len,
                                                        const int* __restrict__ row_start,
                                                        const int* __restrict__ row_slots, float* __restrict__ out,
                                                        int SL, int writes) {
  const int lane = threadIdx.x, sl = lane % SL, col = lane / SL;
  const int cols = WAVE / SL;
  const int e = blockIdx.x * cols + col, h = blockIdx.y, r = blockIdx.z;
  const bool live = e < E;
  const int first = row_first[r], len = row_len[r], slot = row_slots[r];
  const float lam = decay[h];
  const int d0 = sl * SCAN_DPER;
  float S[SCAN_DPER];
  float* kept = slot >= 0 ? state + (((size_t)slot * H + h) * D) * E : nullptr;
  const bool resume = kept && row_start[r] > 0;
#pragma unroll
  for (int i = 0; i < SCAN_DPER; ++i) S[i] = (resume && live && d0 + i < D) ? kept[(size_t)(d0 + i) * E + e] : 0.f;
  float qn[SCAN_DPER], kn[SCAN_DPER], vn = 0.f;
  auto fetch = [&](int t) {
    const T* row = proj + (size_t)t * ld;
#pragma unroll
    for (int i = 0; i < SCAN_DPER; ++i) {
      const bool in = d0 + i < D;
      qn[i] = in ? to_f32(row[q_off + h * D + d0 + i]) : 0.f;
      kn[i] = in ? to_f32(row[k_off + h * D + d0 + i]) : 0.f;
    }
    vn = live ? to_f32(row[v_off + h * E + e]) : 0.f;
  };
  fetch(first);
  for (int t = first; t < first + len; ++t) {
    float q[SCAN_DPER], k[SCAN_DPER];
    const float v = apply_act(vn, act);
#pragma unroll
    for (int i = 0; i < SCAN_DPER; ++i) { q[i] = apply_act(qn[i], act); k[i] = apply_act(kn[i], act) * k_scale; }
    if (t + 1 < first + len) fetch(t + 1);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < SCAN_DPER; ++i) {
      S[i] = fmaf(lam, S[i], k[i] * v);
      acc = fmaf(S[i], q[i], acc);
    }
    for (int off = 1; off < SL; off <<= 1) acc += __shfl_xor(acc, off, WAVE);
    if (live && sl == 0) out[((size_t)t * H + h) * E + e] = acc;
  }
  if (kept && writes && live) {
#pragma unroll
    for (int i = 0; i < SCAN_DPER; ++i)
      if (d0 + i < D) kept[(size_t)(d0 + i) * E + e] = S[i];
  }
}

extern "C" int as_decay_scan(const void* proj, int dtype, int ld, int q_off, int k_off, int v_off, int H, int D, int E,
                             int act, float k_scale, const float* decay, float* state, const int* row_first,
                             const int* row_len, const int* row_start, const int* row_slots, int num_rows, float* out,
                             int writes, hipStream_t stream) {
  if (num_rows <= 0) return AS_OK;
  if (H <= 0 || D <= 0 || E <= 0 || D > 16 * SCAN_DPER || act < 0 || act > 2) return AS_BAD_SHAPE;
  int SL = 1;
  while (SL * SCAN_DPER < D) SL <<= 1;
  const int cols = WAVE / SL;
  dim3 grid((E + cols - 1) / cols, H, num_rows);
  if (grid.y > 65535 || grid.z > 65535) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    decay_scan_kernel<float><<<grid, 64, 0, stream>>>((const float*)proj, ld, q_off, k_off, v_off, H, D, E, act, k_scale, decay,
                                                      state, row_first, row_len, row_start, row_slots, out, SL, writes);
  else if (dtype == DT_BF16)
    decay_scan_kernel<bf16><<<grid, 64, 0, stream>>>((const bf16*)proj, ld, q_off, k_off, v_off, H, D, E, act, k_scale, decay,
                                                     state, row_first, row_len, row_start, row_slots, out, SL, writes);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- the output's norm and gate ---------------------------------------------------------------------------
// o [T, n] fp32 is normed in `groups` equal parts (a head each, or 1: all heads together; eps inside the root),
// multiplied by gain [n] (null: none) and by act(gate[t, g_off + i]); out [T, n] in the compute dtype.
template <typename T>
__global__ __launch_bounds__(256) void decay_finish_kernel(const float* __restrict__ o, int n, int groups, float eps,
                                                           const float* __restrict__ gain, const T* __restrict__ proj,
                                                           int ld, int g_off, int gate_act, T* __restrict__ out) {
  extern __shared__ float inv[];  // [groups]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
  const float* row = o + (size_t)t * n;
  const int gs = n / groups;
  if (groups == 1) {
    __shared__ float red[17];
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(row[i], row[i], ss);
    ss = block_sum(ss, red);
    if (threadIdx.x == 0) inv[0] = 1.0f / sqrtf(ss / (float)n + eps);
  } else {
    for (int g = wave; g < groups; g += waves) {
      float ss = 0.f;
      for (int i = lane; i < gs; i += WAVE) ss = fmaf(row[g * gs + i], row[g * gs + i], ss);
      ss = wave_sum(ss);
      if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)gs + eps);
    }
  }
  __syncthreads();
  const T* gate = proj + (size_t)t * ld + g_off;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = row[i] * inv[i / gs];
    if (gain) v *= gain[i];
    out[(size_t)t * n + i] = from_f32<T>(v * apply_act(to_f32(gate[i]), gate_act));
  }
}

extern "C" int as_decay_finish(const float* o, int n, int groups, float eps, const float* gain, const void* proj,
                               int dtype, int ld, int g_off, int gate_act, void* out, int num_tokens,
                               hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (n <= 0 || groups <= 0 || n % groups || groups > 8192 || gate_act < 0 || gate_act > 2) return AS_BAD_SHAPE;
  const size_t lds = (size_t)groups * sizeof(float);
  if (dtype == DT_F32)
    decay_finish_kernel<float><<<num_tokens, 256, lds, stream>>>(o, n, groups, eps, gain, (const float*)proj, ld, g_off, gate_act, (float*)out);
  else if (dtype == DT_BF16)
    decay_finish_kernel<bf16><<<num_tokens, 256, lds, stream>>>(o, n, groups, eps, gain, (const bf16*)proj, ld, g_off, gate_act, (bf16*)out);
  else return AS_BAD_DTYPE;
  return launch_status();
}
