// Linear attention with a fixed decay per head: a state S [D, E] per head and request,
//
//   S_t = lam_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
//
// with q, k [D] and v [E] columns of one input product (an activation and a factor applied as they are read).
// The state is fp32 and lives in a slot per request; a row that starts its sequence starts from zero whatever its
// slot holds, a later row goes on from what the row before left.  Everything after the products is fp32.
//
//   decay_scan    token by token: a lane keeps a slice of one column of the state in registers for all of a row's tokens
//   decay_step    a step of single tokens: the state read and written in whole lines (keys of up to 128, values in fours)
//   decay_chunks  32 tokens at a time as four fp32 products on the matrix cores (keys of up to 128 coordinates)
//   decay_finish  o normed in groups (per head, or all heads together) with an optional gain, times act(gate)
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

#define ACT_NONE 0
#define ACT_SILU 1
#define ACT_SIGMOID 2

__device__ __forceinline__ float apply_act(float v, int act) {
  if (act == ACT_SILU) return v / (1.0f + expf(-v));
  if (act == ACT_SIGMOID) return 1.0f / (1.0f + expf(-v));
  return v;
}

// The same for inputs that arrive in bfloat16: the hardware's exponential and reciprocal (an ulp or two, far below
// what the inputs' own rounding left), a third of the instructions.
template <typename T> __device__ __forceinline__ float act_of(float v, int act) { return apply_act(v, act); }
template <> __device__ __forceinline__ float act_of<bf16>(float v, int act) {
  if (act == ACT_NONE) return v;
  const float s = __builtin_amdgcn_rcpf(1.0f + __expf(-v));
  return act == ACT_SILU ? v * s : s;
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

// ---- one token a row (a decode step) ------------------------------------------------------------------------
// A step of single tokens is the state read once and written once: the wave's loads are whole 128-byte lines.  A
// lane owns four neighbouring columns e of sixteen rows d of one head's state (eight lanes a line of 32 columns,
// eight slices of d, whose partial sums meet by lane swaps).  Needs D <= 128 and E % 4 == 0.
#define STEP_DPER 16

template <typename T>
__global__ __launch_bounds__(64) void decay_step_kernel(const T* __restrict__ proj, int ld, int q_off, int k_off,
                                                        int v_off, int H, int D, int E, int act, float k_scale,
                                                        const float* __restrict__ decay, float* __restrict__ state,
                                                        const int* __restrict__ row_first,
                                                        const int* __restrict__ row_start,
                                                        const int* __restrict__ row_slots, float* __restrict__ out,
                                                        int writes) {
  const int lane = threadIdx.x, quad = lane & 7, sl = lane >> 3;
  const int e = blockIdx.x * 32 + 4 * quad, h = blockIdx.y, r = blockIdx.z;
  const bool live = e < E;  // E % 4 == 0: a lane's four columns are all there or none
  const int t = row_first[r], slot = row_slots[r];
  const float lam = decay[h];
  const int d0 = sl * STEP_DPER;
  float* kept = slot >= 0 ? state + (((size_t)slot * H + h) * D) * E : nullptr;
  const bool resume = kept && row_start[r] > 0;
  float S[STEP_DPER][4];
#pragma unroll
  for (int i = 0; i < STEP_DPER; ++i) {
    if (resume && live && d0 + i < D) load4(kept + (size_t)(d0 + i) * E + e, S[i]);
    else S[i][0] = S[i][1] = S[i][2] = S[i][3] = 0.f;
  }
  const T* row = proj + (size_t)t * ld;
  float q[STEP_DPER], k[STEP_DPER], v[4];
#pragma unroll
  for (int i = 0; i < STEP_DPER; ++i) {
    const bool in = d0 + i < D;
    q[i] = in ? to_f32(row[q_off + h * D + d0 + i]) : 0.f;
    k[i] = in ? to_f32(row[k_off + h * D + d0 + i]) : 0.f;
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) v[c] = live ? apply_act(to_f32(row[v_off + h * E + e + c]), act) : 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < STEP_DPER; ++i) {
    const float qa = apply_act(q[i], act), ka = apply_act(k[i], act) * k_scale;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      S[i][c] = fmaf(lam, S[i][c], ka * v[c]);
      acc[c] = fmaf(S[i][c], qa, acc[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c)
    for (int off = 8; off < WAVE; off <<= 1) acc[c] += __shfl_xor(acc[c], off, WAVE);
  if (live && sl == 0) store4(out + ((size_t)t * H + h) * E + e, acc);
  if (kept && writes && live) {
#pragma unroll
    for (int i = 0; i < STEP_DPER; ++i)
      if (d0 + i < D) store4(kept + (size_t)(d0 + i) * E + e, S[i]);
  }
}

extern "C" int as_decay_step(const void* proj, int dtype, int ld, int q_off, int k_off, int v_off, int H, int D, int E,
                             int act, float k_scale, const float* decay, float* state, const int* row_first,
                             const int* row_start, const int* row_slots, int num_rows, float* out, int writes,
                             hipStream_t stream) {
  if (num_rows <= 0) return AS_OK;
  if (H <= 0 || D <= 0 || E <= 0 || D > 8 * STEP_DPER || E % 4 || act < 0 || act > 2) return AS_BAD_SHAPE;
  dim3 grid((E + 31) / 32, H, num_rows);
  if (grid.y > 65535 || grid.z > 65535) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    decay_step_kernel<float><<<grid, 64, 0, stream>>>((const float*)proj, ld, q_off, k_off, v_off, H, D, E, act, k_scale, decay,
                                                      state, row_first, row_start, row_slots, out, writes);
  else if (dtype == DT_BF16)
    decay_step_kernel<bf16><<<grid, 64, 0, stream>>>((const bf16*)proj, ld, q_off, k_off, v_off, H, D, E, act, k_scale, decay,
                                                     state, row_first, row_start, row_slots, out, writes);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- a row's tokens in chunks, on the matrix cores in fp32 ---------------------------------------------------
// Over a chunk of n <= 32 tokens that starts from the state S (token t counts from 0 within the chunk):
//
//   o_t = lam^(t+1) S^T q_t + sum_(j <= t) lam^(t-j) (q_t . k_j) v_j          S' = lam^n S + sum_j lam^(n-1-j) k_j v_j^T
//
// which is four products: A = Q K^T (masked and weighed), A V, Q S and K^T V, all of fp32 operands with fp32 sums
// (v_mfma_f32_32x32x2f32).  grid (column groups of 32, heads, rows), four waves a workgroup.  Wave w keeps rows
// 32 w .. 32 w + 31 of the state's 32 columns in its accumulator registers from the row's first token to its last,
// sums A and o over the same 32 key coordinates, and the waves' parts meet in LDS.  An accumulator register i of
// lane l is element (row 8 (i / 4) + 4 (l / 32) + i % 4, column l % 32); as the second operand of the next product
// it stands for exactly that row, so the state never leaves its registers.
#define CHUNK 32
#define CHUNK_DP 128  // keys are padded with zeros to this width: four waves of 32 coordinates
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <typename T>
__global__ __launch_bounds__(256) void decay_chunk_kernel(const T* __restrict__ proj, int ld, int q_off, int k_off,
                                                         int v_off, int H, int D, int E, int act, float k_scale,
                                                         const float* __restrict__ decay, float* __restrict__ state,
                                                         const int* __restrict__ row_first,
                                                         const int* __restrict__ row_len,
                                                         const int* __restrict__ row_start,
                                                         const int* __restrict__ row_slots, float* __restrict__ out,
                                                         int writes) {
  __shared__ float Qs[CHUNK][CHUNK_DP + 1];
  __shared__ float Ks[CHUNK][CHUNK_DP + 1];
  __shared__ float Vs[CHUNK][CHUNK + 1];
  __shared__ float Part[4][CHUNK][CHUNK + 1];
  __shared__ float As[CHUNK][CHUNK + 1];
  __shared__ float pw[CHUNK + 1];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, col = lane & 31, half = lane >> 5;
  const int e0 = blockIdx.x * CHUNK, h = blockIdx.y, r = blockIdx.z;
  const int first = row_first[r], len = row_len[r], slot = row_slots[r];
  const float lam = decay[h];
  float* kept = slot >= 0 ? state + (((size_t)slot * H + h) * D) * E : nullptr;
  const bool resume = kept && row_start[r] > 0;
  const bool e_live = e0 + col < E;
  if (tid <= CHUNK) pw[tid] = powf(lam, (float)tid);
  floatx16 S;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int d = 32 * w + 8 * (i / 4) + 4 * half + i % 4;
    S[i] = (resume && e_live && d < D) ? kept[(size_t)d * E + e0 + col] : 0.f;
  }
  // A chunk's inputs are asked for a chunk ahead and wait in registers as they were projected, so that the loads
  // run under the products of the chunk before.
  constexpr int QK_EACH = CHUNK * CHUNK_DP / 256, V_EACH = CHUNK * CHUNK / 256;
  T q_next[QK_EACH], k_next[QK_EACH], v_next[V_EACH];
  auto fetch = [&](int c0) {
    const int n = min(CHUNK, len - c0);
#pragma unroll
    for (int it = 0; it < QK_EACH; ++it) {
      const int idx = tid + 256 * it, t = idx / CHUNK_DP, d = idx % CHUNK_DP;
      const bool in = t < n && d < D;
      const T* row = proj + (size_t)(first + c0 + (in ? t : 0)) * ld + h * D + (in ? d : 0);
      q_next[it] = in ? row[q_off] : from_f32<T>(0.f);
      k_next[it] = in ? row[k_off] : from_f32<T>(0.f);
    }
#pragma unroll
    for (int it = 0; it < V_EACH; ++it) {
      const int idx = tid + 256 * it, t = idx / CHUNK, e = idx % CHUNK;
      const bool in = t < n && e0 + e < E;
      v_next[it] = in ? proj[(size_t)(first + c0 + t) * ld + v_off + h * E + e0 + e] : from_f32<T>(0.f);
    }
  };
  if (len > 0) fetch(0);
  for (int c0 = 0; c0 < len; c0 += CHUNK) {
    const int n = min(CHUNK, len - c0);
    __syncthreads();  // the chunk before has been read (and pw written)
#pragma unroll
    for (int it = 0; it < QK_EACH; ++it) {
      const int idx = tid + 256 * it, t = idx / CHUNK_DP, d = idx % CHUNK_DP;
      const bool in = t < n && d < D;
      Qs[t][d] = in ? act_of<T>(to_f32(q_next[it]), act) : 0.f;
      Ks[t][d] = in ? act_of<T>(to_f32(k_next[it]), act) * k_scale : 0.f;
    }
#pragma unroll
    for (int it = 0; it < V_EACH; ++it) {
      const int idx = tid + 256 * it, t = idx / CHUNK, e = idx % CHUNK;
      Vs[t][e] = (t < n && e0 + e < E) ? act_of<T>(to_f32(v_next[it]), act) : 0.f;
    }
    if (c0 + CHUNK < len) fetch(c0 + CHUNK);
    __syncthreads();
    // A = Q K^T over this wave's 32 coordinates
    floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = 32 * w + 8 * (i / 4) + 4 * half + i % 4;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(Qs[col][d], Ks[col][d], acc, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) Part[w][8 * (i / 4) + 4 * half + i % 4][col] = acc[i];
    __syncthreads();
    for (int idx = tid; idx < CHUNK * CHUNK; idx += 256) {
      const int t = idx / CHUNK, j = idx % CHUNK;
      const float a = (Part[0][t][j] + Part[1][t][j]) + (Part[2][t][j] + Part[3][t][j]);
      As[t][j] = j <= t ? a * pw[t - j] : 0.f;
    }
    __syncthreads();
    // o = A V over this wave's 8 tokens, + lam^(t+1) Q S over its 32 coordinates
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int j = 8 * w + 2 * s + half;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[col][j], Vs[j][col], acc, 0, 0, 0);
    }
    const float grow = pw[col + 1];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = 32 * w + 8 * (i / 4) + 4 * half + i % 4;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(Qs[col][d] * grow, S[i], acc, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) Part[w][8 * (i / 4) + 4 * half + i % 4][col] = acc[i];
    // S = lam^n S + K^T V, key j weighed by lam^(n-1-j)
    const float shrink = pw[n];
#pragma unroll
    for (int i = 0; i < 16; ++i) S[i] *= shrink;
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      const int j = 2 * s + half;
      const float kw = j < n ? Ks[j][32 * w + col] * pw[n - 1 - j] : 0.f;
      S = __builtin_amdgcn_mfma_f32_32x32x2f32(kw, Vs[j][col], S, 0, 0, 0);
    }
    __syncthreads();
    for (int idx = tid; idx < CHUNK * CHUNK; idx += 256) {
      const int t = idx / CHUNK, e = idx % CHUNK;
      if (t < n && e0 + e < E)
        out[((size_t)(first + c0 + t) * H + h) * E + e0 + e] = (Part[0][t][e] + Part[1][t][e]) + (Part[2][t][e] + Part[3][t][e]);
    }
  }
  if (kept && writes && e_live) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = 32 * w + 8 * (i / 4) + 4 * half + i % 4;
      if (d < D) kept[(size_t)d * E + e0 + col] = S[i];
    }
  }
}

extern "C" int as_decay_chunks(const void* proj, int dtype, int ld, int q_off, int k_off, int v_off, int H, int D, int E,
                               int act, float k_scale, const float* decay, float* state, const int* row_first,
                               const int* row_len, const int* row_start, const int* row_slots, int num_rows, float* out,
                               int writes, hipStream_t stream) {
  if (num_rows <= 0) return AS_OK;
  if (H <= 0 || D <= 0 || E <= 0 || D > CHUNK_DP || act < 0 || act > 2) return AS_BAD_SHAPE;
  dim3 grid((E + CHUNK - 1) / CHUNK, H, num_rows);
  if (grid.y > 65535 || grid.z > 65535) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    decay_chunk_kernel<float><<<grid, 256, 0, stream>>>((const float*)proj, ld, q_off, k_off, v_off, H, D, E, act, k_scale, decay,
                                                        state, row_first, row_len, row_start, row_slots, out, writes);
  else if (dtype == DT_BF16)
    decay_chunk_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)proj, ld, q_off, k_off, v_off, H, D, E, act, k_scale, decay,
                                                       state, row_first, row_len, row_start, row_slots, out, writes);
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
  const bool by_four = gs % 4 == 0 && ld % 4 == 0 && g_off % 4 == 0;  // every row and group starts on 16 (8) bytes
  if (groups == 1) {
    __shared__ float red[17];
    float ss = 0.f;
    if (by_four) {
      for (int i = 4 * threadIdx.x; i < n; i += 4 * blockDim.x) {
        float v[4];
        load4(row + i, v);
#pragma unroll
        for (int c = 0; c < 4; ++c) ss = fmaf(v[c], v[c], ss);
      }
    } else {
      for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(row[i], row[i], ss);
    }
    ss = block_sum(ss, red);
    if (threadIdx.x == 0) inv[0] = 1.0f / sqrtf(ss / (float)n + eps);
  } else {
    for (int g = wave; g < groups; g += waves) {
      float ss = 0.f;
      if (by_four) {
        for (int i = 4 * lane; i < gs; i += 4 * WAVE) {
          float v[4];
          load4(row + g * gs + i, v);
#pragma unroll
          for (int c = 0; c < 4; ++c) ss = fmaf(v[c], v[c], ss);
        }
      } else {
        for (int i = lane; i < gs; i += WAVE) ss = fmaf(row[g * gs + i], row[g * gs + i], ss);
      }
      ss = wave_sum(ss);
      if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)gs + eps);
    }
  }
  __syncthreads();
  const T* gate = proj + (size_t)t * ld + g_off;
  if (by_four) {
    for (int i = 4 * threadIdx.x; i < n; i += 4 * blockDim.x) {
      float v[4], gt[4], gn[4] = {1.f, 1.f, 1.f, 1.f};
      load4(row + i, v);
      load4(gate + i, gt);
      if (gain) load4(gain + i, gn);
      const float scale = inv[i / gs];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        float r = v[c] * scale;
        if (gain) r *= gn[c];
        v[c] = r * apply_act(gt[c], gate_act);
      }
      store4(out + (size_t)t * n + i, v);
    }
    return;
  }
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
