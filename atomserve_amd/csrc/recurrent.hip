// Mixers that carry a fixed-size state from token to token: short causal convolutions, the gated
// delta rule and the gated linear recurrence.  Everything that enters a recurrence (decays, step
// sizes, gates, unit norms, the state itself) is fp32 in both precisions; only what the matrix
// products hand over (T) and the activations handed on to the next product are bf16 when serving.
//
// A step's rows are described as everywhere else: tok_row [T] (the row of a token), and per row its
// first flat token, its length, the position of its first token and its slot in the state tables.  A
// row that starts at position 0 starts from a zero state whatever its slot holds (slots are used
// again); a portion of a prompt goes on from what the portion before left.  State tables are fp32
// [slots, ...]; a row's state is written back only when `writes`.
#include "common.h"

#define CONV_MAX_TAPS 8

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float gelu_tanhf_(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---- short causal convolution per channel ------------------------------------------------------
// in [T, ld]: the C channels start at column col0; in_bias [C] (or none) is added to every input that
// exists (the zeros before a sequence stay zeros).  w [C, taps], the last column multiplying the
// current token; bias [C] or none; act 1: silu.  history [slots, taps - 1, C]: the inputs of the last
// taps - 1 tokens before the row, oldest first.  out fp32 [T, C].
template <typename T, typename W>
__global__ void short_conv_kernel(const T* __restrict__ in, int ld, int col0, int C, const W* __restrict__ in_bias,
                                  const W* __restrict__ w, const W* __restrict__ bias, int taps, int act,
                                  const float* __restrict__ history, const int* __restrict__ tok_row,
                                  const int* __restrict__ row_first, const int* __restrict__ row_start,
                                  const int* __restrict__ row_slots, float* __restrict__ out) {
  const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r = tok_row ? tok_row[t] : t;
  const int first = row_first[r], j = t - first;
  const bool carried = row_start[r] > 0 && row_slots[r] >= 0;
  const float* old = history + (size_t)(carried ? row_slots[r] : 0) * (taps - 1) * C;
  const float ib = in_bias ? to_f32(in_bias[c]) : 0.f;
  float acc = 0.f;
  for (int i = 0; i < taps; ++i) {
    const int src = j - (taps - 1 - i);
    float v = 0.f;
    if (src >= 0) v = to_f32(in[(size_t)(first + src) * ld + col0 + c]) + ib;
    else if (carried) v = old[(size_t)(taps - 1 + src) * C + c];
    acc = fmaf(to_f32(w[(size_t)c * taps + i]), v, acc);
  }
  if (bias) acc += to_f32(bias[c]);
  out[(size_t)t * C + c] = act == 1 ? siluf_(acc) : acc;
}

// After the convolution: the history of every row moves on by the row's tokens.
template <typename T, typename W>
__global__ void conv_history_kernel(const T* __restrict__ in, int ld, int col0, int C, const W* __restrict__ in_bias,
                                    int taps, float* __restrict__ history, const int* __restrict__ row_first,
                                    const int* __restrict__ row_len, const int* __restrict__ row_start,
                                    const int* __restrict__ row_slots) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C || row_slots[r] < 0) return;
  const int first = row_first[r], len = row_len[r], keep = taps - 1;
  float* mine = history + (size_t)row_slots[r] * keep * C;
  const bool carried = row_start[r] > 0;
  const float ib = in_bias ? to_f32(in_bias[c]) : 0.f;
  float fresh[CONV_MAX_TAPS];
  for (int h = 0; h < keep; ++h) {
    const int src = len - keep + h;  // among the row's tokens; negative: among the old history
    if (src >= 0) fresh[h] = to_f32(in[(size_t)(first + src) * ld + col0 + c]) + ib;
    else fresh[h] = carried ? mine[(size_t)(keep + src) * C + c] : 0.f;
  }
  for (int h = 0; h < keep; ++h) mine[(size_t)h * C + c] = fresh[h];
}

// A decode step (every row one token: token t is row t): the convolution and the history's move in one
// kernel.  A thread owns a channel of a row, so it reads the old inputs before it writes the new ones.
template <typename T, typename W>
__global__ void short_conv_step_kernel(const T* __restrict__ in, int ld, int col0, int C, const W* __restrict__ in_bias,
                                       const W* __restrict__ w, const W* __restrict__ bias, int taps, int act,
                                       float* __restrict__ history, const int* __restrict__ row_start,
                                       const int* __restrict__ row_slots, int writes, float* __restrict__ out) {
  const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int keep = taps - 1, slot = row_slots[t];
  const bool carried = row_start[t] > 0 && slot >= 0;
  float* mine = history + (size_t)(slot < 0 ? 0 : slot) * keep * C;
  float seen[CONV_MAX_TAPS];
  for (int i = 0; i < keep; ++i) seen[i] = carried ? mine[(size_t)i * C + c] : 0.f;
  seen[keep] = to_f32(in[(size_t)t * ld + col0 + c]) + (in_bias ? to_f32(in_bias[c]) : 0.f);
  float acc = 0.f;
  for (int i = 0; i < taps; ++i) acc = fmaf(to_f32(w[(size_t)c * taps + i]), seen[i], acc);
  if (bias) acc += to_f32(bias[c]);
  out[(size_t)t * C + c] = act == 1 ? siluf_(acc) : acc;
  if (writes && slot >= 0)
    for (int i = 0; i < keep; ++i) mine[(size_t)i * C + c] = seen[i + 1];
}

extern "C" int as_short_conv(const void* in, int dtype, int ld, int col0, int C, const void* in_bias, const void* w,
                             const void* bias, int w_dtype, int taps, int act, float* history, const int* tok_row,
                             const int* row_first, const int* row_len, const int* row_start, const int* row_slots,
                             float* out, int num_tokens, int num_rows, int writes, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (C <= 0 || taps < 1 || taps > CONV_MAX_TAPS || ld < col0 + C || num_rows <= 0) return AS_BAD_SHAPE;
  const int threads = C >= 256 ? 256 : 64;
  dim3 grid(num_tokens, (C + threads - 1) / threads), rows_grid(num_rows, (C + threads - 1) / threads);
  if (grid.y > 65535) return AS_BAD_SHAPE;
#define LAUNCH(T, W)                                                                                              \
  do {                                                                                                            \
    if (!tok_row && num_rows == num_tokens) { /* every row one token */                                           \
      short_conv_step_kernel<T, W><<<grid, threads, 0, stream>>>((const T*)in, ld, col0, C, (const W*)in_bias,   \
                                                                 (const W*)w, (const W*)bias, taps, act, history, \
                                                                 row_start, row_slots, writes, out);             \
      break;                                                                                                      \
    }                                                                                                             \
    short_conv_kernel<T, W><<<grid, threads, 0, stream>>>((const T*)in, ld, col0, C, (const W*)in_bias,          \
                                                          (const W*)w, (const W*)bias, taps, act, history,       \
                                                          tok_row, row_first, row_start, row_slots, out);        \
    if (writes && taps > 1)                                                                                       \
      conv_history_kernel<T, W><<<rows_grid, threads, 0, stream>>>((const T*)in, ld, col0, C, (const W*)in_bias, \
                                                                   taps, history, row_first, row_len, row_start, \
                                                                   row_slots);                                    \
  } while (0)
  if (dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ---- gated delta rule ----------------------------------------------------------------------------
// Before the scan, per token: the query and key heads (G of them, `dim` wide, in qkv [T, C] at columns
// 0 and G * dim) become unit vectors, x / sqrt(sum(x^2) + 1e-6), the query also times dim^(-1/2); per
// value head beta = sigmoid(b) and the decay g = exp(-exp(A_log) * softplus(a + dt_bias)), with b and a
// taken from the projection's output proj [T, ld] at columns b_off and a_off.
template <typename T, typename W>
__global__ __launch_bounds__(256) void delta_prepare_kernel(float* __restrict__ qkv, int C, int G, int dim, int H,
                                                            const T* __restrict__ proj, int ld, int b_off, int a_off,
                                                            const W* __restrict__ a_log, const W* __restrict__ dt_bias,
                                                            float* __restrict__ beta, float* __restrict__ decay) {
  // a workgroup of four waves per token and four heads (blockIdx.y), so that a decode step's few tokens are many workgroups
  const int t = blockIdx.x, lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
  float* row = qkv + (size_t)t * C;
  for (int head = blockIdx.y * waves + wave; head < 2 * G; head += gridDim.y * waves) {
    float* x = row + (size_t)head * dim;  // query heads first, then key heads
    float ss = 0.f;
    for (int d = lane; d < dim; d += WAVE) ss += x[d] * x[d];
    ss = wave_sum(ss);
    float f = 1.0f / sqrtf(ss + 1e-6f);
    if (head < G) f *= 1.0f / sqrtf((float)dim);
    for (int d = lane; d < dim; d += WAVE) x[d] *= f;
  }
  for (int h = blockIdx.y * blockDim.x + threadIdx.x; h < H; h += gridDim.y * blockDim.x) {
    const float b = to_f32(proj[(size_t)t * ld + b_off + h]), a = to_f32(proj[(size_t)t * ld + a_off + h]);
    beta[(size_t)t * H + h] = sigmoidf_(b);
    decay[(size_t)t * H + h] = expf(-expf(to_f32(a_log[h])) * softplusf_(a + to_f32(dt_bias[h])));
  }
}

extern "C" int as_delta_prepare(float* qkv, int C, int G, int dim, int H, const void* proj, int dtype, int ld, int b_off,
                                int a_off, const void* a_log, const void* dt_bias, int w_dtype, float* beta,
                                float* decay, int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (G <= 0 || dim <= 0 || H <= 0 || C < 2 * G * dim) return AS_BAD_SHAPE;
  const int across = num_tokens >= 512 ? 1 : (2 * G + 3) / 4 > 64 ? 64 : (2 * G + 3) / 4;  // many tokens fill the GPU by themselves
  dim3 grid(num_tokens, across);
#define LAUNCH(T, W)                                                                                               \
  delta_prepare_kernel<T, W><<<grid, 256, 0, stream>>>(qkv, C, G, dim, H, (const T*)proj, ld, b_off, a_off,        \
                                                       (const W*)a_log, (const W*)dt_bias, beta, decay)
  if (dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// The scan.  Per head the state S [dim, vdim] moves on token by token:
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q     (o sees the token's own write)
// The columns of S never meet, so a wave owns CJ columns of one head of one row and keeps them in
// registers for all the row's tokens: lane = column * SL + slice, a slice being RPL rows of S
// (SL = 64 / CJ slices cover dim; the slices of a column are neighbouring lanes, whose partial sums
// meet through DPP moves within a row of 16 lanes, not through LDS).  With p = S_old^T k and r = S_old^T q, both taken in one pass over the
// old state:  u = beta (v - g p),  S_new = g S_old + k u^T,  o = g r + u (k . q).
// Keys and queries of DELTA_TB tokens at a time go through LDS: a round's loads (16 bytes a lane, all asked
// for together, with the lanes' own values, betas and decays) are in flight while the round before is
// worked on, so the chain of dependent steps is the arithmetic alone.
#define DELTA_TB 8
#define DELTA_STAGE 8  // 16-byte pieces a lane brings per pass of a round's staging
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
// The sum over SL neighbouring lanes (SL = 1, 2, 4, 8, 16), in every one of them: lane ^ 1, lane ^ 2, then
// the mirror image within eight lanes (which lies in the other four) and within sixteen (the other eight).
template <int SL> __device__ __forceinline__ float slices_sum(float v) {
  if (SL >= 2) v += dpp_move<0xB1>(v);   // quad_perm [1, 0, 3, 2]
  if (SL >= 4) v += dpp_move<0x4E>(v);   // quad_perm [2, 3, 0, 1]
  if (SL >= 8) v += dpp_move<0x141>(v);  // row_half_mirror
  if (SL >= 16) v += dpp_move<0x140>(v);  // row_mirror
  return v;
}

// MODE 0: the rule above.  MODE 1: a decay per head and key channel, chan [T, H, dim], on the rows of S:
//   S <- diag(g) S, then as above; with p = S_old^T (g k), r = S_old^T (g q): u = beta (v - p), S_new = g S_old + k u^T,
//   o = r + u (k . q).  The decays of a token go through LDS beside its key and query.
// MODE 2: a matrix memory with exponential gates: `beta` holds the logarithm of the input gate i, `decay` that of the
//   forget gate f, [T, H]; beside S the head keeps a normaliser n [dim] and a running maximum m (0 at the start):
//   m' = max(f + m, i);  S' = e^(f + m - m') S + e^(i - m') k v^T;  n' = e^(f + m - m') n + e^(i - m') k;
//   o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6).  norm_state [slots, H, dim], max_state [slots, H].
template <int RPL, int SL, int MODE>
__global__ __launch_bounds__(64) void delta_scan_kernel(const float* __restrict__ qkv, int C, int G, int dim, int H,
                                                        int vdim, const float* __restrict__ beta,
                                                        const float* __restrict__ decay,
                                                        const float* __restrict__ chan, float* __restrict__ state,
                                                        float* __restrict__ norm_state, float* __restrict__ max_state,
                                                        const int* __restrict__ row_first,
                                                        const int* __restrict__ row_len,
                                                        const int* __restrict__ row_start,
                                                        const int* __restrict__ row_slots, int writes,
                                                        float* __restrict__ out) {
  constexpr int NV = MODE == 1 ? 3 : 2;  // vectors of a token that go through LDS: key, query (, decays)
  extern __shared__ __attribute__((aligned(16))) float lds[];  // [DELTA_TB][NV][dimp], dimp = SL * RPL
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  constexpr int CJ = WAVE / SL;
  const int col = lane / SL, slice = lane % SL;
  constexpr int dimp = SL * RPL;
  const int j = blockIdx.z * CJ + col;
  const bool live = j < vdim;
  const int g = h / (H / G);
  const int first = row_first[r], len = row_len[r], slot = row_slots[r];
  const int i0 = slice * RPL;
  float S[RPL];
  float N[MODE == 2 ? RPL : 1];
  float m_run = 0.f;
  float* mine = state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * dim * vdim;
  const bool carried = row_start[r] > 0 && slot >= 0;
#pragma unroll
  for (int i = 0; i < RPL; ++i) S[i] = (carried && live && i0 + i < dim) ? mine[(size_t)(i0 + i) * vdim + j] : 0.f;
  if (MODE == 2) {
    const float* n_mine = norm_state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * dim;
#pragma unroll
    for (int i = 0; i < RPL; ++i) N[i] = (carried && i0 + i < dim) ? n_mine[i0 + i] : 0.f;
    m_run = carried ? max_state[(size_t)slot * H + h] : 0.f;
  }
  const int q_col = g * dim, k_col = (G + g) * dim, v_col = 2 * G * dim + h * vdim;
  // a round's keys and queries as 16-byte pieces: piece -> (token, which vector, four coordinates)
  const int quads = dimp >> 2, per_token = NV * quads, pieces = DELTA_TB * per_token;
  const int passes = (pieces + WAVE * DELTA_STAGE - 1) / (WAVE * DELTA_STAGE);
  float4 stage[DELTA_STAGE];
  float vj[DELTA_TB], bt[DELTA_TB], gt[DELTA_TB];
  const bool whole = ((dim | C) & 3) == 0;  // every key and query starts on 16 bytes
  auto fetch = [&](int t0, int pass) {
    const int nt = min(DELTA_TB, len - t0);
#pragma unroll
    for (int u = 0; u < DELTA_STAGE; ++u) {
      const int piece = (pass * DELTA_STAGE + u) * WAVE + lane;
      const int tt = piece / per_token, rest = piece - tt * per_token, which = rest / quads, i = (rest - which * quads) * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (tt < nt && i < dim && piece < pieces) {
        const size_t t = (size_t)(first + t0 + tt);
        const float* src = which == 2 ? chan + (t * H + h) * dim + i : qkv + t * C + (which ? q_col : k_col) + i;
        if (whole) {
          v = *reinterpret_cast<const float4*>(src);
        } else {  // widths that are no multiples of 4: value by value
          v.x = src[0];
          if (i + 1 < dim) v.y = src[1];
          if (i + 2 < dim) v.z = src[2];
          if (i + 3 < dim) v.w = src[3];
        }
      }
      stage[u] = v;
    }
  };
  auto fetch_own = [&](int t0) {
    const int nt = min(DELTA_TB, len - t0);
#pragma unroll
    for (int tt = 0; tt < DELTA_TB; ++tt) {
      const size_t t = (size_t)first + t0 + (tt < nt ? tt : 0);
      vj[tt] = live ? qkv[t * C + v_col + j] : 0.f;
      bt[tt] = beta[t * H + h];
      gt[tt] = MODE == 1 ? 1.f : decay[t * H + h];
    }
  };
  auto put = [&](int pass) {
#pragma unroll
    for (int u = 0; u < DELTA_STAGE; ++u) {
      const int piece = (pass * DELTA_STAGE + u) * WAVE + lane;
      if (piece < pieces) *reinterpret_cast<float4*>(lds + (size_t)piece * 4) = stage[u];
    }
  };
  if (len > 0) {
    fetch(0, 0);
    fetch_own(0);
  }
  for (int t0 = 0; t0 < len; t0 += DELTA_TB) {
    const int nt = min(DELTA_TB, len - t0);
    __syncthreads();  // the round before has been read
    put(0);
    for (int pass = 1; pass < passes; ++pass) {  // heads wider than a pass brings: the rest, pass by pass
      fetch(t0, pass);
      put(pass);
    }
    float v_now[DELTA_TB], b_now[DELTA_TB], g_now[DELTA_TB];
#pragma unroll
    for (int tt = 0; tt < DELTA_TB; ++tt) { v_now[tt] = vj[tt]; b_now[tt] = bt[tt]; g_now[tt] = gt[tt]; }
    __syncthreads();
    if (t0 + DELTA_TB < len) {  // in flight while this round is worked on
      fetch(t0 + DELTA_TB, 0);
      fetch_own(t0 + DELTA_TB);
    }
#pragma unroll
    for (int tt = 0; tt < DELTA_TB; ++tt) {
      if (tt < nt) {
        // this lane's slice of the token's key and query, 16 bytes at a time (i0 is a multiple of 8)
        const float4* k4 = reinterpret_cast<const float4*>(lds + tt * NV * dimp + i0);
        const float4* q4 = reinterpret_cast<const float4*>(lds + tt * NV * dimp + dimp + i0);
        float kk[RPL], qq[RPL];
#pragma unroll
        for (int i = 0; i < RPL / 4; ++i) {
          const float4 a = k4[i], b = q4[i];
          kk[4 * i] = a.x; kk[4 * i + 1] = a.y; kk[4 * i + 2] = a.z; kk[4 * i + 3] = a.w;
          qq[4 * i] = b.x; qq[4 * i + 1] = b.y; qq[4 * i + 2] = b.z; qq[4 * i + 3] = b.w;
        }
        if (MODE == 2) {
          const float fl = g_now[tt], il = b_now[tt];
          const float m_new = fmaxf(fl + m_run, il);
          const float keep = expf(fl + m_run - m_new), take = expf(il - m_new);
          m_run = m_new;
          const float tv = take * v_now[tt];
          float num = 0.f, nq = 0.f, num2 = 0.f, nq2 = 0.f;
#pragma unroll
          for (int i = 0; i < RPL; i += 2) {
            S[i] = fmaf(kk[i], tv, keep * S[i]);
            N[i] = fmaf(kk[i], take, keep * N[i]);
            num = fmaf(S[i], qq[i], num);
            nq = fmaf(N[i], qq[i], nq);
            S[i + 1] = fmaf(kk[i + 1], tv, keep * S[i + 1]);
            N[i + 1] = fmaf(kk[i + 1], take, keep * N[i + 1]);
            num2 = fmaf(S[i + 1], qq[i + 1], num2);
            nq2 = fmaf(N[i + 1], qq[i + 1], nq2);
          }
          num = slices_sum<SL>(num + num2);
          nq = slices_sum<SL>(nq + nq2);
          if (live && slice == 0)
            out[((size_t)(first + t0 + tt) * H + h) * vdim + j] = num / (fmaxf(fabsf(nq), expf(-m_new)) + 1e-6f);
          continue;
        }
        if (MODE == 1) {  // the decays act on the rows of the old state
          const float4* g4 = reinterpret_cast<const float4*>(lds + tt * NV * dimp + 2 * dimp + i0);
#pragma unroll
          for (int i = 0; i < RPL / 4; ++i) {
            const float4 a = g4[i];
            S[4 * i] *= a.x; S[4 * i + 1] *= a.y; S[4 * i + 2] *= a.z; S[4 * i + 3] *= a.w;
          }
        }
        float p = 0.f, rr = 0.f, kq = 0.f, p2 = 0.f, rr2 = 0.f, kq2 = 0.f;  // two chains each: half the dependent steps
#pragma unroll
        for (int i = 0; i < RPL; i += 2) {
          p = fmaf(S[i], kk[i], p);
          rr = fmaf(S[i], qq[i], rr);
          kq = fmaf(kk[i], qq[i], kq);
          p2 = fmaf(S[i + 1], kk[i + 1], p2);
          rr2 = fmaf(S[i + 1], qq[i + 1], rr2);
          kq2 = fmaf(kk[i + 1], qq[i + 1], kq2);
        }
        p = slices_sum<SL>(p + p2);
        rr = slices_sum<SL>(rr + rr2);
        kq = slices_sum<SL>(kq + kq2);
        const float gg = g_now[tt];
        const float u = b_now[tt] * (v_now[tt] - gg * p);
#pragma unroll
        for (int i = 0; i < RPL; ++i) S[i] = fmaf(kk[i], u, gg * S[i]);
        if (live && slice == 0) out[((size_t)(first + t0 + tt) * H + h) * vdim + j] = fmaf(gg, rr, u * kq);
      }
    }
  }
  if (writes && live && slot >= 0) {
#pragma unroll
    for (int i = 0; i < RPL; ++i)
      if (i0 + i < dim) mine[(size_t)(i0 + i) * vdim + j] = S[i];
  }
  if (MODE == 2 && writes && slot >= 0 && blockIdx.z == 0 && col == 0) {  // every column group keeps the same n and m: one writes
    float* n_mine = norm_state + ((size_t)slot * H + h) * dim;
#pragma unroll
    for (int i = 0; i < RPL; ++i)
      if (i0 + i < dim) n_mine[i0 + i] = N[i];
    if (slice == 0) max_state[(size_t)slot * H + h] = m_run;
  }
}

template <int MODE>
static int launch_delta_scan(const float* qkv, int C, int G, int dim, int H, int vdim, const float* beta,
                             const float* decay, const float* chan, float* state, float* norm_state, float* max_state,
                             const int* row_first, const int* row_len, const int* row_start, const int* row_slots,
                             int writes, float* out, int num_rows, int force_slices, hipStream_t stream) {
  if (num_rows <= 0) return AS_OK;
  if (G <= 0 || H <= 0 || H % G || dim <= 0 || vdim <= 0 || C < 2 * G * dim + H * vdim || H > 65535)
    return AS_BAD_SHAPE;
  if (dim > 16 * 64) return AS_BAD_SHAPE;  // sixteen slices of 64 rows
  int slices = 1;
  while ((dim + slices - 1) / slices > 64) slices *= 2;  // a lane keeps at most 64 rows of its column
  if (MODE == 2)  // the normaliser's rows lie beside the state's: half as many to a lane
    while ((dim + slices - 1) / slices > 32) slices *= 2;
  // few rows and heads: narrower column groups (more slices of fewer rows) until the waves fill the GPU
  while (slices < 16 && (dim + 2 * slices - 1) / (2 * slices) >= 8 &&
         (long)num_rows * H * ((vdim + WAVE / slices - 1) / (WAVE / slices)) < 8L * compute_units())
    slices *= 2;
  if (force_slices > 0) {  // measurements and tests: 1, 2, 4, 8 or 16 slices, if a lane's share then fits
    if ((force_slices & (force_slices - 1)) || force_slices > 16 || (dim + force_slices - 1) / force_slices > 64)
      return AS_BAD_SHAPE;
    slices = force_slices;
  }
  if (slices > 16) return AS_BAD_SHAPE;
  const int rows_per_lane = (dim + slices - 1) / slices;
  const int RPL = rows_per_lane <= 8 ? 8 : rows_per_lane <= 16 ? 16 : rows_per_lane <= 32 ? 32 : 64;
  const int CJ = WAVE / slices;
  dim3 grid(num_rows, H, (vdim + CJ - 1) / CJ);
  const size_t lds = (size_t)DELTA_TB * (MODE == 1 ? 3 : 2) * slices * RPL * sizeof(float);
  if (lds > 64 * 1024) return AS_BAD_SHAPE;
#define LAUNCH(R, SLV)                                                                                            \
  delta_scan_kernel<R, SLV, MODE><<<grid, 64, lds, stream>>>(qkv, C, G, dim, H, vdim, beta, decay, chan, state,   \
                                                             norm_state, max_state, row_first, row_len, row_start, \
                                                             row_slots, writes, out)
#define LAUNCH_SL(R)              \
  do {                            \
    if (slices == 1) LAUNCH(R, 1);      \
    else if (slices == 2) LAUNCH(R, 2); \
    else if (slices == 4) LAUNCH(R, 4); \
    else if (slices == 8) LAUNCH(R, 8); \
    else LAUNCH(R, 16);                 \
  } while (0)
  if (RPL == 8) LAUNCH_SL(8);
  else if (RPL == 16) LAUNCH_SL(16);
  else if (RPL == 32) LAUNCH_SL(32);
  else LAUNCH_SL(64);
#undef LAUNCH_SL
#undef LAUNCH
  return launch_status();
}

extern "C" int as_delta_scan(const float* qkv, int C, int G, int dim, int H, int vdim, const float* beta,
                             const float* decay, float* state, const int* row_first, const int* row_len,
                             const int* row_start, const int* row_slots, int writes, float* out, int num_rows,
                             int force_slices, hipStream_t stream) {
  return launch_delta_scan<0>(qkv, C, G, dim, H, vdim, beta, decay, nullptr, state, nullptr, nullptr, row_first, row_len,
                              row_start, row_slots, writes, out, num_rows, force_slices, stream);
}

// The same rule with a decay per head and key channel: chan [T, H, dim].
extern "C" int as_delta_scan_channels(const float* qkv, int C, int G, int dim, int H, int vdim, const float* beta,
                                      const float* chan, float* state, const int* row_first, const int* row_len,
                                      const int* row_start, const int* row_slots, int writes, float* out,
                                      int num_rows, int force_slices, hipStream_t stream) {
  if (!chan) return AS_BAD_SHAPE;
  return launch_delta_scan<1>(qkv, C, G, dim, H, vdim, beta, nullptr, chan, state, nullptr, nullptr, row_first, row_len,
                              row_start, row_slots, writes, out, num_rows, force_slices, stream);
}

// The matrix memory: qkv [T, C] holds H query heads (already times dim^(-1/2)), H key heads and H value heads.
extern "C" int as_memory_scan(const float* qkv, int C, int dim, int H, int vdim, const float* i_log, const float* f_log,
                              float* state, float* norm_state, float* max_state, const int* row_first,
                              const int* row_len, const int* row_start, const int* row_slots, int writes, float* out,
                              int num_rows, int force_slices, hipStream_t stream) {
  if (!norm_state || !max_state) return AS_BAD_SHAPE;
  return launch_delta_scan<2>(qkv, C, H, dim, H, vdim, i_log, f_log, nullptr, state, norm_state, max_state, row_first,
                              row_len, row_start, row_slots, writes, out, num_rows, force_slices, stream);
}

// After the scan: every head's output over its root mean square (over vdim, eps inside the root), times
// a weight (w [vdim] shared by the heads with w_stride 0, w [H, vdim] with w_stride vdim), times silu (gate_act 0)
// or sigmoid (1) of a gate projection's output (gate [T, ld] at g_off, laid out heads x vdim), times scale: the
// input of the output projection, act [T, ld_out] from column out_off on.
template <typename T, typename W>
__global__ __launch_bounds__(64) void delta_finish_kernel(const float* __restrict__ o, int H, int vdim,
                                                          const W* __restrict__ w, int w_stride, float eps,
                                                          const T* __restrict__ gate, int ld, int g_off, int gate_act,
                                                          float scale, T* __restrict__ act, int ld_out, int out_off) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* x = o + ((size_t)t * H + h) * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += WAVE) ss += x[d] * x[d];
  ss = wave_sum(ss);
  const float inv = scale / sqrtf(ss / (float)vdim + eps);
  for (int d = lane; d < vdim; d += WAVE) {
    const float z = to_f32(gate[(size_t)t * ld + g_off + h * vdim + d]);
    const float gv = gate_act == 1 ? sigmoidf_(z) : siluf_(z);
    act[(size_t)t * ld_out + out_off + h * vdim + d] = from_f32<T>(x[d] * inv * to_f32(w[(size_t)h * w_stride + d]) * gv);
  }
}

extern "C" int as_delta_finish(const float* o, int H, int vdim, const void* w, int w_dtype, int w_per_head, float eps,
                               const void* gate, int dtype, int ld, int g_off, int gate_act, float scale, void* act,
                               int ld_out, int out_off, int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || H > 65535 || vdim <= 0 || gate_act < 0 || gate_act > 1 || ld < g_off + H * vdim ||
      ld_out < out_off + H * vdim)
    return AS_BAD_SHAPE;
  dim3 grid(num_tokens, H);
  const int w_stride = w_per_head ? vdim : 0;
#define LAUNCH(T, W)                                                                                               \
  delta_finish_kernel<T, W><<<grid, 64, 0, stream>>>(o, H, vdim, (const W*)w, w_stride, eps, (const T*)gate, ld,  \
                                                     g_off, gate_act, scale, (T*)act, ld_out, out_off)
  if (dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// Before the scan with a decay per channel: unit vectors as in delta_prepare; beta = sigmoid(proj[t, b_off + h]);
// chan[t, h, d] = exp(-exp(a_log[h]) * softplus(steps[t, a_off + h * dim + d] + dt_bias[h * dim + d])), `steps` being
// the output of the step sizes' second projection, [T, ld_s].  a_log and dt_bias fp32.
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_channels_kernel(float* __restrict__ qkv, int C, int G, int dim, int H,
                                                                     const T* __restrict__ proj, int ld, int b_off,
                                                                     const T* __restrict__ steps, int ld_s, int a_off,
                                                                     const float* __restrict__ a_log,
                                                                     const float* __restrict__ dt_bias,
                                                                     float* __restrict__ beta, float* __restrict__ chan) {
  const int t = blockIdx.x, lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
  float* row = qkv + (size_t)t * C;
  for (int head = blockIdx.y * waves + wave; head < 2 * G; head += gridDim.y * waves) {
    float* x = row + (size_t)head * dim;  // query heads first, then key heads
    float ss = 0.f;
    for (int d = lane; d < dim; d += WAVE) ss += x[d] * x[d];
    ss = wave_sum(ss);
    float f = 1.0f / sqrtf(ss + 1e-6f);
    if (head < G) f *= 1.0f / sqrtf((float)dim);
    for (int d = lane; d < dim; d += WAVE) x[d] *= f;
  }
  for (int h = blockIdx.y * blockDim.x + threadIdx.x; h < H; h += gridDim.y * blockDim.x)
    beta[(size_t)t * H + h] = sigmoidf_(to_f32(proj[(size_t)t * ld + b_off + h]));
  const int HD = H * dim;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < HD; c += gridDim.y * blockDim.x) {
    const float a = to_f32(steps[(size_t)t * ld_s + a_off + c]);
    chan[(size_t)t * HD + c] = expf(-expf(a_log[c / dim]) * softplusf_(a + dt_bias[c]));
  }
}

extern "C" int as_delta_prepare_channels(float* qkv, int C, int G, int dim, int H, const void* proj, int dtype, int ld,
                                         int b_off, const void* steps, int ld_s, int a_off, const float* a_log,
                                         const float* dt_bias, float* beta, float* chan, int num_tokens,
                                         hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (G <= 0 || dim <= 0 || H <= 0 || C < 2 * G * dim || ld < b_off + H || ld_s < a_off + H * dim) return AS_BAD_SHAPE;
  int across = num_tokens >= 512 ? 1 : (H * dim + 255) / 256;
  if (across > 64) across = 64;
  dim3 grid(num_tokens, across);
  if (dtype == DT_F32)
    delta_prepare_channels_kernel<float><<<grid, 256, 0, stream>>>(qkv, C, G, dim, H, (const float*)proj, ld, b_off,
                                                                   (const float*)steps, ld_s, a_off, a_log, dt_bias,
                                                                   beta, chan);
  else if (dtype == DT_BF16)
    delta_prepare_channels_kernel<bf16><<<grid, 256, 0, stream>>>(qkv, C, G, dim, H, (const bf16*)proj, ld, b_off,
                                                                  (const bf16*)steps, ld_s, a_off, a_log, dt_bias, beta,
                                                                  chan);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// Before the scan of a matrix memory: proj [T, ld] holds H query heads at q_off, H key heads at k_off (`dim` wide) and
// H value heads at v_off (`vdim` wide), and the gates' logits at i_off and f_off [H].  qkv fp32 [T, 2 H dim + H vdim]
// receives the queries times dim^(-1/2), the keys and the values; i_log = cap tanh((z_i + b_i) / cap), f_log =
// logsigmoid(cap tanh((z_f + b_f) / cap)), both [T, H]; biases fp32 [H].
__device__ __forceinline__ float log_sigmoidf_(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T>
__global__ __launch_bounds__(256) void memory_prepare_kernel(const T* __restrict__ proj, int ld, int q_off, int k_off,
                                                             int v_off, int i_off, int f_off, int H, int dim, int vdim,
                                                             const float* __restrict__ i_bias,
                                                             const float* __restrict__ f_bias, float cap,
                                                             float* __restrict__ qkv, float* __restrict__ i_log,
                                                             float* __restrict__ f_log) {
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * ld;
  const int HD = H * dim, C = 2 * HD + H * vdim;
  const float qs = 1.0f / sqrtf((float)dim);
  float* dst = qkv + (size_t)t * C;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float v;
    if (c < HD) v = to_f32(row[q_off + c]) * qs;
    else if (c < 2 * HD) v = to_f32(row[k_off + c - HD]);
    else v = to_f32(row[v_off + c - 2 * HD]);
    dst[c] = v;
  }
  for (int h = blockIdx.y * blockDim.x + threadIdx.x; h < H; h += gridDim.y * blockDim.x) {
    const float zi = to_f32(row[i_off + h]) + i_bias[h], zf = to_f32(row[f_off + h]) + f_bias[h];
    i_log[(size_t)t * H + h] = cap * tanhf(zi / cap);
    f_log[(size_t)t * H + h] = log_sigmoidf_(cap * tanhf(zf / cap));
  }
}

extern "C" int as_memory_prepare(const void* proj, int dtype, int ld, int q_off, int k_off, int v_off, int i_off,
                                 int f_off, int H, int dim, int vdim, const float* i_bias, const float* f_bias,
                                 float cap, float* qkv, float* i_log, float* f_log, int num_tokens,
                                 hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (H <= 0 || dim <= 0 || vdim <= 0 || !(cap > 0.f) || ld < q_off + H * dim || ld < k_off + H * dim ||
      ld < v_off + H * vdim || ld < i_off + H || ld < f_off + H)
    return AS_BAD_SHAPE;
  int across = num_tokens >= 512 ? 1 : ((2 * dim + vdim) * H + 255) / 256;
  if (across > 64) across = 64;
  dim3 grid(num_tokens, across);
  if (dtype == DT_F32)
    memory_prepare_kernel<float><<<grid, 256, 0, stream>>>((const float*)proj, ld, q_off, k_off, v_off, i_off, f_off, H,
                                                           dim, vdim, i_bias, f_bias, cap, qkv, i_log, f_log);
  else if (dtype == DT_BF16)
    memory_prepare_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)proj, ld, q_off, k_off, v_off, i_off, f_off, H,
                                                          dim, vdim, i_bias, f_bias, cap, qkv, i_log, f_log);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// ---- gated linear recurrence ----------------------------------------------------------------------
// The gates.  u fp32 [T, width] is cut into `blocks` parts of bw channels; in part b
//   r = sigmoid(ra[b] u_b + ra_b[b]),  i = sigmoid(ri[b] u_b + ri_b[b])     (ra, ri [blocks, bw, bw], out x in)
//   a = exp(-c r softplus(lam));  a_out = a,  x_out = sqrt(1 - a^2) i u.
// A workgroup takes 64 tokens by 64 outputs of one part and a thread four by four of them for both gates;
// tokens and weights meet in LDS in pieces of 32 inputs, laid out input-major so that a thread reads its
// four tokens and its four outputs 16 bytes at a time; every output is one fma chain over its inputs in
// order, whatever shares the launch.
#define GATE_TT 64
#define GATE_TO 64
#define GATE_KC 32
template <typename W>
__global__ __launch_bounds__(256) void rglru_gates_kernel(const float* __restrict__ u, int width, int bw,
                                                          const W* __restrict__ ra, const W* __restrict__ ra_b,
                                                          const W* __restrict__ ri, const W* __restrict__ ri_b,
                                                          const W* __restrict__ lam, float c, float* __restrict__ a_out,
                                                          float* __restrict__ x_out, int num_tokens) {
  __shared__ __attribute__((aligned(16))) float us[GATE_KC][GATE_TT + 4];
  __shared__ __attribute__((aligned(16))) float wr[GATE_KC][GATE_TO + 4];
  __shared__ __attribute__((aligned(16))) float wi[GATE_KC][GATE_TO + 4];
  const int b = blockIdx.y, t0 = blockIdx.x * GATE_TT, o0 = blockIdx.z * GATE_TO;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // outputs o0 + 4 tx .., tokens t0 + 4 ty ..
  float accr[4][4] = {}, acci[4][4] = {};
  const W* rab = ra + (size_t)b * bw * bw;
  const W* rib = ri + (size_t)b * bw * bw;
  const int lk = threadIdx.x & 31, lrow = threadIdx.x >> 5;  // loads: input k0 + lk of rows lrow + 8 i
  for (int k0 = 0; k0 < bw; k0 += GATE_KC) {
    float uu[8], rr[8], ii[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = lrow + 8 * i, k = k0 + lk;
      uu[i] = (t0 + row < num_tokens && k < bw) ? u[(size_t)(t0 + row) * width + b * bw + k] : 0.f;
      const bool in = o0 + row < bw && k < bw;
      rr[i] = in ? to_f32(rab[(size_t)(o0 + row) * bw + k]) : 0.f;
      ii[i] = in ? to_f32(rib[(size_t)(o0 + row) * bw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      us[lk][lrow + 8 * i] = uu[i];
      wr[lk][lrow + 8 * i] = rr[i];
      wi[lk][lrow + 8 * i] = ii[i];
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < GATE_KC; ++kk) {
      const float4 u4 = *reinterpret_cast<const float4*>(&us[kk][4 * ty]);
      const float4 r4 = *reinterpret_cast<const float4*>(&wr[kk][4 * tx]);
      const float4 i4 = *reinterpret_cast<const float4*>(&wi[kk][4 * tx]);
      const float uv[4] = {u4.x, u4.y, u4.z, u4.w}, rv[4] = {r4.x, r4.y, r4.z, r4.w}, iv[4] = {i4.x, i4.y, i4.z, i4.w};
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int oo = 0; oo < 4; ++oo) {
          accr[tt][oo] = fmaf(rv[oo], uv[tt], accr[tt][oo]);
          acci[tt][oo] = fmaf(iv[oo], uv[tt], acci[tt][oo]);
        }
    }
  }
#pragma unroll
  for (int oo = 0; oo < 4; ++oo) {
    const int o = o0 + 4 * tx + oo;
    if (o >= bw) continue;
    const int ch = b * bw + o;
    const float rb = to_f32(ra_b[ch]), ib = to_f32(ri_b[ch]), sp = softplusf_(to_f32(lam[ch]));
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      const int t = t0 + 4 * ty + tt;
      if (t >= num_tokens) continue;
      const float rg = sigmoidf_(accr[tt][oo] + rb), ig = sigmoidf_(acci[tt][oo] + ib);
      const float log_a = -c * rg * sp;
      a_out[(size_t)t * width + ch] = expf(log_a);
      x_out[(size_t)t * width + ch] = sqrtf(-expm1f(2.0f * log_a)) * ig * u[(size_t)t * width + ch];
    }
  }
}

// The same for a few tokens (a decode step): the two matrices are streamed once.  Sixteen lanes share an
// output channel (a wave four channels): each takes four inputs in sixteen (16-byte loads, a row of the
// matrix read in whole lines), and their sums meet through DPP moves within the sixteen; eight tokens at a
// time.  Blocks whose rows do not start on 16 bytes are read value by value.
template <typename W>
__global__ __launch_bounds__(256) void rglru_gates_few_kernel(const float* __restrict__ u, int width, int bw,
                                                              const W* __restrict__ ra, const W* __restrict__ ra_b,
                                                              const W* __restrict__ ri, const W* __restrict__ ri_b,
                                                              const W* __restrict__ lam, float c,
                                                              float* __restrict__ a_out, float* __restrict__ x_out,
                                                              int num_tokens) {
  const int part = threadIdx.x & 15, ch = blockIdx.x * (blockDim.x / 16) + threadIdx.x / 16;
  const bool mine = ch < width;  // lanes without a channel walk an existing one and store nothing
  const int chc = mine ? ch : width - 1;
  const int b = chc / bw, o = chc - b * bw;
  const W* wr = ra + ((size_t)b * bw + o) * bw;
  const W* wi = ri + ((size_t)b * bw + o) * bw;
  const float rb = to_f32(ra_b[chc]), ib = to_f32(ri_b[chc]), sp = softplusf_(to_f32(lam[chc]));
  const bool quads = (bw & 3) == 0 && (width & 3) == 0 && sizeof(W) == 4;  // rows start on 16 bytes: four inputs a load
  for (int t0 = 0; t0 < num_tokens; t0 += 8) {
    float accr[8] = {}, acci[8] = {};
    if (quads) {
      for (int k = 4 * part; k < bw; k += 64) {
        const float4 a4 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(wr) + k);
        const float4 b4 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(wi) + k);
        float4 u4[8];
#pragma unroll
        for (int tt = 0; tt < 8; ++tt)
          u4[tt] = t0 + tt < num_tokens ? *reinterpret_cast<const float4*>(u + (size_t)(t0 + tt) * width + b * bw + k)
                                        : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) {
          accr[tt] = fmaf(a4.w, u4[tt].w, fmaf(a4.z, u4[tt].z, fmaf(a4.y, u4[tt].y, fmaf(a4.x, u4[tt].x, accr[tt]))));
          acci[tt] = fmaf(b4.w, u4[tt].w, fmaf(b4.z, u4[tt].z, fmaf(b4.y, u4[tt].y, fmaf(b4.x, u4[tt].x, acci[tt]))));
        }
      }
    } else {
      for (int k = part; k < bw; k += 16) {
        const float a = to_f32(wr[k]), bb = to_f32(wi[k]);
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) {
          const float uu = t0 + tt < num_tokens ? u[(size_t)(t0 + tt) * width + b * bw + k] : 0.f;
          accr[tt] = fmaf(a, uu, accr[tt]);
          acci[tt] = fmaf(bb, uu, acci[tt]);
        }
      }
    }
#pragma unroll
    for (int tt = 0; tt < 8; ++tt) {
      const float sr = slices_sum<16>(accr[tt]), si = slices_sum<16>(acci[tt]);
      const int t = t0 + tt;
      if (mine && part == 0 && t < num_tokens) {
        const float rg = sigmoidf_(sr + rb), ig = sigmoidf_(si + ib);
        const float log_a = -c * rg * sp;
        a_out[(size_t)t * width + ch] = expf(log_a);
        x_out[(size_t)t * width + ch] = sqrtf(-expm1f(2.0f * log_a)) * ig * u[(size_t)t * width + ch];
      }
    }
  }
}

#define GATE_FEW_TOKENS 16
extern "C" int as_rglru_gates(const float* u, int width, int blocks, const void* ra, const void* ra_b, const void* ri,
                              const void* ri_b, const void* lam, int w_dtype, float c, float* a_out, float* x_out,
                              int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return AS_OK;
  if (width <= 0 || blocks <= 0 || width % blocks || blocks > 65535) return AS_BAD_SHAPE;
  const int bw = width / blocks;
  if (num_tokens <= GATE_FEW_TOKENS) {
    const int blocks_few = (width + 15) / 16;  // sixteen channels a workgroup of 256
    if (w_dtype == DT_F32)
      rglru_gates_few_kernel<float><<<blocks_few, 256, 0, stream>>>(u, width, bw, (const float*)ra, (const float*)ra_b,
                                                                   (const float*)ri, (const float*)ri_b,
                                                                   (const float*)lam, c, a_out, x_out, num_tokens);
    else if (w_dtype == DT_BF16)
      rglru_gates_few_kernel<bf16><<<blocks_few, 256, 0, stream>>>(u, width, bw, (const bf16*)ra, (const bf16*)ra_b,
                                                                  (const bf16*)ri, (const bf16*)ri_b, (const bf16*)lam,
                                                                  c, a_out, x_out, num_tokens);
    else return AS_BAD_DTYPE;
    return launch_status();
  }
  dim3 grid((num_tokens + GATE_TT - 1) / GATE_TT, blocks, (bw + GATE_TO - 1) / GATE_TO);
  if (grid.z > 65535) return AS_BAD_SHAPE;
  if (w_dtype == DT_F32)
    rglru_gates_kernel<float><<<grid, 256, 0, stream>>>(u, width, bw, (const float*)ra, (const float*)ra_b,
                                                        (const float*)ri, (const float*)ri_b, (const float*)lam, c,
                                                        a_out, x_out, num_tokens);
  else if (w_dtype == DT_BF16)
    rglru_gates_kernel<bf16><<<grid, 256, 0, stream>>>(u, width, bw, (const bf16*)ra, (const bf16*)ra_b,
                                                       (const bf16*)ri, (const bf16*)ri_b, (const bf16*)lam, c, a_out,
                                                       x_out, num_tokens);
  else return AS_BAD_DTYPE;
  return launch_status();
}

// The scan: S = a S + x per channel, from zero at the start of a sequence; what leaves is
// scale * S * gelu_tanh(y + y_bias) with y from proj [T, ld] at y_off, into out [T, ld_out] at out_off.
// A workgroup owns 64 channels of a row and cuts the row's tokens into SCAN_SEGS equal stretches, a wave
// each: every wave first runs its stretch from zero (keeping the product of its decays and what it ends
// with), the stretches' ends are chained in LDS in order, and every wave runs its stretch again from its
// true start, now writing.  The chain of dependent steps is a row's length / 8 instead of its length.
#define SCAN_SEGS 16
template <typename T, typename W>
__global__ __launch_bounds__(64 * SCAN_SEGS) void rglru_scan_kernel(
    const float* __restrict__ a, const float* __restrict__ x, int width, const T* __restrict__ proj, int ld, int y_off,
    const W* __restrict__ y_bias, float scale, float* __restrict__ state, const int* __restrict__ row_first,
    const int* __restrict__ row_len, const int* __restrict__ row_start, const int* __restrict__ row_slots, int writes,
    T* __restrict__ out, int ld_out, int out_off) {
  __shared__ float seg_a[SCAN_SEGS][WAVE], seg_b[SCAN_SEGS][WAVE];
  const int lane = threadIdx.x & (WAVE - 1), seg = threadIdx.x / WAVE;
  const int r = blockIdx.y, c = blockIdx.x * WAVE + lane;
  const bool live = c < width;
  const int first = row_first[r], len = row_len[r], slot = row_slots[r];
  const int per = (len + SCAN_SEGS - 1) / SCAN_SEGS;
  const int lo = min(len, seg * per), hi = min(len, lo + per);
  float A = 1.f, B = 0.f;
  if (live) {
#pragma unroll 4
    for (int j = lo; j < hi; ++j) {
      const size_t t = (size_t)first + j;
      const float av = a[t * width + c];
      B = fmaf(av, B, x[t * width + c]);
      A *= av;
    }
  }
  seg_a[seg][lane] = A;
  seg_b[seg][lane] = B;
  __syncthreads();
  if (!live) return;
  float* mine = state + (size_t)(slot < 0 ? 0 : slot) * width + c;
  float S = (row_start[r] > 0 && slot >= 0) ? *mine : 0.f;
  for (int s = 0; s < seg; ++s) S = fmaf(seg_a[s][lane], S, seg_b[s][lane]);
  const float yb = y_bias ? to_f32(y_bias[c]) : 0.f;
#pragma unroll 4
  for (int j = lo; j < hi; ++j) {
    const size_t t = (size_t)first + j;
    S = fmaf(a[t * width + c], S, x[t * width + c]);
    out[t * ld_out + out_off + c] = from_f32<T>(scale * S * gelu_tanhf_(to_f32(proj[t * ld + y_off + c]) + yb));
  }
  if (writes && slot >= 0 && seg == SCAN_SEGS - 1) *mine = S;  // the last stretch ends where the row ends
}

extern "C" int as_rglru_scan(const float* a, const float* x, int width, const void* proj, int dtype, int ld, int y_off,
                             const void* y_bias, int w_dtype, float scale, float* state, const int* row_first,
                             const int* row_len, const int* row_start, const int* row_slots, int writes, void* out,
                             int ld_out, int out_off, int num_rows, hipStream_t stream) {
  if (num_rows <= 0) return AS_OK;
  if (width <= 0 || num_rows > 65535 || ld < y_off + width || ld_out < out_off + width) return AS_BAD_SHAPE;
  const int threads = WAVE * SCAN_SEGS;
  dim3 grid((width + WAVE - 1) / WAVE, num_rows);
#define LAUNCH(T, W)                                                                                              \
  rglru_scan_kernel<T, W><<<grid, threads, 0, stream>>>(a, x, width, (const T*)proj, ld, y_off, (const W*)y_bias, \
                                                        scale, state, row_first, row_len, row_start, row_slots,  \
                                                        writes, (T*)out, ld_out, out_off)
  if (dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16, bf16);
  else if (dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16, float);
  else return AS_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}
