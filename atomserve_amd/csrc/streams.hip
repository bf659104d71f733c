// Several residual streams.  Instead of one stream x a model keeps S copies x_1 .. x_S per token, fp32
// [T, S, n].  A sublayer reads them as one weighted sum through its norm and writes its output y back into all
// of them through a mixing matrix:
//     u = sum_s a[s] x_s;   y = part(norm(u));   x_r <- sum_s M[s, r] x_s + mult c[r] y     (M indexed [from, to])
// One kernel does what lies between two parts: the write of the part before (y still pending), the read for the
// part that follows and its RMS norm, x / sqrt(mean(x^2) + eps) * gain.  Everything is fp32; only y (as the
// part's product left it) and the normed rows (the next product's input) are in the compute dtype.
#include "common.h"

#define STREAMS_MAX 16

// first:    the streams do not exist yet: all of them are x0 [T, n] (what the embedding gave)
// y != 0:   the pending write (mix [S, S], out_c [S], mult)
// in_c != 0: the read and the norm: normed [T, n] = norm(sum_s in_c[s] x_s) * gain
// total != 0: total [T, n] = sum_s x_s (the one stream that the model's last norm reads)
// The streams are written back whenever they changed (first or y).
// A workgroup per token; a thread takes V neighbouring columns at a time (V = 4: 16-byte accesses, for rows whose
// width is a multiple of 4) and keeps up to KEEP such pieces of the weighted sum between the two passes of the norm.
// SC: the number of streams where it is known when the kernel is compiled (the coefficients then live in registers and
// every loop over streams is unrolled), 0: any number up to STREAMS_MAX, coefficients from LDS.
#define STREAMS_KEEP 4
template <typename T, int V, int SC>
__global__ __launch_bounds__(1024) void streams_step_kernel(float* __restrict__ xs, const float* __restrict__ x0, int S_run,
                                                            int n, const T* __restrict__ y,
                                                            const float* __restrict__ mix,
                                                            const float* __restrict__ out_c, float mult,
                                                            const float* __restrict__ in_c,
                                                            const float* __restrict__ gain, float eps,
                                                            T* __restrict__ normed, float* __restrict__ total) {
  __shared__ float red[17];
  __shared__ float m_s[STREAMS_MAX * STREAMS_MAX], c_s[STREAMS_MAX], a_s[STREAMS_MAX];
  constexpr int SM = SC ? SC : STREAMS_MAX;
  const int S = SC ? SC : S_run;
  const int t = blockIdx.x;
  float m_r[SC ? SC * SC : 1], c_r[SC ? SC : 1], a_r[SC ? SC : 1];
  if (SC) {
#pragma unroll
    for (int i = 0; i < SC * SC; ++i) m_r[i] = mix ? mix[i] : (i / SC == i % SC ? 1.f : 0.f);
#pragma unroll
    for (int i = 0; i < SC; ++i) {
      c_r[i] = out_c ? out_c[i] : 0.f;
      a_r[i] = in_c ? in_c[i] : 0.f;
    }
  } else {
    for (int i = threadIdx.x; i < S * S; i += blockDim.x) m_s[i] = mix ? mix[i] : (i / S == i % S ? 1.f : 0.f);
    for (int i = threadIdx.x; i < S; i += blockDim.x) {
      c_s[i] = out_c ? out_c[i] : 0.f;
      a_s[i] = in_c ? in_c[i] : 0.f;
    }
    __syncthreads();
  }
  auto m_at = [&](int from, int to) { return SC ? m_r[from * SM + to] : m_s[from * S + to]; };
  auto c_at = [&](int i) { return SC ? c_r[i] : c_s[i]; };
  auto a_at = [&](int i) { return SC ? a_r[i] : a_s[i]; };
  float* mine = xs + (size_t)t * S * n;
  const bool writes = x0 != nullptr || y != nullptr;
  float kept[STREAMS_KEEP][V];
  float ss = 0.f;
  int slot = 0;
  for (int c = threadIdx.x * V; c < n; c += blockDim.x * V, ++slot) {
    float old[SM][V], now[SM][V], yv[V];
    if (x0) {
      float first[V];
      if (V == 4) *reinterpret_cast<float4*>(first) = *reinterpret_cast<const float4*>(x0 + (size_t)t * n + c);
      else first[0] = x0[(size_t)t * n + c];
#pragma unroll
      for (int s = 0; s < SM; ++s)
#pragma unroll
        for (int v = 0; v < V; ++v) old[s][v] = first[v];
    } else {
#pragma unroll
      for (int s = 0; s < SM; ++s) {
        if (s < S) {
          if (V == 4) *reinterpret_cast<float4*>(old[s]) = *reinterpret_cast<const float4*>(mine + (size_t)s * n + c);
          else old[s][0] = mine[(size_t)s * n + c];
        }
      }
    }
    if (y) {
#pragma unroll
      for (int v = 0; v < V; ++v) yv[v] = mult * to_f32(y[(size_t)t * n + c + v]);
#pragma unroll
      for (int to = 0; to < SM; ++to) {
        if (to < S) {
#pragma unroll
          for (int v = 0; v < V; ++v) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < SM; ++s)
              if (s < S) acc = fmaf(m_at(s, to), old[s][v], acc);
            now[to][v] = fmaf(c_at(to), yv[v], acc);
          }
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < SM; ++s)
#pragma unroll
        for (int v = 0; v < V; ++v) now[s][v] = old[s][v];
    }
    float u[V], sum[V];
#pragma unroll
    for (int v = 0; v < V; ++v) u[v] = sum[v] = 0.f;
#pragma unroll
    for (int s = 0; s < SM; ++s) {
      if (s < S) {
        if (writes) {
          if (V == 4) *reinterpret_cast<float4*>(mine + (size_t)s * n + c) = *reinterpret_cast<const float4*>(now[s]);
          else mine[(size_t)s * n + c] = now[s][0];
        }
#pragma unroll
        for (int v = 0; v < V; ++v) {
          u[v] = fmaf(a_at(s), now[s][v], u[v]);
          sum[v] += now[s][v];
        }
      }
    }
    if (total) {
      if (V == 4) *reinterpret_cast<float4*>(total + (size_t)t * n + c) = *reinterpret_cast<const float4*>(sum);
      else total[(size_t)t * n + c] = sum[0];
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
      if (slot < STREAMS_KEEP) kept[slot < STREAMS_KEEP ? slot : 0][v] = u[v];
      ss = fmaf(u[v], u[v], ss);
    }
  }
  if (!normed) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  slot = 0;
  for (int c = threadIdx.x * V; c < n; c += blockDim.x * V, ++slot) {
#pragma unroll
    for (int v = 0; v < V; ++v) {
      float u;
      if (slot < STREAMS_KEEP) {
        u = kept[slot < STREAMS_KEEP ? slot : 0][v];
      } else {  // rows wider than a thread keeps: the sum once more, from the streams as they are now (this thread wrote them)
        u = 0.f;
        for (int s = 0; s < S; ++s) u = fmaf(a_at(s), mine[(size_t)s * n + c + v], u);
      }
      normed[(size_t)t * n + c + v] = from_f32<T>(u * inv * gain[c + v]);
    }
  }
}

template <typename T>
static void launch_streams_step(float* xs, const float* x0, int S, int n, const T* y, const float* mix,
                                const float* out_c, float mult, const float* in_c, const float* gain, float eps,
                                T* normed, float* total, int num_rows, hipStream_t stream) {
  const bool quads = (n & 3) == 0;
  const int per = quads ? 4 : 1;
  int threads = (n / per + 63) / 64 * 64;
  threads = threads > 1024 ? 1024 : threads < 64 ? 64 : threads;
#define LAUNCH(V, SC)                                                                                                 \
  streams_step_kernel<T, V, SC><<<num_rows, threads, 0, stream>>>(xs, x0, S, n, y, mix, out_c, mult, in_c, gain, eps, \
                                                                  normed, total)
#define LAUNCH_S(V)               \
  do {                            \
    if (S == 1) LAUNCH(V, 1);     \
    else if (S == 2) LAUNCH(V, 2);\
    else if (S == 3) LAUNCH(V, 3);\
    else if (S == 4) LAUNCH(V, 4);\
    else LAUNCH(V, 0);            \
  } while (0)
  if (quads) LAUNCH_S(4);
  else LAUNCH_S(1);
#undef LAUNCH_S
#undef LAUNCH
}

extern "C" int as_streams_step(float* xs, const float* x0, int S, int n, const void* y, int dtype, const float* mix,
                               const float* out_c, float mult, const float* in_c, const float* gain, float eps,
                               void* normed, float* total, int num_rows, hipStream_t stream) {
  if (num_rows <= 0) return AS_OK;
  if (S < 1 || S > STREAMS_MAX || n < 1) return AS_BAD_SHAPE;
  if ((normed != nullptr) != (in_c != nullptr) || (normed && !gain)) return AS_BAD_SHAPE;
  if (y && !out_c) return AS_BAD_SHAPE;
  if (dtype == DT_F32)
    launch_streams_step<float>(xs, x0, S, n, (const float*)y, mix, out_c, mult, in_c, gain, eps, (float*)normed, total,
                               num_rows, stream);
  else if (dtype == DT_BF16)
    launch_streams_step<bf16>(xs, x0, S, n, (const bf16*)y, mix, out_c, mult, in_c, gain, eps, (bf16*)normed, total,
                              num_rows, stream);
  else return AS_BAD_DTYPE;
  return launch_status();
}
