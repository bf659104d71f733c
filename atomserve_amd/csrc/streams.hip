// Several residual streams.  Instead of one stream x a model keeps S copies x_1 .. x_S per token, fp32
// [T, S, n].  A sublayer reads them as one weighted sum through its norm and writes its output y back into all
// of them through a mixing matrix:
//     u = sum_s a[s] x_s;   y = part(norm(u));   x_r <- sum_s M[s, r] x_s + mult c[r] y     (M indexed [from, to])
// One kernel does what lies between two parts: the write of the part before (y still pending), the read for the
// part that follows and its RMS norm, x / sqrt(mean(x^2) + eps) * gain.  Everything is fp32; only y (as the
// part's product left it) and the normed rows (the next product's input) are in the compute dtype.
#include "common.h"

#define STREAMS_MAX 16
#define STREAMS_KEEP 8  // columns of a row that a thread keeps between the two passes of the norm

// first:    the streams do not exist yet: all of them are x0 [T, n] (what the embedding gave)
// y != 0:   the pending write (mix [S, S], out_c [S], mult)
// in_c != 0: the read and the norm: normed [T, n] = norm(sum_s in_c[s] x_s) * gain
// total != 0: total [T, n] = sum_s x_s (the one stream that the model's last norm reads)
// The streams are written back whenever they changed (first or y).
template <typename T>
__global__ __launch_bounds__(1024) void streams_step_kernel(float* __restrict__ xs, const float* __restrict__ x0, int S,
                                                            int n, const T* __restrict__ y,
                                                            const float* __restrict__ mix,
                                                            const float* __restrict__ out_c, float mult,
                                                            const float* __restrict__ in_c,
                                                            const float* __restrict__ gain, float eps,
                                                            T* __restrict__ normed,
                                                            float* __restrict__ total) {
  __shared__ float red[17];
  __shared__ float m_s[STREAMS_MAX * STREAMS_MAX], c_s[STREAMS_MAX], a_s[STREAMS_MAX];
  const int t = blockIdx.x;
  if (threadIdx.x < S * S) m_s[threadIdx.x] = mix ? mix[threadIdx.x] : (threadIdx.x / S == threadIdx.x % S ? 1.f : 0.f);
  if (threadIdx.x < S) {
    c_s[threadIdx.x] = out_c ? out_c[threadIdx.x] : 0.f;
    a_s[threadIdx.x] = in_c ? in_c[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float* mine = xs + (size_t)t * S * n;
  const bool writes = x0 != nullptr || y != nullptr;
  float kept[STREAMS_KEEP];
  float ss = 0.f;
  int slot = 0;
  for (int c = threadIdx.x; c < n; c += blockDim.x, ++slot) {
    float old[STREAMS_MAX], now[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < S) old[s] = x0 ? x0[(size_t)t * n + c] : mine[(size_t)s * n + c];
    if (y) {
      const float yv = mult * to_f32(y[(size_t)t * n + c]);
#pragma unroll
      for (int to = 0; to < STREAMS_MAX; ++to) {
        if (to < S) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < S) acc = fmaf(m_s[s * S + to], old[s], acc);
          now[to] = fmaf(c_s[to], yv, acc);
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < STREAMS_MAX; ++s)
        if (s < S) now[s] = old[s];
    }
    float u = 0.f, sum = 0.f;
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s) {
      if (s < S) {
        if (writes) mine[(size_t)s * n + c] = now[s];
        u = fmaf(a_s[s], now[s], u);
        sum += now[s];
      }
    }
    if (total) total[(size_t)t * n + c] = sum;
    if (slot < STREAMS_KEEP) kept[slot] = u;
    ss = fmaf(u, u, ss);
  }
  if (!normed) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  slot = 0;
  for (int c = threadIdx.x; c < n; c += blockDim.x, ++slot) {
    float u;
    if (slot < STREAMS_KEEP) {
      u = kept[slot];
    } else {  // rows wider than a thread keeps: the sum once more, from the streams as they are now (this thread wrote them)
      u = 0.f;
      for (int s = 0; s < S; ++s) u = fmaf(a_s[s], mine[(size_t)s * n + c], u);
    }
    normed[(size_t)t * n + c] = from_f32<T>(u * inv * gain[c]);
  }
}

extern "C" int as_streams_step(float* xs, const float* x0, int S, int n, const void* y, int dtype, const float* mix,
                               const float* out_c, float mult, const float* in_c, const float* gain, float eps,
                               void* normed, float* total, int num_rows, hipStream_t stream) {
  if (num_rows <= 0) return AS_OK;
  if (S < 1 || S > STREAMS_MAX || n < 1) return AS_BAD_SHAPE;
  if ((normed != nullptr) != (in_c != nullptr) || (normed && !gain)) return AS_BAD_SHAPE;
  if (y && !out_c) return AS_BAD_SHAPE;
  int threads = n >= 4096 ? 1024 : n >= 1024 ? 512 : 256;
  if (dtype == DT_F32)
    streams_step_kernel<float><<<num_rows, threads, 0, stream>>>(xs, x0, S, n, (const float*)y, mix, out_c, mult, in_c,
                                                                 gain, eps, (float*)normed, total);
  else if (dtype == DT_BF16)
    streams_step_kernel<bf16><<<num_rows, threads, 0, stream>>>(xs, x0, S, n, (const bf16*)y, mix, out_c, mult, in_c,
                                                                gain, eps, (bf16*)normed, total);
  else return AS_BAD_DTYPE;
  return launch_status();
}
