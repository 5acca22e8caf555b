// Several residual streams (hyper-connections): instead of one float32 residual row a token has S of them,
// xs[s, token, :]. A sublayer reads u = sum_s in[s] xs[s] and, once it has produced y from norm(u), all streams are
// rewritten at once from the old ones: xs'[t] = sum_s mix[s, t] xs[s] + out[t] y.
//
// As the framework's other norms take the pending delta of the single stream with them, the kernel here takes the
// pending rewrite with it: it applies the rewrite that the sublayer before left (its y, as a tensor or as partial sums
// over runs of k, and that sublayer's mix and out coefficients), writes the streams back, reads the coming sublayer's
// input with its in coefficients, and norms it. Everything is float32; the coefficients are float32 on the device.
#include "common.h"

#define ME_MAX_STREAMS 8

// xs[s] = xs[0] for s = 1 .. S-1 (the streams all start as the embedding rows).
__global__ void streams_spread_kernel(float* __restrict__ xs, size_t per_stream, int S) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= per_stream) return;
  const float v = xs[i];
  for (int s = 1; s < S; ++s) xs[(size_t)s * per_stream + i] = v;
}

extern "C" int me_streams_spread(float* xs, long long per_stream, int S, hipStream_t stream) {
  if (per_stream <= 0 || S <= 1) return 0;
  if (S > ME_MAX_STREAMS) return me_fail("me_streams_spread: %d streams, at most %d", S, ME_MAX_STREAMS);
  streams_spread_kernel<<<(unsigned)((per_stream + 255) / 256), 256, 0, stream>>>(xs, (size_t)per_stream, S);
  return me_check_launch("me_streams_spread");
}

// For output row r (token src = rows ? rows[r] : r), element c:
//   y      = delta[src, c] (+ the partial sums in their order)           (only with mix_out)
//   new[t] = mix_out ? sum_s mix[s, t] old[s] + out[t] y : old[t]         (written back when write_x)
//   u      = sum_t (w_in ? w_in[t] : 1) new[t]
//   h[r]   = u * rsqrt(mean(u^2) + eps) * w
// mix_out is float32 [S * S + S]: mix[s, t] at s * S + t (from stream s to stream t), then out[t].
// One block per row; u of the row waits in LDS between the two passes.
template <typename T>
__global__ void streams_norm_kernel(float* __restrict__ xs, size_t per_stream, int S, const T* __restrict__ delta,
                                    const float* __restrict__ parts, int num_parts, size_t part_stride,
                                    const float* __restrict__ mix_out, const float* __restrict__ w_in,
                                    const float* __restrict__ w, T* __restrict__ h, const int* __restrict__ rows, int dim,
                                    float eps, int write_x) {
  extern __shared__ float u_row[];
  __shared__ float scratch[16];
  __shared__ float coef[ME_MAX_STREAMS * ME_MAX_STREAMS + 2 * ME_MAX_STREAMS];
  float* mix = coef;
  float* outc = coef + ME_MAX_STREAMS * ME_MAX_STREAMS;
  float* inc = outc + ME_MAX_STREAMS;
  if (threadIdx.x < S * S) mix[threadIdx.x] = mix_out ? mix_out[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    outc[threadIdx.x] = mix_out ? mix_out[S * S + threadIdx.x] : 0.f;
    inc[threadIdx.x] = w_in ? w_in[threadIdx.x] : 1.f;
  }
  __syncthreads();
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const size_t base = (size_t)src * dim;
  float ss = 0.f;
  for (int c = threadIdx.x; c < dim; c += blockDim.x) {
    // every load of the element is asked for before the first is used: the streams, the result, its partial sums eight at a time
    float old[ME_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < ME_MAX_STREAMS; ++s) old[s] = s < S ? xs[(size_t)s * per_stream + base + c] : 0.f;
    float u = 0.f;
    if (mix_out) {
      float y = delta ? to_float(delta[base + c]) : 0.f;
      if (parts) {
        float d = 0.f;
        for (int p0 = 0; p0 < num_parts; p0 += 8) {
          float v[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) v[q] = p0 + q < num_parts ? parts[(size_t)(p0 + q) * part_stride + base + c] : 0.f;
#pragma unroll
          for (int q = 0; q < 8; ++q)
            if (p0 + q < num_parts) d = p0 + q == 0 ? v[q] : d + v[q];
        }
        y += d;
      }
      for (int t = 0; t < S; ++t) {
        float nv = outc[t] * y;
#pragma unroll
        for (int s = 0; s < ME_MAX_STREAMS; ++s)
          if (s < S) nv = fmaf(mix[s * S + t], old[s], nv);
        if (write_x) xs[(size_t)t * per_stream + base + c] = nv;
        u = fmaf(inc[t], nv, u);
      }
    } else {
#pragma unroll
      for (int s = 0; s < ME_MAX_STREAMS; ++s)
        if (s < S) u = fmaf(inc[s], old[s], u);
    }
    u_row[c] = u;
    ss = fmaf(u, u, ss);
  }
  const float total = block_sum(ss, scratch);
  const float inv = rsqrtf(total / (float)dim + eps);
  T* hr = h + (size_t)r * dim;
  for (int c = threadIdx.x; c < dim; c += blockDim.x) hr[c] = from_float<T>(u_row[c] * inv * w[c]);
}

// xs: float32 [S, total rows, dim] (per_stream = total rows * dim). delta / parts: the pending result of the sublayer
// before (both null with mix_out null: nothing is pending). rows (or null): the tokens whose normed input is wanted.
extern "C" int me_streams_norm(float* xs, long long per_stream, int S, const void* delta, const float* parts, int num_parts,
                               long long part_stride, const float* mix_out, const float* w_in, const float* w, void* h,
                               const int* rows, int num_rows, int dim, float eps, int write_x, int dtype, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (S < 1 || S > ME_MAX_STREAMS) return me_fail("me_streams_norm: %d streams, 1 to %d are taken", S, ME_MAX_STREAMS);
  if (dim <= 0 || dim > 16384) return me_fail("me_streams_norm: rows of %d elements, at most 16384", dim);
  if ((delta || parts) && !mix_out) return me_fail("me_streams_norm: a pending result needs its coefficients");
  if (parts && (num_parts < 1 || part_stride < (long long)dim)) return me_fail("me_streams_norm: %d partial sums", num_parts);
  // a thread an element up to 1,024 of them (all loads of a row in flight at once), then two, four, ..
  // (many rows hide each other's loads: blocks of 256 then)
  const int threads = num_rows >= 256 ? (dim >= 256 ? 256 : (dim + 63) / 64 * 64) : (dim >= 1024 ? 1024 : (dim + 63) / 64 * 64);
  const size_t lds = (size_t)dim * sizeof(float);
  if (lds > 48 * 1024) {
    const void* fn = dtype == ME_F32 ? (const void*)streams_norm_kernel<float> : (const void*)streams_norm_kernel<bf16_t>;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return me_fail("me_streams_norm: %zu bytes of block memory are refused", lds);
  }
  if (dtype == ME_F32)
    streams_norm_kernel<float><<<num_rows, threads, lds, stream>>>(xs, (size_t)per_stream, S, (const float*)delta, parts, num_parts,
                                                                   (size_t)part_stride, mix_out, w_in, w, (float*)h, rows, dim, eps,
                                                                   write_x);
  else
    streams_norm_kernel<bf16_t><<<num_rows, threads, lds, stream>>>(xs, (size_t)per_stream, S, (const bf16_t*)delta, parts,
                                                                    num_parts, (size_t)part_stride, mix_out, w_in, w, (bf16_t*)h,
                                                                    rows, dim, eps, write_x);
  return me_check_launch("me_streams_norm");
}
