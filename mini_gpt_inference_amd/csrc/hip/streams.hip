// Several residual streams (hyper-connections), the scaled token embedding that starts them, and
// the scaled, soft-capped logits.
//
// The residual of a token is S rows of `width` floats, stored one after the other:
// x[n][s][c].  A sublayer reads u = sum_s a[s] x[n][s] and, once it has its output y, every
// stream is rewritten from the old ones: x'[n][t] = sum_s M[s][t] x[n][s] + b[t] y[n].
// All of it in 32-bit.
#include "common.h"
#include "launchers.h"

#define MGPT_MAX_STREAMS 8

template <typename WT>
__global__ void embed_scaled_kernel(const int* __restrict__ ids, const WT* __restrict__ tok,
                                    float* __restrict__ x, int n_tokens, int width, float scale, int copies) {
  const int n = blockIdx.x;
  if (n >= n_tokens) return;
  const WT* trow = tok + (long)ids[n] * width;
  float* xr = x + (long)n * copies * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = to_float<WT>(trow[c]) * scale;
    for (int s = 0; s < copies; ++s) xr[(long)s * width + c] = v;
  }
}

// x[n][s] = tok[ids[n]] * scale for every s < copies
extern "C" int mgpt_embed_scaled(const int* ids, const void* tok, float* x, int n_tokens, int width,
                                 int table_dtype, float scale, int copies, hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!ids || !tok || !x) return MGPT_ERR_NULL;
  if (n_tokens < 0 || width <= 0 || copies <= 0) return MGPT_ERR_BAD_SHAPE;
  const int threads = width >= 256 ? 256 : 64;
  if (table_dtype == MGPT_F32) {
    hipLaunchKernelGGL(embed_scaled_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream, ids,
                       (const float*)tok, x, n_tokens, width, scale, copies);
  } else if (table_dtype == MGPT_BF16) {
    hipLaunchKernelGGL(embed_scaled_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream, ids,
                       (const bf16_t*)tok, x, n_tokens, width, scale, copies);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
  return mgpt_last_error();
}

__global__ void streams_read_kernel(const float* __restrict__ x, const float* __restrict__ coef,
                                    float* __restrict__ u, float* __restrict__ zero, long total, int width,
                                    int streams) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long n = i / width;
  const int c = (int)(i - n * width);
  const float* xr = x + n * (long)streams * width + c;
  float acc = 0.f;
  for (int s = 0; s < streams; ++s) {
    const float v = xr[(long)s * width];
    acc = coef ? fmaf(coef[s], v, acc) : acc + v;
  }
  u[i] = acc;
  if (zero) zero[i] = 0.f;
}

// u[n] = sum_s coef[s] x[n][s] (coef null: the plain sum); `zero` (optional, [n_rows, width]) is cleared
extern "C" int mgpt_streams_read(const float* x, const float* coef, float* u, float* zero, int n_rows,
                                 int width, int streams, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!x || !u) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || streams <= 0 || streams > MGPT_MAX_STREAMS) return MGPT_ERR_BAD_SHAPE;
  const long total = (long)n_rows * width;
  const long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(streams_read_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, coef, u, zero, total,
                     width, streams);
  return mgpt_last_error();
}

__global__ void streams_write_kernel(float* __restrict__ x, const float* __restrict__ mix,
                                     const float* __restrict__ out, const float* __restrict__ y, long total,
                                     int width, int streams) {
  const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long n = i / width;
  const int c = (int)(i - n * width);
  float* xr = x + n * (long)streams * width + c;
  float old[MGPT_MAX_STREAMS];
#pragma unroll
  for (int s = 0; s < MGPT_MAX_STREAMS; ++s) old[s] = s < streams ? xr[(long)s * width] : 0.f;
  const float yv = y[i];
  for (int t = 0; t < streams; ++t) {
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < MGPT_MAX_STREAMS; ++s)
      if (s < streams) acc = fmaf(mix[s * streams + t], old[s], acc);
    xr[(long)t * width] = fmaf(out[t], yv, acc);
  }
}

// x[n][t] = sum_s mix[s][t] x[n][s] + out[t] y[n], every t from the old streams
extern "C" int mgpt_streams_write(float* x, const float* mix, const float* out, const float* y, int n_rows,
                                  int width, int streams, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!x || !mix || !out || !y) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || streams <= 0 || streams > MGPT_MAX_STREAMS) return MGPT_ERR_BAD_SHAPE;
  const long total = (long)n_rows * width;
  const long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(streams_write_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, mix, out, y, total,
                     width, streams);
  return mgpt_last_error();
}

template <bool FAST>
__global__ void scale_softcap_kernel(float* __restrict__ logits, long ld, int n_rows, int vocab, float scale,
                                     float cap) {
  const int row = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= n_rows || c >= vocab) return;
  float* p = logits + (long)row * ld + c;
  float v = *p * scale;
  if (cap > 0.f) {
    const float z = v / cap;
    if (FAST) {
      const float e = __builtin_amdgcn_exp2f(z * 2.8853900817779268f);   // exp(2z)
      v = cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
    } else {
      v = cap * tanhf(z);
    }
  }
  *p = v;
}

// logits = cap * tanh(logits * scale / cap) in place (cap <= 0: only the scale)
extern "C" int mgpt_scale_softcap(float* logits, long ld, int n_rows, int vocab, float scale, float cap,
                                  int fast, hipStream_t stream) {
  if (n_rows == 0 || vocab == 0) return MGPT_OK;
  if (!logits) return MGPT_ERR_NULL;
  if (n_rows < 0 || vocab < 0 || ld < vocab) return MGPT_ERR_BAD_SHAPE;
  if (n_rows > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid((vocab + 255) / 256, n_rows), block(256);
  if (fast)
    hipLaunchKernelGGL(scale_softcap_kernel<true>, grid, block, 0, stream, logits, ld, n_rows, vocab, scale, cap);
  else
    hipLaunchKernelGGL(scale_softcap_kernel<false>, grid, block, 0, stream, logits, ld, n_rows, vocab, scale, cap);
  return mgpt_last_error();
}
