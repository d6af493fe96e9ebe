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

// A sublayer's write, the next sublayer's read and its LayerNorm in one pass over a token's streams:
//   x[t] <- sum_s mix[s][t] x[s] + out[t] y   (left out when y is null: the streams are as they are)
//   y <- 0                                      (the next sublayer adds its output into it)
//   u = sum_t coef[t] x[t];  h = (u - mean) / sqrt(var + eps) * gain (+ beta)
// One workgroup a token; a thread keeps its share of u in registers (up to SS_KEEP columns a thread,
// wider rows are read back from `u`).  Mean first, then the centred squares, as the LayerNorm kernel.
#define SS_KEEP 16

template <int T>
__device__ __forceinline__ float ss_block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();   // the last use of red is over
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < T / 64; ++w) total += red[w];
  return total;
}

// T threads a token: 256 for a step of many tokens, 1024 for few (a decode step), where a token's
// columns should be few a thread so that one round of loads covers them.
template <typename OT, int T>
__global__ __launch_bounds__(T) void streams_step_kernel(
    float* __restrict__ x, const float* __restrict__ mix, const float* __restrict__ out, float* __restrict__ y,
    int fold, int clear, const float* __restrict__ coef, float* __restrict__ u, const float* __restrict__ gain,
    const float* __restrict__ beta, float eps, OT* __restrict__ h, int width, int streams) {
  __shared__ float red[T / 64];
  const int tid = threadIdx.x;
  const long n = blockIdx.x;
  // the coefficients are the same for every thread: read where they are used, they come through the
  // scalar cache together with the first round of loads (no staging in LDS, no barrier before it)
  const float* m_s = mix;
  const float* o_s = out;
  const float* c_s = coef;
  float* xr = x + n * (long)streams * width;
  // column c of the token, from its old streams and y: the streams rewritten (if a write is pending),
  // y cleared, u returned
  auto column = [&](int c, const float* old, float yv) -> float {
    float uv = 0.f;
    if (fold) {
      for (int t = 0; t < streams; ++t) {
        float acc = 0.f;
#pragma unroll
        for (int s = 0; s < MGPT_MAX_STREAMS; ++s)
          if (s < streams) acc = fmaf(m_s[s * streams + t], old[s], acc);
        acc = fmaf(o_s[t], yv, acc);
        xr[(long)t * width + c] = acc;
        uv = fmaf(c_s[t], acc, uv);
      }
    } else {
#pragma unroll
      for (int s = 0; s < MGPT_MAX_STREAMS; ++s)
        if (s < streams) uv = fmaf(c_s[s], old[s], uv);
    }
    if (clear) y[n * width + c] = 0.f;
    u[n * width + c] = uv;
    return uv;
  };
  auto load = [&](int c, float* old, float& yv) {
#pragma unroll
    for (int s = 0; s < MGPT_MAX_STREAMS; ++s) old[s] = s < streams ? xr[(long)s * width + c] : 0.f;
    yv = fold ? y[n * width + c] : 0.f;
  };
  float keep[SS_KEEP], gk[SS_KEEP], bk[SS_KEEP];
  float sum = 0.f;
  // four columns at a time: all their loads are asked for before the first of them is waited for,
  // the gain and bias that the last pass needs among them
#pragma unroll
  for (int i0 = 0; i0 < SS_KEEP; i0 += 4) {
    float old[4][MGPT_MAX_STREAMS], yv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = tid + (i0 + j) * T;
      load(c < width ? c : 0, old[j], yv[j]);
      gk[i0 + j] = gain[c < width ? c : 0];
      bk[i0 + j] = beta ? beta[c < width ? c : 0] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = tid + (i0 + j) * T;
      keep[i0 + j] = c < width ? column(c, old[j], yv[j]) : 0.f;
      sum += keep[i0 + j];
    }
  }
  for (int c = tid + SS_KEEP * T; c < width; c += T) {
    float old[MGPT_MAX_STREAMS], yv;
    load(c, old, yv);
    sum += column(c, old, yv);
  }
  const float mean = ss_block_sum<T>(sum, red) / (float)width;
  float e = 0.f, v2 = 0.f;
#pragma unroll
  for (int i = 0; i < SS_KEEP; ++i) {
    const float d = tid + i * T < width ? keep[i] - mean : 0.f;
    keep[i] = d;
    e += d;
    v2 = fmaf(d, d, v2);
  }
  for (int c = tid + SS_KEEP * T; c < width; c += T) {
    const float d = u[n * width + c] - mean;
    e += d;
    v2 = fmaf(d, d, v2);
  }
  const float corr = ss_block_sum<T>(e, red) / (float)width;
  const float var = fmaxf(ss_block_sum<T>(v2, red) / (float)width - corr * corr, 0.f);
  const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
  for (int i = 0; i < SS_KEEP; ++i) {
    const int c = tid + i * T;
    if (c < width) h[n * width + c] = from_float<OT>((keep[i] - corr) * rstd * gk[i] + bk[i]);
  }
  for (int c = tid + SS_KEEP * T; c < width; c += T) {
    float v = ((u[n * width + c] - mean) - corr) * rstd * gain[c];
    if (beta) v += beta[c];
    h[n * width + c] = from_float<OT>(v);
  }
}

// y [n_rows, width]: with fold, the output of the sublayer whose write is still to be made (without, the
// streams are read as they are); with clear, it is zero afterwards.  u: float32 [n_rows, width]; h:
// [n_rows, width] in h_dtype.  x, y, u and h are four different buffers.
extern "C" int mgpt_streams_step(float* x, const float* mix, const float* out, float* y, int fold, int clear,
                                 const float* coef, float* u, const float* gain, const float* beta, float eps, void* h,
                                 int h_dtype, int n_rows, int width, int streams, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!x || !coef || !u || !gain || !h || (fold && (!mix || !out)) || ((fold || clear) && !y)) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0 || streams <= 0 || streams > MGPT_MAX_STREAMS) return MGPT_ERR_BAD_SHAPE;
  const bool few = n_rows <= 128 && width > 1024;   // more than four columns a thread otherwise
#define SS_LAUNCH(OT, T)                                                                                          \
  hipLaunchKernelGGL((streams_step_kernel<OT, T>), dim3(n_rows), dim3(T), 0, stream, x, mix, out, y, fold, clear, \
                     coef, u, gain, beta, eps, (OT*)h, width, streams)
  if (h_dtype == MGPT_F32) { if (few) SS_LAUNCH(float, 1024); else SS_LAUNCH(float, 256); }
  else if (h_dtype == MGPT_BF16) { if (few) SS_LAUNCH(bf16_t, 1024); else SS_LAUNCH(bf16_t, 256); }
  else return MGPT_ERR_BAD_DTYPE;
#undef SS_LAUNCH
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
