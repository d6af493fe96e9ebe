// What happens to projected queries, keys and values before attention reads them, in one pass over
// a token (one workgroup a token, its waves dealt out over the heads):
//
//  - rotation by position: channel i of a head's first `rot_dims` channels is paired with channel
//    i + rot_dims/2; the pair (u, w) becomes (u cos a - w sin a, w cos a + u sin a) with
//    a = position * freq[i].  freq is a float32 table made by the host (so base, scaling and any
//    other rule for the frequencies are the caller's); position, angle, sine and cosine are
//    float32, with the full-range sine and cosine.  The other channels pass unchanged.
//  - optionally each query and key head divided by its root mean square over its `head_dim` real
//    channels (eps inside the root), after the rotation;
//  - optionally values mixed with those that another layer made for the same token:
//    v <- (1 - lambda) v + lambda v_other (mode 2), or kept for such layers (mode 1);
//  - queries written back in place; keys and values stored into their page (slot_mapping).
//
// Heads lie `head_stride` channels apart (a head may be padded with zero channels beyond head_dim,
// or value_dim for the values); the values kept for other layers lie value_dim apart.
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

#define QKP_MAX_DIM 512

__global__ __launch_bounds__(256) void qk_prepare_kernel(
    void* __restrict__ z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head, int n_kv_head,
    int head_dim, int value_dim, int head_stride, const int* __restrict__ positions, const float* __restrict__ freq, int rot_dims,
    float norm_eps, const float* __restrict__ mix_lambda, void* __restrict__ v_other, long ld_other, int mix_mode,
    void* __restrict__ kpool, void* __restrict__ vpool, const int* __restrict__ slot_mapping, int page_size,
    int n_tokens) {
  __shared__ float cos_s[QKP_MAX_DIM / 2], sin_s[QKP_MAX_DIM / 2];
  __shared__ float head_s[4][QKP_MAX_DIM];
  const int n = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int half = rot_dims / 2;
  if (freq) {
    const float p = (float)positions[n];
    for (int i = threadIdx.x; i < half; i += 256) {
      const float a = p * freq[i];
      cos_s[i] = cosf(a);
      sin_s[i] = sinf(a);
    }
  }
  __syncthreads();
  const int slot = slot_mapping ? slot_mapping[n] : -1;
  const long page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot - (int)page * page_size : 0;
  float* s = head_s[wave];
  const long row = (long)n * ldz;
  for (int hh = wave; hh < n_head + n_kv_head; hh += 4) {
    const bool is_q = hh < n_head;
    const int g = is_q ? hh : hh - n_head;
    if (!is_q && !kpool) continue;
    const long src = row + (is_q ? q_off : k_off) + (long)g * head_stride;
    for (int c = lane; c < head_dim; c += 64) s[c] = load_f(z, dtype, src + c);
    __builtin_amdgcn_wave_barrier();
    if (freq) {
      for (int i = lane; i < half; i += 64) {
        const float u = s[i], w = s[i + half], co = cos_s[i], si = sin_s[i];
        s[i] = u * co - w * si;
        s[i + half] = w * co + u * si;
      }
      __builtin_amdgcn_wave_barrier();
    }
    float r = 1.0f;
    if (norm_eps >= 0.f) {
      float ss = 0.f;
      for (int c = lane; c < head_dim; c += 64) ss = fmaf(s[c], s[c], ss);
      r = 1.0f / sqrtf(wave_sum(ss) / (float)head_dim + norm_eps);
    }
    if (is_q) {
      for (int c = lane; c < head_dim; c += 64) store_f(z, dtype, src + c, s[c] * r);
    } else if (slot >= 0) {
      const long dst = ((page * n_kv_head + g) * page_size + off) * (long)head_stride;
      for (int c = lane; c < head_stride; c += 64) store_f(kpool, dtype, dst + c, c < head_dim ? s[c] * r : 0.f);
      const long vsrc = row + v_off + (long)g * head_stride;
      const long osrc = (long)n * ld_other + (long)g * value_dim;
      const float lam = mix_mode == 2 ? mix_lambda[0] : 0.f;
      for (int c = lane; c < head_stride; c += 64) {
        float v = load_f(z, dtype, vsrc + c);
        if (mix_mode == 1 && c < value_dim) store_f(v_other, dtype, osrc + c, v);
        if (mix_mode == 2 && c < value_dim) v = (1.0f - lam) * v + lam * load_f(v_other, dtype, osrc + c);
        store_f(vpool, dtype, dst + c, v);
      }
    } else if (mix_mode == 1) {
      // a token without a slot (padding of a bucket) still leaves its values: rows are independent
      const long vsrc = row + v_off + (long)g * head_stride;
      const long osrc = (long)n * ld_other + (long)g * value_dim;
      for (int c = lane; c < value_dim; c += 64) store_f(v_other, dtype, osrc + c, load_f(z, dtype, vsrc + c));
    }
    __builtin_amdgcn_wave_barrier();
  }
}

extern "C" int mgpt_qk_prepare(void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head, int n_kv_head,
                               int head_dim, int value_dim, int head_stride, const int* positions, const float* freq, int rot_dims,
                               float norm_eps, const float* mix_lambda, void* v_other, long ld_other, int mix_mode,
                               void* kpool, void* vpool, const int* slot_mapping, int page_size, int n_tokens,
                               hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!z || (freq && !positions) || (kpool && (!vpool || !slot_mapping))) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  if (n_tokens < 0 || n_head <= 0 || n_kv_head <= 0 || head_dim <= 0 || head_dim > QKP_MAX_DIM || head_stride < head_dim || value_dim <= 0 || value_dim > head_stride ||
      rot_dims < 0 || (rot_dims & 1) || rot_dims > head_dim || (kpool && page_size <= 0) || mix_mode < 0 || mix_mode > 2)
    return MGPT_ERR_BAD_SHAPE;
  if (mix_mode && (!v_other || (mix_mode == 2 && !mix_lambda))) return MGPT_ERR_NULL;
  hipLaunchKernelGGL(qk_prepare_kernel, dim3(n_tokens), dim3(256), 0, stream, z, dtype, ldz, q_off, k_off, v_off, n_head,
                     n_kv_head, head_dim, value_dim, head_stride, positions, rot_dims ? freq : nullptr, rot_dims, norm_eps, mix_lambda,
                     v_other, ld_other, mix_mode, kpool, vpool, slot_mapping, page_size, n_tokens);
  return mgpt_last_error();
}
