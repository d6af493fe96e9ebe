// Linear attention with a fixed decay per head: a mixer whose memory is one float32 matrix per
// request and head instead of a cache of keys and values.
//
//   S_t = decay_h S_(t-1) + k_t v_t^T      (S: [D, E], zero before a request's first token)
//   o_t = S_t^T q_t
//
// q, k [H, D] and v [H, E] of a token lie in one row of `z` (the output of the stacked projection),
// in the compute dtype.  On their way in they may pass an activation (silu), q and k a rotation by
// position (pairs (i, i + rot_dims/2), angle position * freq[i], all float32), and k a constant
// scale.  Everything from there on is float32: the state, its decay, the products that enter it and
// the output.  On the way out a head's output may be divided by its root mean square (eps inside
// the root) and multiplied by silu(gate); the result is stored as float32 or in the compute dtype.
//
// One workgroup per (request, head) walks the request's tokens of this step in order, whatever
// their number (a prompt, a portion of one, one decoded token), from the state that the step
// before left in the request's slot, and leaves the new state there.  The state lives in
// registers: thread (dg, e) owns S[d][e] for d = dg, dg + NG, ... (256 threads a workgroup, or 1,024 for a
// large state, so that a thread's share stays small); the tokens' q, k, v are staged
// through LDS eight at a time, and the partial sums over dg meet there once per eight tokens.
#include "common.h"
#include "dtype_io.h"
#include "launchers.h"

#define DS_MAX 256  // largest D and E
#define DS_TC 8     // tokens staged at once

__device__ __forceinline__ float ds_act(float v, int act) { return act == 1 ? v / (1.0f + expf(-v)) : v; }

template <int R, int NT>     // state values a thread, threads a workgroup
__global__ __launch_bounds__(NT) void decay_state_kernel(
    const void* __restrict__ z, int dtype, long ldz, int q_off, int k_off, int v_off, int g_off, int n_head, int D, int E,
    int act, const int* __restrict__ positions, const float* __restrict__ freq, int rot_dims, float k_scale,
    const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ state_slots,
    const int* __restrict__ cu_q, float norm_eps, void* __restrict__ out, int out_dtype, long ldo) {
  __shared__ float q_s[DS_TC][DS_MAX], k_s[DS_TC][DS_MAX], v_s[DS_TC][DS_MAX], red[DS_TC][NT];
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int slot = state_slots[r];
  const int t_begin = cu_q[r], t_end = cu_q[r + 1];
  if (slot < 0 || t_end <= t_begin) return;     // a request of the padding
  const int NG = NT / E < D ? NT / E : D;       // groups of threads over d (at least 1: E <= 256)
  const bool owner = tid < NG * E;
  const int e = tid % E, dg = tid / E;
  const int count = owner ? (D - dg + NG - 1) / NG : 0;
  const float lambda = decay[h];
  float S[R];
  float* st = state + ((long)slot * n_head + h) * (long)D * E;
  const bool fresh = positions[t_begin] == 0;   // the request's first token: its state starts at zero
#pragma unroll
  for (int j = 0; j < R; ++j) S[j] = (j < count && !fresh) ? st[(long)(dg + j * NG) * E + e] : 0.f;
  const int half = rot_dims / 2;
  const int wave = tid >> 6, lane = tid & 63;

  for (int t0 = t_begin; t0 < t_end; t0 += DS_TC) {
    const int nt = t_end - t0 < DS_TC ? t_end - t0 : DS_TC;
    __syncthreads();     // the chunk before is read
    for (int i = tid; i < nt * D; i += NT) {
      const int tt = i / D, d = i - tt * D;
      const long row = (long)(t0 + tt) * ldz + (long)h * D + d;
      q_s[tt][d] = ds_act(load_f(z, dtype, row + q_off), act);
      k_s[tt][d] = ds_act(load_f(z, dtype, row + k_off), act);
    }
    for (int i = tid; i < nt * E; i += NT) {
      const int tt = i / E, c = i - tt * E;
      v_s[tt][c] = ds_act(load_f(z, dtype, (long)(t0 + tt) * ldz + v_off + (long)h * E + c), act);
    }
    __syncthreads();
    if (freq) {
      for (int i = tid; i < nt * half; i += NT) {
        const int tt = i / half, c = i - tt * half;
        const float a = (float)positions[t0 + tt] * freq[c];
        const float co = cosf(a), si = sinf(a);
        const float qu = q_s[tt][c], qw = q_s[tt][c + half], ku = k_s[tt][c], kw = k_s[tt][c + half];
        q_s[tt][c] = qu * co - qw * si;
        q_s[tt][c + half] = qw * co + qu * si;
        k_s[tt][c] = (ku * co - kw * si) * k_scale;
        k_s[tt][c + half] = (kw * co + ku * si) * k_scale;
      }
      if (k_scale != 1.0f)
        for (int i = tid; i < nt * (D - rot_dims); i += NT) {
          const int tt = i / (D - rot_dims), c = rot_dims + i - tt * (D - rot_dims);
          k_s[tt][c] *= k_scale;
        }
    } else if (k_scale != 1.0f) {
      for (int i = tid; i < nt * D; i += NT) k_s[i / D][i % D] *= k_scale;
    }
    __syncthreads();
    if (owner) {
      for (int tt = 0; tt < nt; ++tt) {
        const float ve = v_s[tt][e];
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
          if (j < count) {
            const int d = dg + j * NG;
            S[j] = fmaf(lambda, S[j], k_s[tt][d] * ve);
            acc = fmaf(S[j], q_s[tt][d], acc);
          }
        }
        red[tt][tid] = acc;
      }
    }
    __syncthreads();
    // a wave a token: the sums over dg in order, the head's norm, the gate, the store
    for (int tt = wave; tt < nt; tt += NT / 64) {
      float ss = 0.f;
      for (int c = lane; c < E; c += 64) {
        float o = 0.f;
        for (int g = 0; g < NG; ++g) o += red[tt][g * E + c];
        red[tt][c] = o;
        ss = fmaf(o, o, ss);
      }
      float scale = 1.0f;
      if (norm_eps >= 0.f) scale = 1.0f / sqrtf(wave_sum(ss) / (float)E + norm_eps);
      const long n = t0 + tt;
      for (int c = lane; c < E; c += 64) {
        float o = red[tt][c] * scale;
        if (g_off >= 0) {
          const float g = load_f(z, dtype, n * ldz + g_off + (long)h * E + c);
          o *= g / (1.0f + expf(-g));
        }
        store_f(out, out_dtype, n * ldo + (long)h * E + c, o);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < R; ++j)
    if (j < count) st[(long)(dg + j * NG) * E + e] = S[j];
}

// z: [n_tokens, ldz] rows in `dtype`; q at q_off, k at k_off, v at v_off, the gate at g_off (-1: none), head by head.
// state: [slots, n_head * D * E] float32; state_slots[r] the slot of request r (-1: none), cu_q its tokens.
extern "C" int mgpt_decay_state(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int g_off, int n_head,
                                int head_dim, int value_dim, int act, const int* positions, const float* freq,
                                int rot_dims, float k_scale, const float* decay, float* state, const int* state_slots,
                                const int* cu_q, int n_req, float norm_eps, void* out, int out_dtype, long ldo,
                                hipStream_t stream) {
  if (n_req == 0) return MGPT_OK;
  if (!z || !positions || !decay || !state || !state_slots || !cu_q || !out) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype) || !dtype_ok(out_dtype)) return MGPT_ERR_BAD_DTYPE;
  const int D = head_dim, E = value_dim;
  if (n_req < 0 || n_head <= 0 || D <= 0 || E <= 0 || D > DS_MAX || E > DS_MAX || rot_dims < 0 || (rot_dims & 1) ||
      rot_dims > D || (act != 0 && act != 1))
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  // a workgroup of 256 threads while a thread then owns at most 16 values of the state, else one of 1,024
  auto per_thread = [&](int threads) {
    const int ng = threads / E < D ? threads / E : D;
    return (D + ng - 1) / ng;
  };
  dim3 grid(n_req, n_head);
#define DS_LAUNCH(R, NT)                                                                                                   \
  hipLaunchKernelGGL((decay_state_kernel<R, NT>), grid, dim3(NT), 0, stream, z, dtype, ldz, q_off, k_off, v_off, g_off, n_head, \
                     D, E, act, positions, rot_dims ? freq : nullptr, rot_dims, k_scale, decay, state, state_slots, cu_q,   \
                     norm_eps, out, out_dtype, ldo)
  if (per_thread(256) <= 8) DS_LAUNCH(8, 256);
  else if (per_thread(256) <= 16) DS_LAUNCH(16, 256);
  else if (per_thread(1024) <= 16) DS_LAUNCH(16, 1024);
  else if (per_thread(1024) <= 32) DS_LAUNCH(32, 1024);
  else if (per_thread(1024) <= 64) DS_LAUNCH(64, 1024);
  else return MGPT_ERR_BAD_SHAPE;
#undef DS_LAUNCH
  return mgpt_last_error();
}

// ---------------------------------------------------------------------------------------------
// Prompt portions: the same recurrence a chunk of 32 tokens at a time, as matrix products on the
// float32 matrix cores (v_mfma_f32_16x16x4_f32: true 32-bit products and sums).  For a chunk whose
// tokens have in-chunk indices i = 0 .. n-1, with L = decay:
//   P[i][j] = (q_i . k_j) L^(i-j) for j <= i, else 0
//   o_i     = sum_j P[i][j] v_j + L^(i+1) S^T q_i
//   S      <- L^n S + sum_j L^(n-1-j) k_j v_j^T
// A workgroup owns (request, head, 32 or 16 value channels): the columns of S are independent of each
// other, so a head's value channels are dealt out over workgroups, each of which makes P for itself.
// Queries and keys come ready (activation, rotation, scale) as float32 from state_inputs_kernel.

#define DC_C 32        // tokens a chunk
#define DC_DMAX 128    // largest head size of this path
#define DC_LDQ (DC_DMAX + 4)
#define DC_LDP (DC_C + 4)

typedef float f32x4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void state_inputs_kernel(const void* __restrict__ z, int dtype, long ldz, int q_off,
                                                           int k_off, int n_head, int D, int act,
                                                           const int* __restrict__ positions, const float* __restrict__ freq,
                                                           int rot_dims, float k_scale, float* __restrict__ qk, int n_tokens) {
  __shared__ float cos_s[DS_MAX / 2], sin_s[DS_MAX / 2];
  const int n = blockIdx.x, half = rot_dims / 2;
  if (freq) {
    const float p = (float)positions[n];
    for (int i = threadIdx.x; i < half; i += 256) {
      const float a = p * freq[i];
      cos_s[i] = cosf(a);
      sin_s[i] = sinf(a);
    }
  }
  __syncthreads();
  const int HD = n_head * D;
  float* dst = qk + (long)n * 2 * HD;
  // thread: one channel of one head; a rotated pair is made by the thread of its first channel
  for (int i = threadIdx.x; i < HD; i += 256) {
    const int d = i % D;
    if (d >= half && d < rot_dims) continue;
    const long at = (long)n * ldz + i;
    float q = ds_act(load_f(z, dtype, at + q_off), act), k = ds_act(load_f(z, dtype, at + k_off), act);
    if (d < half) {
      const float q2 = ds_act(load_f(z, dtype, at + half + q_off), act), k2 = ds_act(load_f(z, dtype, at + half + k_off), act);
      const float co = cos_s[d], si = sin_s[d];
      dst[i + half] = q2 * co + q * si;
      dst[HD + i + half] = (k2 * co + k * si) * k_scale;
      const float qr = q * co - q2 * si, kr = k * co - k2 * si;
      q = qr;
      k = kr;
    }
    dst[i] = q;
    dst[HD + i] = k * k_scale;
  }
}

template <int EB>     // value channels a workgroup: 32, or 16 where that is what fills the machine
__global__ __launch_bounds__(256) void decay_state_chunk_kernel(
    const float* __restrict__ qk, const void* __restrict__ z, int dtype, long ldz, int v_off, int n_head, int D, int E,
    int act, const int* __restrict__ positions, const float* __restrict__ decay, float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_q, float* __restrict__ out, long ldo) {
  constexpr int NJ = EB / 16;     // column tiles of the workgroup's value channels
  // queries and keys [token][d]; the state and the values transposed, [value channel][d] and [value channel][token];
  // P [token][token].  Every product's index of summation runs along a row, so that a lane's operands of four
  // matrix instructions are one 16-byte read: instruction s of such a group takes k = k0 + 4 g + s from lane (r16, g)
  // (any dealing of a stretch's 16 values of k over four instructions gives the same sum, if both operands agree).
  __shared__ __attribute__((aligned(16))) float Qs[DC_C][DC_LDQ], Ks[DC_C][DC_LDQ], St[EB][DC_LDQ], Vt[EB][DC_LDP],
      Ps[DC_C][DC_LDP];
  __shared__ float pw[DC_C + 1];
  const int r = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * EB, tid = threadIdx.x;
  const int slot = state_slots[r];
  const int t_begin = cu_q[r], t_end = cu_q[r + 1];
  if (slot < 0 || t_end <= t_begin) return;     // a request of the padding
  const int wave = tid >> 6, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
  const int Dp = (D + 15) & ~15;                // rows of S and steps along d, padded with zeros
  const int HD = n_head * D;
  const float lambda = decay[h];
  const float log_l = logf(lambda);
  if (tid <= DC_C) pw[tid] = tid == 0 ? 1.0f : expf((float)tid * log_l);
  float* st = state + ((long)slot * n_head + h) * (long)D * E;
  const bool fresh = positions[t_begin] == 0;
  for (int i = tid; i < Dp * EB; i += 256) {
    const int d = i / EB, c = i - d * EB;
    St[c][d] = (!fresh && d < D && e0 + c < E) ? st[(long)d * E + e0 + c] : 0.f;
  }
  const int ti = wave >> 1, tj = wave & 1;      // this wave's 16 x 16 tile of P and of the chunk's outputs

  // A chunk's rows travel from memory into registers while the chunk before is multiplied: thread tid holds
  // elements tid, tid + 256, ... of the chunk's [32, Dp] queries and keys and of its [32, 32] values.
  constexpr int QK_PT = DC_C * DC_DMAX / 256, V_PT = DC_C * EB / 256;
  float q_r[QK_PT], k_r[QK_PT], v_r[V_PT];
  auto fetch = [&](int t0) {
    const int nt = t_end - t0 < DC_C ? t_end - t0 : DC_C;      // may be <= 0
#pragma unroll
    for (int u = 0; u < QK_PT; ++u) {
      const int i = tid + u * 256, tt = i / Dp, d = i - tt * Dp;
      const bool ok = i < DC_C * Dp && tt < nt && d < D;
      const long at = (long)(t0 + tt) * 2 * HD + (long)h * D + d;
      q_r[u] = ok ? qk[at] : 0.f;
      k_r[u] = ok ? qk[at + HD] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < V_PT; ++u) {
      const int i = tid + u * 256, tt = i / EB, c = i - tt * EB;
      v_r[u] = (tt < nt && e0 + c < E)
                   ? ds_act(load_f(z, dtype, (long)(t0 + tt) * ldz + v_off + (long)h * E + e0 + c), act) : 0.f;
    }
  };
  fetch(t_begin);

  for (int t0 = t_begin; t0 < t_end; t0 += DC_C) {
    const int nt = t_end - t0 < DC_C ? t_end - t0 : DC_C;
    __syncthreads();     // the chunk before is done with the staged rows; S is whole
#pragma unroll
    for (int u = 0; u < QK_PT; ++u) {
      const int i = tid + u * 256, tt = i / Dp, d = i - tt * Dp;
      if (i < DC_C * Dp) {
        Qs[tt][d] = q_r[u];
        Ks[tt][d] = k_r[u];
      }
    }
#pragma unroll
    for (int u = 0; u < V_PT; ++u) {
      const int i = tid + u * 256;
      Vt[i % EB][i / EB] = v_r[u];
    }
    __syncthreads();
    fetch(t0 + DC_C);     // (behind the last chunk: no token is left, nothing is loaded)
    // ---- P = Q K^T with the decay of the distance, lower triangle
    {
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      if (tj <= ti) {
#pragma unroll 2
        for (int k0 = 0; k0 < Dp; k0 += 16) {
          const f32x4_t a = *reinterpret_cast<const f32x4_t*>(&Qs[ti * 16 + r16][k0 + 4 * g]);
          const f32x4_t b = *reinterpret_cast<const f32x4_t*>(&Ks[tj * 16 + r16][k0 + 4 * g]);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], acc, 0, 0, 0);
        }
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int i = ti * 16 + 4 * g + v, j = tj * 16 + r16;
        Ps[i][j] = j <= i ? acc[v] * pw[i - j] : 0.f;
      }
    }
    __syncthreads();
    // ---- o = P V + L^(i+1) Q S: the tiles (oi, oj) of the chunk's [32, EB] outputs
    for (int t = wave; t < 2 * NJ; t += 4) {
      const int oi = t / NJ, oj = t - oi * NJ;
      f32x4_t a1 = {0.f, 0.f, 0.f, 0.f}, a2 = {0.f, 0.f, 0.f, 0.f};
      for (int k0 = 0; k0 < (oi + 1) * 16; k0 += 16) {
        const f32x4_t a = *reinterpret_cast<const f32x4_t*>(&Ps[oi * 16 + r16][k0 + 4 * g]);
        const f32x4_t b = *reinterpret_cast<const f32x4_t*>(&Vt[oj * 16 + r16][k0 + 4 * g]);
#pragma unroll
        for (int e = 0; e < 4; ++e) a1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], a1, 0, 0, 0);
      }
#pragma unroll 2
      for (int k0 = 0; k0 < Dp; k0 += 16) {
        const f32x4_t a = *reinterpret_cast<const f32x4_t*>(&Qs[oi * 16 + r16][k0 + 4 * g]);
        const f32x4_t b = *reinterpret_cast<const f32x4_t*>(&St[oj * 16 + r16][k0 + 4 * g]);
#pragma unroll
        for (int e = 0; e < 4; ++e) a2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], a2, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int i = oi * 16 + 4 * g + v, c = e0 + oj * 16 + r16;
        if (i < nt && c < E) out[(long)(t0 + i) * ldo + (long)h * E + c] = a1[v] + pw[i + 1] * a2[v];
      }
    }
    __syncthreads();     // every wave has read the old S
    // ---- S <- L^n S + sum_t L^(n-1-t) k_t v_t^T: the tiles (di, sj) of the [Dp, EB] state, dealt out over the waves
    for (int t = wave; t < (Dp >> 4) * NJ; t += 4) {
      const int di = t / NJ, sj = t - di * NJ;
      f32x4_t* mine = reinterpret_cast<f32x4_t*>(&St[sj * 16 + r16][di * 16 + 4 * g]);     // rows d = 4 g + v of column r16
      f32x4_t acc = *mine;
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[v] *= pw[nt];
#pragma unroll
      for (int k0 = 0; k0 < DC_C; k0 += 16) {
        const f32x4_t b = *reinterpret_cast<const f32x4_t*>(&Vt[sj * 16 + r16][k0 + 4 * g]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int tk = k0 + 4 * g + e;
          const float w = tk < nt ? pw[nt - 1 - tk] : 0.f;
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(Ks[tk][di * 16 + r16] * w, b[e], acc, 0, 0, 0);
        }
      }
      *mine = acc;
    }
  }
  __syncthreads();
  for (int i = tid; i < D * EB; i += 256) {
    const int d = i / EB, c = i - d * EB;
    if (e0 + c < E) st[(long)d * E + e0 + c] = St[c][d];
  }
}

// The chunked form for steps with prompt portions: qk is scratch, float32 [n_tokens, 2 * n_head * head_dim]; out is
// float32 [n_tokens, >= n_head * value_dim]: the heads' raw outputs (norm and gate are the caller's next kernel).
// Head sizes up to 128 (value sizes up to 256); others are refused with MGPT_ERR_BAD_SHAPE and nothing launched.
extern "C" int mgpt_decay_state_chunked(const void* z, int dtype, long ldz, int q_off, int k_off, int v_off, int n_head,
                                        int head_dim, int value_dim, int act, const int* positions, const float* freq,
                                        int rot_dims, float k_scale, const float* decay, float* state,
                                        const int* state_slots, const int* cu_q, int n_req, int n_tokens, float* qk,
                                        float* out, long ldo, hipStream_t stream) {
  if (n_req == 0 || n_tokens == 0) return MGPT_OK;
  if (!z || !positions || !decay || !state || !state_slots || !cu_q || !out || !qk) return MGPT_ERR_NULL;
  if (!dtype_ok(dtype)) return MGPT_ERR_BAD_DTYPE;
  const int D = head_dim, E = value_dim;
  if (n_req < 0 || n_tokens < 0 || n_head <= 0 || D <= 0 || E <= 0 || D > DC_DMAX || E > DS_MAX || rot_dims < 0 ||
      (rot_dims & 1) || rot_dims > D || (act != 0 && act != 1))
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(state_inputs_kernel, dim3(n_tokens), dim3(256), 0, stream, z, dtype, ldz, q_off, k_off, n_head, D, act,
                     positions, rot_dims ? freq : nullptr, rot_dims, k_scale, qk, n_tokens);
  // 32 value channels a workgroup; 16 where that many workgroups would leave compute units idle
  if ((long)n_req * n_head * ((E + 31) / 32) >= 256)
    hipLaunchKernelGGL(decay_state_chunk_kernel<32>, dim3(n_req, n_head, (E + 31) / 32), dim3(256), 0, stream, qk, z, dtype,
                       ldz, v_off, n_head, D, E, act, positions, decay, state, state_slots, cu_q, out, ldo);
  else
    hipLaunchKernelGGL(decay_state_chunk_kernel<16>, dim3(n_req, n_head, (E + 15) / 16), dim3(256), 0, stream, qk, z, dtype,
                       ldz, v_off, n_head, D, E, act, positions, decay, state, state_slots, cu_q, out, ldo);
  return mgpt_last_error();
}
