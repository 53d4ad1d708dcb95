// Gated linear attention: a matrix-valued recurrent state per head with a decay per key channel,
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   alpha_t = sigmoid(z_t)^(1/tau),
// walked token by token in float.  The state of a request lives in its state slot
// [slots, heads, dk, dv] (float) and is carried from step to step.
//
// A wave owns kCols value columns of one head of one entry: the columns of S are independent of
// each other, so an entry's work is spread over heads x ceil(dv / kCols) waves, and the walk along
// the entry's tokens is the only thing that is sequential.  Lane (g, j) holds rows g, g + 4,
// g + 8, ... of column j (RPL rows a lane).  Per token the lane scales its rows by alpha, adds
// k[row] * v[j], and sums S[row][j] * q[row] over its rows; the four row groups are then added by
// two exchanges between lanes.  Every sum's order depends on (dk, dv) alone: a token's output has
// the same bits however its request's tokens were cut into steps.
//
// q, k, alpha of kStage tokens are staged in LDS by the whole wave (alpha computed there, in
// float, as exp(log_sigmoid(z + bias) / tau)), so the walk itself reads LDS broadcasts only.
#include "common.h"

constexpr int kCols = 16;      // value columns a wave owns
constexpr int kGroups = 4;     // row groups (kWave / kCols)
constexpr int kStage = 8;      // tokens staged at a time

// log(sigmoid(z)) without overflow: min(z, 0) - log1p(exp(-|z|))
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T, int RPL>
__global__ __launch_bounds__(kWave) void gla_walk_kernel(
    const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, const float* __restrict__ z,
    const float* __restrict__ z_bias, float inv_tau, float q_scale, float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_tokens, float* __restrict__ out, int nh, int dk,
    int dv) {
  __shared__ float qs[kStage][RPL * kGroups];
  __shared__ float ks[kStage][RPL * kGroups];
  __shared__ float as[kStage][RPL * kGroups];
  const int e = blockIdx.z, h = blockIdx.y, c0 = blockIdx.x * kCols;
  const int lane = threadIdx.x;
  const int j = lane % kCols, g = lane / kCols;
  const int col = c0 + j;
  const bool col_ok = col < dv;
  const int first = cu_tokens[e], len = cu_tokens[e + 1] - first;
  float* S = state + (((size_t)state_slots[e] * nh + h) * dk) * dv;
  float s[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) {
    const int rowi = g + kGroups * r;
    s[r] = (col_ok && rowi < dk) ? S[(size_t)rowi * dv + col] : 0.f;
  }
  constexpr int DKP = RPL * kGroups;   // rows the lanes cover; rows beyond dk stay zero
  for (int t0 = 0; t0 < len; t0 += kStage) {
    const int nt = min(kStage, len - t0);
    __syncthreads();
    for (int i = lane; i < nt * DKP; i += kWave) {
      const int tt = i / DKP, d = i % DKP;
      const size_t tok = (size_t)(first + t0 + tt);
      float qv = 0.f, kv = 0.f, av = 1.f;
      if (d < dk) {
        qv = to_f32<T>(proj[tok * stride + q_off + h * dk + d]) * q_scale;
        kv = to_f32<T>(proj[tok * stride + k_off + h * dk + d]);
        av = expf(log_sigmoid(z[tok * (size_t)(nh * dk) + h * dk + d] + z_bias[h * dk + d]) * inv_tau);
      }
      qs[tt][d] = qv;
      ks[tt][d] = kv;
      as[tt][d] = av;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const size_t tok = (size_t)(first + t0 + tt);
      const float v = col_ok ? to_f32<T>(proj[tok * stride + v_off + h * dv + col]) : 0.f;
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        const int rowi = g + kGroups * r;
        s[r] = fmaf(as[tt][rowi], s[r], ks[tt][rowi] * v);
        o = fmaf(s[r], qs[tt][rowi], o);
      }
      o += __shfl_xor(o, 16, kWave);
      o += __shfl_xor(o, 32, kWave);
      if (g == 0 && col_ok) out[tok * (size_t)(nh * dv) + h * dv + col] = o;
    }
  }
#pragma unroll
  for (int r = 0; r < RPL; ++r) {
    const int rowi = g + kGroups * r;
    if (col_ok && rowi < dk) S[(size_t)rowi * dv + col] = s[r];
  }
}

// Each head's output normed over its dv elements (learned weights shared by the heads), times
// silu(gate): one wave a (token, head).  o float [T, nh * dv]; gate columns of proj.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                              float eps, const T* __restrict__ proj, int stride,
                                                              int g_off, T* __restrict__ out, int n_tokens, int nh,
                                                              int dv) {
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);     // (token, head), heads fastest
  const int lane = threadIdx.x & (kWave - 1);
  if (pair >= n_tokens * nh) return;
  const int t = pair / nh, h = pair % nh;
  const float* x = o + (size_t)pair * dv;
  float ss = 0.f;
  for (int d = lane; d < dv; d += kWave) ss = fmaf(x[d], x[d], ss);
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)dv + eps);
  const T* gate = proj ? proj + (size_t)t * stride + g_off + h * dv : nullptr;
  for (int d = lane; d < dv; d += kWave) {
    float y = x[d] * inv * w[d];
    if (gate) {
      const float gt = to_f32<T>(gate[d]);
      y *= gt / (1.0f + expf(-gt));
    }
    out[(size_t)pair * dv + d] = from_f32<T>(y);
  }
}

template <typename T>
static int launch_walk(const void* proj, int stride, int q_off, int k_off, int v_off, const float* z, const float* z_bias,
                       float inv_tau, float q_scale, float* state, const int* state_slots, const int* cu_tokens,
                       float* out, int n_entries, int nh, int dk, int dv, hipStream_t stream) {
  dim3 grid(ceil_div(dv, kCols), nh, n_entries);
#define WALK(RPL)                                                                                                   \
  gla_walk_kernel<T, RPL><<<grid, kWave, 0, stream>>>((const T*)proj, stride, q_off, k_off, v_off, z, z_bias, inv_tau, \
                                                      q_scale, state, state_slots, cu_tokens, out, nh, dk, dv)
  if (dk <= 32) WALK(8);
  else if (dk <= 64) WALK(16);
  else if (dk <= 128) WALK(32);
  else if (dk <= 256) WALK(64);
  else return SHARPI_ERR_ARG;
#undef WALK
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// proj [T, stride] of `dtype` holds q (nh * dk columns at q_off), k (at k_off) and v (nh * dv at
// v_off); z float [T, nh * dk] are the decay logits before their bias z_bias [nh * dk]; state float
// [slots, nh, dk, dv]; out float [T, nh * dv].  Entries (cu_tokens [entries + 1]) are walked in
// parallel, each from the state of its slot, which is left advanced.
SHARPI_EXPORT int sharpi_gla_walk(const void* proj, int dtype, int stride, int q_off, int k_off, int v_off, const float* z,
                                  const float* z_bias, float tau, float q_scale, float* state, const int* state_slots,
                                  const int* cu_tokens, float* out, int n_entries, int nh, int dk, int dv,
                                  hipStream_t stream) {
  if (n_entries <= 0) return SHARPI_OK;
  if (nh <= 0 || nh > 65535 || n_entries > 65535 || dk <= 0 || dk > 256 || dv <= 0 || !(tau > 0.f)) return SHARPI_ERR_ARG;
  if (dtype == DT_F32)
    return launch_walk<float>(proj, stride, q_off, k_off, v_off, z, z_bias, 1.0f / tau, q_scale, state, state_slots,
                              cu_tokens, out, n_entries, nh, dk, dv, stream);
  if (dtype == DT_BF16)
    return launch_walk<bf16_t>(proj, stride, q_off, k_off, v_off, z, z_bias, 1.0f / tau, q_scale, state, state_slots,
                               cu_tokens, out, n_entries, nh, dk, dv, stream);
  return SHARPI_ERR_ARG;
}

// o float [T, nh * dv] -> out [T, nh * dv] of `dtype`: per (token, head) unit RMS over dv, times w
// [dv], times silu of the gate at proj[t, g_off + h * dv + d] (proj null: no gate).
SHARPI_EXPORT int sharpi_head_norm_gate(const float* o, const float* w, float eps, const void* proj, int dtype, int stride,
                                        int g_off, void* out, int n_tokens, int nh, int dv, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (nh <= 0 || dv <= 0) return SHARPI_ERR_ARG;
  const int blocks = ceil_div(n_tokens * nh, 4);
  if (dtype == DT_F32)
    head_norm_gate_kernel<float><<<blocks, 256, 0, stream>>>(o, w, eps, (const float*)proj, stride, g_off, (float*)out,
                                                              n_tokens, nh, dv);
  else if (dtype == DT_BF16)
    head_norm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(o, w, eps, (const bf16_t*)proj, stride, g_off,
                                                               (bf16_t*)out, n_tokens, nh, dv);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
