// Gated linear attention: a matrix-valued recurrent state per head with a decay per key channel,
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   alpha_t = sigmoid(z_t)^(1/tau),
// walked token by token in float.  The state of a request lives in its state slot and is carried
// from step to step.  It is kept column slice by column slice and, inside a slice, in the order the
// walking wave's lanes hold it: [slots, heads, ceil(dv / 8), DKP, 8] floats with DKP the rows the
// lanes cover (dk rounded up to 32, 64, 128 or 256), row g * RPL + r of the slice at place
// r * 8 + g: the 8 columns a block owns are one contiguous piece of memory which the block alone
// reads and writes, 256 bytes a load of the wave.
//
// A long entry (a prompt alone in its step leaves most of the chip idle: 256 blocks for 16 heads of 128
// value columns) can be walked in segments: phase 1 walks every segment but an entry's last from a
// zero state and leaves its local state and the product D of its decays; a short kernel then turns the
// local states into the segments' true start states, S_start(n + 1) = D_n S_start(n) + S_local(n), one
// after the other from the slot's state; phase 2 walks every segment again from its start state, now
// writing outputs, and the last segment leaves the entry's new state in the slot.  Twice the sums
// on as many times the blocks as an entry has segments; the results differ from the unsegmented
// walk's by rounding only (the state at a segment's start is summed in another order).
//
// Three forms: stages of 16 tokens (8 for the widest heads) for whole entries of steps that bring
// portions of prompts; stages of 8 tokens for the segmented walk, whose many blocks then sit six to a
// compute unit instead of three; and stages of 2 tokens for steps of single tokens, whose blocks take
// 3 KB of LDS instead of 50 and fill the chip (a decode step at batch 64 has 16,384 of them).
//
// The columns of S are independent of each other, so an entry's work is spread over heads x
// ceil(dv / 16) blocks, and the walk along
// the entry's tokens is the only thing that is sequential.  A block is two waves and takes kCPL
// adjacent slices of kCols columns (a lane holds its rows of one column of each: every q, k and decay
// read from LDS then feeds two columns' sums; with one column a lane the walk was bound by LDS reads).
// The walking wave:
// lane (g, j) holds RPL consecutive rows of column j (rows g * RPL ...); per token it scales its rows
// by alpha, adds k[row] * v[j], and sums S[row][j] * q[row] over its rows; the row groups are then
// added by exchanges between lanes.  The staging wave runs a stage ahead: it fetches q, k, v and the
// decays of the next kStage tokens (16 bytes a load where sizes and offsets are multiples of
// eight) and leaves them in the other half of LDS, so that the walking wave reads LDS only and
// never waits for memory.  Every sum's order depends on (dk, dv) alone: a token's output has the
// same bits however its request's tokens were cut into steps.
//
// The decays are made from their logits once per (token, channel) by a kernel of their own, in
// float: alpha = exp(log_sigmoid(z + bias) / tau), in place over the logits.
#include "common.h"

constexpr int kCols = 8;                 // value columns a walking wave owns
constexpr int kGroups = kWave / kCols;   // row groups
constexpr int kCPL = 2;                  // columns a lane holds: a wave walks kCPL adjacent slices of kCols columns

// log(sigmoid(z)) without overflow: min(z, 0) - log1p(exp(-|z|))
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

__global__ void gla_decays_kernel(float* __restrict__ z, const float* __restrict__ bias, float inv_tau, size_t n, int N) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    z[i] = expf(log_sigmoid(z[i] + bias[i % N]) * inv_tau);
}

// The decays straight from the narrow middle of their projection: alpha[t, c] = sigmoid(sum_r a1[t, r]
// W[c, r] + bias[c])^(1 / tau).  a1 are `rank` columns of a wider row (the step's fused projection).  A
// block takes kDecayTokens tokens and 256 channels; a thread one channel, whose weight row it reads
// once for all the block's tokens; the sum is one ascending chain of float FMAs.
constexpr int kDecayTokens = 8;
constexpr int kDecayMaxRank = 256;

template <typename T>
__global__ __launch_bounds__(256) void gla_decays_fused_kernel(const T* __restrict__ proj, int stride, int a_off, int rank,
                                                               const T* __restrict__ w, const float* __restrict__ bias,
                                                               float inv_tau, float* __restrict__ alpha, int n_tokens, int N) {
  __shared__ float a1[kDecayTokens][kDecayMaxRank];
  const int t0 = blockIdx.x * kDecayTokens;
  const int nt = min(kDecayTokens, n_tokens - t0);
  for (int i = threadIdx.x; i < kDecayTokens * rank; i += blockDim.x) {
    const int tt = i / rank, r = i % rank;
    a1[tt][r] = tt < nt ? to_f32<T>(proj[(size_t)(t0 + tt) * stride + a_off + r]) : 0.f;
  }
  __syncthreads();
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= N) return;
  float acc[kDecayTokens];
#pragma unroll
  for (int tt = 0; tt < kDecayTokens; ++tt) acc[tt] = 0.f;
  const T* wr = w + (size_t)c * rank;
  for (int r = 0; r < rank; ++r) {
    const float wv = to_f32<T>(wr[r]);
#pragma unroll
    for (int tt = 0; tt < kDecayTokens; ++tt) acc[tt] = fmaf(a1[tt][r], wv, acc[tt]);
  }
  const float b = bias[c];
#pragma unroll
  for (int tt = 0; tt < kDecayTokens; ++tt)
    if (tt < nt) alpha[(size_t)(t0 + tt) * N + c] = expf(log_sigmoid(acc[tt] + b) * inv_tau);
}

template <typename T, int RPL, bool VEC, int STAGE>
__global__ __launch_bounds__(2 * kWave) void gla_walk_kernel(
    const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, const float* __restrict__ alpha,
    float q_scale, float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_tokens, float* __restrict__ out, int nh, int dk,
    int dv, int ncb, const int* __restrict__ segs, int phase, float* __restrict__ seg_state, float* __restrict__ seg_decay) {
  constexpr int DKP = RPL * kGroups;               // rows the lanes cover; rows beyond dk stay zero
  constexpr int kStage = (STAGE > 8 && DKP > 128) ? 8 : STAGE;   // tokens staged at a time (two stages fit in LDS)
  __shared__ __attribute__((aligned(16))) float qs[2][kStage][DKP];
  __shared__ __attribute__((aligned(16))) float ks[2][kStage][DKP];
  __shared__ __attribute__((aligned(16))) float as[2][kStage][DKP];
  __shared__ float vs[2][kStage][kCPL * kCols];
  __shared__ float part[kStage][kGroups][kCPL * kCols];   // the row groups' shares of a stage's outputs
  // whole entries (segs null, phase 0): blockIdx.z is an entry.  Segments: blockIdx.z is a segment
  // (entry, first token, tokens, 1 if the entry's last); phase 1 walks from zero and keeps the local
  // state and the decays' product, phase 2 walks from the segment's start state and writes outputs.
  int e = blockIdx.z, seg_first = 0, seg_len = 0;
  bool seg_last = true;
  if (segs) {
    e = segs[4 * blockIdx.z];
    seg_first = segs[4 * blockIdx.z + 1];
    seg_len = segs[4 * blockIdx.z + 2];
    seg_last = segs[4 * blockIdx.z + 3] != 0;
    if (phase == 1 && seg_last) return;             // (nobody reads the local state of an entry's last segment)
  }
  const int h = blockIdx.y;
  const int slice = blockIdx.x * kCPL;              // the first of the block's 8-column slices of the state
  const int c0 = slice * kCols;
  const int lane = threadIdx.x & (kWave - 1);
  const bool walker = threadIdx.x < kWave;
  const int j = lane % kCols, g = lane / kCols;     // the lane's columns: c0 + j and c0 + kCols + j; its rows: g * RPL ...
  const int first = segs ? seg_first : cu_tokens[e], len = segs ? seg_len : cu_tokens[e + 1] - first;
  float* S_slot = state + ((((size_t)state_slots[e] * nh + h) * ncb + slice) * DKP) * kCols;
  float* S_seg = segs ? seg_state + ((((size_t)blockIdx.z * nh + h) * ncb + slice) * DKP) * kCols : nullptr;
  const float* S_in = phase == 0 ? S_slot : phase == 2 ? S_seg : nullptr;
  float* S = phase == 0 ? S_slot : phase == 1 ? S_seg : (seg_last ? S_slot : nullptr);    // where the state is left
  const bool track = phase == 1;
  float s[kCPL][RPL], dprod[RPL];
  bool col_ok[kCPL];
#pragma unroll
  for (int c = 0; c < kCPL; ++c) col_ok[c] = c0 + c * kCols + j < dv;
  if (walker) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int rowi = g * RPL + r;
#pragma unroll
      for (int c = 0; c < kCPL; ++c)      // (slice c of the block lies DKP * kCols floats behind slice c - 1)
        s[c][r] = (S_in && col_ok[c] && rowi < dk) ? S_in[(size_t)c * DKP * kCols + (r * kGroups + g) * kCols + j] : 0.f;
      dprod[r] = 1.f;
    }
  }
  auto stage = [&](int t0, int buf) {
    const int nt = min(kStage, len - t0);
    if constexpr (VEC) {     // dk, the row strides and the offsets are multiples of eight
      // every load of the stage is requested before the first is used, none behind a branch (addresses
      // are clamped into the stage and what lies outside is replaced afterwards)
      constexpr int ITER = (kStage * (DKP / 8) + kWave - 1) / kWave;
      float qv[ITER][8], kv[ITER][8], av[ITER][8];
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int i = lane + it * kWave;
        const int tt = min(i / (DKP / 8), nt - 1), d = min((i % (DKP / 8)) * 8, dk - 8);
        const size_t tok = (size_t)(first + t0 + tt);
        load8(proj + tok * stride + q_off + h * dk + d, qv[it]);
        load8(proj + tok * stride + k_off + h * dk + d, kv[it]);
        load8(alpha + tok * (size_t)(nh * dk) + h * dk + d, av[it]);
      }
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int i = lane + it * kWave;
        const int tt = i / (DKP / 8), d = (i % (DKP / 8)) * 8;
        if (tt >= kStage) continue;
        const bool in = d < dk;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          qv[it][x] = in ? qv[it][x] * q_scale : 0.f;
          kv[it][x] = in ? kv[it][x] : 0.f;
          av[it][x] = in ? av[it][x] : 1.f;
        }
        store8(&qs[buf][tt][d], qv[it]);
        store8(&ks[buf][tt][d], kv[it]);
        store8(&as[buf][tt][d], av[it]);
      }
    } else {
      for (int i = lane; i < nt * DKP; i += kWave) {
        const int tt = i / DKP, d = i % DKP;
        const size_t tok = (size_t)(first + t0 + tt);
        float qv = 0.f, kv = 0.f, av = 1.f;
        if (d < dk) {
          qv = to_f32<T>(proj[tok * stride + q_off + h * dk + d]) * q_scale;
          kv = to_f32<T>(proj[tok * stride + k_off + h * dk + d]);
          av = alpha[tok * (size_t)(nh * dk) + h * dk + d];
        }
        qs[buf][tt][d] = qv;
        ks[buf][tt][d] = kv;
        as[buf][tt][d] = av;
      }
    }
    constexpr int VC = kCPL * kCols;                                 // the block's value columns
    for (int i = lane; i < nt * VC; i += kWave) {
      const int tt = i / VC, c = blockIdx.x * VC + i % VC;
      vs[buf][tt][i % VC] = c < dv ? to_f32<T>(proj[(size_t)(first + t0 + tt) * stride + v_off + h * dv + c]) : 0.f;
    }
  };
  // The outputs of a stage: its tokens' sums over the eight row groups, added in the order of the groups
  // and written 64 bytes a token.  The walking wave does it at the start of the next stage (a barrier lies
  // between; its own reads of `part` come before its next writes in program order), so that no exchange
  // between lanes stands between one token's sums and the next one's.
  int done_t0 = -1, done_nt = 0;
  auto flush = [&]() {
    constexpr int VC = kCPL * kCols;
    for (int i = lane; i < done_nt * VC; i += kWave) {
      const int tt = i / VC, c = i % VC;
      float o = 0.f;
#pragma unroll
      for (int gg = 0; gg < kGroups; ++gg) o += part[tt][gg][c];
      if (c0 + c < dv) out[(size_t)(first + done_t0 + tt) * (size_t)(nh * dv) + h * dv + c0 + c] = o;
    }
  };
  if (!walker) stage(0, 0);
  __syncthreads();
  int buf = 0;
  for (int t0 = 0; t0 < len; t0 += kStage, buf ^= 1) {
    if (!walker) {
      if (t0 + kStage < len) stage(t0 + kStage, buf ^ 1);
    } else {
      const int nt = min(kStage, len - t0);
      if (!track && done_t0 >= 0) flush();
      done_t0 = t0;
      done_nt = nt;
      auto one_token = [&](int tt) {
        const float v0 = vs[buf][tt][j], v1 = vs[buf][tt][kCols + j];
        const float* qrow = &qs[buf][tt][g * RPL];
        const float* krow = &ks[buf][tt][g * RPL];
        const float* arow = &as[buf][tt][g * RPL];
        float o0 = 0.f, o1 = 0.f;
#pragma unroll
        for (int r = 0; r < RPL; r += 4) {
          const float4 a4 = *reinterpret_cast<const float4*>(arow + r);
          const float4 k4 = *reinterpret_cast<const float4*>(krow + r);
          const float4 q4 = *reinterpret_cast<const float4*>(qrow + r);
          const float av[4] = {a4.x, a4.y, a4.z, a4.w}, kv[4] = {k4.x, k4.y, k4.z, k4.w}, qv[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            s[0][r + x] = fmaf(av[x], s[0][r + x], kv[x] * v0);
            o0 = fmaf(s[0][r + x], qv[x], o0);
            s[1][r + x] = fmaf(av[x], s[1][r + x], kv[x] * v1);
            o1 = fmaf(s[1][r + x], qv[x], o1);
            if (track) dprod[r + x] *= av[x];
          }
        }
        if (track) return;                            // (phase 1 wants the state and the decays only)
        part[tt][g][j] = o0;                          // the groups' shares meet in `flush`, a stage later
        part[tt][g][kCols + j] = o1;
      };
      if (nt == kStage) {
        // a full stage, unrolled: the LDS reads of the tokens ahead are requested while this one is summed
#pragma unroll 2
        for (int tt = 0; tt < kStage; ++tt) one_token(tt);
      } else {
        for (int tt = 0; tt < nt; ++tt) one_token(tt);
      }
    }
    __syncthreads();
  }
  if (walker && !track && done_t0 >= 0) flush();     // (the loop's last barrier lies before this)
  if (walker && S) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int rowi = g * RPL + r;
#pragma unroll
      for (int c = 0; c < kCPL; ++c)
        if (col_ok[c] && rowi < dk) S[(size_t)c * DKP * kCols + (r * kGroups + g) * kCols + j] = s[c][r];
    }
  }
  if (walker && track && slice == 0 && j == 0) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) seg_decay[((size_t)blockIdx.z * nh + h) * DKP + g * RPL + r] = dprod[r];
  }
}

// Between the two phases of a segmented walk: an entry's segments one after the other.  The state at the
// first segment's start is the slot's; S_start(n + 1) = D_n S_start(n) + S_local(n).  seg_state holds
// S_local on entry and S_start on exit.  One wave a (column slice, head, entry), lanes as in the walk.
template <int RPL>
__global__ __launch_bounds__(kWave) void gla_combine_kernel(const float* __restrict__ state, const int* __restrict__ state_slots,
                                                            const int* __restrict__ ent_segs, float* __restrict__ seg_state,
                                                            const float* __restrict__ seg_decay, int nh) {
  constexpr int DKP = RPL * kGroups;
  const int e = blockIdx.z, h = blockIdx.y;
  const int lane = threadIdx.x, j = lane % kCols, g = lane / kCols;
  const int seg0 = ent_segs[2 * e], n = ent_segs[2 * e + 1];
  const float* S_slot = state + ((((size_t)state_slots[e] * nh + h) * gridDim.x + blockIdx.x) * DKP) * kCols;
  float s[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) s[r] = S_slot[(r * kGroups + g) * kCols + j];
  // (a segment's local state and decays are requested one segment ahead of their use: the chain of
  // sums is short, the loads are what takes time)
  float local[RPL] = {}, dec[RPL] = {};
  auto fetch = [&](int i) {
    const size_t seg = (size_t)(seg0 + i);
    const float* p = seg_state + (((seg * nh + h) * gridDim.x + blockIdx.x) * DKP) * kCols;
    const float* d = seg_decay + (seg * nh + h) * DKP + g * RPL;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      local[r] = p[(r * kGroups + g) * kCols + j];
      dec[r] = d[r];
    }
  };
  if (n > 1) fetch(0);
  for (int i = 0; i < n; ++i) {
    float* p = seg_state + ((((size_t)(seg0 + i) * nh + h) * gridDim.x + blockIdx.x) * DKP) * kCols;
    float next[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      p[(r * kGroups + g) * kCols + j] = s[r];
      next[r] = fmaf(dec[r], s[r], local[r]);
    }
    if (i + 2 < n) fetch(i + 1);                       // (the last segment has no local state to read)
    if (i + 1 < n) {
#pragma unroll
      for (int r = 0; r < RPL; ++r) s[r] = next[r];
    }
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
static int launch_walk(const void* proj, int stride, int q_off, int k_off, int v_off, const float* alpha, float q_scale,
                       float* state, const int* state_slots, const int* cu_tokens, float* out, int n_entries, int nh,
                       int dk, int dv, int max_entry_len, hipStream_t stream) {
  const int ncb = ceil_div(dv, kCols);
  dim3 grid(ceil_div(ncb, kCPL), nh, n_entries);
  const bool vec = dk % 8 == 0 && stride % 8 == 0 && q_off % 8 == 0 && k_off % 8 == 0 &&
                   ((uintptr_t)proj % 32 == 0) && ((uintptr_t)alpha % 32 == 0);
  const bool brief = max_entry_len <= 2;
#define WALK_AS(RPL, VEC, STAGE)                                                                                      \
  gla_walk_kernel<T, RPL, VEC, STAGE><<<grid, 2 * kWave, 0, stream>>>(                                       \
      (const T*)proj, stride, q_off, k_off, v_off, alpha, q_scale, state, state_slots, cu_tokens, out, nh, dk, dv, ncb, nullptr, 0, \
      nullptr, nullptr)
#define WALK(RPL)                         \
  do {                                    \
    if (brief) {                          \
      if (vec) WALK_AS(RPL, true, 2);     \
      else WALK_AS(RPL, false, 2);        \
    } else {                              \
      if (vec) WALK_AS(RPL, true, 16);    \
      else WALK_AS(RPL, false, 16);       \
    }                                     \
  } while (0)
  if (dk <= 32) WALK(4);
  else if (dk <= 64) WALK(8);
  else if (dk <= 128) WALK(16);
  else if (dk <= 256) WALK(32);
  else return SHARPI_ERR_ARG;
#undef WALK
#undef WALK_AS
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

template <typename T>
static int launch_segmented(const void* proj, int stride, int q_off, int k_off, int v_off, const float* alpha, float q_scale,
                            float* state, const int* state_slots, const int* cu_tokens, float* out, int n_entries, int nh,
                            int dk, int dv, const int* segs, const int* ent_segs, int n_segs, float* seg_state,
                            float* seg_decay, hipStream_t stream) {
  const int ncb = ceil_div(dv, kCols);
  dim3 grid(ceil_div(ncb, kCPL), nh, n_segs), cgrid(ncb, nh, n_entries);
  const bool vec = dk % 8 == 0 && stride % 8 == 0 && q_off % 8 == 0 && k_off % 8 == 0 &&
                   ((uintptr_t)proj % 32 == 0) && ((uintptr_t)alpha % 32 == 0);
#define PHASE(RPL, VEC, PH)                                                                                            \
  gla_walk_kernel<T, RPL, VEC, 8><<<grid, 2 * kWave, 0, stream>>>(                                         \
      (const T*)proj, stride, q_off, k_off, v_off, alpha, q_scale, state, state_slots, cu_tokens, out, nh, dk, dv, ncb, segs, PH, \
      seg_state, seg_decay)
#define SEGMENTED(RPL)                                                                                       \
  do {                                                                                                       \
    if (vec) PHASE(RPL, true, 1);                                                                            \
    else PHASE(RPL, false, 1);                                                                               \
    gla_combine_kernel<RPL><<<cgrid, kWave, 0, stream>>>(state, state_slots, ent_segs, seg_state, seg_decay, nh); \
    if (vec) PHASE(RPL, true, 2);                                                                            \
    else PHASE(RPL, false, 2);                                                                               \
  } while (0)
  if (dk <= 32) SEGMENTED(4);
  else if (dk <= 64) SEGMENTED(8);
  else if (dk <= 128) SEGMENTED(16);
  else if (dk <= 256) SEGMENTED(32);
  else return SHARPI_ERR_ARG;
#undef SEGMENTED
#undef PHASE
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// The walk of gla_walk with long entries cut into segments that are walked side by side (see the head of
// this file).  segs int [n_segs, 4] = (entry, first token of the step's rows, tokens, 1 if the entry's last
// segment), an entry's segments consecutive and in order; ent_segs int [n_entries, 2] = (first segment,
// segments); seg_state float [n_segs, nh, ceil(dv / 8), DKP, 8] and seg_decay float [n_segs, nh, DKP]: scratch.
SHARPI_EXPORT int sharpi_gla_walk_segmented(const void* proj, int dtype, int stride, int q_off, int k_off, int v_off,
                                            const float* alpha, float q_scale, float* state, const int* state_slots,
                                            const int* cu_tokens, float* out, int n_entries, int nh, int dk, int dv,
                                            const int* segs, const int* ent_segs, int n_segs, float* seg_state,
                                            float* seg_decay, hipStream_t stream) {
  if (n_entries <= 0 || n_segs <= 0) return SHARPI_OK;
  if (nh <= 0 || nh > 65535 || n_entries > 65535 || n_segs > 65535 || dk <= 0 || dk > 256 || dv <= 0) return SHARPI_ERR_ARG;
  if (!segs || !ent_segs || !seg_state || !seg_decay) return SHARPI_ERR_ARG;
  if (dtype == DT_F32)
    return launch_segmented<float>(proj, stride, q_off, k_off, v_off, alpha, q_scale, state, state_slots, cu_tokens, out,
                                   n_entries, nh, dk, dv, segs, ent_segs, n_segs, seg_state, seg_decay, stream);
  if (dtype == DT_BF16)
    return launch_segmented<bf16_t>(proj, stride, q_off, k_off, v_off, alpha, q_scale, state, state_slots, cu_tokens, out,
                                    n_entries, nh, dk, dv, segs, ent_segs, n_segs, seg_state, seg_decay, stream);
  return SHARPI_ERR_ARG;
}

// columns of the state that lie together in memory (the state's layout is [.., ceil(dv / this), dk, this])
SHARPI_EXPORT int sharpi_gla_state_cols() { return kCols; }

SHARPI_EXPORT int sharpi_gla_decays(float* z, const float* bias, float tau, int n_rows, int N, hipStream_t stream) {
  if (n_rows <= 0) return SHARPI_OK;
  if (N <= 0 || !(tau > 0.f) || !bias) return SHARPI_ERR_ARG;
  const size_t n = (size_t)n_rows * N;
  gla_decays_kernel<<<(unsigned)min((size_t)8192, (n + 255) / 256), 256, 0, stream>>>(z, bias, 1.0f / tau, n, N);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// proj [T, stride] of `dtype`: its columns a_off .. a_off + rank are the narrow middle of the decay
// projection; w [N, rank] of the same dtype, bias float [N]; alpha float [T, N] receives
// sigmoid(a1 w^T + bias)^(1 / tau).
SHARPI_EXPORT int sharpi_gla_decays_fused(const void* proj, int dtype, int stride, int a_off, int rank, const void* w,
                                          const float* bias, float tau, float* alpha, int n_tokens, int N,
                                          hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (N <= 0 || rank <= 0 || rank > kDecayMaxRank || !(tau > 0.f) || !bias || !w) return SHARPI_ERR_ARG;
  dim3 grid(ceil_div(n_tokens, kDecayTokens), ceil_div(N, 256));
  if (grid.y > 65535) return SHARPI_ERR_ARG;
  if (dtype == DT_F32)
    gla_decays_fused_kernel<float><<<grid, 256, 0, stream>>>((const float*)proj, stride, a_off, rank, (const float*)w, bias,
                                                             1.0f / tau, alpha, n_tokens, N);
  else if (dtype == DT_BF16)
    gla_decays_fused_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)proj, stride, a_off, rank, (const bf16_t*)w,
                                                              bias, 1.0f / tau, alpha, n_tokens, N);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// proj [T, stride] of `dtype` holds q (nh * dk columns at q_off), k (at k_off) and v (nh * dv at
// v_off); alpha float [T, nh * dk] are the decays; state float [slots, nh, ceil(dv / 8), DKP, 8] (see above);
// max_entry_len bounds the tokens of an entry (it picks the form: stages of 2 tokens up to 2); out float
// [T, nh * dv].  Entries (cu_tokens [entries + 1]) are walked in parallel, each from the state of
// its slot, which is left advanced.
SHARPI_EXPORT int sharpi_gla_walk(const void* proj, int dtype, int stride, int q_off, int k_off, int v_off,
                                  const float* alpha, float q_scale, float* state, const int* state_slots,
                                  const int* cu_tokens, float* out, int n_entries, int nh, int dk, int dv,
                                  int max_entry_len, hipStream_t stream) {
  if (n_entries <= 0) return SHARPI_OK;
  if (nh <= 0 || nh > 65535 || n_entries > 65535 || dk <= 0 || dk > 256 || dv <= 0) return SHARPI_ERR_ARG;
  if (dtype == DT_F32)
    return launch_walk<float>(proj, stride, q_off, k_off, v_off, alpha, q_scale, state, state_slots, cu_tokens, out,
                              n_entries, nh, dk, dv, max_entry_len, stream);
  if (dtype == DT_BF16)
    return launch_walk<bf16_t>(proj, stride, q_off, k_off, v_off, alpha, q_scale, state, state_slots, cu_tokens, out,
                               n_entries, nh, dk, dv, max_entry_len, stream);
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
