// Kernels of latent attention and of layers whose norms sit on the branch outputs.
//
// norm_add:        h[t] += unit_rms(delta[t]) * w, optionally with a copy of the new h[t] in the
//                  activations' storage type (what the next branch reads).  delta may be an expert
//                  sum still to be formed (rows of the experts' outputs, their places and weights).
// latent_prep:     per token: the latent c = rms_norm(first R of the down projection) and the one
//                  rotated key part, stored side by side as the token's cache row [R + dr]; the
//                  rotated parts of the queries go to the tails of the query rows [H, R + dr].
// head_gemm:       out[t, h, n] = sum_k x[t, h, k] * w[h, n, k], one product per head, with an
//                  optional sigmoid gate on the result (float FMA chains in ascending k: a row's
//                  bits do not depend on the batch).
// attn_latent:     attention of H query heads over ONE shared row per key: the score is q . row
//                  over all R + dr elements, the value is the row's first R elements; softmax in
//                  float with an optional per-head sink term exp(sink_h) in the denominator.
#include "common.h"

constexpr int kMaxPairs = 128;   // rotated pairs of a head's rotated part

// ---------------------------------------------------------------------------
template <typename TD, typename TO>
__global__ __launch_bounds__(256) void norm_add_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                       const float* __restrict__ w, TO* __restrict__ out, int hidden,
                                                       float eps, const int* __restrict__ sum_pos,
                                                       const float* __restrict__ sum_w, int sum_k) {
  extern __shared__ float rowbuf[];
  __shared__ float red[16];
  const int t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float d;
    if (!sum_pos) {
      d = to_f32<TD>(delta[(size_t)t * hidden + c]);
    } else {
      d = 0.f;
      for (int q = 0; q < sum_k; ++q) {
        const float v = to_f32<TD>(delta[(size_t)sum_pos[t * sum_k + q] * hidden + c]);
        d += sum_w ? sum_w[t * sum_k + q] * v : v;
      }
      d = to_f32<TD>(from_f32<TD>(d));   // the sum is rounded once to the storage type, as the combine kernel stores it
    }
    rowbuf[c] = d;
    ss += d * d;
  }
  const float total = block_sum(ss, red);
  const float s = 1.0f / sqrtf(total / (float)hidden + eps);
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float x = h[(size_t)t * hidden + c] + (rowbuf[c] * s) * w[c];
    h[(size_t)t * hidden + c] = x;
    if (out) out[(size_t)t * hidden + c] = from_f32<TO>(x);
  }
}

// h float [T, hidden]; delta [T, hidden] (or the experts' rows with sum_pos int32 [T, k], sum_w float
// [T, k] or null); w float [hidden]; out [T, hidden] of out_dtype or null.
SHARPI_EXPORT int sharpi_norm_add(float* h, const void* delta, int d_dtype, const float* w, void* out, int out_dtype,
                                  int n_tokens, int hidden, float eps, const int* sum_pos, const float* sum_w,
                                  int sum_k, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (hidden <= 0 || hidden > 12288 || !(eps > 0.f) || !delta || !w || (sum_pos && sum_k <= 0)) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens), block(256);
  const size_t lds = (size_t)hidden * sizeof(float);
#define NORM_ADD(TDV, TOV)                                                                                       \
  norm_add_kernel<TDV, TOV><<<grid, block, lds, stream>>>(h, (const TDV*)delta, w, (TOV*)out, hidden, eps,       \
                                                          sum_pos, sum_w, sum_k)
  const int od = out ? out_dtype : d_dtype;
  if (d_dtype == DT_F32 && od == DT_F32) NORM_ADD(float, float);
  else if (d_dtype == DT_BF16 && od == DT_BF16) NORM_ADD(bf16_t, bf16_t);
  else if (d_dtype == DT_F32 && od == DT_BF16) NORM_ADD(float, bf16_t);
  else if (d_dtype == DT_BF16 && od == DT_F32) NORM_ADD(bf16_t, float);
  else return SHARPI_ERR_ARG;
#undef NORM_ADD
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// One element of a rotated part: element j of `src` (dr wide) at the angles cs/sn; pairs (2i, 2i+1)
// for i < n_pairs rotate, the rest passes.
template <typename T>
__device__ __forceinline__ float rotated_elem(const T* __restrict__ src, int j, int n_pairs, const float* cs,
                                              const float* sn) {
  if (j >= 2 * n_pairs) return to_f32<T>(src[j]);
  const int i = j >> 1;
  const float a = to_f32<T>(src[2 * i]), b = to_f32<T>(src[2 * i + 1]);
  return (j & 1) ? b * cs[i] + a * sn[i] : a * cs[i] - b * sn[i];
}

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const T* __restrict__ proj, int ld, int q_off, int kv_off,
                                                          T* __restrict__ q_full, T* __restrict__ k_cache,
                                                          const int* __restrict__ slots,
                                                          const int* __restrict__ positions,
                                                          const float* __restrict__ inv_freq, int n_pairs,
                                                          const float* __restrict__ norm_w, float eps, int H, int dn,
                                                          int dr, int R) {
  __shared__ float red[16];
  __shared__ float cs[kMaxPairs], sn[kMaxPairs];
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    const float ang = p * inv_freq[i];
    cs[i] = cosf(ang);
    sn[i] = sinf(ang);
  }
  __syncthreads();
  const T* row = proj + (size_t)t * ld;
  const int D = R + dr;
  for (int idx = threadIdx.x; idx < H * dr; idx += blockDim.x) {
    const int h = idx / dr, j = idx - h * dr;
    const T* qr = row + q_off + (size_t)h * (dn + dr) + dn;
    q_full[((size_t)t * H + h) * D + R + j] = from_f32<T>(rotated_elem<T>(qr, j, n_pairs, cs, sn));
  }
  if (kv_off < 0) return;                  // (the same for every thread)
  const T* kv = row + kv_off;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += blockDim.x) {
    const float x = to_f32<T>(kv[c]);
    ss += x * x;
  }
  const float total = block_sum(ss, red);
  const int slot = slots[t];
  if (slot < 0) return;
  const float s = 1.0f / sqrtf(total / (float)R + eps);
  T* dst = k_cache + (size_t)slot * D;
  for (int c = threadIdx.x; c < R; c += blockDim.x) dst[c] = from_f32<T>((to_f32<T>(kv[c]) * s) * norm_w[c]);
  for (int j = threadIdx.x; j < dr; j += blockDim.x) dst[R + j] = from_f32<T>(rotated_elem<T>(kv + R, j, n_pairs, cs, sn));
}

// proj [T, ld]: queries at column q_off as [H, dn + dr], the down projection [R + dr] at column
// kv_off (< 0: this layer makes no latent).  q_full [T, H, R + dr] receives the rotated query parts
// (columns R ..); k_cache rows [R + dr] at `slots` (< 0: nothing stored) receive the latent and the
// rotated key part.  inv_freq float [n_pairs], norm_w float [R].
SHARPI_EXPORT int sharpi_latent_prep(const void* proj, int dtype, int ld, int q_off, int kv_off, void* q_full,
                                     void* k_cache, const int* slots, const int* positions, const float* inv_freq,
                                     int n_pairs, const float* norm_w, float eps, int n_tokens, int H, int dn, int dr,
                                     int R, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (H <= 0 || dn <= 0 || dr <= 0 || R <= 0 || n_pairs < 0 || n_pairs > kMaxPairs || 2 * n_pairs > dr) return SHARPI_ERR_ARG;
  if (q_off < 0 || q_off + H * (dn + dr) > ld || (kv_off >= 0 && kv_off + R + dr > ld)) return SHARPI_ERR_ARG;
  if (kv_off >= 0 && (!k_cache || !slots || !norm_w || !(eps > 0.f))) return SHARPI_ERR_ARG;
  if (n_pairs > 0 && !inv_freq) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens), block(256);
  if (dtype == DT_F32)
    latent_prep_kernel<float><<<grid, block, 0, stream>>>((const float*)proj, ld, q_off, kv_off, (float*)q_full,
                                                          (float*)k_cache, slots, positions, inv_freq, n_pairs,
                                                          norm_w, eps, H, dn, dr, R);
  else if (dtype == DT_BF16)
    latent_prep_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)proj, ld, q_off, kv_off, (bf16_t*)q_full,
                                                           (bf16_t*)k_cache, slots, positions, inv_freq, n_pairs,
                                                           norm_w, eps, H, dn, dr, R);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
constexpr int kHgTile = 64, kHgK = 16;

template <typename T>
__global__ __launch_bounds__(256) void head_gemm_kernel(const T* __restrict__ x, int ldx, int sx,
                                                        const T* __restrict__ w, T* __restrict__ out, int ldo, int so,
                                                        const T* __restrict__ gate, int ldg, int n_tokens, int N,
                                                        int K) {
  __shared__ float xs[kHgK][kHgTile + 1], ws[kHgK][kHgTile + 1];
  const int h = blockIdx.z, t0 = blockIdx.x * kHgTile, n0 = blockIdx.y * kHgTile;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  const T* xh = x + (size_t)h * sx;
  const T* wh = w + (size_t)h * N * K;
  for (int k0 = 0; k0 < K; k0 += kHgK) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int idx = threadIdx.x + r * 256;
      const int row = idx >> 4, kk = idx & 15;
      const bool kin = k0 + kk < K;
      xs[kk][row] = (kin && t0 + row < n_tokens) ? to_f32<T>(xh[(size_t)(t0 + row) * ldx + k0 + kk]) : 0.f;
      ws[kk][row] = (kin && n0 + row < N) ? to_f32<T>(wh[(size_t)(n0 + row) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kHgK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty * 4 + i;
    if (t >= n_tokens) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (gate) v *= 1.0f / (1.0f + expf(-to_f32<T>(gate[(size_t)t * ldg + (size_t)h * N + n])));
      out[(size_t)t * ldo + (size_t)h * so + n] = from_f32<T>(v);
    }
  }
}

// The same on the matrix cores (bfloat16): a block of four waves computes 64 tokens x 64 outputs of
// one head, a wave 32 x 32 as 2 x 2 tiles of v_mfma_f32_16x16x32_bf16 with the weights as the A
// operand (out^T = W x^T); both operands come straight from memory in runs of 8 elements (a head's
// weights are small and stay in cache).  Every output is one chain over k in the same order whatever
// the number of tokens.  K, the heads' input stride and the row strides are multiples of 8 elements,
// the output's of 4.
typedef __attribute__((ext_vector_type(8))) __bf16 hg_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hg_f32x4;

__global__ __launch_bounds__(256) void head_gemm_mfma_kernel(const bf16_t* __restrict__ x, int ldx, int sx,
                                                             const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
                                                             int ldo, int so, const bf16_t* __restrict__ gate, int ldg,
                                                             int n_tokens, int N, int K) {
  const int h = blockIdx.z;
  const int wv = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int g = lane >> 4, m = lane & 15;
  const int t_base = blockIdx.x * 64 + (wv >> 1) * 32, n_base = blockIdx.y * 64 + (wv & 1) * 32;
  if (t_base >= n_tokens || n_base >= N) return;
  const bf16_t* xp[2];
  const bf16_t* wp[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    xp[a] = x + (size_t)min(t_base + 16 * a + m, n_tokens - 1) * ldx + (size_t)h * sx + 8 * g;
    wp[a] = w + ((size_t)h * N + min(n_base + 16 * a + m, N - 1)) * K + 8 * g;
  }
  hg_f32x4 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) acc[a][b] = hg_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool in = k0 + 8 * g < K;
    uint4 xa[2], wa[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      xa[a] = in ? *reinterpret_cast<const uint4*>(xp[a] + k0) : make_uint4(0, 0, 0, 0);
      wa[a] = in ? *reinterpret_cast<const uint4*>(wp[a] + k0) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<hg_bf16x8*>(&wa[a]),
                                                            *reinterpret_cast<hg_bf16x8*>(&xa[b]), acc[a][b], 0, 0, 0);
  }
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int t = t_base + 16 * b + m;
    if (t >= n_tokens) continue;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int n = n_base + 16 * a + 4 * g;
      if (n >= N) continue;                       // (N is a multiple of 4: the four outputs are in or out together)
      float v[4] = {acc[a][b][0], acc[a][b][1], acc[a][b][2], acc[a][b][3]};
      if (gate) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= 1.0f / (1.0f + expf(-bf16_to_f32(gate[(size_t)t * ldg + (size_t)h * N + n + i])));
      }
      uint2 o;
      o.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
      o.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
      *reinterpret_cast<uint2*>(out + (size_t)t * ldo + (size_t)h * so + n) = o;
    }
  }
}

// x rows of ldx elements, head h's K inputs at column h * sx; w [H, N, K]; out rows of ldo elements,
// head h's N outputs at column h * so; gate (or null) rows of ldg elements, head h's at column h * N:
// the result is multiplied by sigmoid(gate).  All of one storage type.
SHARPI_EXPORT int sharpi_head_gemm(const void* x, int dtype, int ldx, int sx, const void* w, void* out, int ldo,
                                   int so, const void* gate, int ldg, int n_tokens, int H, int N, int K,
                                   hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (H <= 0 || H > 65535 || N <= 0 || K <= 0 || sx < K || so < N || ldx < (H - 1) * sx + K || ldo < (H - 1) * so + N) return SHARPI_ERR_ARG;
  if (gate && ldg < H * N) return SHARPI_ERR_ARG;
  dim3 grid(ceil_div(n_tokens, kHgTile), ceil_div(N, kHgTile), H), block(256);
  if (grid.y > 65535) return SHARPI_ERR_ARG;
  if (dtype == DT_F32)
    head_gemm_kernel<float><<<grid, block, 0, stream>>>((const float*)x, ldx, sx, (const float*)w, (float*)out, ldo, so,
                                                        (const float*)gate, ldg, n_tokens, N, K);
  else if (dtype == DT_BF16 && K % 8 == 0 && sx % 8 == 0 && ldx % 8 == 0 && N % 4 == 0 && so % 4 == 0 && ldo % 4 == 0 &&
           ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 7) == 0)
    head_gemm_mfma_kernel<<<grid, block, 0, stream>>>((const bf16_t*)x, ldx, sx, (const bf16_t*)w, (bf16_t*)out, ldo, so,
                                                      (const bf16_t*)gate, ldg, n_tokens, N, K);
  else if (dtype == DT_BF16)
    head_gemm_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, ldx, sx, (const bf16_t*)w, (bf16_t*)out, ldo,
                                                         so, (const bf16_t*)gate, ldg, n_tokens, N, K);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// Attention over shared rows, float arithmetic: one block per (token, four heads), a wave a head.
// Tiles of KT keys are staged in LDS once for the block's heads.  A lane owns key (lane % KT) of a
// tile and, where KT < 64, a slice of the row's elements (the slices are summed across lanes in a
// fixed order); the value sum has a lane per element.  The order of every sum depends on the
// row width, the storage type and (first visible key, position) alone.
constexpr int kLatWaves = 4;
constexpr int kLatMaxAcc = 8;            // value elements per lane: R <= 512
constexpr int kLatTileBytes = 48 * 1024;

template <typename T, int NA>
__global__ __launch_bounds__(kLatWaves* kWave) void attn_latent_kernel(
    const T* __restrict__ q, const T* __restrict__ kc, const int* __restrict__ block_table,
    const int* __restrict__ entry_of_token, const int* __restrict__ positions, const float* __restrict__ sink,
    T* __restrict__ out, int window_kind, int window, float scale, int H, int R, int dr, int page_size,
    int max_blocks, int num_pages, int KT, int ldk) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int D = R + dr;
  float* qs = reinterpret_cast<float*>(smem);                       // [waves][D]
  int* ok = reinterpret_cast<int*>(qs + kLatWaves * D);             // [64]: key r of the tile exists
  T* kt = reinterpret_cast<T*>(ok + kWave);                         // [KT][ldk]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x >> 6;
  const int h_raw = blockIdx.y * kLatWaves + w;
  const bool live = h_raw < H;
  const int h = live ? h_raw : H - 1;
  const int e = entry_of_token[t];
  const int p = positions[t];
  int start = 0;
  if (window_kind == 1) start = (p / window) * window;
  else if (window_kind == 2) start = p - window + 1 > 0 ? p - window + 1 : 0;
  const int* bt = block_table + (size_t)e * max_blocks;
  const T* qrow = q + ((size_t)t * H + h) * D;
  for (int d = lane; d < D; d += kWave) qs[w * D + d] = to_f32<T>(qrow[d]);

  const int nparts = kWave / KT;
  const int key_l = lane % KT, part = lane / KT;
  const int Dp = (D + nparts - 1) / nparts;
  const int d0 = part * Dp, d1 = min(D, d0 + Dp);
  float m = -INFINITY, l = 0.f;
  float acc[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) acc[i] = 0.f;

  for (int tile0 = start; tile0 <= p; tile0 += KT) {
    __syncthreads();                     // the tile before is used up (and qs is written, the first time)
    for (int r = w; r < KT; r += kLatWaves) {
      const int key = tile0 + r;
      const T* src = nullptr;
      if (key <= p) {
        const int blk = key / page_size;
        const int page = blk < max_blocks ? bt[blk] : -1;
        if (page >= 0 && page < num_pages) src = kc + ((size_t)page * page_size + key % page_size) * D;
      }
      if (lane == 0) ok[r] = src != nullptr;
      for (int d = lane; d < D; d += kWave) kt[r * ldk + d] = src ? src[d] : from_f32<T>(0.f);
    }
    __syncthreads();
    float dot = 0.f;
    const T* kr = kt + key_l * ldk;
    const float* qw = qs + w * D;
    for (int d = d0; d < d1; ++d) dot = fmaf(qw[d], to_f32<T>(kr[d]), dot);
    for (int off = KT; off < kWave; off <<= 1) dot += __shfl_xor(dot, off, kWave);
    const bool valid = ok[key_l] != 0;
    const float s = valid ? dot * scale : -INFINITY;
    const float mb = wave_max(s);
    if (mb > -INFINITY) {
      const float m_new = fmaxf(m, mb);
      const float pe = (valid && part == 0) ? expf(s - m_new) : 0.f;
      const float corr = expf(m - m_new);
      l = l * corr + wave_sum(pe);
#pragma unroll
      for (int i = 0; i < NA; ++i) acc[i] *= corr;
      m = m_new;
      for (int j = 0; j < KT; ++j) {
        const float pj = __shfl(pe, j, kWave);
        if (pj == 0.f) continue;
        const T* vr = kt + j * ldk;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
          const int d = lane + i * kWave;
          if (d < R) acc[i] = fmaf(pj, to_f32<T>(vr[d]), acc[i]);
        }
      }
    }
  }
  if (!live) return;
  float M = m, denom = l;
  if (sink) {
    const float sk = sink[h];
    M = fmaxf(m, sk);
    denom = l * expf(m - M) + expf(sk - M);
  }
  const float f = denom > 0.f ? expf(m - M) / denom : 0.f;
  T* orow = out + ((size_t)t * H + h) * R;
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int d = lane + i * kWave;
    if (d < R) orow[d] = from_f32<T>(acc[i] * f);
  }
}

// q [T, H, R + dr]; rows [pages * page_size, R + dr] (the cache of one shared key head); sink float
// [H] or null; out [T, H, R].
SHARPI_EXPORT int sharpi_attention_latent(const void* q, const void* rows, int dtype, const int* block_table,
                                          const int* entry_of_token, const int* positions, const float* sink,
                                          void* out, int window_kind, int window, float scale, int n_tokens, int H,
                                          int R, int dr, int page_size, int max_blocks, int num_pages,
                                          hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (H <= 0 || H > 65535 * kLatWaves || R <= 0 || R > kLatMaxAcc * kWave || dr < 0) return SHARPI_ERR_ARG;
  if (page_size <= 0 || max_blocks <= 0 || num_pages <= 0) return SHARPI_ERR_ARG;
  if (window_kind < 0 || window_kind > 2 || (window_kind != 0 && window <= 0)) return SHARPI_ERR_ARG;
  if (dtype != DT_F32 && dtype != DT_BF16) return SHARPI_ERR_ARG;
  const int D = R + dr;
  const int width = dtype == DT_F32 ? 4 : 2;
  // rows of the tile a bank apart: an odd number of 4-byte words
  int ldk = dtype == DT_F32 ? (D | 1) : ((D + 1) & ~1);
  if (dtype == DT_BF16 && ((ldk / 2) & 1) == 0) ldk += 2;
  int KT = kWave;
  while (KT > 16 && (size_t)KT * ldk * width > (size_t)kLatTileBytes) KT >>= 1;
  if ((size_t)KT * ldk * width > (size_t)kLatTileBytes) return SHARPI_ERR_ARG;
  const size_t lds = (size_t)kLatWaves * D * sizeof(float) + kWave * sizeof(int) + (size_t)KT * ldk * width;
  dim3 grid(n_tokens, ceil_div(H, kLatWaves)), block(kLatWaves * kWave);
  const int na = ceil_div(R, kWave);
#define LAT_LAUNCH(TV, NAV)                                                                                      \
  attn_latent_kernel<TV, NAV><<<grid, block, lds, stream>>>((const TV*)q, (const TV*)rows, block_table,          \
                                                            entry_of_token, positions, sink, (TV*)out,           \
                                                            window_kind, window, scale, H, R, dr, page_size,     \
                                                            max_blocks, num_pages, KT, ldk)
#define LAT_BY_NA(TV)                                  \
  do {                                                 \
    if (na <= 1) LAT_LAUNCH(TV, 1);                    \
    else if (na <= 2) LAT_LAUNCH(TV, 2);               \
    else if (na <= 4) LAT_LAUNCH(TV, 4);               \
    else LAT_LAUNCH(TV, 8);                            \
  } while (0)
  if (dtype == DT_F32) LAT_BY_NA(float); else LAT_BY_NA(bf16_t);
#undef LAT_BY_NA
#undef LAT_LAUNCH
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
