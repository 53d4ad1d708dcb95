// Latent attention on the matrix cores (bfloat16): H query heads over ONE cached row per key,
// [c (R) | rotated key part (dr)], score = q . row over D = R + dr elements, value = the row's
// first R elements.
//
// A block of eight waves works on up to 64 (token, head) rows of one request against one run of
// keys [run * RUN, (run + 1) * RUN): 16 rows (16 heads of a token, or all heads of several
// consecutive tokens where a layer has fewer than 16) belong to a pair of waves, each of which
// forms the scores and the softmax state of the rows (the same bits in both) and one half of their
// output elements, so that a wave's accumulators take 64 registers for a latent of 512 and two
// waves fit a SIMD.
// Keys come in chunks of 32, staged in LDS once for the block: the rows as they lie in the cache
// (the A operand of S^T = K Q^T, contraction over elements), and their first R elements once more,
// transposed [element][key] (the A operand of O^T = V^T P^T, contraction over keys), made from the
// staged rows by the block itself, so the cache holds every latent once.  Probabilities enter the
// second product as a bfloat16 pair hi + lo; the softmax state is float.  A row whose keys lie in
// one run is finished here (with the sink term, if any); a row with more runs leaves (max, sum,
// unnormalised output) per run, and the merge kernel adds the runs in ascending order and applies
// the sink.  Runs start at multiples of RUN whatever the batch, so a row's sums depend on
// (position, RUN) alone.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kLmWaves = 4;           // row groups of 16 rows a block
constexpr int kLmHalves = 2;          // waves a row group: each takes half of the output elements
constexpr int kLmChunk = 32;          // keys a chunk
constexpr int kLmVtLd = kLmChunk + 8; // elements a row of the transposed tile (rows 16 bytes apart in banks)

struct LmGeom {
  int H, R, D, d32, r16;   // heads, latent width, row width, 32-element steps of a row, 16-element tiles of the output
  int hpw, tb;             // heads and tokens of a wave's 16 rows
  int htb, tgb;            // head tiles and token groups of a block's four waves
  int ldk;                 // elements a staged row takes in LDS
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  return (uint32_t)f32_to_bf16(a).bits | ((uint32_t)f32_to_bf16(b).bits << 16);
}

template <int MAXD32, int MAXR16>
__global__ __launch_bounds__(kLmWaves* kLmHalves* kWave) void attn_latent_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ rows, const int* __restrict__ block_table,
    const int* __restrict__ entry_of_token, const int* __restrict__ positions, const int* __restrict__ tiles,
    const int* __restrict__ token_list, int tile_subs, const float* __restrict__ sink, bf16_t* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, float scale, LmGeom gm, int run_keys, int max_runs,
    int page_size, int max_blocks, int num_pages) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16_t* kt = reinterpret_cast<bf16_t*>(smem);                    // [32][ldk]
  bf16_t* vt = kt + kLmChunk * gm.ldk;                             // [R][kLmVtLd], keys in the order the second product wants
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int w = (tid >> 6) & (kLmWaves - 1), half = tid >> 8;
  const int g = lane >> 4, m16 = lane & 15;
  const int tpb = gm.tgb * gm.tb;
  // this wave's 16-element tiles of the output: the first or the second half of them
  constexpr int MAXH = (MAXR16 + 1) / 2;
  const int r_lo = half ? (gm.r16 + 1) / 2 : 0;
  const int r_n = half ? gm.r16 - r_lo : (gm.r16 + 1) / 2;

  // the block's tokens: a piece of a prompt tile, or one listed token
  int tok0, cnt, e;
  if (tiles) {
    const int tile = blockIdx.x / tile_subs, sb = blockIdx.x - tile * tile_subs;
    e = tiles[tile * 3];
    tok0 = tiles[tile * 3 + 1] + sb * tpb;
    cnt = min(tpb, tiles[tile * 3 + 2] - sb * tpb);
  } else {
    tok0 = token_list ? token_list[blockIdx.x] : blockIdx.x;
    e = entry_of_token[tok0];
    cnt = 1;
  }
  if (cnt <= 0) return;
  const int p0 = positions[tok0];
  const int run = blockIdx.y;
  const int k_begin = run * run_keys;
  const int k_end = min(k_begin + run_keys, p0 + cnt);
  if (k_begin >= k_end) return;
  const int* bt = block_table + (size_t)e * max_blocks;

  // this lane's row (column of the transposed products)
  const int tg = w / gm.htb, ht = blockIdx.z * gm.htb + (w - tg * gm.htb);
  const int ti = tg * gm.tb + m16 / gm.hpw;
  const int head = ht * gm.hpw + m16 % gm.hpw;
  const bool row_ok = ti < cnt && head < gm.H;
  const int token = tok0 + (row_ok ? ti : 0);
  const int p_row = p0 + ti;
  const bool wave_ok = __any(row_ok);

  bf16x8 qf[MAXD32];
  {
    const bf16_t* qrow = q + ((size_t)token * gm.H + (row_ok ? head : 0)) * gm.D;
#pragma unroll
    for (int j = 0; j < MAXD32; ++j) {
      uint4 v = make_uint4(0, 0, 0, 0);
      const int d = 32 * j + 8 * g;
      if (j < gm.d32 && row_ok && d < gm.D) v = *reinterpret_cast<const uint4*>(qrow + d);
      qf[j] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  // the columns of the staged rows beyond D stay zero
  for (int i = tid; i < kLmChunk * gm.ldk / 8; i += blockDim.x) reinterpret_cast<uint4*>(kt)[i] = make_uint4(0, 0, 0, 0);

  f32x4 acc[MAXH];
#pragma unroll
  for (int d = 0; d < MAXH; ++d) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const int d8 = gm.D >> 3;
  // Staging: a thread owns row (tid / 16) of every chunk and the pieces of 8 elements c, c + 16, ... of
  // it (sixteen lanes read 256 bytes on end), so a chunk costs it ONE page lookup, which is made a
  // chunk ahead, and NJ independent loads, which are requested before the chunk before is multiplied.
  constexpr int NJ = (MAXD32 * 4 + 15) / 16;
  const int st_r = tid >> 4, st_c = tid & 15;
  auto row_of = [&](int c0) -> const bf16_t* {
    const int key = c0 + st_r;
    if (key >= k_end) return nullptr;
    const int blk = key / page_size;
    const int page = blk < max_blocks ? bt[blk] : -1;
    return (page >= 0 && page < num_pages) ? rows + ((size_t)page * page_size + key % page_size) * gm.D : nullptr;
  };
  uint4 stage[NJ];
  auto fetch = [&](const bf16_t* src) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int c8 = st_c + 16 * j;
      stage[j] = (src && c8 < d8) ? *reinterpret_cast<const uint4*>(src + 8 * c8) : make_uint4(0, 0, 0, 0);
    }
  };
  // (with the widest rows the registers do not reach for rows held across the products: they are
  // then requested where they are stored, and the SIMD's other wave covers the wait)
  constexpr bool kAhead = MAXD32 <= 10;
  const bf16_t* cur_row = row_of(k_begin);
  if (kAhead) fetch(cur_row);
  const bf16_t* next_row = row_of(k_begin + kLmChunk);

  for (int c0 = k_begin; c0 < k_end; c0 += kLmChunk) {
    if (!kAhead) fetch(cur_row);
    __syncthreads();                       // the chunk before is used up (the first time: the zero fill is done)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int c8 = st_c + 16 * j;
      if (c8 < d8) *reinterpret_cast<uint4*>(kt + st_r * gm.ldk + 8 * c8) = stage[j];
    }
    if (kAhead) fetch(next_row);           // the next chunk's rows are on their way while this one is transposed and multiplied
    cur_row = next_row;
    next_row = row_of(c0 + 2 * kLmChunk);
    __syncthreads();
    // element d of keys {4 gq + i, 16 + 4 gq + i} -> vt[d][8 gq ..]: the order in which a lane of the
    // first product holds its probabilities
    for (int gq = 0; gq < 4; ++gq)
      for (int d = tid; d < gm.R; d += blockDim.x) {
        const uint16_t* col = reinterpret_cast<const uint16_t*>(kt) + d;
        uint32_t x[4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          x[i] = (uint32_t)col[(4 * gq + 2 * i) * gm.ldk] | ((uint32_t)col[(4 * gq + 2 * i + 1) * gm.ldk] << 16);
          x[2 + i] = (uint32_t)col[(16 + 4 * gq + 2 * i) * gm.ldk] | ((uint32_t)col[(16 + 4 * gq + 2 * i + 1) * gm.ldk] << 16);
        }
        *reinterpret_cast<uint4*>(vt + d * kLmVtLd + 8 * gq) = make_uint4(x[0], x[1], x[2], x[3]);
      }
    __syncthreads();
    if (!wave_ok) continue;

    f32x4 s[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int j = 0; j < MAXD32; ++j) {
      if (j < gm.d32) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(kt + (16 * u + m16) * gm.ldk + 32 * j + 8 * g);
          s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[j], s[u], 0, 0, 0);
        }
      }
    }
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = c0 + 16 * u + 4 * g + i;
        const bool ok = row_ok && key < k_end && key <= p_row;
        sv[4 * u + i] = ok ? s[u][i] * scale : -INFINITY;
        mx = fmaxf(mx, sv[4 * u + i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m_run, mx);
    const float corr = m_run > -INFINITY ? expf(m_run - m_new) : 0.f;
    float pe[8], ps = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pe[i] = sv[i] > -INFINITY ? expf(sv[i] - m_new) : 0.f;
      ps += pe[i];
    }
    ps += __shfl_xor(ps, 16, kWave);
    ps += __shfl_xor(ps, 32, kWave);
    l_run = l_run * corr + ps;
    m_run = m_new;
    uint4 hi, lo;
    {
      float r[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) r[i] = pe[i] - bf16_to_f32(f32_to_bf16(pe[i]));
      hi = make_uint4(pack_bf16(pe[0], pe[1]), pack_bf16(pe[2], pe[3]), pack_bf16(pe[4], pe[5]), pack_bf16(pe[6], pe[7]));
      lo = make_uint4(pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]), pack_bf16(r[4], r[5]), pack_bf16(r[6], r[7]));
    }
    const bf16x8 pf_hi = *reinterpret_cast<bf16x8*>(&hi), pf_lo = *reinterpret_cast<bf16x8*>(&lo);
    if (__any(corr != 1.0f)) {             // some row's maximum moved: seldom, once the first chunks are through
#pragma unroll
      for (int d = 0; d < MAXH; ++d) {
        acc[d][0] *= corr; acc[d][1] *= corr; acc[d][2] *= corr; acc[d][3] *= corr;
      }
    }
#pragma unroll
    for (int d = 0; d < MAXH; ++d) {
      if (d < r_n) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vt + (16 * (r_lo + d) + m16) * kLmVtLd + 8 * g);
        const f32x4 a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_hi, acc[d], 0, 0, 0);
        acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_lo, a, 0, 0, 0);
      }
    }
  }

  if (!row_ok) return;
  const int n_runs = p_row / run_keys + 1;      // runs that hold keys of this row
  if (run >= n_runs) return;
  const size_t rh = (size_t)token * gm.H + head;
  if (n_runs == 1) {
    float M = m_run, denom = l_run;
    if (sink) {
      const float sk = sink[head];
      M = fmaxf(m_run, sk);
      denom = l_run * expf(m_run - M) + expf(sk - M);
    }
    const float f = denom > 0.f ? expf(m_run - M) / denom : 0.f;
    bf16_t* orow = out + rh * gm.R + 16 * r_lo;
#pragma unroll
    for (int d = 0; d < MAXH; ++d) {
      if (d < r_n) {
        uint2 v;
        v.x = pack_bf16(acc[d][0] * f, acc[d][1] * f);
        v.y = pack_bf16(acc[d][2] * f, acc[d][3] * f);
        *reinterpret_cast<uint2*>(orow + 16 * d + 4 * g) = v;
      }
    }
    return;
  }
  float* po = part_o + (rh * max_runs + run) * gm.R + 16 * r_lo;
#pragma unroll
  for (int d = 0; d < MAXH; ++d) {
    if (d < r_n) *reinterpret_cast<float4*>(po + 16 * d + 4 * g) = make_float4(acc[d][0], acc[d][1], acc[d][2], acc[d][3]);
  }
  if (g == 0 && half == 0) {
    part_ml[(rh * max_runs + run) * 2] = m_run;
    part_ml[(rh * max_runs + run) * 2 + 1] = l_run;
  }
}

// The rows with more than one run: out = sum_r o_r e^(m_r - M) / (sum_r l_r e^(m_r - M) + e^(sink - M)), a wave a
// (token, head) row, four rows a block.  The maximum and the denominator are taken with a lane a run
// (wave reductions in a fixed order), the output with a lane per four elements, runs in ascending order.
constexpr int kLmMergeWaves = 4;

__global__ __launch_bounds__(kLmMergeWaves* kWave) void attn_latent_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ positions,
    const int* __restrict__ token_list, const float* __restrict__ sink, bf16_t* __restrict__ out, int H, int R,
    int run_keys, int max_runs) {
  const int token = token_list ? token_list[blockIdx.x] : blockIdx.x;
  const int head = blockIdx.y * kLmMergeWaves + (threadIdx.x >> 6);
  const int lane = threadIdx.x & (kWave - 1);
  if (head >= H) return;
  const int n_runs = positions[token] / run_keys + 1;
  if (n_runs <= 1) return;
  const size_t rh = (size_t)token * H + head;
  bf16_t* orow = out + rh * R;
  if (n_runs > max_runs) {          // the launch was sized for fewer keys than this token sees: never a result over fewer keys
    for (int d = lane; d < R; d += kWave) orow[d].bits = 0x7fc0;
    return;
  }
  const float* ml = part_ml + rh * max_runs * 2;
  float mx = -INFINITY;
  for (int r = lane; r < n_runs; r += kWave) mx = fmaxf(mx, ml[2 * r]);
  float M = wave_max(mx);
  if (sink) M = fmaxf(M, sink[head]);
  float dl = 0.f;
  for (int r = lane; r < n_runs; r += kWave) dl += ml[2 * r + 1] * expf(ml[2 * r] - M);
  const float denom = wave_sum(dl) + (sink ? expf(sink[head] - M) : 0.f);
  const float inv = denom > 0.f ? 1.0f / denom : 0.f;
  const float w_lane = lane < n_runs ? expf(ml[2 * lane] - M) : 0.f;     // run r's weight sits in lane r (the first 64 runs)
  const float* po = part_o + rh * max_runs * R;
  for (int d0 = 0; d0 < R; d0 += 4 * kWave) {      // (every lane walks the loop: the weights come from other lanes)
    const int d = d0 + 4 * lane;
    const bool on = d < R;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int r = 0; r < n_runs; ++r) {
      const float wr = r < kWave ? __shfl(w_lane, r, kWave) : expf(ml[2 * r] - M);
      if (on) {
        const float4 v = *reinterpret_cast<const float4*>(po + (size_t)r * R + d);
        o.x += v.x * wr; o.y += v.y * wr; o.z += v.z * wr; o.w += v.w * wr;
      }
    }
    if (on) {
      uint2 pk;
      pk.x = pack_bf16(o.x * inv, o.y * inv);
      pk.y = pack_bf16(o.z * inv, o.w * inv);
      *reinterpret_cast<uint2*>(orow + d) = pk;
    }
  }
}

static int pow2_ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

static LmGeom lm_geom(int H, int R, int dr) {
  LmGeom g;
  g.H = H; g.R = R; g.D = R + dr;
  g.d32 = (g.D + 31) / 32;
  g.r16 = R / 16;
  g.hpw = H >= 16 ? 16 : pow2_ceil(H);
  g.tb = 16 / g.hpw;
  const int ht = ceil_div(H, g.hpw);
  g.htb = ht >= 4 ? 4 : pow2_ceil(ht);
  g.tgb = kLmWaves / g.htb;
  g.ldk = g.d32 * 32 + 8;
  return g;
}

// Whether the kernel takes these sizes: R a multiple of 16 up to 512, rows a multiple of 8 up to 640 wide.
SHARPI_EXPORT int sharpi_attention_latent_mfma_takes(int R, int dr) {
  return R > 0 && dr >= 0 && R % 16 == 0 && (R + dr) % 8 == 0 && R <= 512 && R + dr <= 640;
}

// Tokens of one request that a block of the kernel works on (the prompt tiles are cut into pieces of this many).
SHARPI_EXPORT int sharpi_attention_latent_mfma_block_tokens(int H) {
  const LmGeom g = lm_geom(H, 16, 0);
  return g.tgb * g.tb;
}

// q [T, H, R + dr] bfloat16; rows [pages * page_size, R + dr]; either tiles int32 [n_items, 3] = (entry,
// first token, rows <= tile_tokens) of consecutive tokens of one request, or n_items single tokens
// (token_list int32 [n_items], or null: tokens 0 .. n_items - 1).  part_o float [T * H * max_runs * R],
// part_ml float [T * H * max_runs * 2]: scratch for rows with keys in more than one run of run_keys
// (a multiple of 32); max_runs runs cover every token's keys.  out [T, H, R] bfloat16.
SHARPI_EXPORT int sharpi_attention_latent_mfma(const void* q, const void* rows, const int* block_table,
                                               const int* entry_of_token, const int* positions, const int* tiles,
                                               const int* token_list, int n_items, int tile_tokens,
                                               const float* sink, void* out, float* part_o, float* part_ml,
                                               float scale, int H, int R, int dr, int run_keys, int max_runs,
                                               int page_size, int max_blocks, int num_pages, hipStream_t stream) {
  if (n_items <= 0) return SHARPI_OK;
  if (!sharpi_attention_latent_mfma_takes(R, dr) || H <= 0) return SHARPI_ERR_ARG;
  if (run_keys <= 0 || run_keys % kLmChunk || max_runs <= 0 || max_runs > 65535) return SHARPI_ERR_ARG;
  if (page_size <= 0 || max_blocks <= 0 || num_pages <= 0 || (tiles && tile_tokens <= 0)) return SHARPI_ERR_ARG;
  const LmGeom g = lm_geom(H, R, dr);
  const int tpb = g.tgb * g.tb;
  const int subs = tiles ? ceil_div(tile_tokens, tpb) : 1;
  const int head_blocks = ceil_div(ceil_div(H, g.hpw), g.htb);
  if (head_blocks > 65535) return SHARPI_ERR_ARG;
  dim3 grid(n_items * subs, max_runs, head_blocks), block(kLmWaves * kLmHalves * kWave);
  const size_t lds = ((size_t)kLmChunk * g.ldk + (size_t)R * kLmVtLd) * sizeof(bf16_t);
#define LM_LAUNCH(MD, MR)                                                                                         \
  do {                                                                                                            \
    auto kern = attn_latent_mfma_kernel<MD, MR>;                                                                  \
    static size_t allowed = 48 * 1024;       /* dynamic LDS this instantiation may take (raised once per size) */  \
    if (lds > allowed) {                                                                                          \
      hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e_ != hipSuccess) return (int)e_;                                                                       \
      allowed = lds;                                                                                              \
    }                                                                                                             \
    kern<<<grid, block, lds, stream>>>((const bf16_t*)q, (const bf16_t*)rows, block_table, entry_of_token,        \
                                       positions, tiles, token_list, subs, sink, (bf16_t*)out, part_o, part_ml,   \
                                       scale, g, run_keys, max_runs, page_size, max_blocks, num_pages);           \
  } while (0)
  if (g.d32 <= 5 && g.r16 <= 8) LM_LAUNCH(5, 8);
  else if (g.d32 <= 10 && g.r16 <= 16) LM_LAUNCH(10, 16);
  else if (g.d32 <= 18) LM_LAUNCH(18, 32);      // rows of up to 576: eight registers fewer than the widest form, which spills
  else LM_LAUNCH(20, 32);
#undef LM_LAUNCH
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// The merge of the rows with more than one run: n_tokens tokens (token_list, or 0 .. n_tokens - 1).
SHARPI_EXPORT int sharpi_attention_latent_merge(const float* part_o, const float* part_ml, const int* positions,
                                                const int* token_list, int n_tokens, const float* sink, void* out,
                                                int H, int R, int run_keys, int max_runs, hipStream_t stream) {
  if (n_tokens <= 0 || max_runs <= 1) return SHARPI_OK;
  if (H <= 0 || H > 65535 || R <= 0 || R % 4 || run_keys <= 0) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens, ceil_div(H, kLmMergeWaves)), block(kLmMergeWaves * kWave);
  attn_latent_merge_kernel<<<grid, block, 0, stream>>>(part_o, part_ml, positions, token_list, sink, (bf16_t*)out, H, R,
                                                       run_keys, max_runs);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
