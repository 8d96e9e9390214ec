// Attention over a shared low-rank latent (one cached row per token for all heads).
//
// A token's cache row is [latent c (R lanes) | rotated key part (Dr lanes)]; the key page layout is that
// of every other attention of this library with one key head of R + Dr lanes, and there are no value
// pages: the values are the latent lanes of the same rows.  Queries come "absorbed": per head
// [W_uk^T q_plain (R lanes) | rotated query part (Dr lanes)] in float, so a score is one dot product of
// R + Dr lanes against the cache row, and a head's result is the probability-weighted sum of latents
// (R lanes), which the caller expands with W_uv.
//
// Kernels: the write of a step's tokens into the cache (RMS norm of the latent, rotation of the shared
// key part and of the queries' rotated parts), a small batched product per head, and the attention.
#include "common.h"

// ---------------------------------------------------------------------------------------
// down [T][ld_down]: R latent lanes then Dr key lanes.  q [T][ld_q], head h at h * (dn + Dr).  cos_sin [positions][half_t]
// (cos, sin), of which the first rot/2 pairs turn lanes (i, i + rot/2) of the Dr part, or (adjacent) lanes (2i, 2i + 1).
// qabs [T][H][R + Dr] (float or the cache's type) gets the rotated query parts at lane R.  vcache (may be null):
// pages [R][page] that receive the latent transposed, for the matrix-core attention.
// ---------------------------------------------------------------------------------------
template <typename TA, typename TQ>
__global__ void latent_write_kernel(const TA* __restrict__ down, int ld_down, const TA* __restrict__ q, int ld_q, int H, int dn,
                                    const float* __restrict__ norm_w, float eps, const float2* __restrict__ cos_sin,
                                    int half_t, int rot, TQ* __restrict__ qabs, TA* __restrict__ kcache, TA* __restrict__ vcache,
                                    const int* __restrict__ positions, const int* __restrict__ token_seq,
                                    const int* __restrict__ block_table, int table_width, int page_size, int R, int Dr,
                                    int write_kv, int adjacent) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  const int b = token_seq[t];
  if (b < 0) return;
  const int pos = positions[t];
  const float2* cs = cos_sin + (size_t)pos * half_t;
  const int half = rot >> 1;
  // queries: rotated parts into the absorbed rows
  for (int i = threadIdx.x; i < H * Dr; i += blockDim.x) {
    const int h = i / Dr, d = i - h * Dr;
    const TA* src = q + (size_t)t * ld_q + (size_t)h * (dn + Dr) + dn;
    float v = to_float(src[d]);
    if (d < rot) {
      const bool first = adjacent ? !(d & 1) : d < half;
      const int pair = adjacent ? d >> 1 : (d < half ? d : d - half);
      const float2 c = cs[pair];
      const float other = to_float(src[adjacent ? d ^ 1 : (d < half ? d + half : d - half)]);
      v = first ? v * c.x - other * c.y : v * c.x + other * c.y;
    }
    qabs[((size_t)t * H + h) * (R + Dr) + R + d] = from_float<TQ>(v);
  }
  const int page = block_table[(size_t)b * table_width + pos / page_size];
  if (!write_kv || page < 0) return;
  const TA* row = down + (size_t)t * ld_down;
  TA* dst = kcache + ((size_t)page * page_size + (pos % page_size)) * (R + Dr);
  float ss = 0.f;
  for (int d = threadIdx.x; d < R; d += blockDim.x) {
    const float v = to_float(row[d]);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum<true>(ss, red) / (float)R + eps);
  TA* vdst = vcache ? vcache + (size_t)page * R * page_size + (pos % page_size) : nullptr;   // transposed page [R][page]
  for (int d = threadIdx.x; d < R; d += blockDim.x) {
    const TA c = from_float<TA>(to_float(row[d]) * inv * norm_w[d]);
    dst[d] = c;
    if (vdst) vdst[(size_t)d * page_size] = c;
  }
  for (int d = threadIdx.x; d < Dr; d += blockDim.x) {
    float v = to_float(row[R + d]);
    if (d < rot) {
      const bool first = adjacent ? !(d & 1) : d < half;
      const int pair = adjacent ? d >> 1 : (d < half ? d : d - half);
      const float2 c = cs[pair];
      const float other = to_float(row[R + (adjacent ? d ^ 1 : (d < half ? d + half : d - half))]);
      v = first ? v * c.x - other * c.y : v * c.x + other * c.y;
    }
    dst[R + d] = from_float<TA>(v);
  }
}

extern "C" int blm_latent_write(const void* down, int ld_down, const void* q, int ld_q, int dtype, int T, int H, int dn,
                                const float* norm_w, float eps, const void* cos_sin, int half_t, int rot, void* qabs,
                                int qabs_dtype, void* kcache, void* vcache, const int* positions, const int* token_seq, const int* block_table,
                                int table_width, int page_size, int R, int Dr, int write_kv, int adjacent, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && H > 0 && dn >= 0 && R > 0 && Dr >= 0, "latent_write: bad sizes");
  BLM_REQUIRE(rot % 2 == 0 && rot >= 0 && rot <= Dr && rot / 2 <= half_t, "latent_write: %d turning lanes do not fit %d", rot, Dr);
  BLM_REQUIRE(page_size > 0 && table_width > 0 && ld_down >= R + Dr && ld_q >= H * (dn + Dr), "latent_write: bad geometry");
#define BLM_LW(TA, TQ)                                                                                                  \
  hipLaunchKernelGGL((latent_write_kernel<TA, TQ>), dim3(T), dim3(256), 0, stream, (const TA*)down, ld_down, (const TA*)q, \
                     ld_q, H, dn, norm_w, eps, (const float2*)cos_sin, half_t, rot, (TQ*)qabs, (TA*)kcache, (TA*)vcache,  \
                     positions, token_seq, block_table, table_width, page_size, R, Dr, write_kv, adjacent)
  if (dtype == BLM_F32 && qabs_dtype == BLM_F32) BLM_LW(float, float);
  else if (dtype == BLM_BF16 && qabs_dtype == BLM_F32) BLM_LW(bf16, float);
  else if (dtype == BLM_BF16 && qabs_dtype == BLM_BF16) BLM_LW(bf16, bf16);
  else return blm_fail("latent_write: unsupported dtypes %d / %d", dtype, qabs_dtype);
#undef BLM_LW
  BLM_LAUNCH_CHECK("latent_write");
  return 0;
}

// ---------------------------------------------------------------------------------------
// RMS norm of a slice of rows: out[t][d] = x[t][d] / sqrt(mean_d(x[t]^2) + eps) * w[d] for d < N; x [T][ld] (any row
// stride), out [T][N] contiguous in x's type, w float.  Sums and scaling in float.  (A latent between two projections.)
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void rmsnorm_rows_kernel(const TA* __restrict__ x, int ld, const float* __restrict__ w, float eps,
                                    TA* __restrict__ out, int N) {
  __shared__ float red[17];
  const TA* row = x + (size_t)blockIdx.x * ld;
  float ss = 0.f;
  for (int d = threadIdx.x; d < N; d += blockDim.x) {
    const float v = to_float(row[d]);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum<true>(ss, red) / (float)N + eps);
  TA* o = out + (size_t)blockIdx.x * N;
  for (int d = threadIdx.x; d < N; d += blockDim.x) o[d] = from_float<TA>(to_float(row[d]) * inv * w[d]);
}

extern "C" int blm_rmsnorm_rows(const void* x, int ld, int dtype, const float* w, float eps, void* out, int T, int N,
                                hipStream_t stream) {
  BLM_REQUIRE(T > 0 && N > 0 && ld >= N, "rmsnorm_rows: bad sizes T=%d N=%d rows of %d", T, N, ld);
  const int threads = N <= 64 ? 64 : N <= 128 ? 128 : 256;
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(rmsnorm_rows_kernel<float>, dim3(T), dim3(threads), 0, stream, (const float*)x, ld, w, eps, (float*)out, N);
  else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(rmsnorm_rows_kernel<bf16>, dim3(T), dim3(threads), 0, stream, (const bf16*)x, ld, w, eps, (bf16*)out, N);
  else
    return blm_fail("rmsnorm_rows: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("rmsnorm_rows");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Batched product per head: out[t][h][n] = sum_k in[t][h][k] * w[h][n][k], float accumulation.
// in: rows of `in_row` elements, head h at h * in_head; out likewise; w [H][N][K] contiguous.
// 64 x 64 tile per block of 256 threads, 16 of K per stage in shared memory, 4 x 4 results per thread.
// ---------------------------------------------------------------------------------------
#define HP_TILE 64
#define HP_K 16
template <typename TI, typename TW, typename TO>
__global__ void __launch_bounds__(256)
    head_project_kernel(const TI* __restrict__ in, long long in_row, int in_head, const TW* __restrict__ w,
                        TO* __restrict__ out, long long out_row, int out_head, int T, int N, int K) {
  __shared__ float sa[HP_K][HP_TILE + 1], sb[HP_K][HP_TILE + 1];
  const int h = blockIdx.z;
  const int t0 = blockIdx.x * HP_TILE, n0 = blockIdx.y * HP_TILE;
  const TI* a = in + (size_t)h * in_head;
  const TW* bw = w + (size_t)h * N * K;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += HP_K) {
    for (int i = threadIdx.x; i < HP_TILE * HP_K; i += 256) {
      const int r = i / HP_K, k = i - r * HP_K;
      const int t = t0 + r, n = n0 + r, kk = k0 + k;
      sa[k][r] = (t < T && kk < K) ? to_float(a[(size_t)t * in_row + kk]) : 0.f;
      sb[k][r] = (n < N && kk < K) ? to_float(bw[(size_t)n * K + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < HP_K; ++k) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = sa[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = sb[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty * 4 + i;
    if (t >= T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[(size_t)t * out_row + (size_t)h * out_head + n] = from_float<TO>(acc[i][j]);
    }
  }
}

// The same for few rows (decoding): one wavefront per output column (h, n) streams that row of w once, its lanes
// taking k = lane, lane + 64, ...; the rows' inputs come from the caches.  Up to HP_FEW rows.
#define HP_FEW 16
template <typename TI, typename TW, typename TO>
__global__ void __launch_bounds__(256)
    head_project_few_kernel(const TI* __restrict__ in, long long in_row, int in_head, const TW* __restrict__ w,
                            TO* __restrict__ out, long long out_row, int out_head, int T, int H, int N, int K) {
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long col = (long long)blockIdx.x * 4 + wave;
  if (col >= (long long)H * N) return;
  const int h = (int)(col / N), n = (int)(col - (long long)h * N);
  const TW* wr = w + ((size_t)h * N + n) * K;
  const TI* a = in + (size_t)h * in_head;
  float acc[HP_FEW];
#pragma unroll
  for (int t = 0; t < HP_FEW; ++t) acc[t] = 0.f;
  for (int k = lane; k < K; k += BLM_WAVE) {
    const float wv = to_float(wr[k]);
#pragma unroll
    for (int t = 0; t < HP_FEW; ++t)
      if (t < T) acc[t] = fmaf(to_float(a[(size_t)t * in_row + k]), wv, acc[t]);
  }
#pragma unroll
  for (int t = 0; t < HP_FEW; ++t) {
    if (t < T) {
      const float v = wave_sum(acc[t]);
      if (lane == 0) out[(size_t)t * out_row + (size_t)h * out_head + n] = from_float<TO>(v);
    }
  }
}

extern "C" int blm_head_project(const void* in, int in_dtype, long long in_row, int in_head, const void* w, int w_dtype,
                                void* out, int out_dtype, long long out_row, int out_head, int T, int H, int N, int K,
                                hipStream_t stream) {
  BLM_REQUIRE(T > 0 && H > 0 && N > 0 && K > 0 && H <= 65535, "head_project: bad sizes T=%d H=%d N=%d K=%d", T, H, N, K);
  dim3 grid((T + HP_TILE - 1) / HP_TILE, (N + HP_TILE - 1) / HP_TILE, H), block(256);
  BLM_REQUIRE(grid.y <= 65535, "head_project: too many columns");
  const unsigned few_blocks = (unsigned)(((long long)H * N + 3) / 4);
#define BLM_HP(TI, TW, TO)                                                                                       \
  if (T <= HP_FEW)                                                                                               \
    hipLaunchKernelGGL((head_project_few_kernel<TI, TW, TO>), dim3(few_blocks), block, 0, stream, (const TI*)in, \
                       in_row, in_head, (const TW*)w, (TO*)out, out_row, out_head, T, H, N, K);                  \
  else                                                                                                           \
    hipLaunchKernelGGL((head_project_kernel<TI, TW, TO>), grid, block, 0, stream, (const TI*)in, in_row, in_head, \
                       (const TW*)w, (TO*)out, out_row, out_head, T, N, K)
  if (in_dtype == BLM_F32 && w_dtype == BLM_F32 && out_dtype == BLM_F32) { BLM_HP(float, float, float); }
  else if (in_dtype == BLM_BF16 && w_dtype == BLM_BF16 && out_dtype == BLM_F32) { BLM_HP(bf16, bf16, float); }
  else if (in_dtype == BLM_F32 && w_dtype == BLM_BF16 && out_dtype == BLM_BF16) { BLM_HP(float, bf16, bf16); }
  else if (in_dtype == BLM_BF16 && w_dtype == BLM_BF16 && out_dtype == BLM_BF16) { BLM_HP(bf16, bf16, bf16); }
  else if (in_dtype == BLM_F32 && w_dtype == BLM_BF16 && out_dtype == BLM_F32) { BLM_HP(float, bf16, float); }
  else return blm_fail("head_project: unsupported dtypes in=%d w=%d out=%d", in_dtype, w_dtype, out_dtype);
#undef BLM_HP
  BLM_LAUNCH_CHECK("head_project");
  return 0;
}

// ---------------------------------------------------------------------------------------
// The attention, generic form: one wavefront per (query token, head); prompts and decoding alike.
// Query at position p of its sequence sees rows j <= p of the same sequence.  A chunk of 64 rows at a
// time: every lane scores one row (R + Dr lanes against the query in shared memory), the running maximum
// and sum follow, then every lane owns latent lanes lane, lane + 64, ... of the weighted sum and walks the
// chunk's rows.  With n_splits > 1 the rows of a (token, head) are cut into pieces for different
// wavefronts, whose partial results the last one to arrive merges (as in the generic attention).
// olat [T][H][R] float.
// ---------------------------------------------------------------------------------------
#define LAT_WAVES 4
#define LAT_MAX_R 1024
template <typename TA>
__global__ void __launch_bounds__(LAT_WAVES* BLM_WAVE)
    latent_attn_kernel(const float* __restrict__ qabs, float* __restrict__ olat, const int* __restrict__ positions,
                       const int* __restrict__ token_seq, const int* __restrict__ block_table, int table_width,
                       const TA* __restrict__ kcache, int page_size, int T, int H, int R, int Dr, float scale,
                       int n_splits, float* part_o, float* part_ml, int* arrivals) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int W = R + Dr;
  const long long item = (long long)blockIdx.x * LAT_WAVES + wave;
  const bool active = item < (long long)T * H;
  const int t = active ? (int)(item / H) : 0;
  const int b = active ? token_seq[t] : -1;
  float* qs = smem + (size_t)wave * W;
  if (active && b >= 0) {
    const float* qrow = qabs + (size_t)item * W;
    for (int d = lane; d < W; d += BLM_WAVE) qs[d] = qrow[d];
  }
  __syncthreads();
  if (!active) return;
  float* orow = olat + (size_t)item * R;
  if (b < 0) {
    for (int d = lane; d < R; d += BLM_WAVE) orow[d] = 0.f;
    return;
  }
  const int pos = positions[t];
  const int* bt = block_table + (size_t)b * table_width;
  const int split = blockIdx.y;
  const int n_chunks = pos / BLM_WAVE + 1;
  const int per_split = (n_chunks + n_splits - 1) / n_splits;
  const int j_begin = split * per_split * BLM_WAVE;
  const int j_end = min(pos, j_begin + per_split * BLM_WAVE - 1);

  float m = -INFINITY, l = 0.f;
  float acc[LAT_MAX_R / BLM_WAVE];
#pragma unroll
  for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) acc[i] = 0.f;
  const bool vec = (W % 8) == 0;

  for (int j0 = j_begin; j0 <= j_end; j0 += BLM_WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= j_end;
    float s = -INFINITY;
    if (valid) {
      const int page = bt[j / page_size];
      const TA* krow = kcache + ((size_t)page * page_size + (j % page_size)) * W;
      float dot = 0.f;
      if (vec && sizeof(TA) == 2) {
        for (int d = 0; d < W; d += 8) {
          const uint4 raw = *reinterpret_cast<const uint4*>(krow + d);
          const uint32_t ws[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            dot = fmaf(qs[d + 2 * i], __uint_as_float(ws[i] << 16), dot);
            dot = fmaf(qs[d + 2 * i + 1], __uint_as_float(ws[i] & 0xffff0000u), dot);
          }
        }
      } else {
        for (int d = 0; d < W; ++d) dot = fmaf(qs[d], to_float(krow[d]), dot);
      }
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) acc[i] *= corr;
    const int cnt = (j_end - j0 + 1) < BLM_WAVE ? (j_end - j0 + 1) : BLM_WAVE;
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = __shfl(p, jj, BLM_WAVE);
      const int ja = j0 + jj;
      const int page = bt[ja / page_size];
      const TA* crow = kcache + ((size_t)page * page_size + (ja % page_size)) * W;
#pragma unroll
      for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) {
        const int d = lane + i * BLM_WAVE;
        if (d < R) acc[i] = fmaf(pj, to_float(crow[d]), acc[i]);
      }
    }
    m = m_new;
  }
  if (n_splits == 1) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) {
      const int d = lane + i * BLM_WAVE;
      if (d < R) orow[d] = acc[i] * inv;
    }
    return;
  }
  float* po = part_o + ((size_t)item * n_splits + split) * R;
#pragma unroll
  for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) {
    const int d = lane + i * BLM_WAVE;
    if (d < R) __hip_atomic_store(po + d, acc[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (lane == 0) {
    __hip_atomic_store(part_ml + ((size_t)item * n_splits + split) * 2, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(part_ml + ((size_t)item * n_splits + split) * 2 + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the wavefront's stores have been acknowledged
  int last = 0;
  if (lane == 0) {
    const int before = __hip_atomic_fetch_add(arrivals + item, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = before == n_splits - 1;
    if (last) __hip_atomic_store(arrivals + item, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  last = __shfl(last, 0, BLM_WAVE);
  if (!last) return;
  float M = -INFINITY, L = 0.f;
  float O[LAT_MAX_R / BLM_WAVE];
#pragma unroll
  for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) O[i] = 0.f;
  for (int sp = 0; sp < n_splits; ++sp) {
    const float* ml = part_ml + ((size_t)item * n_splits + sp) * 2;
    const float ms = __hip_atomic_load(ml, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float ls = __hip_atomic_load(ml + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (ls == 0.f) continue;
    const float Mn = fmaxf(M, ms);
    const float keep = expf(M - Mn), take = expf(ms - Mn);
    L = L * keep + ls * take;
    const float* ps = part_o + ((size_t)item * n_splits + sp) * R;
#pragma unroll
    for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) {
      const int d = lane + i * BLM_WAVE;
      if (d < R) O[i] = O[i] * keep + __hip_atomic_load(ps + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * take;
    }
    M = Mn;
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int i = 0; i < LAT_MAX_R / BLM_WAVE; ++i) {
    const int d = lane + i * BLM_WAVE;
    if (d < R) orow[d] = O[i] * inv;
  }
}

// part_o: T*H*n_splits*R floats, part_ml: T*H*n_splits*2 floats, arrivals: T*H ints, zero before the
// first call and left zero; all three may be null when n_splits is 1.
extern "C" int blm_latent_attn(const float* qabs, float* olat, int cache_dtype, const int* positions,
                               const int* token_seq, const int* block_table, int table_width, const void* kcache,
                               int page_size, int T, int H, int R, int Dr, float scale, int n_splits, float* part_o,
                               float* part_ml, int* arrivals, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && H > 0 && R > 0 && Dr >= 0, "latent_attn: bad sizes T=%d H=%d R=%d Dr=%d", T, H, R, Dr);
  BLM_REQUIRE(R <= LAT_MAX_R, "latent_attn: a latent of %d lanes is more than %d", R, LAT_MAX_R);
  BLM_REQUIRE(page_size > 0 && table_width > 0, "latent_attn: bad cache geometry");
  BLM_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || (part_o && part_ml && arrivals)),
              "latent_attn: %d splits need their workspace", n_splits);
  const long long items = (long long)T * H;
  const long long blocks = (items + LAT_WAVES - 1) / LAT_WAVES;
  BLM_REQUIRE(blocks < 2147483647LL, "latent_attn: too many (token, head) pairs");
  const size_t smem = (size_t)LAT_WAVES * (R + Dr) * sizeof(float);
  BLM_REQUIRE(smem <= 64 * 1024, "latent_attn: query rows of %d lanes do not fit shared memory", R + Dr);
  dim3 grid((unsigned)blocks, (unsigned)n_splits), block(LAT_WAVES * BLM_WAVE);
  if (cache_dtype == BLM_F32)
    hipLaunchKernelGGL(latent_attn_kernel<float>, grid, block, smem, stream, qabs, olat, positions, token_seq, block_table,
                       table_width, (const float*)kcache, page_size, T, H, R, Dr, scale, n_splits, part_o, part_ml, arrivals);
  else if (cache_dtype == BLM_BF16)
    hipLaunchKernelGGL(latent_attn_kernel<bf16>, grid, block, smem, stream, qabs, olat, positions, token_seq, block_table,
                       table_width, (const bf16*)kcache, page_size, T, H, R, Dr, scale, n_splits, part_o, part_ml, arrivals);
  else
    return blm_fail("latent_attn: unsupported dtype %d", cache_dtype);
  BLM_LAUNCH_CHECK("latent_attn");
  return 0;
}

// ---------------------------------------------------------------------------------------
// The attention on the matrix cores (bfloat16 cache and queries, float softmax and accumulation).
//
// All heads share the cached rows, so the 16 "query columns" of a wavefront are 16 consecutive (token, head)
// pairs of one sequence, each with its own position.  Per page of 64 rows:
//   S^T = K Q^T      A = 16 cache rows x 32 lanes of [latent | key part] per instruction, B = Q^T; lane
//                    (kg, c) gets the scores of column c for rows kg*4 .. kg*4+3 of each 16-row tile
//   O^T += V^T P^T   A = 16 latent lanes x 32 rows from the transposed latent pages ([R][64] per page),
//                    B = the probabilities the lane has just computed.  The rows of a page are dealt to the
//                    four score tiles so that the eight rows a lane supplies are neighbours in the
//                    transposed page (lat_key_of), as in this library's other matrix-core attention.
// Fragments come straight from global memory (the pages of a sequence are shared by all its wavefronts and
// stay in the caches); no shared memory, no barriers.  With n_splits > 1 the pages of a wavefront's columns
// are cut into pieces whose partial results a second kernel adds up.
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 lat_bf16x8;
typedef __attribute__((ext_vector_type(4))) float lat_f32x4;

__device__ __forceinline__ constexpr int lat_key_of(int t, int i) { return (t >> 1) * 32 + (i >> 2) * 8 + (t & 1) * 4 + (i & 3); }

// keep the first n (0..8) bf16 of a 16-byte group, zero the rest
__device__ __forceinline__ uint4 lat_keep_first(uint4 v, int n) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int left = n - 2 * i;
    w[i] = left >= 2 ? w[i] : (left == 1 ? (w[i] & 0xffffu) : 0u);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

#define LATM_WAVES 4
template <int R, int DR>
__global__ void __launch_bounds__(LATM_WAVES* BLM_WAVE)
    latent_attn_mfma_kernel(const bf16* __restrict__ q, float* __restrict__ olat, const int* __restrict__ cu_seqlens,
                            const int* __restrict__ lens_after, const int* __restrict__ block_table, int table_width,
                            const bf16* __restrict__ kcache, const bf16* __restrict__ vcache, int B, int H,
                            int tiles_per_seq, float scale2, int n_splits, float* part_o, float* part_ml) {
  constexpr int W = R + DR;
  constexpr int KS = (W + 31) / 32;
  constexpr int DT = R / 16;
  static_assert(R % 16 == 0 && W % 8 == 0, "latent lanes in tiles of 16, rows in pieces of 16 bytes");
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int c = lane & 15, kg = lane >> 4;
  const int tile_id = blockIdx.x * LATM_WAVES + wave;          // over sequences x tiles of 16 columns
  const int b = tile_id / tiles_per_seq, tile = tile_id - b * tiles_per_seq;
  if (b >= B) return;                                            // the last block's surplus wavefronts
  const int split = blockIdx.y;
  const int t_first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_first;
  const int n_cols = n_new * H;
  if (tile * 16 >= n_cols) return;                               // also a padding sequence
  const int after = lens_after[b];
  const int past = after - n_new;
  // this lane's column
  const int idx = tile * 16 + c;
  const bool valid = idx < n_cols;
  const int tok = valid ? idx / H : 0, head = valid ? idx - tok * H : 0;
  const int qpos = valid ? past + tok : -1;
  const size_t item = (size_t)(t_first + tok) * H + head;
  // the last column of the tile sees the most
  const int last_idx = min(tile * 16 + 15, n_cols - 1);
  const int max_qpos = past + last_idx / H;
  const int max_key = after - 1;
  const int n_pages = max_qpos / 64 + 1;
  const int per = (n_pages + n_splits - 1) / n_splits;
  const int p_begin = split * per, p_end = min(n_pages, p_begin + per);
  const int* bt = block_table + (size_t)b * table_width;

  uint4 qf[KS];
  {
    const bf16* qrow = q + item * W;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + kg * 8;
      qf[ks] = (valid && (W % 32 == 0 || d < W)) ? *reinterpret_cast<const uint4*>(qrow + d) : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  float m = -INFINITY;
  lat_f32x4 l = {0.f, 0.f, 0.f, 0.f};
  lat_f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = lat_f32x4{0.f, 0.f, 0.f, 0.f};

  for (int pi = p_begin; pi < p_end; ++pi) {
    const int page = bt[pi];
    const int key0 = pi * 64;
    const bf16* kp = kcache + (size_t)page * 64 * W;
    const bf16* vp = vcache + (size_t)page * R * 64;
    float s[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bf16* krow = kp + (size_t)lat_key_of(t, c) * W;
      uint4 kf[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + kg * 8;
        kf[ks] = (W % 32 == 0 || d < W) ? *reinterpret_cast<const uint4*>(krow + d) : make_uint4(0u, 0u, 0u, 0u);
      }
      lat_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lat_bf16x8, kf[ks]),
                                                      __builtin_bit_cast(lat_bf16x8, qf[ks]), acc, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kj = key0 + lat_key_of(t, kg * 4 + r);
        s[t][r] = kj <= qpos ? acc[r] : -INFINITY;      // whatever the rows past the data hold, it is replaced here
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = blm_max(mx, s[t][r]);
    mx = rows_max(mx);
    const float m_new = blm_max(m, mx * scale2);
    const float corr = (m == m_new) ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        s[t][r] = (s[t][r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], scale2, -m_new));
    if (__any(m != m_new)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[dt][r] *= corr;
#pragma unroll
      for (int r = 0; r < 4; ++r) l[r] *= corr;
    }
    m = m_new;
    const bool tail = key0 + 63 > max_key;       // the page holds places past the data: 0 * garbage must stay 0
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint4 pf;
      pf.x = f32x2_to_bf16x2_bits(s[2 * h][0], s[2 * h][1]);
      pf.y = f32x2_to_bf16x2_bits(s[2 * h][2], s[2 * h][3]);
      pf.z = f32x2_to_bf16x2_bits(s[2 * h + 1][0], s[2 * h + 1][1]);
      pf.w = f32x2_to_bf16x2_bits(s[2 * h + 1][2], s[2 * h + 1][3]);
      // the softmax's denominator: a row of ones in place of V^T sums the rounded probabilities of every column
      l = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          __builtin_bit_cast(lat_bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u)),
          __builtin_bit_cast(lat_bf16x8, pf), l, 0, 0, 0);
      const int keep = max_key - (key0 + h * 32 + kg * 8) + 1;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        uint4 va = *reinterpret_cast<const uint4*>(vp + (size_t)(dt * 16 + c) * 64 + h * 32 + kg * 8);
        if (tail) va = lat_keep_first(va, keep);
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lat_bf16x8, va),
                                                        __builtin_bit_cast(lat_bf16x8, pf), o[dt], 0, 0, 0);
      }
    }
  }
  float* orow = olat + item * R;
  if (n_splits == 1) {
    if (valid) {
      const float inv = 1.0f / l[0];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        *reinterpret_cast<float4*>(orow + dt * 16 + kg * 4) = make_float4(o[dt][0] * inv, o[dt][1] * inv, o[dt][2] * inv, o[dt][3] * inv);
    }
    return;
  }
  // leave this piece: per column its maximum, sum and unnormalised result; latent_merge_kernel adds the pieces up
  const size_t gcol = (size_t)tile_id * 16 + c;
  float* po = part_o + (gcol * n_splits + split) * R;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    *reinterpret_cast<float4*>(po + dt * 16 + kg * 4) = make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
  if (kg == 0) {
    part_ml[(gcol * n_splits + split) * 2] = m;
    part_ml[(gcol * n_splits + split) * 2 + 1] = l[0];
  }
}

// The pieces of a split run added up, one block per column (a (token, head) pair): maxima in base 2.  A piece
// that saw nothing has sum 0, maximum -infinity and a result of zeros, and gets weight 0.
#define LATM_MERGE_THREADS 256
#define LATM_MAX_PIECES 64
__global__ void __launch_bounds__(LATM_MERGE_THREADS)
    latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, float* __restrict__ olat,
                        const int* __restrict__ cu_seqlens, int H, int R, int tiles_per_seq, int n_splits) {
  __shared__ float wgt[LATM_MAX_PIECES];
  __shared__ float inv_sum;
  const int gcol = blockIdx.x;
  const int per_seq = tiles_per_seq * 16;
  const int b = gcol / per_seq, idx = gcol - b * per_seq;
  const int t_first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_first;
  if (idx >= n_new * H) return;
  const int tok = idx / H, head = idx - tok * H;
  float* orow = olat + ((size_t)(t_first + tok) * H + head) * R;
  const float* ml = part_ml + (size_t)gcol * n_splits * 2;
  if (threadIdx.x < BLM_WAVE) {          // n_splits <= 64: one lane per piece
    const bool has = (int)threadIdx.x < n_splits;
    const float ms = has ? ml[threadIdx.x * 2] : -INFINITY, ls = has ? ml[threadIdx.x * 2 + 1] : 0.f;
    const float M = wave_max(ls != 0.f ? ms : -INFINITY);
    const float w = ls != 0.f ? __builtin_amdgcn_exp2f(ms - M) : 0.f;
    const float L = wave_sum(ls * w);
    if (has) wgt[threadIdx.x] = w;
    if (threadIdx.x == 0) inv_sum = 1.0f / L;
  }
  __syncthreads();
  const float* po = part_o + (size_t)gcol * n_splits * R;
  for (int d = threadIdx.x; d < R; d += LATM_MERGE_THREADS) {
    float acc = 0.f;
    for (int sp = 0; sp < n_splits; ++sp) acc = fmaf(po[(size_t)sp * R + d], wgt[sp], acc);
    orow[d] = acc * inv_sum;
  }
}

// the sizes the matrix-core form is built for (latent lanes, turned key lanes)
#define BLM_LATM_SIZES(X)                                                                                    \
  X(512, 64) X(512, 32) X(384, 64) X(256, 64) X(256, 32) X(192, 64) X(192, 32) X(160, 32) X(128, 64) X(128, 32) \
  X(128, 16) X(96, 32) X(96, 16) X(64, 64) X(64, 32) X(64, 16) X(48, 16) X(32, 16) X(32, 8)

extern "C" int blm_latent_attn_mfma_supported(int R, int Dr) {
#define BLM_LATM_HAS(r, d) if (R == r && Dr == d) return 1;
  BLM_LATM_SIZES(BLM_LATM_HAS)
#undef BLM_LATM_HAS
  return 0;
}

// q: bfloat16 [T][H][R + Dr]; olat float [T][H][R]; key pages [pages][1][64][R + Dr], transposed latent pages
// [pages][1][R][64], both bfloat16.  B sequences of at most max_new tokens.  Workspace for n_splits > 1:
// part_o (B * tiles * 16 * n_splits * R floats), part_ml (... * 2), with tiles = ceil(max_new * H / 16).
extern "C" int blm_latent_attn_mfma(const void* q, float* olat, const int* cu_seqlens, const int* lens_after,
                                    const int* block_table, int table_width, const void* kcache, const void* vcache,
                                    int page_size, int B, int max_new, int H, int R, int Dr, float scale, int n_splits,
                                    float* part_o, float* part_ml, hipStream_t stream) {
  BLM_REQUIRE(B > 0 && max_new > 0 && H > 0, "latent_attn_mfma: bad sizes B=%d max_new=%d H=%d", B, max_new, H);
  BLM_REQUIRE(page_size == 64 && table_width > 0, "latent_attn_mfma: pages of 64 rows");
  BLM_REQUIRE(n_splits >= 1 && n_splits <= LATM_MAX_PIECES && (n_splits == 1 || (part_o && part_ml)),
              "latent_attn_mfma: %d pieces (1 to %d, with their workspace)", n_splits, LATM_MAX_PIECES);
  const long long tiles = ((long long)max_new * H + 15) / 16;
  const long long waves = (long long)B * tiles;
  BLM_REQUIRE(waves < 2147483647LL, "latent_attn_mfma: too many tiles");
  const unsigned blocks = (unsigned)((waves + LATM_WAVES - 1) / LATM_WAVES);
  const float scale2 = scale * 1.4426950408889634f;
  dim3 grid(blocks, (unsigned)n_splits);
#define BLM_LATM_CASE(r, d)                                                                                            \
  if (R == r && Dr == d) {                                                                                             \
    hipLaunchKernelGGL((latent_attn_mfma_kernel<r, d>), grid, dim3(LATM_WAVES * BLM_WAVE), 0, stream, (const bf16*)q,  \
                       olat, cu_seqlens, lens_after, block_table, table_width, (const bf16*)kcache, (const bf16*)vcache, \
                       B, H, (int)tiles, scale2, n_splits, part_o, part_ml);                                           \
    BLM_LAUNCH_CHECK("latent_attn_mfma");                                                                              \
    if (n_splits > 1) {                                                                                                \
      hipLaunchKernelGGL(latent_merge_kernel, dim3((unsigned)(waves * 16)), dim3(LATM_MERGE_THREADS), 0, stream, part_o, part_ml, \
                         olat, cu_seqlens, H, R, (int)tiles, n_splits);                                                \
      BLM_LAUNCH_CHECK("latent_merge");                                                                                \
    }                                                                                                                  \
    return 0;                                                                                                          \
  }
  BLM_LATM_SIZES(BLM_LATM_CASE)
#undef BLM_LATM_CASE
  return blm_fail("latent_attn_mfma: a latent of %d + %d lanes is not among the sizes it is built for", R, Dr);
}
