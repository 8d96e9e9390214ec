// Attention over the paged cache whose softmax has a sink (one learned logit per head that takes its share of
// the denominator and has no key and no value) and whose weights are mixed between the heads afterwards
// ("talking heads": weight'_h(i, j) = sum_g M[h][g] weight_g(i, j), head h then reads the values of its own
// key-value head).  Keys and values may have head sizes of their own; a window limits how far back a query sees.
//
// The mixing is linear, so it is moved behind the sum over the keys:
//   out_h = sum_g M[h][g] * A[g][c(h)],   A[g][c] = sum_j weight_g(i, j) v_c(j),   c(h) the key-value head of h
// One wavefront per (token, head g) walks the visible keys once with a running maximum and sum (which start
// at the sink's logit and at one), and keeps one accumulator per key-value head c; a second kernel mixes.
// Scores, maxima, sums and accumulators are float.  Key pages [kv head][token][dk], value pages [kv head][dv][token].
//
// Also here: what comes between the q/k/v projection and the attention: bias, rotation of the first lanes of
// every query and key head by the token's position (lane i paired with lane i + rot/2), and the write of the
// rotated keys and the values into the token's place of the pages.
#include "common.h"

#define SA_MAX_DV_REGS 4      // value lanes per head up to 64 * this
#define SA_MAX_DK 512

// ---------------------------------------------------------------------------------------
// qkv [T][ld]: queries at column 0 (H * dk), then (if keys are written) keys (G * dk) and values (G * dv).
// bias [H*dk (+ G*dk + G*dv)] float or null.  cos_sin [positions][rot/2][2] float.  adjacent: pair i of the turning
// lanes is (2i, 2i + 1) instead of (i, i + rot/2).  values_are_keys (dv = dk): there are no value columns; a token's
// values are its keys as projected (with their bias), before the rotation.  q_scale [H] float or null: every lane of
// query head h is multiplied by q_scale[h] behind the rotation (a temperature per head: the scores are linear in it).
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void qkv_prepare_kernel(TA* __restrict__ qkv, int ld, const float* __restrict__ bias,
                                   const float* __restrict__ cos_sin, int rot, const int* __restrict__ positions,
                                   const int* __restrict__ token_seq, const int* __restrict__ block_table, int table_width,
                                   TA* __restrict__ kcache, TA* __restrict__ vcache, int page_size, int H, int G, int dk,
                                   int dv, int write_kv, int adjacent, int values_are_keys,
                                   const float* __restrict__ q_scale) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  if (b < 0) return;
  const int pos = positions[t];
  TA* row = qkv + (size_t)t * ld;
  const int half = rot / 2;
  const float* cs = cos_sin + (size_t)pos * half * 2;
  const int n_rot_heads = H + (write_kv ? G : 0);
  int page = 0, in_page = 0;
  if (write_kv) {
    page = block_table[(size_t)b * table_width + pos / page_size];
    in_page = pos % page_size;
  }
  // rotating pairs and the lanes behind them, head by head (queries, then keys)
  const int per_head = half + (dk - rot);
  for (int e = threadIdx.x; e < n_rot_heads * per_head; e += blockDim.x) {
    const int head = e / per_head, i = e - head * per_head;
    const int col = head * dk;
    TA* krow = head >= H ? kcache + (((size_t)page * G + (head - H)) * page_size + in_page) * dk : nullptr;
    const float f = (q_scale && head < H) ? q_scale[head] : 1.0f;
    if (i < half) {
      const int la = adjacent ? 2 * i : i, lb = adjacent ? 2 * i + 1 : i + half;
      float u = to_float(row[col + la]), v = to_float(row[col + lb]);
      if (bias) { u += bias[col + la]; v += bias[col + lb]; }
      const float c = cs[2 * i], s = cs[2 * i + 1];
      const float ru = (u * c - v * s) * f, rv = (v * c + u * s) * f;
      if (krow) { krow[la] = from_float<TA>(ru); krow[lb] = from_float<TA>(rv); }
      else { row[col + la] = from_float<TA>(ru); row[col + lb] = from_float<TA>(rv); }
    } else {
      const int lane = rot + (i - half);
      float u = to_float(row[col + lane]);
      if (bias) u += bias[col + lane];
      if (krow) krow[lane] = from_float<TA>(u);
      else row[col + lane] = from_float<TA>(u * f);
    }
  }
  if (write_kv) {
    // the keys' columns of the row still hold what was projected (rotated keys went to the pages only)
    const int v0 = values_are_keys ? H * dk : (H + G) * dk;
    for (int e = threadIdx.x; e < G * dv; e += blockDim.x) {
      float u = to_float(row[v0 + e]);
      if (bias) u += bias[v0 + e];
      const int c = e / dv, d = e - c * dv;
      vcache[(((size_t)page * G + c) * dv + d) * page_size + in_page] = from_float<TA>(u);
    }
  }
}

extern "C" int blm_qkv_prepare(void* qkv, int dtype, int ld, const float* bias, const float* cos_sin, int rot,
                               const int* positions, const int* token_seq, const int* block_table, int table_width,
                               void* kcache, void* vcache, int page_size, int T, int H, int G, int dk, int dv, int write_kv,
                               int adjacent, int values_are_keys, const float* q_scale, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && H > 0 && G > 0 && dk > 0 && dv > 0, "qkv_prepare: bad sizes T=%d H=%d G=%d dk=%d dv=%d", T, H, G, dk, dv);
  BLM_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk, "qkv_prepare: %d turning lanes of %d (even, at most the head size)", rot, dk);
  BLM_REQUIRE(!values_are_keys || dv == dk, "qkv_prepare: values that are the keys have the keys' head size, not %d", dv);
  BLM_REQUIRE(ld >= H * dk + (write_kv ? G * (dk + (values_are_keys ? 0 : dv)) : 0), "qkv_prepare: rows of %d are too short", ld);
  BLM_REQUIRE(!write_kv || (kcache && vcache && block_table && page_size > 0 && table_width > 0), "qkv_prepare: the pages are missing");
  BLM_REQUIRE(rot == 0 || cos_sin, "qkv_prepare: the table of angles is missing");
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(qkv_prepare_kernel<float>, dim3(T), dim3(256), 0, stream, (float*)qkv, ld, bias, cos_sin, rot, positions,
                       token_seq, block_table, table_width, (float*)kcache, (float*)vcache, page_size, H, G, dk, dv, write_kv, adjacent, values_are_keys, q_scale);
  else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(qkv_prepare_kernel<bf16>, dim3(T), dim3(256), 0, stream, (bf16*)qkv, ld, bias, cos_sin, rot, positions,
                       token_seq, block_table, table_width, (bf16*)kcache, (bf16*)vcache, page_size, H, G, dk, dv, write_kv, adjacent, values_are_keys, q_scale);
  else
    return blm_fail("qkv_prepare: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("qkv_prepare");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Output gate: x[t][c] *= sigmoid(g[t][c]) for c < N, in float, rounded once.  x [T][ld_x], g [T][ld_g] (the gate's
// columns of the projection's rows).
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void sigmoid_gate_kernel(TA* __restrict__ x, int ld_x, const TA* __restrict__ g, int ld_g, long long n, int N) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / N;
    const int c = (int)(e - t * N);
    TA* px = x + (size_t)t * ld_x + c;
    *px = from_float<TA>(to_float(*px) / (1.0f + __expf(-to_float(g[(size_t)t * ld_g + c]))));
  }
}

// eight bfloat16 at a time (N, both row strides and both addresses multiples of eight elements)
__global__ void sigmoid_gate8_kernel(bf16* __restrict__ x, int ld_x, const bf16* __restrict__ g, int ld_g, long long n8, int N8) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n8; e += stride) {
    const long long t = e / N8;
    const int c = (int)(e - t * N8) * 8;
    uint4* px = reinterpret_cast<uint4*>(x + (size_t)t * ld_x + c);
    const uint4 xv = *px, gv = *reinterpret_cast<const uint4*>(g + (size_t)t * ld_g + c);
    const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, gw[4] = {gv.x, gv.y, gv.z, gv.w};
    uint32_t r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float x0 = __uint_as_float(xw[k] << 16), x1 = __uint_as_float(xw[k] & 0xffff0000u);
      const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
      r[k] = f32x2_to_bf16x2_bits(x0 / (1.0f + __expf(-g0)), x1 / (1.0f + __expf(-g1)));
    }
    *px = make_uint4(r[0], r[1], r[2], r[3]);
  }
}

extern "C" int blm_sigmoid_gate(void* x, int ld_x, const void* g, int ld_g, int dtype, int T, int N, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && N > 0 && ld_x >= N && ld_g >= N, "sigmoid_gate: bad sizes T=%d N=%d rows of %d and %d", T, N, ld_x, ld_g);
  const long long n = (long long)T * N;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, dim3(blocks), dim3(256), 0, stream, (float*)x, ld_x, (const float*)g, ld_g, n, N);
  else if (dtype == BLM_BF16 && N % 8 == 0 && ld_x % 8 == 0 && ld_g % 8 == 0 && ((size_t)x & 15) == 0 && ((size_t)g & 15) == 0) {
    const long long n8 = n / 8;
    const unsigned b8 = (unsigned)((n8 + 255) / 256 < 65535 ? (n8 + 255) / 256 : 65535);
    hipLaunchKernelGGL(sigmoid_gate8_kernel, dim3(b8), dim3(256), 0, stream, (bf16*)x, ld_x, (const bf16*)g, ld_g, n8, N / 8);
  } else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (bf16*)x, ld_x, (const bf16*)g, ld_g, n, N);
  else
    return blm_fail("sigmoid_gate: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("sigmoid_gate");
  return 0;
}

// ---------------------------------------------------------------------------------------
// One wavefront per (token, head g, batch of GB key-value heads).  acc out: A [T][H][G][dv] float, already divided
// by the head's denominator.  all_groups = 0: only the head's own key-value head, written at A[t][g][0] of a
// [T][H][1][dv] array.
// ---------------------------------------------------------------------------------------
template <typename TA, int GB>
__global__ void sink_attn_kernel(const TA* __restrict__ q, int ldq, float* __restrict__ A, const float* __restrict__ sinks,
                                 const int* __restrict__ positions, const int* __restrict__ token_seq,
                                 const int* __restrict__ block_table, int table_width, const TA* __restrict__ kcache,
                                 const TA* __restrict__ vcache, int page_size, int T, int H, int G, int dk, int dv,
                                 float scale, int window, int all_groups) {
  extern __shared__ float sa_sm[];
  const int waves = blockDim.x / BLM_WAVE;
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long w = (long long)blockIdx.x * waves + wave;
  if (w >= (long long)T * H) return;         // no block-wide barrier below: a wavefront may leave alone
  const int t = (int)(w / H), head = (int)(w - (long long)t * H);
  const int b = token_seq[t];
  const int n_out = all_groups ? G : 1;
  const int c0 = all_groups ? blockIdx.y * GB : head / (H / G);
  float* qs = sa_sm + (size_t)wave * (dk + BLM_WAVE * (dv + 1));
  float* vt = qs + dk;                      // [64 keys][dv + 1]
  float* arow = A + ((size_t)t * H + head) * n_out * dv;
  if (b < 0) {
    for (int c = 0; c < GB; ++c) {
      const int cc = all_groups ? c0 + c : 0;
      if (all_groups ? cc < G : c == 0)
        for (int d = lane; d < dv; d += BLM_WAVE) arow[(size_t)cc * dv + d] = 0.f;
    }
    return;
  }
  const TA* qrow = q + (size_t)t * ldq + (size_t)head * dk;
  for (int d = lane; d < dk; d += BLM_WAVE) qs[d] = to_float(qrow[d]);
  __builtin_amdgcn_wave_barrier();
  const int pos = positions[t];
  const int kvh = head / (H / G);
  const int* bt = block_table + (size_t)b * table_width;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  float m = sinks ? sinks[head] : -INFINITY;
  float l = sinks ? 1.f : 0.f;
  float acc[GB][SA_MAX_DV_REGS];
#pragma unroll
  for (int c = 0; c < GB; ++c)
#pragma unroll
    for (int i = 0; i < SA_MAX_DV_REGS; ++i) acc[c][i] = 0.f;

  for (int j0 = first; j0 <= pos; j0 += BLM_WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    int page = 0, in_page = 0;
    if (valid) {
      page = bt[j / page_size];
      in_page = j % page_size;
      const TA* krow = kcache + (((size_t)page * G + kvh) * page_size + in_page) * dk;
      float dot = 0.f;
      for (int d = 0; d < dk; ++d) dot = fmaf(qs[d], to_float(krow[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);      // m is finite with a sink; without one, -inf only before the first chunk
    l = l * corr + wave_sum(p);
    m = m_new;
    const int cnt = (pos - j0 + 1) < BLM_WAVE ? (pos - j0 + 1) : BLM_WAVE;
#pragma unroll
    for (int c = 0; c < GB; ++c) {
      const int cc = c0 + c;
      if (cc < G && (all_groups || c == 0)) {
        if (valid) {
          const TA* vcol = vcache + ((size_t)page * G + cc) * dv * page_size + in_page;
          float* mine = vt + (size_t)lane * (dv + 1);
          for (int d = 0; d < dv; ++d) mine[d] = to_float(vcol[(size_t)d * page_size]);
        }
        __builtin_amdgcn_wave_barrier();      // the tile is the wavefront's own: its reads follow its writes in order
#pragma unroll
        for (int i = 0; i < SA_MAX_DV_REGS; ++i) acc[c][i] *= corr;
        for (int jj = 0; jj < cnt; ++jj) {
          const float pj = __shfl(p, jj, BLM_WAVE);
          const float* vrow = vt + (size_t)jj * (dv + 1);
#pragma unroll
          for (int i = 0; i < SA_MAX_DV_REGS; ++i) {
            const int d = lane + i * BLM_WAVE;
            if (d < dv) acc[c][i] = fmaf(pj, vrow[d], acc[c][i]);
          }
        }
        __builtin_amdgcn_wave_barrier();      // the next tile's writes follow these reads
      }
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < GB; ++c) {
    const int cc = c0 + c;
    if (cc < G && (all_groups || c == 0)) {
      float* o = arow + (size_t)(all_groups ? cc : 0) * dv;
#pragma unroll
      for (int i = 0; i < SA_MAX_DV_REGS; ++i) {
        const int d = lane + i * BLM_WAVE;
        if (d < dv) o[d] = acc[c][i] * inv;
      }
    }
  }
}

// out[t][h][d] = sum_g mix[h][g] * A[t][g][c(h)][d]  (mix null: A has one slot per head and is only converted); a block
// per (token, head)
template <typename TA>
__global__ void talk_mix_kernel(const float* __restrict__ A, const float* __restrict__ mix, TA* __restrict__ out,
                                const int* __restrict__ token_seq, int H, int G, int dv) {
  const int t = blockIdx.x, h = blockIdx.y;
  TA* o = out + ((size_t)t * H + h) * dv;
  if (token_seq[t] < 0) {      // a padding token: nobody wrote its rows of A
    for (int d = threadIdx.x; d < dv; d += blockDim.x) o[d] = from_float<TA>(0.f);
    return;
  }
  const int n_slots = mix ? G : 1;
  const float* a = A + (size_t)t * H * n_slots * dv;
  const int c = h / (H / G);
  for (int d = threadIdx.x; d < dv; d += blockDim.x) {
    float v;
    if (mix) {
      v = 0.f;
      for (int g = 0; g < H; ++g) v = fmaf(mix[h * H + g], a[((size_t)g * G + c) * dv + d], v);
    } else {
      v = a[(size_t)h * dv + d];
    }
    o[d] = from_float<TA>(v);
  }
}

static int launch_talk_mix(const float* A, const float* mix, void* out, int dtype, const int* token_seq, int T, int H, int G,
                           int dv, hipStream_t stream) {
  const int threads = dv > 64 ? 128 : 64;
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(talk_mix_kernel<float>, dim3(T, H), dim3(threads), 0, stream, A, mix, (float*)out, token_seq, H, G, dv);
  else
    hipLaunchKernelGGL(talk_mix_kernel<bf16>, dim3(T, H), dim3(threads), 0, stream, A, mix, (bf16*)out, token_seq, H, G, dv);
  BLM_LAUNCH_CHECK("talk_mix");
  return 0;
}

extern "C" int blm_sink_attn(const void* q, int ldq, void* out, int dtype, float* A, const float* sinks, const float* mix,
                             const int* positions, const int* token_seq, const int* block_table, int table_width,
                             const void* kcache, const void* vcache, int page_size, int T, int H, int G, int dk, int dv,
                             float scale, int window, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && H > 0 && G > 0 && H % G == 0, "sink_attn: bad sizes T=%d heads=%d kv_heads=%d", T, H, G);
  BLM_REQUIRE(dk > 0 && dk <= SA_MAX_DK && dv > 0 && dv <= 64 * SA_MAX_DV_REGS,
              "sink_attn: head sizes %d / %d are not supported (keys up to %d, values up to %d)", dk, dv, SA_MAX_DK, 64 * SA_MAX_DV_REGS);
  BLM_REQUIRE(page_size > 0 && table_width > 0 && window >= 0 && ldq >= H * dk, "sink_attn: bad geometry");
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "sink_attn: unsupported dtype %d", dtype);
  const int all_groups = mix ? 1 : 0;
  const int gb = !all_groups ? 1 : (G >= 8 ? 8 : (G >= 4 ? 4 : (G >= 2 ? 2 : 1)));
  const size_t per_wave = ((size_t)dk + (size_t)BLM_WAVE * (dv + 1)) * sizeof(float);
  int waves = (int)((64 * 1024) / per_wave);
  BLM_REQUIRE(waves >= 1, "sink_attn: head sizes %d / %d need more shared memory than a block gets", dk, dv);
  waves = waves > 4 ? 4 : waves;
  const long long items = (long long)T * H;
  const long long blocks = (items + waves - 1) / waves;
  BLM_REQUIRE(blocks < 2147483647LL, "sink_attn: too many (token, head) pairs: %lld", items);
  dim3 grid((unsigned)blocks, (unsigned)(all_groups ? (G + gb - 1) / gb : 1)), block(waves * BLM_WAVE);
#define SA_CASE(TA, GB)                                                                                               \
  hipLaunchKernelGGL((sink_attn_kernel<TA, GB>), grid, block, per_wave * waves, stream, (const TA*)q, ldq, A, sinks, \
                     positions, token_seq, block_table, table_width, (const TA*)kcache, (const TA*)vcache, page_size, T, H, G, \
                     dk, dv, scale, window, all_groups)
#define SA_PICK(TA)                  \
  do {                               \
    if (gb == 8) SA_CASE(TA, 8);     \
    else if (gb == 4) SA_CASE(TA, 4); \
    else if (gb == 2) SA_CASE(TA, 2); \
    else SA_CASE(TA, 1);             \
  } while (0)
  if (dtype == BLM_F32) SA_PICK(float);
  else SA_PICK(bf16);
#undef SA_PICK
#undef SA_CASE
  BLM_LAUNCH_CHECK("sink_attn");
  return launch_talk_mix(A, mix, out, dtype, token_seq, T, H, G, dv, stream);
}

// ---------------------------------------------------------------------------------------
// The same function on the matrix cores (bfloat16, pages of 64 keys).  A wavefront's 16 query columns are
// 16 (token, head) pairs of one sequence whose heads share a key-value head, so that one tile of keys serves
// them all.  Per page:
//   S^T = K Q^T      A operand = 16 keys x 32 lanes of a key row per instruction, B = Q^T; lane (kg, c) gets the
//                    scores of column c for keys kg*4 .. kg*4+3 of each 16-key tile
//   O_g^T += V_g^T P^T  for every key-value head g of the batch: A = 16 value lanes x 32 keys from the transposed
//                    value pages, B = the probabilities the lane has just computed (the keys of a page are dealt
//                    to the four score tiles so that the eight keys a lane supplies are neighbours there)
// The running maximum starts at the sink's logit and the sum at one (in the first piece of a cut range).  Fragments
// come straight from global memory; the four wavefronts of a block are neighbouring tiles, which read the same
// pages at the same time.  With n_splits > 1 the pages of a tile are cut into pieces that a second kernel adds up.
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 sa_bf16x8;
typedef __attribute__((ext_vector_type(4))) float sa_f32x4;

__device__ __forceinline__ constexpr int sa_key_of(int t, int i) { return (t >> 1) * 32 + (i >> 2) * 8 + (t & 1) * 4 + (i & 3); }

__device__ __forceinline__ uint4 sa_keep_first(uint4 v, int n) {      // the first n (0..8) bf16 of 16 bytes, zeros behind
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int left = n - 2 * i;
    w[i] = left >= 2 ? w[i] : (left == 1 ? (w[i] & 0xffffu) : 0u);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

#define SAM_WAVES 4
#define SAM_MAX_PIECES 64
template <int KS, int DT, int GB>
__global__ void __launch_bounds__(SAM_WAVES* BLM_WAVE)
    sink_attn_mfma_kernel(const bf16* __restrict__ q, int ldq, float* __restrict__ A, const float* __restrict__ sinks,
                          const int* __restrict__ cu_seqlens, const int* __restrict__ lens_after,
                          const int* __restrict__ block_table, int table_width, const bf16* __restrict__ kcache,
                          const bf16* __restrict__ vcache, int B, int H, int G, int dk, int dv, int tiles_per_seq,
                          float scale2, int window, int all_groups, int n_splits, float* __restrict__ part_o,
                          float* __restrict__ part_ml) {
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int c = lane & 15, kg = lane >> 4;
  const long long tile_id = (long long)blockIdx.x * SAM_WAVES + wave;      // over sequences x key-value heads x tiles
  const int tile = (int)(tile_id % tiles_per_seq);
  const int kvh = (int)((tile_id / tiles_per_seq) % G);
  const long long b = tile_id / ((long long)tiles_per_seq * G);
  if (b >= B) return;
  const int split = blockIdx.y;
  const int Hg = H / G;
  const int t_first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_first;
  const int n_cols = n_new * Hg;
  if (tile * 16 >= n_cols) return;                                         // also a padding sequence
  const int after = lens_after[b];
  const int past = after - n_new;
  const int idx = tile * 16 + c;
  const bool valid = idx < n_cols;
  const int tok = valid ? idx / Hg : 0, head = kvh * Hg + (valid ? idx - tok * Hg : 0);
  const int qpos = valid ? past + tok : -1;
  const int min_qpos = past + (tile * 16) / Hg;
  const int max_qpos = past + min(tile * 16 + 15, n_cols - 1) / Hg;
  const int max_key = after - 1;
  const int first_key = (window > 0 && min_qpos - window + 1 > 0) ? min_qpos - window + 1 : 0;
  const int p_lo = first_key / 64, p_hi = max_qpos / 64;
  const int per = (p_hi - p_lo + 1 + n_splits - 1) / n_splits;
  const int p_begin = p_lo + split * per, p_end = min(p_hi + 1, p_begin + per);
  const int* bt = block_table + (size_t)b * table_width;
  const int n_out = all_groups ? G : 1;
  const int g0 = all_groups ? blockIdx.z * GB : kvh;

  uint4 qf[KS];
  {
    const bf16* qrow = q + (size_t)(t_first + tok) * ldq + (size_t)head * dk;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + kg * 8;
      qf[ks] = (valid && d < dk) ? *reinterpret_cast<const uint4*>(qrow + d) : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  const bool sunk = valid && sinks != nullptr && split == 0;
  float m = sunk ? sinks[head] * 1.4426950408889634f : -INFINITY;
  sa_f32x4 l = sunk ? sa_f32x4{1.f, 1.f, 1.f, 1.f} : sa_f32x4{0.f, 0.f, 0.f, 0.f};
  sa_f32x4 o[GB][DT];
#pragma unroll
  for (int gi = 0; gi < GB; ++gi)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[gi][dt] = sa_f32x4{0.f, 0.f, 0.f, 0.f};

  for (int pi = p_begin; pi < p_end; ++pi) {
    const int page = bt[pi];
    const int key0 = pi * 64;
    const bf16* kp = kcache + ((size_t)page * G + kvh) * 64 * dk;
    // one key-value head per wavefront (steps of few tiles): its value fragments are asked for here, in front of the
    // scores, so that a page costs one trip to memory and not two in a row
    uint4 v_early[GB == 1 ? 2 : 1][GB == 1 ? DT : 1];
    if (GB == 1 && g0 < G) {
      const bf16* vp = vcache + ((size_t)page * G + g0) * dv * 64;
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const int row = dt * 16 + c;
          v_early[GB == 1 ? h : 0][GB == 1 ? dt : 0] =
              row < dv ? *reinterpret_cast<const uint4*>(vp + (size_t)row * 64 + h * 32 + kg * 8) : make_uint4(0u, 0u, 0u, 0u);
        }
    }
    float s[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bf16* krow = kp + (size_t)sa_key_of(t, c) * dk;
      uint4 kf[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + kg * 8;
        kf[ks] = d < dk ? *reinterpret_cast<const uint4*>(krow + d) : make_uint4(0u, 0u, 0u, 0u);
      }
      sa_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sa_bf16x8, kf[ks]),
                                                      __builtin_bit_cast(sa_bf16x8, qf[ks]), acc, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kj = key0 + sa_key_of(t, kg * 4 + r);
        const bool seen = kj <= qpos && (window <= 0 || kj > qpos - window);
        s[t][r] = seen ? acc[r] : -INFINITY;      // whatever the places past the data hold, it is replaced here
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[t][r]);
    mx = rows_max(mx);
    const float m_new = fmaxf(m, mx * scale2);
    const float corr = (m == m_new) ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        s[t][r] = (s[t][r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], scale2, -m_new));
    if (__any(m != m_new)) {
#pragma unroll
      for (int gi = 0; gi < GB; ++gi)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[gi][dt][r] *= corr;
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
          __builtin_bit_cast(sa_bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u)),
          __builtin_bit_cast(sa_bf16x8, pf), l, 0, 0, 0);
      const int keep = max_key - (key0 + h * 32 + kg * 8) + 1;
#pragma unroll
      for (int gi = 0; gi < GB; ++gi) {
        const int cc = g0 + gi;
        if (cc < G) {
          const bf16* vp = vcache + ((size_t)page * G + cc) * dv * 64;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const int row = dt * 16 + c;
            uint4 va;
            if (GB == 1) va = v_early[GB == 1 ? h : 0][GB == 1 ? dt : 0];
            else va = row < dv ? *reinterpret_cast<const uint4*>(vp + (size_t)row * 64 + h * 32 + kg * 8) : make_uint4(0u, 0u, 0u, 0u);
            if (tail) va = sa_keep_first(va, keep);
            o[gi][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sa_bf16x8, va),
                                                                __builtin_bit_cast(sa_bf16x8, pf), o[gi][dt], 0, 0, 0);
          }
        }
      }
    }
  }
  if (n_splits == 1) {
    if (valid) {
      const float inv = 1.0f / l[0];
      float* arow = A + ((size_t)(t_first + tok) * H + head) * n_out * dv;
#pragma unroll
      for (int gi = 0; gi < GB; ++gi) {
        const int cc = g0 + gi;
        if (cc < G) {
          float* og = arow + (size_t)(all_groups ? cc : 0) * dv;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int d = dt * 16 + kg * 4 + r;
              if (d < dv) og[d] = o[gi][dt][r] * inv;
            }
        }
      }
    }
    return;
  }
  // leave this piece: per column its maximum, sum and unnormalised results; sink_merge_kernel adds the pieces up
  const size_t gcol = (size_t)tile_id * 16 + c;
  float* po = part_o + (gcol * n_splits + split) * n_out * dv;
#pragma unroll
  for (int gi = 0; gi < GB; ++gi) {
    const int cc = g0 + gi;
    if (cc < G) {
      float* og = po + (size_t)(all_groups ? cc : 0) * dv;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int d = dt * 16 + kg * 4 + r;
          if (d < dv) og[d] = o[gi][dt][r];
        }
    }
  }
  if (kg == 0 && blockIdx.z == 0) {
    part_ml[(gcol * n_splits + split) * 2] = m;
    part_ml[(gcol * n_splits + split) * 2 + 1] = l[0];
  }
}

// The same for steps of many tokens (prompts): the four wavefronts of a block are four neighbouring tiles of one
// sequence and key-value head, which see nearly the same pages; the block brings every page once, keys and the values
// of the batch's key-value heads, into shared memory (16 bytes per thread and load, whole pages in order; rows padded
// by 16 bytes so that the fragment reads of 16 rows fall on different banks), and the wavefronts take their fragments
// from there.  Without it every wavefront fetches every fragment itself, and the second-level cache's rate bounds
// the kernel.  A wavefront skips the pages outside its own tile's range but meets the others at every page.
template <int KS, int DT, int GB>
__global__ void __launch_bounds__(SAM_WAVES* BLM_WAVE)
    sink_attn_mfma_staged_kernel(const bf16* __restrict__ q, int ldq, float* __restrict__ A, const float* __restrict__ sinks,
                                 const int* __restrict__ cu_seqlens, const int* __restrict__ lens_after,
                                 const int* __restrict__ block_table, int table_width, const bf16* __restrict__ kcache,
                                 const bf16* __restrict__ vcache, int B, int H, int G, int dk, int dv, int blocks_per_seq,
                                 float scale2, int window, int all_groups) {
  extern __shared__ __attribute__((aligned(16))) bf16 sam_sm[];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int c = lane & 15, kg = lane >> 4;
  const int blk = blockIdx.x % blocks_per_seq;
  const int kvh = (blockIdx.x / blocks_per_seq) % G;
  const int b = blockIdx.x / (blocks_per_seq * G);
  const int Hg = H / G;
  const int t_first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_first;
  const int n_cols = n_new * Hg;
  if (blk * 64 >= n_cols) return;                                          // the whole block: also a padding sequence
  const int after = lens_after[b];
  const int past = after - n_new;
  const int tile = blk * SAM_WAVES + wave;
  const bool active = tile * 16 < n_cols;
  const int idx = tile * 16 + c;
  const bool valid = active && idx < n_cols;
  const int tok = valid ? idx / Hg : 0, head = kvh * Hg + (valid ? idx - tok * Hg : 0);
  const int qpos = valid ? past + tok : -1;
  const int max_key = after - 1;
  auto first_page = [&](int col) { const int p = past + col / Hg; return (window > 0 && p - window + 1 > 0) ? (p - window + 1) / 64 : 0; };
  auto last_page = [&](int col) { return (past + min(col, n_cols - 1) / Hg) / 64; };
  const int my_lo = active ? first_page(tile * 16) : 1, my_hi = active ? last_page(tile * 16 + 15) : 0;
  const int blk_lo = first_page(blk * 64), blk_hi = last_page(blk * 64 + 63);
  const int* bt = block_table + (size_t)b * table_width;
  const int n_out = all_groups ? G : 1;
  const int g0 = all_groups ? blockIdx.z * GB : kvh;
  const int krs = dk + 8, vrs = 64 + 8;                                    // padded rows, in elements
  bf16* k_sm = sam_sm;                                                     // [64][krs]
  bf16* v_sm = sam_sm + 64 * krs;                                          // [GB][dv][vrs]

  uint4 qf[KS];
  {
    const bf16* qrow = q + (size_t)(t_first + tok) * ldq + (size_t)head * dk;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + kg * 8;
      qf[ks] = (valid && d < dk) ? *reinterpret_cast<const uint4*>(qrow + d) : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  const bool sunk = valid && sinks != nullptr;
  float m = sunk ? sinks[head] * 1.4426950408889634f : -INFINITY;
  sa_f32x4 l = sunk ? sa_f32x4{1.f, 1.f, 1.f, 1.f} : sa_f32x4{0.f, 0.f, 0.f, 0.f};
  sa_f32x4 o[GB][DT];
#pragma unroll
  for (int gi = 0; gi < GB; ++gi)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[gi][dt] = sa_f32x4{0.f, 0.f, 0.f, 0.f};
  const int k_pieces = dk / 8;                                             // 16-byte pieces per key row

  // a page travels in two steps: from memory into registers while the page before is worked on, from there into
  // shared memory once nobody reads that page any more
  constexpr int KP = 4, VP = 4;            // 16-byte pieces per thread: keys (64 rows of up to 128 lanes), values per key-value head
  uint4 k_in[KP], v_in[GB][VP];
#define SAM_FETCH(PI)                                                                                     \
  {                                                                                                       \
    const int page_ = bt[PI];                                                                             \
    const bf16* kp_ = kcache + ((size_t)page_ * G + kvh) * 64 * dk;                                       \
    _Pragma("unroll") for (int u = 0; u < KP; ++u) {                                                      \
      const int e = threadIdx.x + u * SAM_WAVES * BLM_WAVE;                                               \
      k_in[u] = e < 64 * k_pieces ? *reinterpret_cast<const uint4*>(kp_ + (size_t)e * 8) : make_uint4(0u, 0u, 0u, 0u); \
    }                                                                                                     \
    _Pragma("unroll") for (int gi = 0; gi < GB; ++gi) {                                                   \
      const bf16* vp_ = vcache + ((size_t)page_ * G + min(g0 + gi, G - 1)) * dv * 64;                     \
      _Pragma("unroll") for (int u = 0; u < VP; ++u) {                                                    \
        const int e = threadIdx.x + u * SAM_WAVES * BLM_WAVE;                                             \
        v_in[gi][u] = e < dv * 8 ? *reinterpret_cast<const uint4*>(vp_ + (size_t)e * 8) : make_uint4(0u, 0u, 0u, 0u); \
      }                                                                                                   \
    }                                                                                                     \
  }
  SAM_FETCH(blk_lo)
  for (int pi = blk_lo; pi <= blk_hi; ++pi) {
    const int key0 = pi * 64;
    __syncthreads();                                                       // nobody reads the page before any more
    _Pragma("unroll") for (int u = 0; u < KP; ++u) {
      const int e = threadIdx.x + u * SAM_WAVES * BLM_WAVE;
      if (e < 64 * k_pieces) {
        const int row = e / k_pieces, piece = e - row * k_pieces;
        *reinterpret_cast<uint4*>(k_sm + (size_t)row * krs + piece * 8) = k_in[u];
      }
    }
    _Pragma("unroll") for (int gi = 0; gi < GB; ++gi) {
      bf16* vs = v_sm + (size_t)gi * dv * vrs;
      _Pragma("unroll") for (int u = 0; u < VP; ++u) {
        const int e = threadIdx.x + u * SAM_WAVES * BLM_WAVE;
        if (e < dv * 8) *reinterpret_cast<uint4*>(vs + (size_t)(e >> 3) * vrs + (e & 7) * 8) = v_in[gi][u];
      }
    }
    __syncthreads();
    if (pi < blk_hi) SAM_FETCH(pi + 1)                                     // travels while this page is worked on
    if (pi < my_lo || pi > my_hi) continue;
    float s[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bf16* krow = k_sm + (size_t)sa_key_of(t, c) * krs;
      sa_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + kg * 8;
        const uint4 kf = d < dk ? *reinterpret_cast<const uint4*>(krow + d) : make_uint4(0u, 0u, 0u, 0u);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sa_bf16x8, kf), __builtin_bit_cast(sa_bf16x8, qf[ks]),
                                                      acc, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kj = key0 + sa_key_of(t, kg * 4 + r);
        const bool seen = kj <= qpos && (window <= 0 || kj > qpos - window);
        s[t][r] = seen ? acc[r] : -INFINITY;
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[t][r]);
    mx = rows_max(mx);
    const float m_new = fmaxf(m, mx * scale2);
    const float corr = (m == m_new) ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        s[t][r] = (s[t][r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], scale2, -m_new));
    if (__any(m != m_new)) {
#pragma unroll
      for (int gi = 0; gi < GB; ++gi)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[gi][dt][r] *= corr;
#pragma unroll
      for (int r = 0; r < 4; ++r) l[r] *= corr;
    }
    m = m_new;
    const bool tail = key0 + 63 > max_key;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint4 pf;
      pf.x = f32x2_to_bf16x2_bits(s[2 * h][0], s[2 * h][1]);
      pf.y = f32x2_to_bf16x2_bits(s[2 * h][2], s[2 * h][3]);
      pf.z = f32x2_to_bf16x2_bits(s[2 * h + 1][0], s[2 * h + 1][1]);
      pf.w = f32x2_to_bf16x2_bits(s[2 * h + 1][2], s[2 * h + 1][3]);
      l = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          __builtin_bit_cast(sa_bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u)),
          __builtin_bit_cast(sa_bf16x8, pf), l, 0, 0, 0);
      const int keep = max_key - (key0 + h * 32 + kg * 8) + 1;
#pragma unroll
      for (int gi = 0; gi < GB; ++gi) {
        if (g0 + gi < G) {
          const bf16* vs = v_sm + (size_t)gi * dv * vrs;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const int row = dt * 16 + c;
            uint4 va = row < dv ? *reinterpret_cast<const uint4*>(vs + (size_t)row * vrs + h * 32 + kg * 8) : make_uint4(0u, 0u, 0u, 0u);
            if (tail) va = sa_keep_first(va, keep);
            o[gi][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sa_bf16x8, va),
                                                                __builtin_bit_cast(sa_bf16x8, pf), o[gi][dt], 0, 0, 0);
          }
        }
      }
    }
  }
  if (valid) {
    const float inv = 1.0f / l[0];
    float* arow = A + ((size_t)(t_first + tok) * H + head) * n_out * dv;
#pragma unroll
    for (int gi = 0; gi < GB; ++gi) {
      const int cc = g0 + gi;
      if (cc < G) {
        float* og = arow + (size_t)(all_groups ? cc : 0) * dv;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int d = dt * 16 + kg * 4 + r;
            if (d < dv) og[d] = o[gi][dt][r] * inv;
          }
      }
    }
  }
}

#undef SAM_FETCH

// The pieces of a cut range added up, one block per column: maxima in base 2.  A piece that saw nothing and holds
// no sink has sum 0, maximum -infinity and results of zeros, and gets weight 0.
__global__ void __launch_bounds__(256)
    sink_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, float* __restrict__ A,
                      const int* __restrict__ cu_seqlens, int H, int G, int n_out, int dv, int tiles_per_seq, int n_splits) {
  __shared__ float wgt[SAM_MAX_PIECES];
  __shared__ float inv_sum;
  const size_t gcol = blockIdx.x;
  const int c = (int)(gcol & 15);
  const long long tile_id = (long long)(gcol >> 4);
  const int tile = (int)(tile_id % tiles_per_seq);
  const int kvh = (int)((tile_id / tiles_per_seq) % G);
  const long long b = tile_id / ((long long)tiles_per_seq * G);
  const int Hg = H / G;
  const int t_first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_first;
  const int idx = tile * 16 + c;
  if (idx >= n_new * Hg) return;
  const int tok = idx / Hg, head = kvh * Hg + idx - tok * Hg;
  const float* ml = part_ml + gcol * n_splits * 2;
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
  const int n = n_out * dv;
  const float* po = part_o + gcol * n_splits * n;
  float* arow = A + ((size_t)(t_first + tok) * H + head) * n;
  for (int d = threadIdx.x; d < n; d += blockDim.x) {
    float acc = 0.f;
    for (int p = 0; p < n_splits; ++p) acc = fmaf(wgt[p], po[(size_t)p * n + d], acc);
    arow[d] = acc * inv_sum;
  }
}

#define SAM_STAGED_LDS (152 * 1024)
#define SAM_DEVICES 64
static bool g_sam_big_lds[SAM_DEVICES];
#define SAM_ALL_CASES(X) X(2, 2) X(2, 3) X(2, 4) X(2, 8) X(4, 2) X(4, 3) X(4, 4) X(4, 8)
// Once per device, outside any stream capture: lets the form that stages pages ask for more shared memory than a
// kernel gets without asking.  Without it that form is not used.
extern "C" int blm_sink_attn_mfma_init() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  BLM_REQUIRE(e == hipSuccess && dev >= 0, "sink_attn_mfma_init: hipGetDevice failed: %s", hipGetErrorString(e));
  if (dev >= SAM_DEVICES) return 0;
#define SAM_ATTR(KS, DT)                                                                                                  \
  {                                                                                                                       \
    const void* ks_[] = {(const void*)sink_attn_mfma_staged_kernel<KS, DT, 1>, (const void*)sink_attn_mfma_staged_kernel<KS, DT, 2>, \
                         (const void*)sink_attn_mfma_staged_kernel<KS, DT, 4>};                                           \
    for (const void* k : ks_) {                                                                                           \
      e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, SAM_STAGED_LDS);                             \
      BLM_REQUIRE(e == hipSuccess, "sink_attn_mfma_init: cannot raise the shared memory limit: %s", hipGetErrorString(e)); \
    }                                                                                                                     \
  }
  SAM_ALL_CASES(SAM_ATTR)
#undef SAM_ATTR
  g_sam_big_lds[dev] = true;
  return 0;
}

extern "C" int blm_sink_attn_mfma_supported(int dk, int dv) {
  return (dk % 8 == 0 && dk >= 8 && dk <= 128 && dv >= 1 && dv <= 128) ? 1 : 0;
}

// q: bfloat16 rows of ldq elements (queries at column 0, already rotated); out bfloat16 [T][H * dv]; A: float
// [T][H][G or 1][dv] workspace; pages in bfloat16, 64 keys each.  B sequences of at most max_new tokens.  Workspace for
// n_splits > 1: part_o (B * G * tiles * 16 * n_splits * (G or 1) * dv floats), part_ml (B * G * tiles * 16 * n_splits * 2),
// with tiles = ceil(max_new * (H / G) / 16).  group_batch: 0, or the most key-value heads a wavefront accumulates (1, 2, 4).
extern "C" int blm_sink_attn_mfma(const void* q, int ldq, void* out, float* A, const float* sinks, const float* mix,
                                  const int* token_seq, const int* cu_seqlens, const int* lens_after, const int* block_table,
                                  int table_width, const void* kcache, const void* vcache, int page_size, int B, int max_new,
                                  int T, int H, int G, int dk, int dv, float scale, int window, int n_splits, int group_batch,
                                  float* part_o, float* part_ml, hipStream_t stream) {
  BLM_REQUIRE(B > 0 && max_new > 0 && T > 0 && H > 0 && G > 0 && H % G == 0, "sink_attn_mfma: bad sizes B=%d H=%d G=%d", B, H, G);
  BLM_REQUIRE(page_size == 64 && table_width > 0 && window >= 0, "sink_attn_mfma: pages of 64 keys");
  BLM_REQUIRE(blm_sink_attn_mfma_supported(dk, dv), "sink_attn_mfma: head sizes %d / %d are not among those it takes", dk, dv);
  BLM_REQUIRE(scale > 0.f && ldq % 8 == 0 && ldq >= H * dk && ((size_t)q & 15) == 0, "sink_attn_mfma: a positive scale and query rows that start at multiples of 16 bytes");
  BLM_REQUIRE(n_splits >= 1 && n_splits <= SAM_MAX_PIECES && (n_splits == 1 || (part_o && part_ml)),
              "sink_attn_mfma: %d pieces (1 to %d, with their workspace)", n_splits, SAM_MAX_PIECES);
  const int all_groups = mix ? 1 : 0;
  // key-value heads per wavefront: up to four share one walk over the keys; fewer (group_batch) spreads a step of few
  // tiles over more wavefronts, each of which then waits for fewer fragments
  int gb = !all_groups ? 1 : (G >= 4 ? 4 : (G >= 2 ? 2 : 1));
  if (group_batch >= 1 && group_batch < gb) gb = group_batch >= 2 ? 2 : 1;
  const long long tiles = ((long long)max_new * (H / G) + 15) / 16;
  const long long waves = (long long)B * G * tiles;
  BLM_REQUIRE(waves < 2147483647LL, "sink_attn_mfma: too many tiles");
  dim3 grid((unsigned)((waves + SAM_WAVES - 1) / SAM_WAVES), (unsigned)n_splits, (unsigned)(all_groups ? (G + gb - 1) / gb : 1));
  const float scale2 = scale * 1.4426950408889634f;
  const int ks = dk <= 64 ? 2 : 4;
  const int dt = dv <= 32 ? 2 : (dv <= 48 ? 3 : (dv <= 64 ? 4 : 8));
#define SAM_CASE(KS, DT, GB)                                                                                              \
  hipLaunchKernelGGL((sink_attn_mfma_kernel<KS, DT, GB>), grid, dim3(SAM_WAVES * BLM_WAVE), 0, stream, (const bf16*)q, ldq, A, \
                     sinks, cu_seqlens, lens_after, block_table, table_width, (const bf16*)kcache, (const bf16*)vcache, B, H, \
                     G, dk, dv, (int)tiles, scale2, window, all_groups, n_splits, part_o, part_ml)
#define SAM_GB(KS, DT)                  \
  do {                                  \
    if (gb == 4) SAM_CASE(KS, DT, 4);   \
    else if (gb == 2) SAM_CASE(KS, DT, 2); \
    else SAM_CASE(KS, DT, 1);           \
  } while (0)
#define SAM_DT(KS)                      \
  do {                                  \
    if (dt == 2) SAM_GB(KS, 2);         \
    else if (dt == 3) SAM_GB(KS, 3);    \
    else if (dt == 4) SAM_GB(KS, 4);    \
    else SAM_GB(KS, 8);                 \
  } while (0)
  // prompts: the form that stages every page once per block of four tiles, where its pages fit the shared memory
  const int Hg = H / G;
  const size_t staged_lds = ((size_t)64 * (dk + 8) + (size_t)gb * dv * (64 + 8)) * sizeof(bf16);
  int dev = -1;
  const bool big = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < SAM_DEVICES && g_sam_big_lds[dev];
  const bool staged = n_splits == 1 && (long long)max_new * Hg >= 64 && staged_lds <= (size_t)(big ? SAM_STAGED_LDS : 64 * 1024);
  if (staged) {
    const int blocks_per_seq = (int)((tiles + SAM_WAVES - 1) / SAM_WAVES);
    dim3 sgrid((unsigned)((long long)B * G * blocks_per_seq), 1, grid.z);
#undef SAM_CASE
#define SAM_CASE(KS, DT, GB)                                                                                              \
  hipLaunchKernelGGL((sink_attn_mfma_staged_kernel<KS, DT, GB>), sgrid, dim3(SAM_WAVES * BLM_WAVE), staged_lds, stream,    \
                     (const bf16*)q, ldq, A, sinks, cu_seqlens, lens_after, block_table, table_width, (const bf16*)kcache, \
                     (const bf16*)vcache, B, H, G, dk, dv, blocks_per_seq, scale2, window, all_groups)
    if (ks == 2) SAM_DT(2);
    else SAM_DT(4);
  } else {
#undef SAM_CASE
#define SAM_CASE(KS, DT, GB)                                                                                              \
  hipLaunchKernelGGL((sink_attn_mfma_kernel<KS, DT, GB>), grid, dim3(SAM_WAVES * BLM_WAVE), 0, stream, (const bf16*)q, ldq, A, \
                     sinks, cu_seqlens, lens_after, block_table, table_width, (const bf16*)kcache, (const bf16*)vcache, B, H, \
                     G, dk, dv, (int)tiles, scale2, window, all_groups, n_splits, part_o, part_ml)
    if (ks == 2) SAM_DT(2);
    else SAM_DT(4);
  }
#undef SAM_DT
#undef SAM_GB
#undef SAM_CASE
  BLM_LAUNCH_CHECK("sink_attn_mfma");
  if (n_splits > 1) {
    hipLaunchKernelGGL(sink_merge_kernel, dim3((unsigned)(waves * 16)), dim3(256), 0, stream, part_o, part_ml, A, cu_seqlens, H,
                       G, all_groups ? G : 1, dv, (int)tiles, n_splits);
    BLM_LAUNCH_CHECK("sink_merge");
  }
  return launch_talk_mix(A, mix, out, BLM_BF16, token_seq, T, H, G, dv, stream);
}
