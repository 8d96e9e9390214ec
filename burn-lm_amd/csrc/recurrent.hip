// Recurrent mixers whose state is a matrix [key channels][value channels] per head and sequence, kept in
// float in the cache's state tensors: a linear recurrence with one gate that shares a channel between its old state and
// the new value (HGRN2), a delta rule with one decay per key channel, and gated linear attention (a decay per key
// channel, every token's key and value added as an outer product).  The columns of the state (one per value
// channel) never meet: each needs only its own value and what the token brings per key channel (gates, keys,
// queries).  So one wavefront walks the tokens of one (sequence, head) for 16 columns (or 4): the 4 (or 16) lanes of a
// column each keep a share of its rows in registers and add their parts of a dot product with a few cross-lane
// steps, and nothing waits for another wavefront.  What a token brings per key channel is
// computed by the wavefront into its own piece of shared memory, from inputs it loaded one token ahead.  The
// results go out unnormalised in float; a second kernel takes the root mean square over each head's value
// lanes, the weight and (delta rule, gated linear attention) the output gate.  The same kernels serve prompts and
// decoding; gated linear attention also cuts a prompt into segments that several wavefronts walk at once.
//
// Also here: the short causal convolution in front of the delta rule with its per-sequence history.
#include "common.h"

__device__ __forceinline__ float blm_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float blm_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float blm_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// Two shapes of a wavefront (LPC lanes per column, 64 / LPC columns; lane group g holds rows g * ROWS .. + ROWS - 1):
// 4 lanes per column for steps of few tokens per sequence (decoding): 16 neighbouring columns make the state's
// rows come and go in 64-byte pieces, which is what such a step waits for;  16 lanes per column for prompts: a
// token then costs a lane a quarter of the dependent instructions, which is what a long walk in order waits for.
#define SCAN_COLS 16      // most columns of the state per wavefront
#define SCAN_WAVES 4
#define SCAN_MAX_DK 256
// A vector per key channel in shared memory (LPC * (ROWS + 4) floats): channel i at i + 4 * (i / ROWS), so that the
// groups' 16-byte reads (each group's lanes read one address) fall on different banks; channels from dk up to
// LPC * ROWS hold zeros.
template <int ROWS>
__device__ __forceinline__ int scan_place(int i) { return i + 4 * (i / ROWS); }
// sum over the lanes of a column: 4 lanes a row of 16 apart, or the 16 lanes of a row
template <int LPC>
__device__ __forceinline__ float column_sum(float v) {
  if (LPC == 4) return rows_sum(v);
  v += blm_dpp<BLM_DPP_XOR1>(v);
  v += blm_dpp<BLM_DPP_XOR2>(v);
  v += blm_dpp<BLM_DPP_HALF_MIRROR>(v);
  v += blm_dpp<BLM_DPP_MIRROR>(v);
  return v;
}

#define SCAN_CHUNK 8      // tokens whose inputs a wavefront fetches and prepares at a time

// ---------------------------------------------------------------------------------------
// HGRN2.  proj [T][ld]: q at column 0 (H*dk), forget-gate logits at H*dk (H*dk), values at 2*H*dk (H*dv).
//   f = low + (1 - low) * sigmoid(logit + bias);  S = diag(f) S + (1 - f) v^T;  o = S^T silu(q)
// state [slots][H][dk][dv] float; o_raw [T][H*dv] float.
// A wavefront takes its tokens eight at a time: the chunk's inputs were fetched into registers while the chunk
// before ran (a trip to memory takes longer than a token's arithmetic), are turned into gates and activated
// queries for all eight tokens at once, left in the wavefront's piece of shared memory, and walked in order.
// (The gates themselves come from hgrn2_gates_kernel.)
// ---------------------------------------------------------------------------------------
// gates [T][2 * H*dk] float: f = low + (1 - low) * sigmoid(logit + bias), then silu(q): everything about a token that
// does not depend on the state, for all tokens at once, so that the walk in order does no more than it must
template <typename TA>
__global__ void hgrn2_gates_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ f_bias,
                                   const float* __restrict__ low, float* __restrict__ gates, long long n, int HK) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / HK;
    const int c = (int)(e - t * HK);
    const TA* row = proj + (size_t)t * ld;
    const float lo = low[c];
    gates[(size_t)t * 2 * HK + c] = lo + (1.f - lo) * blm_sigmoid(to_float(row[HK + c]) + f_bias[c]);
    gates[(size_t)t * 2 * HK + HK + c] = blm_silu(to_float(row[c]));
  }
}

template <typename TA, int ROWS, int LPC>
__global__ void __launch_bounds__(SCAN_WAVES* BLM_WAVE)
    hgrn2_scan_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ gates,
                      float* __restrict__ state, float* __restrict__ o_raw,
                      const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int H, int dk, int dv,
                      int col_groups, long long n_items) {
  extern __shared__ __attribute__((aligned(16))) float scan_sm[];     // per wavefront: [chunk][f | q][vec], [chunk][16 values]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long item = (long long)blockIdx.x * (blockDim.x / BLM_WAVE) + wave;
  if (item >= n_items) return;
  const int cg = (int)(item % col_groups);
  const int h = (int)((item / col_groups) % H);
  const int b = (int)(item / ((long long)col_groups * H));
  const int slot = seq_slots[b];
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (slot < 0 || t1 <= t0) return;
  constexpr int COLS = BLM_WAVE / LPC;
  const int g = LPC == 4 ? lane >> 4 : lane & 15, cl = LPC == 4 ? lane & 15 : lane >> 4;
  const int col = cg * COLS + cl;
  const bool own = col < dv;
  constexpr int dkp = ROWS * LPC;      // dk rounded up; the channels between stay zero
  constexpr int vec = LPC * (ROWS + 4);
  float* base = scan_sm + (size_t)wave * SCAN_CHUNK * (2 * vec + SCAN_COLS);
  float* v_sm = base + SCAN_CHUNK * 2 * vec;
  float* S_g = state + (((size_t)slot * H + h) * dk) * dv;
  float S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int i = g * ROWS + r;
    S[r] = (own && i < dk) ? S_g[(size_t)i * dv + col] : 0.f;
  }
  // per key channel (lane l prepares channels l, l + 64, ...): constants, and a chunk's raw inputs
  constexpr int PER = (dkp + BLM_WAVE - 1) / BLM_WAVE;
  float raw_f[SCAN_CHUNK][PER], raw_q[SCAN_CHUNK][PER], v_in[SCAN_CHUNK];
  auto fetch = [&](int tc) {
#pragma unroll
    for (int tt = 0; tt < SCAN_CHUNK; ++tt) {
      if (tc + tt < t1) {
        const TA* row = proj + (size_t)(tc + tt) * ld;
        const float* gr = gates + (size_t)(tc + tt) * 2 * H * dk;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
          const int i = lane + k * BLM_WAVE;
          if (i < dk) {
            raw_f[tt][k] = gr[h * dk + i];
            raw_q[tt][k] = gr[(size_t)H * dk + h * dk + i];
          }
        }
        v_in[tt] = own ? to_float(row[(size_t)2 * H * dk + h * dv + col]) : 0.f;
      }
    }
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += SCAN_CHUNK) {
    const int n = min(SCAN_CHUNK, t1 - tc);
#pragma unroll
    for (int tt = 0; tt < SCAN_CHUNK; ++tt) {
      if (tt < n) {
        if (g == 0) v_sm[tt * SCAN_COLS + cl] = v_in[tt];
#pragma unroll
        for (int k = 0; k < PER; ++k) {
          const int i = lane + k * BLM_WAVE;
          if (i < dkp) {
            const int at = scan_place<ROWS>(i);
            base[(tt * 2) * vec + at] = i < dk ? raw_f[tt][k] : 0.f;
            base[(tt * 2 + 1) * vec + at] = i < dk ? raw_q[tt][k] : 0.f;
          }
        }
      }
    }
    if (tc + SCAN_CHUNK < t1) fetch(tc + SCAN_CHUNK);     // the next chunk's inputs travel while this one runs
    __builtin_amdgcn_wave_barrier();      // the piece of shared memory is the wavefront's own: reads follow writes in order
#pragma unroll 1
    for (int tt = 0; tt < n; ++tt) {
      {
        const float* fg = base + (tt * 2) * vec + g * (ROWS + 4);
        const float vv = v_sm[tt * SCAN_COLS + cl];
        float o = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
          const float4 f4 = *reinterpret_cast<const float4*>(fg + r);
          const float4 q4 = *reinterpret_cast<const float4*>(fg + vec + r);
          const float f[4] = {f4.x, f4.y, f4.z, f4.w}, q[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            S[r + e] = fmaf(f[e], S[r + e] - vv, vv);       // f S + (1 - f) v
            o = fmaf(S[r + e], q[e], o);
          }
        }
        o = column_sum<LPC>(o);
        if (own && g == 0) o_raw[(size_t)(tc + tt) * H * dv + h * dv + col] = o;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (own) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int i = g * ROWS + r;
      if (i < dk) S_g[(size_t)i * dv + col] = S[r];
    }
  }
}

// out[t][h][j] = o_raw[t][h][j] / sqrt(mean_j(o_raw^2) + eps) * norm_w[j] (* f(gate[t][h * dv + j])); one wavefront
// per (token, head).  gate rows are gate_ld elements apart; f is the sigmoid (gate_mode 1) or SiLU (gate_mode 2).
// Rows of padding tokens hold whatever o_raw holds (the caller clears it).
template <typename TA>
__global__ void __launch_bounds__(SCAN_WAVES* BLM_WAVE)
    head_norm_kernel(const float* __restrict__ o_raw, const float* __restrict__ norm_w, const TA* __restrict__ gate,
                     int gate_ld, int gate_mode, int H, TA* __restrict__ out, long long n_items, int dv, float eps) {
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long item = (long long)blockIdx.x * SCAN_WAVES + wave;
  if (item >= n_items) return;
  const float* src = o_raw + (size_t)item * dv;
  const TA* grow = gate ? gate + (size_t)(item / H) * gate_ld + (size_t)(item % H) * dv : nullptr;
  float ss = 0.f;
  for (int j = lane; j < dv; j += BLM_WAVE) ss = fmaf(src[j], src[j], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
  for (int j = lane; j < dv; j += BLM_WAVE) {
    float v = src[j] * inv * norm_w[j];
    if (grow) {
      const float z = to_float(grow[j]);
      v *= gate_mode == 2 ? blm_silu(z) : blm_sigmoid(z);
    }
    out[(size_t)item * dv + j] = from_float<TA>(v);
  }
}

// The same for rows of many lanes (a norm over all heads' lanes together): a block of four wavefronts per row, the
// row's values kept in registers between the two passes (up to HEAD_NORM_WIDE_PER per thread, else read again).
#define HEAD_NORM_WIDE_PER 8
template <typename TA>
__global__ void __launch_bounds__(256)
    head_norm_wide_kernel(const float* __restrict__ o_raw, const float* __restrict__ norm_w, const TA* __restrict__ gate,
                          int gate_ld, int gate_mode, int H, TA* __restrict__ out, int dv, float eps) {
  __shared__ float part[4];
  const long long item = blockIdx.x;
  const float* src = o_raw + (size_t)item * dv;
  const TA* grow = gate ? gate + (size_t)(item / H) * gate_ld + (size_t)(item % H) * dv : nullptr;
  float x[HEAD_NORM_WIDE_PER];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < HEAD_NORM_WIDE_PER; ++k) {
    const int j = threadIdx.x + k * 256;
    x[k] = j < dv ? src[j] : 0.f;
    ss = fmaf(x[k], x[k], ss);
  }
  for (int j = threadIdx.x + HEAD_NORM_WIDE_PER * 256; j < dv; j += 256) ss = fmaf(src[j], src[j], ss);
  ss = wave_sum(ss);
  if ((threadIdx.x & (BLM_WAVE - 1)) == 0) part[threadIdx.x / BLM_WAVE] = ss;
  __syncthreads();
  const float inv = 1.0f / sqrtf((part[0] + part[1] + part[2] + part[3]) / (float)dv + eps);
  auto put = [&](int j, float xv) {
    float v = xv * inv * norm_w[j];
    if (grow) {
      const float z = to_float(grow[j]);
      v *= gate_mode == 2 ? blm_silu(z) : blm_sigmoid(z);
    }
    out[(size_t)item * dv + j] = from_float<TA>(v);
  };
#pragma unroll
  for (int k = 0; k < HEAD_NORM_WIDE_PER; ++k) {
    const int j = threadIdx.x + k * 256;
    if (j < dv) put(j, x[k]);
  }
  for (int j = threadIdx.x + HEAD_NORM_WIDE_PER * 256; j < dv; j += 256) put(j, src[j]);
}

static int launch_head_norm(const float* o_raw, const float* norm_w, const void* gate, int gate_ld, int gate_mode, int H,
                            void* out, int dtype, long long items, int dv, float eps, hipStream_t stream) {
  if (dv >= 512 && items < (1ll << 31)) {
    if (dtype == BLM_F32)
      hipLaunchKernelGGL(head_norm_wide_kernel<float>, dim3((unsigned)items), dim3(256), 0, stream, o_raw, norm_w,
                         (const float*)gate, gate_ld, gate_mode, H, (float*)out, dv, eps);
    else
      hipLaunchKernelGGL(head_norm_wide_kernel<bf16>, dim3((unsigned)items), dim3(256), 0, stream, o_raw, norm_w,
                         (const bf16*)gate, gate_ld, gate_mode, H, (bf16*)out, dv, eps);
    BLM_LAUNCH_CHECK("head_norm_wide");
    return 0;
  }
  const unsigned blocks = (unsigned)((items + SCAN_WAVES - 1) / SCAN_WAVES);
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(head_norm_kernel<float>, dim3(blocks), dim3(SCAN_WAVES * BLM_WAVE), 0, stream, o_raw, norm_w,
                       (const float*)gate, gate_ld, gate_mode, H, (float*)out, items, dv, eps);
  else
    hipLaunchKernelGGL(head_norm_kernel<bf16>, dim3(blocks), dim3(SCAN_WAVES * BLM_WAVE), 0, stream, o_raw, norm_w,
                       (const bf16*)gate, gate_ld, gate_mode, H, (bf16*)out, items, dv, eps);
  BLM_LAUNCH_CHECK("head_norm");
  return 0;
}

// Wavefronts per block and shared memory of a scan whose wavefronts each keep `vectors` per-channel vectors for a
// chunk of tokens: as many wavefronts (up to four) as fit the 64 KB a kernel gets without asking.
struct ScanLaunch {
  dim3 grid, block;
  size_t smem;
};
static ScanLaunch scan_launch(int rows, int lpc, int vectors, long long items, int chunk = SCAN_CHUNK) {
  const size_t per_wave = (size_t)chunk * (vectors * lpc * (rows + 4) + (vectors - 1) * SCAN_COLS) * sizeof(float);
  int waves = (int)((64 * 1024) / per_wave);
  waves = waves > SCAN_WAVES ? SCAN_WAVES : (waves < 1 ? 1 : waves);
  ScanLaunch sl;
  sl.grid = dim3((unsigned)((items + waves - 1) / waves));
  sl.block = dim3(waves * BLM_WAVE);
  sl.smem = per_wave * waves;
  return sl;
}

// rows per lane: the key channels dealt to a column's lanes, rounded up to what the kernels are built for; 16 lanes
// per column where the sequences bring many tokens each (see above)
#define BLM_SCAN_PICK(CALL)                                  \
  do {                                                       \
    if (T > 4 * B) {                                         \
      const int rows = (dk + 15) / 16;                       \
      if (rows <= 4) { CALL(4, 16); }                        \
      else if (rows <= 8) { CALL(8, 16); }                   \
      else { CALL(16, 16); }                                 \
    } else {                                                 \
      const int rows = (dk + 3) / 4;                         \
      if (rows <= 4) { CALL(4, 4); }                         \
      else if (rows <= 8) { CALL(8, 4); }                    \
      else if (rows <= 16) { CALL(16, 4); }                  \
      else if (rows <= 32) { CALL(32, 4); }                  \
      else { CALL(64, 4); }                                  \
    }                                                        \
  } while (0)

extern "C" int blm_hgrn2_scan(const void* proj, int dtype, int ld, const float* f_bias, const float* low,
                              const float* norm_w, float eps, float* state, float* gates, float* o_raw, void* out,
                              const int* cu_seqlens, const int* seq_slots, int T, int B, int H, int dk, int dv,
                              hipStream_t stream) {
  BLM_REQUIRE(T > 0 && B > 0 && H > 0, "hgrn2_scan: bad sizes T=%d B=%d H=%d", T, B, H);
  BLM_REQUIRE(dk >= 1 && dk <= SCAN_MAX_DK && dv >= 1, "hgrn2_scan: %d key channels per head are not supported (up to %d)", dk, SCAN_MAX_DK);
  BLM_REQUIRE(ld >= 2 * H * dk + H * dv, "hgrn2_scan: rows of %d are too short", ld);
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "hgrn2_scan: unsupported dtype %d", dtype);
  {   // gates and activated queries of every token [T][2 * H*dk]
    const long long n = (long long)T * H * dk;
    const unsigned gblocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    if (dtype == BLM_F32)
      hipLaunchKernelGGL(hgrn2_gates_kernel<float>, dim3(gblocks), dim3(256), 0, stream, (const float*)proj, ld, f_bias, low, gates, n, H * dk);
    else
      hipLaunchKernelGGL(hgrn2_gates_kernel<bf16>, dim3(gblocks), dim3(256), 0, stream, (const bf16*)proj, ld, f_bias, low, gates, n, H * dk);
    BLM_LAUNCH_CHECK("hgrn2_gates");
  }
#define BLM_HG(ROWS, LPC)                                                                                              \
  const int col_groups = (dv + 64 / LPC - 1) / (64 / LPC);                                                             \
  const long long items = (long long)B * H * col_groups;                                                               \
  const ScanLaunch sl = scan_launch(ROWS, LPC, 2, items);                                                              \
  if (dtype == BLM_F32)                                                                                                \
    hipLaunchKernelGGL((hgrn2_scan_kernel<float, ROWS, LPC>), sl.grid, sl.block, sl.smem, stream, (const float*)proj, ld, gates, \
                       state, o_raw, cu_seqlens, seq_slots, H, dk, dv, col_groups, items);                             \
  else                                                                                                                 \
    hipLaunchKernelGGL((hgrn2_scan_kernel<bf16, ROWS, LPC>), sl.grid, sl.block, sl.smem, stream, (const bf16*)proj, ld, gates,   \
                       state, o_raw, cu_seqlens, seq_slots, H, dk, dv, col_groups, items)
  BLM_SCAN_PICK(BLM_HG);
#undef BLM_HG
  BLM_LAUNCH_CHECK("hgrn2_scan");
  return launch_head_norm(o_raw, norm_w, nullptr, 0, 0, H, out, dtype, (long long)T * H, dv, eps, stream);
}

// ---------------------------------------------------------------------------------------
// Short causal convolution per channel, SiLU, and unit norms of the query and key heads.
// proj [T][ld]: channels 0 .. C-1 are [q: G*dk | k: G*dk | v: rest].  taps_w [C][taps] (last column: the
// current token).  hist [slots][taps-1][C] float: the inputs of the taps-1 tokens before the step, oldest
// first.  out [T][C] float: q / sqrt(sum q^2 + 1e-6) * dk^-1/2, k / sqrt(sum k^2 + 1e-6), v.
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void conv_prepare_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ taps_w, int taps,
                                    const float* __restrict__ hist, float* __restrict__ out,
                                    const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                                    const int* __restrict__ seq_slots, int C, int G, int dk) {
  // block (t, p): channels p * dk .. p * dk + dk - 1 of token t: a query or key head (p < 2 G), or as many values
  __shared__ float red[17];
  const int t = blockIdx.x, c0 = blockIdx.y * dk;
  const int b = token_seq[t];
  float* o = out + (size_t)t * C;
  const int c_end = min(c0 + dk, C);
  if (b < 0) {
    for (int c = c0 + threadIdx.x; c < c_end; c += blockDim.x) o[c] = 0.f;
    return;
  }
  const int start = cu_seqlens[b], slot = seq_slots[b];
  const int off = t - start;
  const bool unit = c0 < 2 * G * dk;
  float ss = 0.f;
  for (int c = c0 + threadIdx.x; c < c_end; c += blockDim.x) {
    float a = 0.f;
    for (int k = 0; k < taps; ++k) {
      const int src = off - (taps - 1) + k;      // offset in the step of the input under tap k
      float x;
      if (src >= 0) x = to_float(proj[(size_t)(start + src) * ld + c]);
      else x = slot >= 0 ? hist[((size_t)slot * (taps - 1) + (taps - 1 + src)) * C + c] : 0.f;
      a = fmaf(taps_w[(size_t)c * taps + k], x, a);
    }
    a = blm_silu(a);
    o[c] = a;
    ss = fmaf(a, a, ss);
  }
  if (!unit) return;
  ss = block_sum<true>(ss, red);
  const float f = (c0 < G * dk ? 1.0f / sqrtf((float)dk) : 1.f) / sqrtf(ss + 1e-6f);
  for (int c = c0 + threadIdx.x; c < c_end; c += blockDim.x) o[c] *= f;      // each thread rescales what it wrote
}

// The history after the step: the last taps-1 inputs of each sequence, taken from the step's rows and,
// where the step brought fewer, from the old history.  One thread per (sequence, channel) reads all it
// needs before it writes.  Runs after conv_prepare.
#define BLM_MAX_TAPS 16
template <typename TA>
__global__ void conv_history_kernel(const TA* __restrict__ proj, int ld, int taps, float* __restrict__ hist,
                                    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int C) {
  const int b = blockIdx.x;
  const int slot = seq_slots[b];
  const int start = cu_seqlens[b], n = cu_seqlens[b + 1] - start;
  if (slot < 0 || n <= 0) return;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float keep[BLM_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < BLM_MAX_TAPS; ++k) {
      if (k < taps - 1) {
        const int src = n - (taps - 1) + k;
        keep[k] = src >= 0 ? to_float(proj[(size_t)(start + src) * ld + c])
                           : hist[((size_t)slot * (taps - 1) + (k + n)) * C + c];
      }
    }
#pragma unroll
    for (int k = 0; k < BLM_MAX_TAPS; ++k)
      if (k < taps - 1) hist[((size_t)slot * (taps - 1) + k) * C + c] = keep[k];
  }
}

extern "C" int blm_conv_prepare(const void* proj, int dtype, int ld, const float* taps_w, int taps, float* hist,
                                float* out, const int* token_seq, const int* cu_seqlens, const int* seq_slots, int T,
                                int B, int C, int G, int dk, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && B > 0 && C > 0 && ld >= C, "conv_prepare: bad sizes T=%d B=%d C=%d ld=%d", T, B, C, ld);
  BLM_REQUIRE(taps >= 1 && taps <= BLM_MAX_TAPS, "conv_prepare: %d taps (1 to %d)", taps, BLM_MAX_TAPS);
  BLM_REQUIRE(G >= 0 && dk >= 1 && 2 * G * dk <= C && true, "conv_prepare: bad head geometry");
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "conv_prepare: unsupported dtype %d", dtype);
  const unsigned ycols = (unsigned)((C + 255) / 256);
  const unsigned pieces = (unsigned)((C + dk - 1) / dk);
  const int threads = dk <= 64 ? 64 : (dk <= 128 ? 128 : 256);
  BLM_REQUIRE(pieces <= 65535, "conv_prepare: too many heads");
  if (dtype == BLM_F32) {
    hipLaunchKernelGGL(conv_prepare_kernel<float>, dim3(T, pieces), dim3(threads), 0, stream, (const float*)proj, ld, taps_w, taps,
                       hist, out, token_seq, cu_seqlens, seq_slots, C, G, dk);
    if (taps > 1)
      hipLaunchKernelGGL(conv_history_kernel<float>, dim3(B, ycols), dim3(256), 0, stream, (const float*)proj, ld, taps, hist,
                         cu_seqlens, seq_slots, C);
  } else {
    hipLaunchKernelGGL(conv_prepare_kernel<bf16>, dim3(T, pieces), dim3(threads), 0, stream, (const bf16*)proj, ld, taps_w, taps,
                       hist, out, token_seq, cu_seqlens, seq_slots, C, G, dk);
    if (taps > 1)
      hipLaunchKernelGGL(conv_history_kernel<bf16>, dim3(B, ycols), dim3(256), 0, stream, (const bf16*)proj, ld, taps, hist,
                         cu_seqlens, seq_slots, C);
  }
  BLM_LAUNCH_CHECK("conv_prepare");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Delta rule with a decay per key channel.  qkv [T][C] float from conv_prepare (q: G*dk, k: G*dk, v: H*dv;
// head h reads q/k head h / (H / G)).  beta = sigmoid(beta_logit[t][h]); decay_i = exp(-exp(a_log[h]) *
// softplus(decay_in[t][h*dk+i] + dt_bias[h*dk+i])); per token, in this order:
//   S = diag(decay) S;  u = beta (v - S^T k);  S = S + k u^T;  o = S^T q
// then out = o / sqrt(mean(o^2) + eps) * norm_w * sigmoid(gate_in[t][h*dv+j]) by head_norm_kernel.
// beta_logit: column `beta_col` of rows of `ld_beta` elements; decay_in, gate_in: [T][H*dk], [T][H*dv].
// ---------------------------------------------------------------------------------------
// gates [T][H*dk + H] float: the decays, then beta = sigmoid(logit) per head: what does not depend on the state
template <typename TA>
__global__ void delta_gates_kernel(const TA* __restrict__ beta_src, int ld_beta, int beta_col,
                                   const TA* __restrict__ decay_in, const float* __restrict__ dt_bias,
                                   const float* __restrict__ a_log, float* __restrict__ gates, long long n, int H, int dk) {
  const int HK = H * dk, per = HK + H;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / per;
    const int c = (int)(e - t * per);
    if (c < HK)
      gates[e] = expf(-expf(a_log[c / dk]) * blm_softplus(to_float(decay_in[(size_t)t * HK + c]) + dt_bias[c]));
    else
      gates[e] = blm_sigmoid(to_float(beta_src[(size_t)t * ld_beta + beta_col + (c - HK)]));
  }
}

template <typename TA, int ROWS, int LPC>
__global__ void __launch_bounds__(SCAN_WAVES* BLM_WAVE)
    delta_scan_kernel(const float* __restrict__ qkv, int C, const float* __restrict__ gates,
                      float* __restrict__ state, float* __restrict__ o_raw, const int* __restrict__ cu_seqlens,
                      const int* __restrict__ seq_slots, int H, int G, int dk, int dv, int col_groups, long long n_items) {
  extern __shared__ __attribute__((aligned(16))) float scan_sm[];     // per wavefront: [chunk][decay | k | q][vec], [chunk][16 values + beta]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long item = (long long)blockIdx.x * (blockDim.x / BLM_WAVE) + wave;
  if (item >= n_items) return;
  const int cg = (int)(item % col_groups);
  const int h = (int)((item / col_groups) % H);
  const int b = (int)(item / ((long long)col_groups * H));
  const int slot = seq_slots[b];
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (slot < 0 || t1 <= t0) return;
  constexpr int COLS = BLM_WAVE / LPC;
  const int g = LPC == 4 ? lane >> 4 : lane & 15, cl = LPC == 4 ? lane & 15 : lane >> 4;
  const int col = cg * COLS + cl;
  const bool own = col < dv;
  const int kh = h / (H / G);
  constexpr int dkp = ROWS * LPC;
  constexpr int vec = LPC * (ROWS + 4);
  float* base = scan_sm + (size_t)wave * SCAN_CHUNK * (3 * vec + 2 * SCAN_COLS);
  float* v_sm = base + SCAN_CHUNK * 3 * vec;        // per token: 16 values, then beta
  float* S_g = state + (((size_t)slot * H + h) * dk) * dv;
  float S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int i = g * ROWS + r;
    S[r] = (own && i < dk) ? S_g[(size_t)i * dv + col] : 0.f;
  }
  constexpr int PER = (dkp + BLM_WAVE - 1) / BLM_WAVE;
  float raw_d[SCAN_CHUNK][PER], raw_k[SCAN_CHUNK][PER], raw_q[SCAN_CHUNK][PER], v_in[SCAN_CHUNK], bl_in[SCAN_CHUNK];
  auto fetch = [&](int tc) {
#pragma unroll
    for (int tt = 0; tt < SCAN_CHUNK; ++tt) {
      if (tc + tt < t1) {
        const int t = tc + tt;
        const float* row = qkv + (size_t)t * C;
        const float* gr = gates + (size_t)t * (H * dk + H);
#pragma unroll
        for (int k = 0; k < PER; ++k) {
          const int i = lane + k * BLM_WAVE;
          if (i < dk) {
            raw_d[tt][k] = gr[h * dk + i];
            raw_k[tt][k] = row[(size_t)G * dk + kh * dk + i];
            raw_q[tt][k] = row[kh * dk + i];
          }
        }
        v_in[tt] = own ? row[(size_t)2 * G * dk + h * dv + col] : 0.f;
        bl_in[tt] = gr[H * dk + h];
      }
    }
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += SCAN_CHUNK) {
    const int n = min(SCAN_CHUNK, t1 - tc);
#pragma unroll
    for (int tt = 0; tt < SCAN_CHUNK; ++tt) {
      if (tt < n) {
        if (g == 0) v_sm[tt * 2 * SCAN_COLS + cl] = v_in[tt];
        if (lane == 0) v_sm[tt * 2 * SCAN_COLS + SCAN_COLS] = bl_in[tt];
#pragma unroll
        for (int k = 0; k < PER; ++k) {
          const int i = lane + k * BLM_WAVE;
          if (i < dkp) {
            const int at = scan_place<ROWS>(i);
            base[(tt * 3) * vec + at] = i < dk ? raw_d[tt][k] : 0.f;
            base[(tt * 3 + 1) * vec + at] = i < dk ? raw_k[tt][k] : 0.f;
            base[(tt * 3 + 2) * vec + at] = i < dk ? raw_q[tt][k] : 0.f;
          }
        }
      }
    }
    if (tc + SCAN_CHUNK < t1) fetch(tc + SCAN_CHUNK);     // the next chunk's inputs travel while this one runs
    __builtin_amdgcn_wave_barrier();
#pragma unroll 1
    for (int tt = 0; tt < n; ++tt) {
      {
        const float* bg = base + (tt * 3) * vec + g * (ROWS + 4);
        const float vv = v_sm[tt * 2 * SCAN_COLS + cl], beta = v_sm[tt * 2 * SCAN_COLS + SCAN_COLS];
        float dot = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
          const float4 d4 = *reinterpret_cast<const float4*>(bg + r);
          const float4 k4 = *reinterpret_cast<const float4*>(bg + vec + r);
          const float d[4] = {d4.x, d4.y, d4.z, d4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            S[r + e] *= d[e];
            dot = fmaf(S[r + e], kk[e], dot);
          }
        }
        const float u = beta * (vv - column_sum<LPC>(dot));
        float o = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
          const float4 k4 = *reinterpret_cast<const float4*>(bg + vec + r);
          const float4 q4 = *reinterpret_cast<const float4*>(bg + 2 * vec + r);
          const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, q[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            S[r + e] = fmaf(kk[e], u, S[r + e]);
            o = fmaf(S[r + e], q[e], o);
          }
        }
        o = column_sum<LPC>(o);
        if (own && g == 0) o_raw[(size_t)(tc + tt) * H * dv + h * dv + col] = o;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (own) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int i = g * ROWS + r;
      if (i < dk) S_g[(size_t)i * dv + col] = S[r];
    }
  }
}

extern "C" int blm_delta_scan(const float* qkv, int C, const void* beta_src, int dtype, int ld_beta, int beta_col,
                              const void* decay_in, const float* dt_bias, const float* a_log, const void* gate_in,
                              const float* norm_w, float eps, float* state, float* gates, float* o_raw, void* out,
                              const int* cu_seqlens, const int* seq_slots, int T, int B, int H, int G, int dk, int dv,
                              hipStream_t stream) {
  BLM_REQUIRE(T > 0 && B > 0 && H > 0 && G > 0 && H % G == 0, "delta_scan: bad sizes T=%d B=%d H=%d G=%d", T, B, H, G);
  BLM_REQUIRE(dk >= 1 && dk <= SCAN_MAX_DK && dv >= 1, "delta_scan: %d key channels per head are not supported (up to %d)", dk, SCAN_MAX_DK);
  BLM_REQUIRE(C >= 2 * G * dk + H * dv, "delta_scan: rows of %d are too short", C);
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "delta_scan: unsupported dtype %d", dtype);
  {   // decays and write strengths of every token [T][H*dk + H]
    const long long n = (long long)T * (H * dk + H);
    const unsigned gblocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    if (dtype == BLM_F32)
      hipLaunchKernelGGL(delta_gates_kernel<float>, dim3(gblocks), dim3(256), 0, stream, (const float*)beta_src, ld_beta, beta_col,
                         (const float*)decay_in, dt_bias, a_log, gates, n, H, dk);
    else
      hipLaunchKernelGGL(delta_gates_kernel<bf16>, dim3(gblocks), dim3(256), 0, stream, (const bf16*)beta_src, ld_beta, beta_col,
                         (const bf16*)decay_in, dt_bias, a_log, gates, n, H, dk);
    BLM_LAUNCH_CHECK("delta_gates");
  }
#define BLM_DS(ROWS, LPC)                                                                                                 \
  const int col_groups = (dv + 64 / LPC - 1) / (64 / LPC);                                                                \
  const long long items = (long long)B * H * col_groups;                                                                  \
  const ScanLaunch sl = scan_launch(ROWS, LPC, 3, items);                                                                 \
  if (dtype == BLM_F32)                                                                                                   \
    hipLaunchKernelGGL((delta_scan_kernel<float, ROWS, LPC>), sl.grid, sl.block, sl.smem, stream, qkv, C, gates, state, o_raw, \
                       cu_seqlens, seq_slots, H, G, dk, dv, col_groups, items);                                           \
  else                                                                                                                    \
    hipLaunchKernelGGL((delta_scan_kernel<bf16, ROWS, LPC>), sl.grid, sl.block, sl.smem, stream, qkv, C, gates, state, o_raw,  \
                       cu_seqlens, seq_slots, H, G, dk, dv, col_groups, items)
  BLM_SCAN_PICK(BLM_DS);
#undef BLM_DS
  BLM_LAUNCH_CHECK("delta_scan");
  return launch_head_norm(o_raw, norm_w, gate_in, H * dv, 1, H, out, dtype, (long long)T * H, dv, eps, stream);
}

// ---------------------------------------------------------------------------------------
// Gated linear attention.  proj [T][ld]: q at column 0 (H*dk), k at H*dk (H*dk), v at 2*H*dk (H*dv), the output
// gate's logits at 2*H*dk + H*dv (H*dv).  decay_in [T][H*dk]: the decay's logits before their bias.
//   alpha = sigmoid(decay_in + bias)^(1/tau) = exp(-softplus(-(decay_in + bias)) / tau)
//   S = diag(alpha) S + k v^T;  o = S^T (q * dk^-1/2)
// then out = o / sqrt(mean(o^2) + eps) * norm_w * silu(gate) by head_norm_kernel.
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void gla_gates_kernel(const TA* __restrict__ decay_in, const float* __restrict__ bias, float inv_tau,
                                 float* __restrict__ gates, long long n, int HK) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride)
    gates[e] = expf(-blm_softplus(-(to_float(decay_in[e]) + bias[e % HK])) * inv_tau);
}

// SiLU in place on the first `cols` columns of every row (queries, keys and values of a step whose sequences are walked
// in segments: there every column group of a head would otherwise activate the head's queries and keys again).  The
// result is rounded to the rows' type, as the walk that activates on the way rounds it.
template <typename TA>
__global__ void silu_rows_kernel(TA* __restrict__ proj, int ld, int cols, long long n) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / cols;
    TA* at = proj + (size_t)t * ld + (e - t * cols);
    *at = from_float<TA>(blm_silu(to_float(*at)));
  }
}

// With SEG a sequence's tokens are cut into n_seg segments of seg_len tokens that different wavefronts walk at the
// same time: the first from the sequence's state, the others from zero.  The recurrence is linear in the state, so
//   S_t = (prod of the segment's decays up to t) S_start + (what the walk from zero gives),
//   o_t = (q_t * that product)^T S_start + (the walk's o_t):
// a segment leaves its end state, the product of all its decays and, per token, the query times the running product;
// gla_carry_kernel then passes the true start states from segment to segment (and leaves the sequence's state), and
// gla_apply_kernel adds the first term to the results.  Decays are at most one, so the products cannot overflow.
template <typename TA, int ROWS, int LPC, bool SEG, int CH>
__global__ void __launch_bounds__(SCAN_WAVES* BLM_WAVE)
    gla_scan_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ gates, int gates_ld, int act, float q_scale,
                    float* __restrict__ state, float* __restrict__ o_raw, const int* __restrict__ cu_seqlens,
                    const int* __restrict__ seq_slots, int H, int dk, int dv, int col_groups, long long n_items,
                    int n_seg, int seg_len, float* __restrict__ seg_end, float* __restrict__ seg_decay,
                    float* __restrict__ q_tilde) {
  extern __shared__ __attribute__((aligned(16))) float scan_sm[];     // per wavefront: [chunk][decay | k | q][vec], [chunk][16 values]
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const long long item = (long long)blockIdx.x * (blockDim.x / BLM_WAVE) + wave;
  if (item >= n_items) return;
  const int cg = (int)(item % col_groups);
  const int h = (int)((item / col_groups) % H);
  const int seg = SEG ? (int)((item / ((long long)col_groups * H)) % n_seg) : 0;
  const int b = (int)(item / ((long long)col_groups * H * (SEG ? n_seg : 1)));
  const int slot = seq_slots[b];
  const int seq_end = cu_seqlens[b + 1];
  const int t0 = cu_seqlens[b] + seg * (SEG ? seg_len : 0);
  const int t1 = SEG ? min(seq_end, t0 + seg_len) : seq_end;
  if (slot < 0 || t1 <= t0) return;
  constexpr int COLS = BLM_WAVE / LPC;
  const int g = LPC == 4 ? lane >> 4 : lane & 15, cl = LPC == 4 ? lane & 15 : lane >> 4;
  const int col = cg * COLS + cl;
  const bool own = col < dv;
  constexpr int dkp = ROWS * LPC;
  constexpr int vec = LPC * (ROWS + 4);
  float* base = scan_sm + (size_t)wave * CH * (3 * vec + 2 * SCAN_COLS);
  float* v_sm = base + CH * 3 * vec;
  float* S_g = state + (((size_t)slot * H + h) * dk) * dv;
  float S[ROWS], D[SEG ? ROWS : 1];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int i = g * ROWS + r;
    S[r] = (own && i < dk && seg == 0) ? S_g[(size_t)i * dv + col] : 0.f;
    if (SEG) D[r] = 1.f;
  }
  const bool writes_rows = SEG && cl == 0 && cg == 0;      // one column's lanes write what belongs to the rows alone
  constexpr int PER = (dkp + BLM_WAVE - 1) / BLM_WAVE;
  float raw_d[CH][PER], raw_k[CH][PER], raw_q[CH][PER], v_in[CH];
  auto fetch = [&](int tc) {
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) {
      if (tc + tt < t1) {
        const int t = tc + tt;
        const TA* row = proj + (size_t)t * ld;
        const float* gr = gates + (size_t)t * gates_ld;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
          const int i = lane + k * BLM_WAVE;
          if (i < dk) {
            raw_d[tt][k] = gr[h * dk + i];
            const float kx = to_float(row[(size_t)H * dk + h * dk + i]), qx = to_float(row[h * dk + i]);
            raw_k[tt][k] = act ? to_float(from_float<TA>(blm_silu(kx))) : kx;
            raw_q[tt][k] = (act ? to_float(from_float<TA>(blm_silu(qx))) : qx) * q_scale;
          }
        }
        v_in[tt] = own ? to_float(row[(size_t)2 * H * dk + h * dv + col]) : 0.f;
        if (act) v_in[tt] = to_float(from_float<TA>(blm_silu(v_in[tt])));
      }
    }
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += CH) {
    const int n = min(CH, t1 - tc);
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) {
      if (tt < n) {
        if (g == 0) v_sm[tt * 2 * SCAN_COLS + cl] = v_in[tt];
#pragma unroll
        for (int k = 0; k < PER; ++k) {
          const int i = lane + k * BLM_WAVE;
          if (i < dkp) {
            const int at = scan_place<ROWS>(i);
            base[(tt * 3) * vec + at] = i < dk ? raw_d[tt][k] : 0.f;
            base[(tt * 3 + 1) * vec + at] = i < dk ? raw_k[tt][k] : 0.f;
            base[(tt * 3 + 2) * vec + at] = i < dk ? raw_q[tt][k] : 0.f;
          }
        }
      }
    }
    if (tc + CH < t1) fetch(tc + CH);     // the next chunk's inputs travel while this one runs
    __builtin_amdgcn_wave_barrier();
#pragma unroll 1
    for (int tt = 0; tt < n; ++tt) {
      const float* bg = base + (tt * 3) * vec + g * (ROWS + 4);
      const float vv = v_sm[tt * 2 * SCAN_COLS + cl];
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < ROWS; r += 4) {
        const float4 d4 = *reinterpret_cast<const float4*>(bg + r);
        const float4 k4 = *reinterpret_cast<const float4*>(bg + vec + r);
        const float4 q4 = *reinterpret_cast<const float4*>(bg + 2 * vec + r);
        const float d[4] = {d4.x, d4.y, d4.z, d4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, q[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[r + e] = fmaf(d[e], S[r + e], kk[e] * vv);
          o = fmaf(S[r + e], q[e], o);
          if (SEG) {
            D[r + e] *= d[e];
            if (writes_rows && seg > 0 && g * ROWS + r + e < dk)
              q_tilde[((size_t)(tc + tt) * H + h) * dk + g * ROWS + r + e] = q[e] * D[r + e];
          }
        }
      }
      o = column_sum<LPC>(o);
      if (own && g == 0) o_raw[(size_t)(tc + tt) * H * dv + h * dv + col] = o;
    }
    __builtin_amdgcn_wave_barrier();
  }
  float* S_out = SEG ? seg_end + ((((size_t)b * n_seg + seg) * H + h) * dk) * dv : S_g;
  if (own) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int i = g * ROWS + r;
      if (i < dk) S_out[(size_t)i * dv + col] = S[r];
    }
  }
  if (writes_rows) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int i = g * ROWS + r;
      if (i < dk) seg_decay[(((size_t)b * n_seg + seg) * H + h) * dk + i] = D[SEG ? r : 0];
    }
  }
}

// From segment to segment: start[s + 1] = decay[s] * start[s] + end[s], with start[1] = end[0] (the first segment
// walked from the sequence's own state); what comes out behind the last segment is the sequence's state.
__global__ void gla_carry_kernel(const float* __restrict__ seg_end, const float* __restrict__ seg_decay,
                                 float* __restrict__ seg_start, float* __restrict__ state, const int* __restrict__ cu_seqlens,
                                 const int* __restrict__ seq_slots, int H, int dk, int dv, int n_seg, int seg_len) {
  const int b = blockIdx.y;
  const int slot = seq_slots[b];
  const int n_new = cu_seqlens[b + 1] - cu_seqlens[b];
  if (slot < 0 || n_new <= 0) return;
  const int ns = (n_new + seg_len - 1) / seg_len;
  const size_t per = (size_t)H * dk * dv;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < per; e += (size_t)gridDim.x * blockDim.x) {
    const size_t row = e / dv;      // h * dk + i
    float S = seg_end[((size_t)b * n_seg) * per + e];
    for (int sgm = 1; sgm < ns; ++sgm) {
      seg_start[((size_t)b * n_seg + sgm) * per + e] = S;
      S = fmaf(seg_decay[((size_t)b * n_seg + sgm) * H * dk + row], S, seg_end[((size_t)b * n_seg + sgm) * per + e]);
    }
    state[(size_t)slot * per + e] = S;
  }
}

// o_raw[t][h][:] += q_tilde[t][h][:]^T start[segment of t][h] for the tokens of every segment but a sequence's first;
// one wavefront per (eight tokens of one segment, head), a lane per value channel (and its neighbours 64 apart).
#define GLA_APPLY_TOKENS 8
#define GLA_APPLY_CPL 4
__global__ void __launch_bounds__(BLM_WAVE)
    gla_apply_kernel(const float* __restrict__ q_tilde, const float* __restrict__ seg_start, float* __restrict__ o_raw,
                     const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int H, int dk, int dv, int n_seg,
                     int seg_len, int tiles_per_seq) {
  extern __shared__ float qt[];      // [8][dk]
  const int b = blockIdx.x / tiles_per_seq, tile = blockIdx.x - b * tiles_per_seq;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - first;
  const int off = tile * GLA_APPLY_TOKENS;
  if (seq_slots[b] < 0 || off >= n_new) return;
  const int seg = off / seg_len;      // seg_len is a multiple of eight: the tile lies in one segment
  if (seg == 0) return;
  const int n = min(GLA_APPLY_TOKENS, n_new - off);
  for (int e = lane; e < n * dk; e += BLM_WAVE) {
    const int tt = e / dk, i = e - tt * dk;
    qt[tt * dk + i] = q_tilde[((size_t)(first + off + tt) * H + h) * dk + i];
  }
  __builtin_amdgcn_wave_barrier();
  const float* Sp = seg_start + ((((size_t)b * n_seg + seg) * H + h) * dk) * dv;
  float acc[GLA_APPLY_TOKENS][GLA_APPLY_CPL];
#pragma unroll
  for (int tt = 0; tt < GLA_APPLY_TOKENS; ++tt)
#pragma unroll
    for (int c = 0; c < GLA_APPLY_CPL; ++c) acc[tt][c] = 0.f;
  for (int i = 0; i < dk; ++i) {
    float sv[GLA_APPLY_CPL];
#pragma unroll
    for (int c = 0; c < GLA_APPLY_CPL; ++c) {
      const int j = lane + c * BLM_WAVE;
      sv[c] = j < dv ? Sp[(size_t)i * dv + j] : 0.f;
    }
#pragma unroll
    for (int tt = 0; tt < GLA_APPLY_TOKENS; ++tt) {
      const float qv = tt < n ? qt[tt * dk + i] : 0.f;
#pragma unroll
      for (int c = 0; c < GLA_APPLY_CPL; ++c) acc[tt][c] = fmaf(qv, sv[c], acc[tt][c]);
    }
  }
#pragma unroll
  for (int tt = 0; tt < GLA_APPLY_TOKENS; ++tt) {
    if (tt < n) {
#pragma unroll
      for (int c = 0; c < GLA_APPLY_CPL; ++c) {
        const int j = lane + c * BLM_WAVE;
        if (j < dv) o_raw[((size_t)(first + off + tt) * H + h) * dv + j] += acc[tt][c];
      }
    }
  }
}

// n_seg > 1 (only where the sequences bring many tokens each, T > 4 B): seg_len a multiple of 8 with n_seg * seg_len >= the
// most tokens of a sequence; seg_end and seg_start [B][n_seg][H][dk][dv], seg_decay [B][n_seg][H][dk], q_tilde [T][H][dk].
// Variants of the same recurrence, for mixers that differ in what surrounds it:
//   fixed_decay [H*dk] float (not null): every token's decays, instead of decay_in, decay_bias and tau (a decay per head that
//     is a constant of the model; gates is then not used);
//   act_mode 1: SiLU on the queries, keys and values (rounded to the rows' type) as they are read, or, where the sequences
//     are walked in segments, in place beforehand: proj is then changed;  q_scale: the queries' factor (<= 0: dk^-1/2);
//   norm_all 1: the root mean square is taken over all heads' value lanes together and norm_w is [H*dv];
//   gate_mode: 1 sigmoid, 2 SiLU of the output gate's logits.
extern "C" int blm_gla_scan(void* proj, int dtype, int ld, const void* decay_in, const float* decay_bias, float tau,
                            const float* norm_w, float eps, float* state, float* gates, float* o_raw, void* out,
                            const int* cu_seqlens, const int* seq_slots, int T, int B, int H, int dk, int dv, int max_new,
                            int n_seg, int seg_len, float* seg_end, float* seg_start, float* seg_decay, float* q_tilde,
                            const float* fixed_decay, int act_mode, float q_scale_in, int norm_all, int gate_mode,
                            hipStream_t stream) {
  BLM_REQUIRE(T > 0 && B > 0 && H > 0 && (fixed_decay || tau > 0.f), "gla_scan: bad sizes T=%d B=%d H=%d tau=%g", T, B, H, (double)tau);
  BLM_REQUIRE(dk >= 1 && dk <= SCAN_MAX_DK && dv >= 1, "gla_scan: %d key channels per head are not supported (up to %d)", dk, SCAN_MAX_DK);
  BLM_REQUIRE(ld >= 2 * H * dk + 2 * H * dv, "gla_scan: rows of %d are too short", ld);
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "gla_scan: unsupported dtype %d", dtype);
  BLM_REQUIRE(n_seg >= 1 && (n_seg == 1 || (T > 4 * B && seg_len >= 8 && seg_len % 8 == 0 && (long long)n_seg * seg_len >= max_new &&
                                            dv <= BLM_WAVE * GLA_APPLY_CPL && seg_end && seg_start && seg_decay && q_tilde)),
              "gla_scan: %d segments of %d tokens do not fit this step", n_seg, seg_len);
  BLM_REQUIRE((act_mode == 0 || act_mode == 1) && (gate_mode == 1 || gate_mode == 2) && (fixed_decay || (decay_in && decay_bias && gates)),
              "gla_scan: unknown activation %d or gate %d, or no decays", act_mode, gate_mode);
  if (!fixed_decay) {
    const long long n = (long long)T * H * dk;
    const unsigned gblocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    if (dtype == BLM_F32)
      hipLaunchKernelGGL(gla_gates_kernel<float>, dim3(gblocks), dim3(256), 0, stream, (const float*)decay_in, decay_bias, 1.0f / tau, gates, n, H * dk);
    else
      hipLaunchKernelGGL(gla_gates_kernel<bf16>, dim3(gblocks), dim3(256), 0, stream, (const bf16*)decay_in, decay_bias, 1.0f / tau, gates, n, H * dk);
    BLM_LAUNCH_CHECK("gla_gates");
  }
  if (act_mode == 1 && n_seg > 1) {
    const int cols = 2 * H * dk + H * dv;
    const long long n = (long long)T * cols;
    const unsigned ablocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
    if (dtype == BLM_F32) hipLaunchKernelGGL(silu_rows_kernel<float>, dim3(ablocks), dim3(256), 0, stream, (float*)proj, ld, cols, n);
    else hipLaunchKernelGGL(silu_rows_kernel<bf16>, dim3(ablocks), dim3(256), 0, stream, (bf16*)proj, ld, cols, n);
    BLM_LAUNCH_CHECK("silu_rows");
    act_mode = 0;
  }
  const float q_scale = q_scale_in > 0.f ? q_scale_in : 1.0f / sqrtf((float)dk);
  const float* decays = fixed_decay ? fixed_decay : gates;
  const int decays_ld = fixed_decay ? 0 : H * dk;
#define BLM_GLA_RUN(ROWS, LPC, SEG, NSEG, CH)                                                                             \
  const int col_groups = (dv + 64 / LPC - 1) / (64 / LPC);                                                                \
  const long long items = (long long)B * NSEG * H * col_groups;                                                           \
  const ScanLaunch sl = scan_launch(ROWS, LPC, 3, items, CH);                                                             \
  if (dtype == BLM_F32)                                                                                                   \
    hipLaunchKernelGGL((gla_scan_kernel<float, ROWS, LPC, SEG, CH>), sl.grid, sl.block, sl.smem, stream, (const float*)proj, ld, decays, decays_ld, act_mode, \
                       q_scale, state, o_raw, cu_seqlens, seq_slots, H, dk, dv, col_groups, items, n_seg, seg_len, seg_end, \
                       seg_decay, q_tilde);                                                                               \
  else                                                                                                                    \
    hipLaunchKernelGGL((gla_scan_kernel<bf16, ROWS, LPC, SEG, CH>), sl.grid, sl.block, sl.smem, stream, (const bf16*)proj, ld, decays, decays_ld, act_mode,   \
                       q_scale, state, o_raw, cu_seqlens, seq_slots, H, dk, dv, col_groups, items, n_seg, seg_len, seg_end, \
                       seg_decay, q_tilde)
  // segments: many wavefronts at once, each waiting for its own chain of dependent instructions; chunks of four tokens halve
  // a wavefront's shared memory, so that twice as many of them share a compute unit
#define BLM_GLA(ROWS, LPC) BLM_GLA_RUN(ROWS, LPC, false, 1, SCAN_CHUNK)
#define BLM_GLA_SEG(ROWS) BLM_GLA_RUN(ROWS, 16, true, n_seg, 4)
  if (n_seg > 1) {
    const int rows = (dk + 15) / 16;
    if (rows <= 4) { BLM_GLA_SEG(4); }
    else if (rows <= 8) { BLM_GLA_SEG(8); }
    else { BLM_GLA_SEG(16); }
  } else {
    BLM_SCAN_PICK(BLM_GLA);
  }
#undef BLM_GLA_SEG
#undef BLM_GLA
#undef BLM_GLA_RUN
  BLM_LAUNCH_CHECK("gla_scan");
  if (n_seg > 1) {
    const size_t per = (size_t)H * dk * dv;
    const unsigned cb = (unsigned)((per + 255) / 256 < 1024 ? (per + 255) / 256 : 1024);
    hipLaunchKernelGGL(gla_carry_kernel, dim3(cb, B), dim3(256), 0, stream, seg_end, seg_decay, seg_start, state, cu_seqlens,
                       seq_slots, H, dk, dv, n_seg, seg_len);
    BLM_LAUNCH_CHECK("gla_carry");
    const int tiles_per_seq = (max_new + GLA_APPLY_TOKENS - 1) / GLA_APPLY_TOKENS;
    hipLaunchKernelGGL(gla_apply_kernel, dim3((unsigned)(B * tiles_per_seq), H), dim3(BLM_WAVE),
                       (size_t)GLA_APPLY_TOKENS * dk * sizeof(float), stream, q_tilde, seg_start, o_raw, cu_seqlens, seq_slots, H,
                       dk, dv, n_seg, seg_len, tiles_per_seq);
    BLM_LAUNCH_CHECK("gla_apply");
  }
  const char* gate = (const char*)proj + (size_t)(2 * H * dk + H * dv) * (dtype == BLM_F32 ? 4 : 2);
  if (norm_all) return launch_head_norm(o_raw, norm_w, gate, ld, gate_mode, 1, out, dtype, (long long)T, H * dv, eps, stream);
  return launch_head_norm(o_raw, norm_w, gate, ld, gate_mode, H, out, dtype, (long long)T * H, dv, eps, stream);
}

// ---------------------------------------------------------------------------------------
// Lightning attention over prompts: chunks of 64 tokens as float32 matrix products.
// With ONE constant decay a per head the recurrence S_t = a S_(t-1) + k_t v_t^T, o_t = S_t^T q_t has a closed form inside
// a chunk of n tokens that starts from the state S0 (i, j count from the chunk's first token):
//   O = (Q K^T * L) V + diag(a^(i+1)) Q S0,   L_ij = a^(i-j) for j <= i, else 0
//   S_end = a^n S0 + (diag(a^(n-1-j)) K)^T V
// All powers are at most one and come from a table pw [H][65] = a^0 .. a^64 (made in double precision), so no quotient or
// running product of decays appears and a fast decay cannot overflow.  Kernels: silu_rows (the activation, once, in
// place), lc_state (every chunk's own contribution (diag(..) K)^T V), lc_carry (the chunks' start states in order, from
// the sequence's state, and its new state), lc_out (the chunk's results).  Operands
// are staged through shared memory in the rows' type, 16 bytes per lane and load, and multiplied by 32x32x2 float32
// matrix instructions: lane l holds row l % 32 of the left operand and column l % 32 of the right one at depth l / 32;
// result register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32.
// Heads of up to 128 key and 128 value channels, padded to multiples of 32 with zeros.
// ---------------------------------------------------------------------------------------
#define LC_CHUNK 64
#define LC_MAX 128
#define LC_THREADS 256
#define LC_A_LD (LC_CHUNK + 1)
#define LC_STEPS 8      // matrix instructions written out per turn of a loop over depth: 16 steps of depth
#define LC_LDS_LIMIT (128 * 1024)
typedef float lc_acc __attribute__((ext_vector_type(16)));

template <typename TA>
__device__ __forceinline__ int lc_row_pad() { return sizeof(TA) == 4 ? 1 : 2; }      // an odd number of 4-byte words per row

// SiLU rounded to the rows' type.  Rows of 16 bits take the hardware's exponential and reciprocal, whose errors (about
// 1e-6 of the result) are far below that rounding; float rows take the exact functions.
template <typename TA>
__device__ __forceinline__ TA lc_silu(TA v) {
  const float x = to_float(v);
  if (sizeof(TA) == 4) return from_float<TA>(blm_silu(x));
  return from_float<TA>(x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * x)));
}

// SiLU in place on the first `cols` columns of every row, 16 bytes per lane (cols and ld multiples of that many elements,
// rows aligned to 16 bytes).
template <typename TA>
__global__ void silu_rows_wide_kernel(TA* __restrict__ proj, int ld, int cols, long long n_vec) {
  constexpr int VEC = 16 / sizeof(TA);
  const int per_row = cols / VEC;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n_vec; e += stride) {
    const long long t = e / per_row;
    uint4* at = reinterpret_cast<uint4*>(proj + (size_t)t * ld + (size_t)(e - t * per_row) * VEC);
    uint4 raw = *at;
    TA* vals = reinterpret_cast<TA*>(&raw);
#pragma unroll
    for (int k = 0; k < VEC; ++k) vals[k] = lc_silu(vals[k]);
    *at = raw;
  }
}

// A chunk's rows of one head into shared memory as they are, for N operands at once (queries, keys, values): operand p
// is `width[p]` channels from column col0[p] on and arrives in dst[p] [64][row_ld[p]]; the tokens from n on and the channels
// from width up to the padded width WP arrive as zeros.  Where rows and widths allow, every lane takes 16 bytes at a
// time, has all its loads of all operands under way before it turns to the first (one trip to memory, not one per
// operand), and leaves them as 4-byte words (row_ld and the 16-byte pieces keep every word aligned).
template <typename TA, int N>
struct LcOperands {
  int col0[N], width[N], WP[N], row_ld[N];
  TA* dst[N];
};

template <typename TA, int N>
__device__ __forceinline__ void lc_stage(const TA* __restrict__ rows, int ld, int n, const LcOperands<TA, N>& op) {
  constexpr int VEC = 16 / sizeof(TA);
  bool wide = ld % VEC == 0 && (reinterpret_cast<uintptr_t>(rows) & 15) == 0;
#pragma unroll
  for (int p = 0; p < N; ++p) wide = wide && op.width[p] % VEC == 0 && op.col0[p] % VEC == 0 && op.width[p] <= LC_MAX;
  if (wide) {
    // up to 64 * 128 / VEC pieces per operand: at most 4 (16-bit rows) or 8 (float rows) per lane
    constexpr int PER = (LC_CHUNK * LC_MAX / VEC + LC_THREADS - 1) / LC_THREADS;
    uint4 raw[N][PER];
    int at[N][PER];
#pragma unroll
    for (int p = 0; p < N; ++p) {
      const int per_row = op.width[p] / VEC, items = LC_CHUNK * per_row;
      const TA* src = rows + op.col0[p];
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int e = threadIdx.x + u * LC_THREADS, j = e / per_row, i = (e - j * per_row) * VEC;
        at[p][u] = e < items ? j * op.row_ld[p] + i : -1;
        raw[p][u] = (e < items && j < n) ? *reinterpret_cast<const uint4*>(src + (size_t)j * ld + i) : uint4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int p = 0; p < N; ++p) {
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        if (at[p][u] >= 0) {
          uint32_t* w = reinterpret_cast<uint32_t*>(op.dst[p] + at[p][u]);
          w[0] = raw[p][u].x; w[1] = raw[p][u].y; w[2] = raw[p][u].z; w[3] = raw[p][u].w;
        }
      }
      if (op.WP[p] > op.width[p]) {
        const int extra = op.WP[p] - op.width[p];
        for (int e = threadIdx.x; e < LC_CHUNK * extra; e += LC_THREADS)
          op.dst[p][(e / extra) * op.row_ld[p] + op.width[p] + e % extra] = from_float<TA>(0.f);
      }
    }
  } else {
#pragma unroll
    for (int p = 0; p < N; ++p) {
      const TA* src = rows + op.col0[p];
      for (int e = threadIdx.x; e < LC_CHUNK * op.WP[p]; e += LC_THREADS) {
        const int j = e / op.WP[p], i = e - j * op.WP[p];
        op.dst[p][j * op.row_ld[p] + i] = (j < n && i < op.width[p]) ? src[(size_t)j * ld + i] : from_float<TA>(0.f);
      }
    }
  }
}

// seg_end [B][n_seg][H][dk][dv]: what the chunk's own tokens add to the state by the chunk's end
template <typename TA>
__global__ void __launch_bounds__(LC_THREADS)
    lc_state_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ pw, float* __restrict__ seg_end,
                    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int H, int dk, int dv, int n_seg) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lc_sm[];
  const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int slot = seq_slots[b], first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - first;
  const int t0 = c * LC_CHUNK;
  if (slot < 0 || t0 >= n_new) return;
  const int n = min(LC_CHUNK, n_new - t0);
  const int DKP = (dk + 31) & ~31, DVP = (dv + 31) & ~31;
  float* wj = reinterpret_cast<float*>(lc_sm);                      // [64]: a^(n-1-j), zero from n on
  TA* Ks = reinterpret_cast<TA*>(wj + LC_CHUNK);                    // [64][DKP]
  TA* Vs = Ks + LC_CHUNK * DKP;                                     // [64][DVP]
  const float* pwh = pw + h * (LC_CHUNK + 1);
  const TA* rows = proj + (size_t)(first + t0) * ld;
  {
    LcOperands<TA, 2> op;
    op.col0[0] = H * dk + h * dk; op.width[0] = dk; op.WP[0] = DKP; op.row_ld[0] = DKP; op.dst[0] = Ks;
    op.col0[1] = 2 * H * dk + h * dv; op.width[1] = dv; op.WP[1] = DVP; op.row_ld[1] = DVP; op.dst[1] = Vs;
    lc_stage<TA, 2>(rows, ld, n, op);
  }
  if (threadIdx.x < LC_CHUNK) wj[threadIdx.x] = threadIdx.x < n ? pwh[n - 1 - threadIdx.x] : 0.f;
  __syncthreads();
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int lr = lane & 31, lk = lane >> 5;
  const int NV = DVP / 32, tiles = (DKP / 32) * NV;
  const int depth = (n + 2 * LC_STEPS - 1) & ~(2 * LC_STEPS - 1);
  lc_acc acc[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[s][r] = 0.f;
  int k_at[4], v_at[4];      // where the wavefront's tiles start in a row of keys and of values
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int t = min(wave + 4 * s, tiles - 1), tr = t / NV;
    k_at[s] = tr * 32 + lr;
    v_at[s] = (t - tr * NV) * 32 + lr;
  }
  // The weight of token j goes onto its values.  Every wavefront multiplies four tiles whether it has that many or not (a
  // wavefront with fewer repeats its last one into accumulators that are never stored): a matrix instruction under a
  // condition would make the compiler move its sixteen result registers about in every turn of the loop.
  // (A loop whose turns are counted at run time is not unrolled around matrix instructions: sixteen steps of depth are
  // written out per turn, and the depth is rounded up to that; what lies behind the chunk's tokens is zeros.)
  for (int kb = 0; kb < depth; kb += 2 * LC_STEPS) {
#pragma unroll
    for (int u = 0; u < LC_STEPS; ++u) {
      const int k0 = kb + 2 * u;
      const TA* krow = Ks + (k0 + lk) * DKP;
      const TA* vrow = Vs + (k0 + lk) * DVP;
      const float w = wj[k0 + lk];
#pragma unroll
      for (int s = 0; s < 4; ++s)
        acc[s] = __builtin_amdgcn_mfma_f32_32x32x2f32(to_float(krow[k_at[s]]), to_float(vrow[v_at[s]]) * w, acc[s], 0, 0, 0);
    }
  }
  const size_t at = (((size_t)b * n_seg + c) * H + h) * (size_t)dk * dv;
  const bool whole = (dk & 31) == 0 && (dv & 31) == 0;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int t = wave + 4 * s;
    if (t < tiles) {
      const int tr = t / NV, tc = t - tr * NV;
      const int col = tc * 32 + lr, i0 = tr * 32 + 4 * lk;
      float* end_p = seg_end + at + (size_t)i0 * dv + col;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int di = 8 * (r / 4) + (r & 3);
        if (whole || (i0 + di < dk && col < dv)) end_p[(size_t)di * dv] = acc[s][r];
      }
    }
  }
}

// From chunk to chunk: start[0] is the sequence's state, start[c + 1] = a^(tokens of chunk c) start[c] + end[c]; what
// comes out behind the last chunk is the sequence's new state.
__global__ void lc_carry_kernel(const float* __restrict__ seg_end, float* __restrict__ seg_start, float* __restrict__ state,
                                const float* __restrict__ pw, const int* __restrict__ cu_seqlens,
                                const int* __restrict__ seq_slots, int H, int dk, int dv, int n_seg) {
  const int b = blockIdx.y;
  const int slot = seq_slots[b];
  const int n_new = cu_seqlens[b + 1] - cu_seqlens[b];
  if (slot < 0 || n_new <= 0) return;
  const int ns = (n_new + LC_CHUNK - 1) / LC_CHUNK;
  const size_t per_head = (size_t)dk * dv, per = (size_t)H * per_head;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < per; e += (size_t)gridDim.x * blockDim.x) {
    const float* pwh = pw + (e / per_head) * (LC_CHUNK + 1);
    const float whole = pwh[LC_CHUNK], last = pwh[n_new - (ns - 1) * LC_CHUNK];
    float S = state[(size_t)slot * per + e];
    for (int c = 0; c < ns; ++c) {
      const size_t at = ((size_t)b * n_seg + c) * per + e;
      seg_start[at] = S;
      S = fmaf(c + 1 < ns ? whole : last, S, seg_end[at]);
    }
    state[(size_t)slot * per + e] = S;
  }
}

template <typename TA>
__global__ void __launch_bounds__(LC_THREADS)
    lc_out_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ pw, const float* __restrict__ seg_start,
                  float* __restrict__ o_raw, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int H, int dk,
                  int dv, int n_seg) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lc_sm[];
  const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int slot = seq_slots[b], first = cu_seqlens[b], n_new = cu_seqlens[b + 1] - first;
  const int t0 = c * LC_CHUNK;
  if (slot < 0 || t0 >= n_new) return;
  const int n = min(LC_CHUNK, n_new - t0);
  const int DKP = (dk + 31) & ~31, DVP = (dv + 31) & ~31;
  const int SK = DKP + lc_row_pad<TA>();
  float* As = reinterpret_cast<float*>(lc_sm);                      // [64][65]: (Q K^T) * L
  float* pws = As + LC_CHUNK * LC_A_LD;                             // [65] (+ 3 unused)
  TA* Qs = reinterpret_cast<TA*>(pws + LC_CHUNK + 4);               // [64][SK]
  TA* Ks = Qs + LC_CHUNK * SK;                                      // [64][SK]
  TA* Vs = Ks + LC_CHUNK * SK;                                      // [64][DVP]
  const TA* rows = proj + (size_t)(first + t0) * ld;
  {
    LcOperands<TA, 3> op;
    op.col0[0] = h * dk; op.width[0] = dk; op.WP[0] = DKP; op.row_ld[0] = SK; op.dst[0] = Qs;
    op.col0[1] = H * dk + h * dk; op.width[1] = dk; op.WP[1] = DKP; op.row_ld[1] = SK; op.dst[1] = Ks;
    op.col0[2] = 2 * H * dk + h * dv; op.width[2] = dv; op.WP[2] = DVP; op.row_ld[2] = DVP; op.dst[2] = Vs;
    lc_stage<TA, 3>(rows, ld, n, op);
  }
  if (threadIdx.x <= LC_CHUNK) pws[threadIdx.x] = pw[h * (LC_CHUNK + 1) + threadIdx.x];
  __syncthreads();
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int lr = lane & 31, lk = lane >> 5;
  // scores of the three tiles at and below the diagonal, times the powers of the decay
  if (wave < 3) {
    const int ti = wave == 0 ? 0 : 1, tj = wave == 2 ? 1 : 0;
    lc_acc sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
    const TA* qrow = Qs + (ti * 32 + lr) * SK + lk;
    const TA* krow = Ks + (tj * 32 + lr) * SK + lk;
    for (int kb = 0; kb < DKP; kb += 2 * LC_STEPS) {
#pragma unroll
      for (int u = 0; u < LC_STEPS; ++u)
        sc = __builtin_amdgcn_mfma_f32_32x32x2f32(to_float(qrow[kb + 2 * u]), to_float(krow[kb + 2 * u]), sc, 0, 0, 0);
    }
    const int j = tj * 32 + lr;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = ti * 32 + 8 * (r / 4) + 4 * lk + (r & 3);
      As[i * LC_A_LD + j] = j <= i ? sc[r] * pws[i - j] : 0.f;
    }
  }
  __syncthreads();
  const int NV = DVP / 32;
  const int ti = wave & 1, tc0 = wave >> 1;
  const bool two = tc0 + 2 < NV;
  // A wavefront without a first or second tile of its own repeats the head's last column tile and stores nothing of it:
  // no matrix instruction stands under a condition (see lc_state_kernel).
  const int ca = min(tc0, NV - 1) * 32 + lr, cb = min(tc0 + 2, NV - 1) * 32 + lr;
  lc_acc acc[2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[s][r] = 0.f;
  // what the chunk's start state gives: Q S0, row i times a^(i+1).  Columns from dv on and the row behind an odd dk are
  // read from the last valid column and row: such columns are never stored, and that row meets zeros of Q.
  {
    const float* S0 = seg_start + (((size_t)b * n_seg + c) * H + h) * (size_t)dk * dv;
    const TA* qrow = Qs + (ti * 32 + lr) * SK + lk;
    const float* s0 = S0 + min(ca, dv - 1);
    const float* s1 = S0 + min(cb, dv - 1);
    for (int kb = 0; kb < DKP; kb += 2 * LC_STEPS) {
      float sa[LC_STEPS], sb[LC_STEPS];
#pragma unroll
      for (int u = 0; u < LC_STEPS; ++u) {
        const size_t row = (size_t)min(kb + 2 * u + lk, dk - 1) * dv;
        sa[u] = s0[row];
        sb[u] = s1[row];
      }
#pragma unroll
      for (int u = 0; u < LC_STEPS; ++u) {
        const float a = to_float(qrow[kb + 2 * u]);
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, sa[u], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, sb[u], acc[1], 0, 0, 0);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float f = pws[ti * 32 + 8 * (r / 4) + 4 * lk + (r & 3) + 1];
      acc[0][r] *= f;
      acc[1][r] *= f;
    }
  }
  // what the chunk's own tokens give: (scores * L) V, over the keys up to the row tile's last row
  {
    const float* arow = As + (ti * 32 + lr) * LC_A_LD + lk;
    const TA* v0 = Vs + lk * DVP + ca;
    const TA* v1 = Vs + lk * DVP + cb;
    const int depth = min((ti + 1) * 32, (n + 2 * LC_STEPS - 1) & ~(2 * LC_STEPS - 1));
    for (int kb = 0; kb < depth; kb += 2 * LC_STEPS) {
#pragma unroll
      for (int u = 0; u < LC_STEPS; ++u) {
        const int k0 = kb + 2 * u;
        const float a = arow[k0];
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, to_float(v0[k0 * DVP]), acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, to_float(v1[k0 * DVP]), acc[1], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const int col = (tc0 + 2 * s) * 32 + lr;
    if ((s == 0 ? tc0 < NV : two) && col < dv) {
      const int i0 = ti * 32 + 4 * lk;
      float* o = o_raw + ((size_t)(first + t0 + i0) * H + h) * dv + col;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int di = 8 * (r / 4) + (r & 3);
        if (i0 + di < n) o[(size_t)di * H * dv] = acc[s][r];
      }
    }
  }
}

static size_t lc_state_lds(int dk, int dv, int dtype) {
  const int DKP = (dk + 31) & ~31, DVP = (dv + 31) & ~31;
  return (size_t)LC_CHUNK * sizeof(float) + (size_t)LC_CHUNK * (DKP + DVP) * (dtype == BLM_F32 ? 4 : 2);
}
static size_t lc_out_lds(int dk, int dv, int dtype) {
  const int DKP = (dk + 31) & ~31, DVP = (dv + 31) & ~31;
  const int es = dtype == BLM_F32 ? 4 : 2, SK = DKP + (dtype == BLM_F32 ? 1 : 2);
  return (size_t)(LC_CHUNK * LC_A_LD + LC_CHUNK + 4) * sizeof(float) + (size_t)LC_CHUNK * (2 * SK + DVP) * es;
}

#define LC_DEVICES 64
static bool g_lc_ready[LC_DEVICES];
// Once per device, outside any stream capture: the chunk kernels take more shared memory than a kernel gets without asking.
extern "C" int blm_lightning_chunks_init() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  BLM_REQUIRE(e == hipSuccess && dev >= 0 && dev < LC_DEVICES, "lightning_chunks_init: hipGetDevice failed or device %d is beyond %d", dev, LC_DEVICES);
  const void* ks[] = {(const void*)lc_state_kernel<float>, (const void*)lc_state_kernel<bf16>, (const void*)lc_out_kernel<float>,
                      (const void*)lc_out_kernel<bf16>};
  for (const void* k : ks) {
    e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, LC_LDS_LIMIT);
    BLM_REQUIRE(e == hipSuccess, "lightning_chunks_init: cannot raise the shared memory limit: %s", hipGetErrorString(e));
  }
  g_lc_ready[dev] = true;
  return 0;
}

extern "C" int blm_lightning_chunks_supported(int dk, int dv) { return (dk >= 1 && dk <= LC_MAX && dv >= 1 && dv <= LC_MAX) ? 1 : 0; }

// proj as for blm_gla_scan (queries, keys, values, output-gate logits); pw [H][65] float: powers 0 .. 64 of every head's
// decay; n_seg: chunks of 64 tokens that cover the longest sequence of the step; seg_end, seg_start [B][n_seg][H][dk][dv]
// float.  state is read and left updated; o_raw [T][H*dv] float; out [T][H*dv] in proj's type.
// act_mode, norm_all, gate_mode as for blm_gla_scan (act_mode 1 activates proj's queries, keys and values in place).
extern "C" int blm_lightning_chunks(void* proj, int dtype, int ld, const float* pw, const float* norm_w, float eps,
                                    float* state, float* o_raw, void* out, const int* cu_seqlens, const int* seq_slots, int T,
                                    int B, int H, int dk, int dv, int max_new, int n_seg, float* seg_end, float* seg_start,
                                    int act_mode, int norm_all, int gate_mode, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && B > 0 && B <= 65535 && H > 0 && H <= 65535, "lightning_chunks: bad sizes T=%d B=%d H=%d", T, B, H);
  BLM_REQUIRE(blm_lightning_chunks_supported(dk, dv), "lightning_chunks: heads of %d x %d channels are not supported (up to %d)", dk, dv, LC_MAX);
  BLM_REQUIRE(ld >= 2 * H * dk + 2 * H * dv, "lightning_chunks: rows of %d are too short", ld);
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "lightning_chunks: unsupported dtype %d", dtype);
  BLM_REQUIRE(max_new >= 1 && n_seg >= 1 && (long long)n_seg * LC_CHUNK >= max_new && pw && seg_end && seg_start,
              "lightning_chunks: %d chunks do not cover %d tokens, or no workspace", n_seg, max_new);
  BLM_REQUIRE((act_mode == 0 || act_mode == 1) && (gate_mode == 1 || gate_mode == 2), "lightning_chunks: unknown activation %d or gate %d", act_mode, gate_mode);
  int dev = -1;
  BLM_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < LC_DEVICES && g_lc_ready[dev],
              "lightning_chunks: blm_lightning_chunks_init has not run on device %d", dev);
  const size_t lds_a = lc_state_lds(dk, dv, dtype), lds_c = lc_out_lds(dk, dv, dtype);
  BLM_REQUIRE(lds_a <= LC_LDS_LIMIT && lds_c <= LC_LDS_LIMIT, "lightning_chunks: %zu bytes of shared memory are too many", lds_c);
  if (act_mode == 1) {
    const int cols = 2 * H * dk + H * dv, vec = dtype == BLM_F32 ? 4 : 8;
    if (cols % vec == 0 && ld % vec == 0 && ((uintptr_t)proj & 15) == 0) {
      const long long n = (long long)T * (cols / vec);
      const unsigned ablocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
      if (dtype == BLM_F32) hipLaunchKernelGGL(silu_rows_wide_kernel<float>, dim3(ablocks), dim3(256), 0, stream, (float*)proj, ld, cols, n);
      else hipLaunchKernelGGL(silu_rows_wide_kernel<bf16>, dim3(ablocks), dim3(256), 0, stream, (bf16*)proj, ld, cols, n);
    } else {
      const long long n = (long long)T * cols;
      const unsigned ablocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
      if (dtype == BLM_F32) hipLaunchKernelGGL(silu_rows_kernel<float>, dim3(ablocks), dim3(256), 0, stream, (float*)proj, ld, cols, n);
      else hipLaunchKernelGGL(silu_rows_kernel<bf16>, dim3(ablocks), dim3(256), 0, stream, (bf16*)proj, ld, cols, n);
    }
    BLM_LAUNCH_CHECK("silu_rows");
  }
  const dim3 grid((unsigned)n_seg, (unsigned)H, (unsigned)B);
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(lc_state_kernel<float>, grid, dim3(LC_THREADS), lds_a, stream, (const float*)proj, ld, pw, seg_end,
                       cu_seqlens, seq_slots, H, dk, dv, n_seg);
  else
    hipLaunchKernelGGL(lc_state_kernel<bf16>, grid, dim3(LC_THREADS), lds_a, stream, (const bf16*)proj, ld, pw, seg_end,
                       cu_seqlens, seq_slots, H, dk, dv, n_seg);
  BLM_LAUNCH_CHECK("lc_state");
  const size_t per = (size_t)H * dk * dv;
  const unsigned cb = (unsigned)((per + 255) / 256 < 1024 ? (per + 255) / 256 : 1024);
  hipLaunchKernelGGL(lc_carry_kernel, dim3(cb, B), dim3(256), 0, stream, seg_end, seg_start, state, pw, cu_seqlens, seq_slots, H,
                     dk, dv, n_seg);
  BLM_LAUNCH_CHECK("lc_carry");
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(lc_out_kernel<float>, grid, dim3(LC_THREADS), lds_c, stream, (const float*)proj, ld, pw, seg_start,
                       o_raw, cu_seqlens, seq_slots, H, dk, dv, n_seg);
  else
    hipLaunchKernelGGL(lc_out_kernel<bf16>, grid, dim3(LC_THREADS), lds_c, stream, (const bf16*)proj, ld, pw, seg_start,
                       o_raw, cu_seqlens, seq_slots, H, dk, dv, n_seg);
  BLM_LAUNCH_CHECK("lc_out");
  const char* gate = (const char*)proj + (size_t)(2 * H * dk + H * dv) * (dtype == BLM_F32 ? 4 : 2);
  if (norm_all) return launch_head_norm(o_raw, norm_w, gate, ld, gate_mode, 1, out, dtype, (long long)T, H * dv, eps, stream);
  return launch_head_norm(o_raw, norm_w, gate, ld, gate_mode, H, out, dtype, (long long)T * H, dv, eps, stream);
}
