// Kernels around the sublayers of a layer whose mixer and feed-forward read the same normalised rows side by
// side: a short causal convolution added to what each sublayer reads, the float residual add of both results,
// a gated per-token side input, an RMS norm that hands on a float delta, a clamped gated activation, and the
// routing and gating of a mixture of experts whose experts run as one stacked product.
#include "common.h"

#define PB_MAX_TAPS 16
#define PB_MAX_READERS 4
#define PB_MAX_TOP 16

__device__ __forceinline__ float pb_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// ---------------------------------------------------------------------------------------
// out_r[t][c] = n[t][c] + sum_k w_r[c][k] * n(t - taps + 1 + k)[c] for every reader r (one or two); rows before the
// step come from hist [slots][taps-1][D] (oldest first; zeros in a fresh slot stand for "before the sequence").  n is
// the float output of the norm; padding tokens (sequence -1) give zeros.
// ---------------------------------------------------------------------------------------
struct PbReaders {
  const float* w[PB_MAX_READERS];   // [D][taps]
  void* out[PB_MAX_READERS];        // [T][D]
};

// A block takes PB_TOKEN_TILE tokens x 256 channels (fewer tokens per block where a step brings few): a thread keeps its
// channel's taps in registers and walks the tile's tokens, so that the taps are read once per tile and a row of n is
// found in the nearest cache by the tokens behind it.
#define PB_TOKEN_TILE 16
template <typename TO>
__global__ void input_conv_kernel(const float* __restrict__ n, float* __restrict__ hist, PbReaders rd, int readers,
                                  int taps, const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                                  const int* __restrict__ seq_slots, int T, int D, int tile, int moves_history) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= D) return;
  float w[2][PB_MAX_TAPS];
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int k = 0; k < PB_MAX_TAPS; ++k) w[r][k] = (r < readers && k < taps) ? rd.w[r][(size_t)c * taps + k] : 0.f;
  const int t_end = min(T, (int)(blockIdx.x + 1) * tile);
  for (int t = blockIdx.x * tile; t < t_end; ++t) {
    const int b = token_seq[t];
    if (b < 0) {
      for (int r = 0; r < readers; ++r) ((TO*)rd.out[r])[(size_t)t * D + c] = from_float<TO>(0.f);
      continue;
    }
    const int start = cu_seqlens[b], slot = seq_slots[b];
    const int off = t - start;
    float x[PB_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < PB_MAX_TAPS; ++k) {
      if (k < taps) {
        const int src = off - (taps - 1) + k;
        x[k] = src >= 0 ? n[(size_t)(start + src) * D + c]
                        : (slot >= 0 ? hist[((size_t)slot * (taps - 1) + (taps - 1 + src)) * D + c] : 0.f);
      }
    }
    const float cur = n[(size_t)t * D + c];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if (r < readers) {
        float a = 0.f;
#pragma unroll
        for (int k = 0; k < PB_MAX_TAPS; ++k)
          if (k < taps) a = fmaf(w[r][k], x[k], a);
        ((TO*)rd.out[r])[(size_t)t * D + c] = from_float<TO>(cur + a);
      }
    }
    // every sequence brings one token (decoding): this thread alone touches the channel's history, and has read it
    if (moves_history && slot >= 0) {
#pragma unroll
      for (int k = 0; k < PB_MAX_TAPS; ++k)
        if (k < taps - 1) hist[((size_t)slot * (taps - 1) + k) * D + c] = x[k + 1];
    }
  }
}

// the history after the step: each sequence's last taps-1 rows, from the step's rows and, where the step brought
// fewer, from the old history; a thread reads all it needs before it writes.  Runs after the convolution.
__global__ void input_history_kernel(const float* __restrict__ n, int taps, float* __restrict__ hist,
                                     const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, int D) {
  const int b = blockIdx.x;
  const int slot = seq_slots[b];
  const int start = cu_seqlens[b], cnt = cu_seqlens[b + 1] - start;
  if (slot < 0 || cnt <= 0) return;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < D; c += gridDim.y * blockDim.x) {
    float keep[PB_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < PB_MAX_TAPS; ++k) {
      if (k < taps - 1) {
        const int src = cnt - (taps - 1) + k;
        keep[k] = src >= 0 ? n[(size_t)(start + src) * D + c] : hist[((size_t)slot * (taps - 1) + (k + cnt)) * D + c];
      }
    }
#pragma unroll
    for (int k = 0; k < PB_MAX_TAPS; ++k)
      if (k < taps - 1) hist[((size_t)slot * (taps - 1) + k) * D + c] = keep[k];
  }
}

extern "C" int blm_input_conv(const float* n, float* hist, const float* w0, const float* w1, void* out0, void* out1,
                              int readers, int out_dtype, int taps, const int* token_seq, const int* cu_seqlens, const int* seq_slots,
                              int T, int B, int D, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && B > 0 && D > 0, "input_conv: bad sizes T=%d B=%d D=%d", T, B, D);
  BLM_REQUIRE(taps >= 1 && taps <= PB_MAX_TAPS, "input_conv: %d taps (1 to %d)", taps, PB_MAX_TAPS);
  BLM_REQUIRE(readers >= 1 && readers <= 2, "input_conv: %d readers (1 or 2)", readers);
  const float* weights[2] = {w0, w1};
  void* outs[2] = {out0, out1};
  BLM_REQUIRE(taps == 1 || hist, "input_conv: the history is missing");
  PbReaders rd;
  for (int r = 0; r < readers; ++r) {
    BLM_REQUIRE(weights[r] && outs[r], "input_conv: reader %d lacks its weights or output", r);
    rd.w[r] = weights[r];
    rd.out[r] = outs[r];
  }
  // few tokens (decoding): a token's channels over several blocks, so that more than a handful of compute units work
  const int threads = 256;
  const unsigned pieces = (unsigned)((D + threads - 1) / threads);
  const int tile = T >= 512 ? PB_TOKEN_TILE : 1;
  const unsigned tiles = (unsigned)((T + tile - 1) / tile);
  const int moves_history = (taps > 1 && T == B) ? 1 : 0;      // as many tokens as sequences: one each (a sequence brings at least one)
  if (out_dtype == BLM_F32)
    hipLaunchKernelGGL(input_conv_kernel<float>, dim3(tiles, pieces), dim3(threads), 0, stream, n, hist, rd, readers, taps, token_seq,
                       cu_seqlens, seq_slots, T, D, tile, moves_history);
  else if (out_dtype == BLM_BF16)
    hipLaunchKernelGGL(input_conv_kernel<bf16>, dim3(tiles, pieces), dim3(threads), 0, stream, n, hist, rd, readers, taps, token_seq,
                       cu_seqlens, seq_slots, T, D, tile, moves_history);
  else
    return blm_fail("input_conv: unsupported dtype %d", out_dtype);
  BLM_LAUNCH_CHECK("input_conv");
  if (taps > 1 && !moves_history) {
    hipLaunchKernelGGL(input_history_kernel, dim3(B, (D + 255) / 256), dim3(256), 0, stream, n, taps, hist, cu_seqlens,
                       seq_slots, D);
    BLM_LAUNCH_CHECK("input_history");
  }
  return 0;
}

// ---------------------------------------------------------------------------------------
// h[t] += a[t] + b[t] (+ bias), in float; copy[t] = the new h[t] in the activation dtype.  a and b: [T][D] in
// the activation dtype or float planes [P][T][D] that are summed in order; b may be missing.
// ---------------------------------------------------------------------------------------
template <typename TA, typename TB, typename TO>
__global__ void residual_add_kernel(float* __restrict__ h, const TA* __restrict__ a, int a_planes, const TB* __restrict__ b,
                                    int b_planes, const float* __restrict__ bias, TO* __restrict__ copy, long long n, int D) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    float da = 0.f, db = 0.f;
    for (int p = 0; p < a_planes; ++p) da += to_float(a[(size_t)p * n + e]);
    if (bias) da += bias[e % D];
    if (b)
      for (int p = 0; p < b_planes; ++p) db += to_float(b[(size_t)p * n + e]);
    const float v = h[e] + (da + db);
    h[e] = v;
    if (copy) copy[e] = from_float<TO>(v);
  }
}

extern "C" int blm_residual_add(float* h, const void* a, int a_dtype, int a_planes, const void* b, int b_dtype, int b_planes,
                                const float* bias, void* copy, int copy_dtype, int T, int D, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && D > 0 && a && a_planes >= 1 && b_planes >= 1, "residual_add: bad sizes T=%d D=%d", T, D);
  const long long n = (long long)T * D;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  if (!b) b_dtype = a_dtype;
  if (!copy) copy_dtype = BLM_F32;
#define PB_RA(TA, TB, TO)                                                                                            \
  hipLaunchKernelGGL((residual_add_kernel<TA, TB, TO>), dim3(blocks), dim3(256), 0, stream, h, (const TA*)a, a_planes, \
                     (const TB*)b, b_planes, bias, (TO*)copy, n, D)
#define PB_RA_O(TA, TB)                       \
  do {                                        \
    if (copy_dtype == BLM_F32) PB_RA(TA, TB, float); \
    else PB_RA(TA, TB, bf16);                 \
  } while (0)
  BLM_REQUIRE((a_dtype == BLM_F32 || a_dtype == BLM_BF16) && (b_dtype == BLM_F32 || b_dtype == BLM_BF16) &&
                  (copy_dtype == BLM_F32 || copy_dtype == BLM_BF16), "residual_add: unsupported dtypes");
  if (a_dtype == BLM_F32 && b_dtype == BLM_F32) PB_RA_O(float, float);
  else if (a_dtype == BLM_F32) PB_RA_O(float, bf16);
  else if (b_dtype == BLM_F32) PB_RA_O(bf16, float);
  else PB_RA_O(bf16, bf16);
#undef PB_RA_O
#undef PB_RA
  BLM_LAUNCH_CHECK("residual_add");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Side input per token: out[t][j] = gelu_tanh(z[t][j]) * table[token of t][col0 + j].  The token of row t is
// ids[t], or (as for the embedding) element source_rows[t] of the array whose address is in the source cell.
// ---------------------------------------------------------------------------------------
template <typename TA, typename TW>
__global__ void side_gate_kernel(const TA* __restrict__ z, const TW* __restrict__ table, int table_ld, int col0,
                                 const int* __restrict__ ids, const int* __restrict__ source_rows,
                                 const int* const* __restrict__ source, int V, TA* __restrict__ out, int T, int dim) {
  const long long n = (long long)T * dim;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const int t = (int)(e / dim), j = (int)(e - (long long)t * dim);
    int id = ids[t];
    if (source_rows) {
      const int r = source_rows[t];
      if (r >= 0) id = (*source)[r];
    }
    float v;
    if ((unsigned)id >= (unsigned)V) {
      v = __builtin_nanf("");
    } else {
      const float x = to_float(z[e]);
      const float g = 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
      v = g * to_float(table[(size_t)id * table_ld + col0 + j]);
    }
    out[e] = from_float<TA>(v);
  }
}

extern "C" int blm_side_gate(const void* z, int dtype, const void* table, int table_dtype, int table_ld, int col0,
                             const int* ids, const int* source_rows, const void* source_cell, int V, void* out, int T,
                             int dim, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && dim > 0 && V > 0 && col0 >= 0 && col0 + dim <= table_ld, "side_gate: bad sizes T=%d dim=%d", T, dim);
  BLM_REQUIRE((source_rows == nullptr) == (source_cell == nullptr), "side_gate: rows and cell of a token source come together");
  const long long n = (long long)T * dim;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  const int* const* cell = (const int* const*)source_cell;
#define PB_SG(TA, TW)                                                                                                 \
  hipLaunchKernelGGL((side_gate_kernel<TA, TW>), dim3(blocks), dim3(256), 0, stream, (const TA*)z, (const TW*)table, \
                     table_ld, col0, ids, source_rows, cell, V, (TA*)out, T, dim)
  if (dtype == BLM_F32 && table_dtype == BLM_F32) PB_SG(float, float);
  else if (dtype == BLM_BF16 && table_dtype == BLM_BF16) PB_SG(bf16, bf16);
  else if (dtype == BLM_F32 && table_dtype == BLM_BF16) PB_SG(float, bf16);
  else return blm_fail("side_gate: unsupported dtypes %d / %d", dtype, table_dtype);
#undef PB_SG
  BLM_LAUNCH_CHECK("side_gate");
  return 0;
}

// ---------------------------------------------------------------------------------------
// out[t] = y[t] / sqrt(mean(y[t]^2) + eps) * w, float out; y in the activation dtype or float planes that are summed.
// ---------------------------------------------------------------------------------------
template <typename TY>
__global__ void rms_scale_kernel(const TY* __restrict__ y, int planes, size_t plane_stride, const float* __restrict__ w,
                                 float* __restrict__ out, int D, float eps) {
  extern __shared__ float row[];
  __shared__ float red[17];
  const int t = blockIdx.x;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float v = 0.f;
    for (int p = 0; p < planes; ++p) v += to_float(y[p * plane_stride + (size_t)t * D + d]);
    row[d] = v;
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum<true>(ss, red) / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += blockDim.x) out[(size_t)t * D + d] = row[d] * inv * w[d];
}

extern "C" int blm_rms_scale(const void* y, int dtype, int planes, const float* w, float* out, int T, int D, float eps,
                             hipStream_t stream) {
  BLM_REQUIRE(T > 0 && D > 0 && D <= 16384 && planes >= 1, "rms_scale: bad sizes T=%d D=%d", T, D);
  const int threads = D >= 1024 ? 512 : (D >= 256 ? 256 : 128);
  const size_t stride = (size_t)T * D;
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(rms_scale_kernel<float>, dim3(T), dim3(threads), (size_t)D * sizeof(float), stream, (const float*)y,
                       planes, stride, w, out, D, eps);
  else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(rms_scale_kernel<bf16>, dim3(T), dim3(threads), (size_t)D * sizeof(float), stream, (const bf16*)y,
                       planes, stride, w, out, D, eps);
  else
    return blm_fail("rms_scale: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("rms_scale");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Clamped gated activation: g = min(gate, limit), u = clamp(up, -limit, limit); out = g * sigmoid(alpha g) * (u + 1).
// gate_up [T][2 I]: gate columns, then up columns.
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void clamped_glu_kernel(const TA* __restrict__ gate_up, TA* __restrict__ out, long long n, int I, float limit,
                                   float alpha) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / I;
    const int i = (int)(e - t * I);
    const float g = fminf(to_float(gate_up[(size_t)t * 2 * I + i]), limit);
    const float u = fminf(fmaxf(to_float(gate_up[(size_t)t * 2 * I + I + i]), -limit), limit);
    out[e] = from_float<TA>(g * pb_sigmoid(alpha * g) * (u + 1.0f));
  }
}

// eight bfloat16 at a time (I a multiple of 8, rows that start at multiples of 16 bytes)
__device__ __forceinline__ float pb_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float pb_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__global__ void clamped_glu8_kernel(const bf16* __restrict__ gate_up, bf16* __restrict__ out, long long n8, int I8, float limit,
                                    float alpha) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n8; e += stride) {
    const long long t = e / I8;
    const int i = (int)(e - t * I8);
    const uint4 g4 = *reinterpret_cast<const uint4*>(gate_up + ((size_t)t * 2 * I8 + i) * 8);
    const uint4 u4 = *reinterpret_cast<const uint4*>(gate_up + ((size_t)t * 2 * I8 + I8 + i) * 8);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float g0 = fminf(pb_lo(gw[k]), limit), g1 = fminf(pb_hi(gw[k]), limit);
      const float u0 = fminf(fmaxf(pb_lo(uw[k]), -limit), limit), u1 = fminf(fmaxf(pb_hi(uw[k]), -limit), limit);
      r[k] = f32x2_to_bf16x2_bits(g0 * pb_sigmoid(alpha * g0) * (u0 + 1.0f), g1 * pb_sigmoid(alpha * g1) * (u1 + 1.0f));
    }
    *reinterpret_cast<uint4*>(out + (size_t)e * 8) = make_uint4(r[0], r[1], r[2], r[3]);
  }
}

extern "C" int blm_clamped_glu(const void* gate_up, void* out, int dtype, int T, int I, float limit, float alpha,
                               hipStream_t stream) {
  BLM_REQUIRE(T > 0 && I > 0 && limit > 0.f, "clamped_glu: bad sizes T=%d I=%d limit=%g", T, I, (double)limit);
  const long long n = (long long)T * I;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(clamped_glu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gate_up, (float*)out, n, I, limit, alpha);
  else if (dtype == BLM_BF16 && I % 8 == 0 && ((size_t)gate_up & 15) == 0 && ((size_t)out & 15) == 0) {
    const long long n8 = n / 8;
    const unsigned b8 = (unsigned)((n8 + 255) / 256 < 65535 ? (n8 + 255) / 256 : 65535);
    hipLaunchKernelGGL(clamped_glu8_kernel, dim3(b8), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, n8, I / 8, limit, alpha);
  } else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(clamped_glu_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, n, I, limit, alpha);
  else
    return blm_fail("clamped_glu: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("clamped_glu");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Gated feed-forward activation with the tanh form of GELU on the gate branch:
//   out = 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * u;   gate_up [T][2 I]: gate columns, then up columns.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float pb_gelu_tanh(float g) {
  const float a = 0.7978845608028654f * (g + 0.044715f * g * g * g);
  // tanh(a) = 1 - 2 / (1 + e^(2a)): exact at both ends (e^(2a) -> inf gives 1, -> 0 gives -1)
  const float th = 1.0f - 2.0f / (1.0f + __expf(2.0f * a));
  return 0.5f * g * (1.0f + th);
}

template <typename TA>
__global__ void gelu_glu_kernel(const TA* __restrict__ gate_up, TA* __restrict__ out, long long n, int I) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / I;
    const int i = (int)(e - t * I);
    const float g = to_float(gate_up[(size_t)t * 2 * I + i]);
    const float u = to_float(gate_up[(size_t)t * 2 * I + I + i]);
    out[e] = from_float<TA>(pb_gelu_tanh(g) * u);
  }
}

__global__ void gelu_glu8_kernel(const bf16* __restrict__ gate_up, bf16* __restrict__ out, long long n8, int I8) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n8; e += stride) {
    const long long t = e / I8;
    const int i = (int)(e - t * I8);
    const uint4 g4 = *reinterpret_cast<const uint4*>(gate_up + ((size_t)t * 2 * I8 + i) * 8);
    const uint4 u4 = *reinterpret_cast<const uint4*>(gate_up + ((size_t)t * 2 * I8 + I8 + i) * 8);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      r[k] = f32x2_to_bf16x2_bits(pb_gelu_tanh(pb_lo(gw[k])) * pb_lo(uw[k]), pb_gelu_tanh(pb_hi(gw[k])) * pb_hi(uw[k]));
    *reinterpret_cast<uint4*>(out + (size_t)e * 8) = make_uint4(r[0], r[1], r[2], r[3]);
  }
}

extern "C" int blm_gelu_glu(const void* gate_up, void* out, int dtype, int T, int I, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && I > 0, "gelu_glu: bad sizes T=%d I=%d", T, I);
  const long long n = (long long)T * I;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(gelu_glu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gate_up, (float*)out, n, I);
  else if (dtype == BLM_BF16 && I % 8 == 0 && ((size_t)gate_up & 15) == 0 && ((size_t)out & 15) == 0) {
    const long long n8 = n / 8;
    const unsigned b8 = (unsigned)((n8 + 255) / 256 < 65535 ? (n8 + 255) / 256 : 65535);
    hipLaunchKernelGGL(gelu_glu8_kernel, dim3(b8), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, n8, I / 8);
  } else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(gelu_glu_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, n, I);
  else
    return blm_fail("gelu_glu: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("gelu_glu");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Soft cap of float logits, in place: z <- cap * tanh(z / cap).
// ---------------------------------------------------------------------------------------
__global__ void softcap_kernel(float* __restrict__ z, long long n, float cap, float inv_cap) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) z[e] = cap * tanhf(z[e] * inv_cap);
}

extern "C" int blm_softcap(float* z, long long n, float cap, hipStream_t stream) {
  BLM_REQUIRE(n > 0 && cap > 0.f, "softcap: bad sizes n=%lld cap=%g", n, (double)cap);
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL(softcap_kernel, dim3(blocks), dim3(256), 0, stream, z, n, cap, 1.0f / cap);
  BLM_LAUNCH_CHECK("softcap");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Routing of a mixture of experts.  logits [T][ld] float: E router logits, then (if shared) one logit of the
// shared expert's gate; bias [E] is added.  The `top` largest logits are chosen (the lower index wins a tie);
// their weights are the softmax over the chosen logits only.  weights [T][E + 1] float: an expert's weight or 0,
// and at E the shared expert's sigmoid gate (1 if there is no gate logit).
// ---------------------------------------------------------------------------------------
__global__ void moe_route_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ bias, int E, int top,
                                 int shared_col, float* __restrict__ weights, int T) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (size_t)t * ld;
  float* w = weights + (size_t)t * (E + 1);
  int chosen[PB_MAX_TOP];
  float val[PB_MAX_TOP];
  for (int e = 0; e < E; ++e) w[e] = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
      const float v = z[e] + bias[e];
      if (!taken && (best < 0 || v > bv)) { best = e; bv = v; }
    }
    chosen[k] = best;
    val[k] = bv;
  }
  float sum = 0.f;
  const float largest = val[0];
  for (int k = 0; k < top; ++k) { val[k] = expf(val[k] - largest); sum += val[k]; }
  for (int k = 0; k < top; ++k) w[chosen[k]] = val[k] / sum;
  w[E] = shared_col >= 0 ? pb_sigmoid(z[shared_col]) : 1.0f;
}

extern "C" int blm_moe_route(const float* logits, int ld, const float* bias, int E, int top, int shared_col, float* weights,
                             int T, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && E > 0 && top >= 1 && top <= E && top <= PB_MAX_TOP && ld >= E && shared_col < ld,
              "moe_route: bad sizes T=%d experts=%d top=%d (top at most %d)", T, E, top, PB_MAX_TOP);
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 127) / 128), dim3(128), 0, stream, logits, ld, bias, E, top, shared_col, weights, T);
  BLM_LAUNCH_CHECK("moe_route");
  return 0;
}

// The experts' gated activations, each scaled by its expert's weight for the token, for experts that run as one
// stacked product.  gate_up [T][2 I] with I = E * ffe + ffs columns of gates (expert e at e * ffe, the shared expert
// behind them), then as many of ups.  out[t][i] = silu(gate) * up * weights[t][expert of column i].
template <typename TA>
__global__ void moe_gate_kernel(const TA* __restrict__ gate_up, const float* __restrict__ weights, TA* __restrict__ out,
                                long long n, int I, int E, int ffe) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / I;
    const int i = (int)(e - t * I);
    const int ex = i / ffe < E ? i / ffe : E;
    const float w = weights[(size_t)t * (E + 1) + ex];
    float v = 0.f;
    if (w != 0.f) {
      const float g = to_float(gate_up[(size_t)t * 2 * I + i]), u = to_float(gate_up[(size_t)t * 2 * I + I + i]);
      v = g * pb_sigmoid(g) * u * w;
    }
    out[e] = from_float<TA>(v);
  }
}

// eight bfloat16 at a time (the experts' inner sizes and I multiples of 8: eight neighbours belong to one expert)
__global__ void moe_gate8_kernel(const bf16* __restrict__ gate_up, const float* __restrict__ weights, bf16* __restrict__ out,
                                 long long n8, int I8, int E, int ffe8) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n8; e += stride) {
    const long long t = e / I8;
    const int i = (int)(e - t * I8);
    const int ex = i / ffe8 < E ? i / ffe8 : E;
    const float w = weights[(size_t)t * (E + 1) + ex];
    uint32_t r[4] = {0u, 0u, 0u, 0u};
    if (w != 0.f) {
      const uint4 g4 = *reinterpret_cast<const uint4*>(gate_up + ((size_t)t * 2 * I8 + i) * 8);
      const uint4 u4 = *reinterpret_cast<const uint4*>(gate_up + ((size_t)t * 2 * I8 + I8 + i) * 8);
      const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float g0 = pb_lo(gw[k]), g1 = pb_hi(gw[k]);
        r[k] = f32x2_to_bf16x2_bits(g0 * pb_sigmoid(g0) * pb_lo(uw[k]) * w, g1 * pb_sigmoid(g1) * pb_hi(uw[k]) * w);
      }
    }
    *reinterpret_cast<uint4*>(out + (size_t)e * 8) = make_uint4(r[0], r[1], r[2], r[3]);
  }
}

extern "C" int blm_moe_gate(const void* gate_up, const float* weights, void* out, int dtype, int T, int I, int E, int ffe,
                            hipStream_t stream) {
  BLM_REQUIRE(T > 0 && E > 0 && ffe > 0 && I >= E * ffe, "moe_gate: bad sizes T=%d I=%d experts=%d of %d", T, I, E, ffe);
  const long long n = (long long)T * I;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(moe_gate_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gate_up, weights, (float*)out, n, I, E, ffe);
  else if (dtype == BLM_BF16 && I % 8 == 0 && ffe % 8 == 0 && ((size_t)gate_up & 15) == 0 && ((size_t)out & 15) == 0) {
    const long long n8 = n / 8;
    const unsigned b8 = (unsigned)((n8 + 255) / 256 < 65535 ? (n8 + 255) / 256 : 65535);
    hipLaunchKernelGGL(moe_gate8_kernel, dim3(b8), dim3(256), 0, stream, (const bf16*)gate_up, weights, (bf16*)out, n8, I / 8, E, ffe / 8);
  } else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(moe_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)gate_up, weights, (bf16*)out, n, I, E, ffe);
  else
    return blm_fail("moe_gate: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("moe_gate");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Several sublayers' results into the residual at once, each with a coefficient per channel and (optionally) per
// token:  h[t][c] += sum_i chan_i[c] * row_i[t] * sum_p y_i[p][t][c]  in float.  A term's y is [T][D] in any kernel
// dtype or float planes [P][T][D]; chan_i (float [D]) or row_i (float, row t at row_i[t * row_ld_i]) may be null
// (a factor of one).  This is how a layer with layer scale and a residual multiplier adds mixer and feed-forward,
// and how a sublayer that passes its input through (an identity expert) adds weight * input.
// ---------------------------------------------------------------------------------------
#define PB_MAX_TERMS 4
struct PbTerms {
  const void* y[PB_MAX_TERMS];
  const float* chan[PB_MAX_TERMS];
  const float* row[PB_MAX_TERMS];
  int row_ld[PB_MAX_TERMS];
  int planes[PB_MAX_TERMS];
  int dtype[PB_MAX_TERMS];
};

__global__ void scaled_add_kernel(float* __restrict__ h, PbTerms tm, int n_terms, long long n, int D) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
    const long long t = e / D;
    const int c = (int)(e - t * D);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < PB_MAX_TERMS; ++i) {
      if (i < n_terms) {
        float y = 0.f;
        if (tm.dtype[i] == BLM_F32) {
          const float* p = (const float*)tm.y[i];
          for (int k = 0; k < tm.planes[i]; ++k) y += p[(size_t)k * n + e];
        } else {
          y = to_float(((const bf16*)tm.y[i])[e]);
        }
        float f = tm.chan[i] ? tm.chan[i][c] : 1.0f;
        if (tm.row[i]) f *= tm.row[i][(size_t)t * tm.row_ld[i]];
        sum = fmaf(f, y, sum);
      }
    }
    h[e] += sum;
  }
}

// The same for four neighbouring channels per lane (D a multiple of four, every tensor aligned to 16 bytes, or 8 for
// 16-bit summands): 16-byte loads and stores, one division per four elements.
__global__ void scaled_add4_kernel(float* __restrict__ h, PbTerms tm, int n_terms, long long n4, int D4) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n4; e += stride) {
    const long long t = e / D4;
    const int c4 = (int)(e - t * D4);
    float4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < PB_MAX_TERMS; ++i) {
      if (i < n_terms) {
        float4 y = {0.f, 0.f, 0.f, 0.f};
        if (tm.dtype[i] == BLM_F32) {
          const float4* p = (const float4*)tm.y[i];
          for (int k = 0; k < tm.planes[i]; ++k) {
            const float4 v = p[(size_t)k * n4 + e];
            y.x += v.x; y.y += v.y; y.z += v.z; y.w += v.w;
          }
        } else {
          const uint2 raw = ((const uint2*)tm.y[i])[e];
          y.x = __uint_as_float(raw.x << 16); y.y = __uint_as_float(raw.x & 0xffff0000u);
          y.z = __uint_as_float(raw.y << 16); y.w = __uint_as_float(raw.y & 0xffff0000u);
        }
        float4 f = {1.f, 1.f, 1.f, 1.f};
        if (tm.chan[i]) f = ((const float4*)tm.chan[i])[c4];
        if (tm.row[i]) {
          const float r = tm.row[i][(size_t)t * tm.row_ld[i]];
          f.x *= r; f.y *= r; f.z *= r; f.w *= r;
        }
        sum.x = fmaf(f.x, y.x, sum.x); sum.y = fmaf(f.y, y.y, sum.y);
        sum.z = fmaf(f.z, y.z, sum.z); sum.w = fmaf(f.w, y.w, sum.w);
      }
    }
    float4 v = ((float4*)h)[e];
    v.x += sum.x; v.y += sum.y; v.z += sum.z; v.w += sum.w;
    ((float4*)h)[e] = v;
  }
}

extern "C" int blm_scaled_add(float* h, int T, int D, int n_terms,
                              const void* y0, int dtype0, int planes0, const float* chan0, const float* row0, int row_ld0,
                              const void* y1, int dtype1, int planes1, const float* chan1, const float* row1, int row_ld1,
                              const void* y2, int dtype2, int planes2, const float* chan2, const float* row2, int row_ld2,
                              const void* y3, int dtype3, int planes3, const float* chan3, const float* row3, int row_ld3,
                              hipStream_t stream) {
  BLM_REQUIRE(h && T > 0 && D > 0 && n_terms >= 1 && n_terms <= PB_MAX_TERMS, "scaled_add: bad sizes T=%d D=%d terms=%d", T, D, n_terms);
  PbTerms tm;
  const void* ys[PB_MAX_TERMS] = {y0, y1, y2, y3};
  const float* chans[PB_MAX_TERMS] = {chan0, chan1, chan2, chan3};
  const float* rows[PB_MAX_TERMS] = {row0, row1, row2, row3};
  const int lds[PB_MAX_TERMS] = {row_ld0, row_ld1, row_ld2, row_ld3};
  const int planes[PB_MAX_TERMS] = {planes0, planes1, planes2, planes3};
  const int dtypes[PB_MAX_TERMS] = {dtype0, dtype1, dtype2, dtype3};
  for (int i = 0; i < PB_MAX_TERMS; ++i) {
    const bool used = i < n_terms;
    BLM_REQUIRE(!used || (ys[i] && planes[i] >= 1 && (dtypes[i] == BLM_F32 || (dtypes[i] == BLM_BF16 && planes[i] == 1)) &&
                          (!rows[i] || lds[i] >= 1)),
                "scaled_add: term %d is not float planes or one bfloat16 plane", i);
    tm.y[i] = used ? ys[i] : nullptr;
    tm.chan[i] = used ? chans[i] : nullptr;
    tm.row[i] = used ? rows[i] : nullptr;
    tm.row_ld[i] = used ? lds[i] : 0;
    tm.planes[i] = used ? planes[i] : 0;
    tm.dtype[i] = used ? dtypes[i] : BLM_F32;
  }
  const long long n = (long long)T * D;
  bool wide = D % 4 == 0 && ((uintptr_t)h & 15) == 0;
  for (int i = 0; i < n_terms; ++i)
    wide = wide && ((uintptr_t)ys[i] & (dtypes[i] == BLM_F32 ? 15 : 7)) == 0 && (!chans[i] || ((uintptr_t)chans[i] & 15) == 0);
  if (wide) {
    const long long n4 = n / 4;
    const unsigned blocks4 = (unsigned)((n4 + 255) / 256 < 65535 ? (n4 + 255) / 256 : 65535);
    hipLaunchKernelGGL(scaled_add4_kernel, dim3(blocks4), dim3(256), 0, stream, h, tm, n_terms, n4, D / 4);
    BLM_LAUNCH_CHECK("scaled_add4");
    return 0;
  }
  const unsigned blocks = (unsigned)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL(scaled_add_kernel, dim3(blocks), dim3(256), 0, stream, h, tm, n_terms, n, D);
  BLM_LAUNCH_CHECK("scaled_add");
  return 0;
}

// ---------------------------------------------------------------------------------------
// Routing by scores with a correction, limited to the best groups.  logits [T][ld] float: N = E + n_identity router
// logits (the last n_identity belong to experts that pass their input through).  s = softmax(logits) over all N;
// choice = s + correction (null: none).  The N experts form `groups` equal groups of neighbours; a group's score is its
// largest choice; only experts of the `keep` best groups can be chosen (groups <= 1: all can).  The `top` largest
// choices are taken (the lower index wins a tie); their weights are s (without the correction) over the sum of the
// chosen s (+ 1e-20).  weights [T][E + 1] float: a real expert's weight or 0, and at E the sum of the weights of the
// chosen pass-through experts.
// ---------------------------------------------------------------------------------------
#define PB_MAX_ROUTED 256
#define PB_ROUTED_PER_LANE (PB_MAX_ROUTED / BLM_WAVE)

// the largest (value, index) pair over a wavefront; of equal values the one with the lower index (indices below 2^24;
// 0x7fffffff stands for "none").  Two reductions across lanes instead of a pair that travels: first the value, then the
// smallest index among the lanes that hold it.
__device__ __forceinline__ void pb_wave_best(float& v, int& i) {
  const float best = wave_max(v);
  const float mine = (v == best && i != 0x7fffffff) ? -(float)i : -3.0e9f;
  const float first = -wave_max(mine);
  v = best;
  i = first < 2.0e9f ? (int)first : 0x7fffffff;
}

// One wavefront per token; lane l holds the experts l, l + 64, ...  Scores and corrected scores stay in registers; the
// groups' ranks and the kept groups pass through the wavefront's piece of shared memory.
__global__ void __launch_bounds__(256)
    moe_route_grouped_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ correction, int E,
                             int n_identity, int groups, int keep, int top, float* __restrict__ weights, int T) {
  __shared__ float sm_choice[4][PB_MAX_ROUTED];
  __shared__ int sm_kept[4][PB_MAX_ROUTED];
  const int wave = threadIdx.x / BLM_WAVE, lane = threadIdx.x & (BLM_WAVE - 1);
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  const int N = E + n_identity;
  const float* z = logits + (size_t)t * ld;
  float* w = weights + (size_t)t * (E + 1);
  float zs[PB_ROUTED_PER_LANE], score[PB_ROUTED_PER_LANE], choice[PB_ROUTED_PER_LANE];
  float largest = -INFINITY;
#pragma unroll
  for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
    const int e = lane + k * BLM_WAVE;
    zs[k] = e < N ? z[e] : -INFINITY;
    largest = fmaxf(largest, zs[k]);
  }
  largest = wave_max(largest);
  float denom = 0.f;
#pragma unroll
  for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
    score[k] = lane + k * BLM_WAVE < N ? expf(zs[k] - largest) : 0.f;
    denom += score[k];
  }
  const float inv = 1.0f / wave_sum(denom);
#pragma unroll
  for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
    const int e = lane + k * BLM_WAVE;
    score[k] *= inv;
    choice[k] = e < N ? score[k] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  if (groups > 1) {
    const int per = N / groups;
#pragma unroll
    for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
      const int e = lane + k * BLM_WAVE;
      if (e < N) { sm_choice[wave][e] = choice[k]; sm_kept[wave][e] = 0; }
    }
    __builtin_amdgcn_wave_barrier();
    float rank[PB_ROUTED_PER_LANE];      // of group lane + k * 64: its largest corrected score
#pragma unroll
    for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
      const int g = lane + k * BLM_WAVE;
      rank[k] = -INFINITY;
      if (g < groups)
        for (int e = g * per; e < (g + 1) * per; ++e) rank[k] = fmaxf(rank[k], sm_choice[wave][e]);
    }
    bool running[PB_ROUTED_PER_LANE];
#pragma unroll
    for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) running[k] = lane + k * BLM_WAVE < groups;
    for (int n = 0; n < keep; ++n) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;      // no group
#pragma unroll
      for (int k = 0; k < PB_ROUTED_PER_LANE; ++k)
        if (running[k] && (bi == 0x7fffffff || rank[k] > bv)) { bv = rank[k]; bi = lane + k * BLM_WAVE; }
      pb_wave_best(bv, bi);
#pragma unroll
      for (int k = 0; k < PB_ROUTED_PER_LANE; ++k)
        if (lane + k * BLM_WAVE == bi) { running[k] = false; sm_kept[wave][bi] = 1; }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
      const int e = lane + k * BLM_WAVE;
      if (e < N && !sm_kept[wave][e / per]) choice[k] = -INFINITY;
    }
  }
  // the `top` largest corrected scores, one after the other; a chosen expert leaves the running
  bool mine[PB_ROUTED_PER_LANE], open[PB_ROUTED_PER_LANE];
#pragma unroll
  for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
    mine[k] = false;
    open[k] = lane + k * BLM_WAVE < N && choice[k] != -INFINITY;      // experts of groups left out never run
  }
  float sum = 0.f;
  for (int n = 0; n < top; ++n) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;      // no expert
#pragma unroll
    for (int k = 0; k < PB_ROUTED_PER_LANE; ++k)
      if (open[k] && (bi == 0x7fffffff || choice[k] > bv)) { bv = choice[k]; bi = lane + k * BLM_WAVE; }
    pb_wave_best(bv, bi);
#pragma unroll
    for (int k = 0; k < PB_ROUTED_PER_LANE; ++k)
      if (lane + k * BLM_WAVE == bi) { mine[k] = true; open[k] = false; sum += score[k]; }
  }
  sum = wave_sum(sum);
  const float norm = 1.0f / (sum + 1e-20f);
  // real experts' weights straight out; the pass-through experts' added up over the wavefront
  float passed = 0.f;
#pragma unroll
  for (int k = 0; k < PB_ROUTED_PER_LANE; ++k) {
    const int e = lane + k * BLM_WAVE;
    if (e < E) w[e] = mine[k] ? score[k] * norm : 0.f;
    else if (e < N && mine[k]) passed += score[k] * norm;
  }
  passed = wave_sum(passed);
  if (lane == 0) w[E] = passed;
}

extern "C" int blm_moe_route_grouped(const float* logits, int ld, const float* correction, int E, int n_identity, int groups,
                                     int keep, int top, float* weights, int T, hipStream_t stream) {
  const int N = E + n_identity;
  BLM_REQUIRE(T > 0 && E >= 0 && n_identity >= 0 && N >= 1 && N <= PB_MAX_ROUTED && ld >= N && top >= 1 && top <= N,
              "moe_route_grouped: bad sizes T=%d experts=%d+%d (at most %d) top=%d", T, E, n_identity, PB_MAX_ROUTED, top);
  BLM_REQUIRE(groups <= 1 || (N % groups == 0 && keep >= 1 && keep <= groups), "moe_route_grouped: %d experts in %d groups, %d kept",
              N, groups, keep);
  BLM_REQUIRE(top <= (groups > 1 ? keep * (N / groups) : N), "moe_route_grouped: top=%d is more than the kept groups hold", top);
  hipLaunchKernelGGL(moe_route_grouped_kernel, dim3((T + 3) / 4), dim3(256), 0, stream, logits, ld, correction, E,
                     n_identity, groups, keep, top, weights, T);
  BLM_LAUNCH_CHECK("moe_route_grouped");
  return 0;
}
