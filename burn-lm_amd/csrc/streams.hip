// Row-wise kernels for residual arrangements with several streams: the write of a sublayer's result
// into the streams, the read of the next sublayer's input out of them and its layer norm in one pass;
// the shift that blends a row with its predecessor in the sequence; the xIELU activation.
// All arithmetic is float.  The streams are float [tokens][streams][width]; small parameter vectors
// (norm weight and bias, per-channel scales, stream coefficients) are float.
#include "common.h"

#define BLM_MAX_STREAMS 16

// ---------------------------------------------------------------------------------------
// For output row i (token r = rows ? rows[i] : i):
//   if y:  x'_t = sum_s mix[s][t] x_s + outw[t] * (sum of y's planes) * scale_y      (all t from the old x_s)
//          written back if write_x
//   u = sum_t readw[t] x'_t     (readw null: every coefficient 1)
//   out[i] = ((u - mean(u)) / sqrt(var(u) + eps) * gamma + beta) * out_scale
//   if stash: the first token of sequence b in this step leaves stash[b] = position > 0 ? carry[slot of b] : 0
//   (what a later kernel needs of the sequence's state before anything of this step overwrites it)
// ---------------------------------------------------------------------------------------
template <typename TD, typename TO>
__global__ void streams_norm_kernel(float* __restrict__ x, int S, const TD* __restrict__ y, int n_planes,
                                    size_t plane_stride, const float* __restrict__ scale_y,
                                    const float* __restrict__ mix, const float* __restrict__ outw,
                                    const float* __restrict__ readw, const float* __restrict__ gamma,
                                    const float* __restrict__ beta, TO* __restrict__ out,
                                    const int* __restrict__ rows, int D, float eps, float out_scale, int write_x,
                                    const float* __restrict__ carry, float* __restrict__ stash,
                                    const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                                    const int* __restrict__ seq_slots, const int* __restrict__ positions) {
  extern __shared__ float u_row[];
  __shared__ float red[17];
  __shared__ float s_mix[BLM_MAX_STREAMS * BLM_MAX_STREAMS], s_out[BLM_MAX_STREAMS], s_read[BLM_MAX_STREAMS];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  if (y)
    for (int k = threadIdx.x; k < S * S; k += blockDim.x) s_mix[k] = mix[k];
  if (threadIdx.x < S) {
    if (y) s_out[threadIdx.x] = outw[threadIdx.x];
    s_read[threadIdx.x] = readw ? readw[threadIdx.x] : 1.f;
  }
  __syncthreads();
  float* xr = x + (size_t)r * S * D;
  float sum = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float xs[BLM_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < BLM_MAX_STREAMS; ++s) xs[s] = s < S ? xr[(size_t)s * D + d] : 0.f;
    float u = 0.f;
    if (y) {
      float yy = 0.f;
      for (int p = 0; p < n_planes; ++p) yy += to_float(y[p * plane_stride + (size_t)r * D + d]);
      yy *= scale_y[d];
#pragma unroll
      for (int t = 0; t < BLM_MAX_STREAMS; ++t) {
        if (t < S) {
          float v = s_out[t] * yy;
#pragma unroll
          for (int s = 0; s < BLM_MAX_STREAMS; ++s)
            if (s < S) v = fmaf(s_mix[s * S + t], xs[s], v);
          if (write_x) xr[(size_t)t * D + d] = v;
          u = fmaf(s_read[t], v, u);
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < BLM_MAX_STREAMS; ++s)
        if (s < S) u = fmaf(s_read[s], xs[s], u);
    }
    u_row[d] = u;
    sum += u;
  }
  const float mean = block_sum<true>(sum, red) / (float)D;
  float sq = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float c = u_row[d] - mean;
    sq += c * c;
  }
  const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)D + eps);
  TO* o = out + (size_t)i * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x)
    o[d] = from_float<TO>(((u_row[d] - mean) * inv * gamma[d] + beta[d]) * out_scale);
  if (stash) {
    const int b = token_seq[r];
    if (b >= 0 && cu_seqlens[b] == r) {
      const int slot = seq_slots[b];
      const bool has_past = positions[r] > 0 && slot >= 0;
      for (int d = threadIdx.x; d < D; d += blockDim.x)
        stash[(size_t)b * D + d] = has_past ? carry[(size_t)slot * D + d] : 0.f;
    }
  }
}

template <typename TD, typename TO>
static int launch_streams_norm(float* x, int S, const void* y, int n_planes, long long plane_stride, const float* scale_y,
                               const float* mix, const float* outw, const float* readw, const float* gamma,
                               const float* beta, void* out, const int* rows, int n_out, int D, float eps,
                               float out_scale, int write_x, const float* carry, float* stash, const int* token_seq,
                               const int* cu_seqlens, const int* seq_slots, const int* positions, hipStream_t stream) {
  // few rows (decoding): a row's loads are what the kernel waits for, so as many threads as the row has pairs of lanes
  const int wide = ((D / 2 + BLM_WAVE - 1) / BLM_WAVE) * BLM_WAVE;
  const int threads = n_out <= 512 ? (wide < 128 ? 128 : (wide > 1024 ? 1024 : wide)) : (D >= 1024 ? 512 : (D >= 256 ? 256 : 128));
  hipLaunchKernelGGL((streams_norm_kernel<TD, TO>), dim3(n_out), dim3(threads), (size_t)D * sizeof(float), stream, x, S,
                     (const TD*)y, n_planes, (size_t)plane_stride, scale_y, mix, outw, readw, gamma, beta, (TO*)out, rows, D,
                     eps, out_scale, write_x, carry, stash, token_seq, cu_seqlens, seq_slots, positions);
  BLM_LAUNCH_CHECK("streams_norm");
  return 0;
}

extern "C" int blm_streams_norm(float* x, int S, const void* y, int y_dtype, int n_planes, long long plane_stride,
                                const float* scale_y, const float* mix, const float* outw, const float* readw,
                                const float* gamma, const float* beta, void* out, int out_dtype, const int* rows,
                                int n_out, int D, float eps, float out_scale, int write_x, const float* carry,
                                float* stash, const int* token_seq, const int* cu_seqlens, const int* seq_slots,
                                const int* positions, hipStream_t stream) {
  BLM_REQUIRE(n_out > 0 && D > 0 && D <= 16384, "streams_norm: bad sizes n=%d D=%d (width at most 16384)", n_out, D);
  BLM_REQUIRE(S >= 1 && S <= BLM_MAX_STREAMS, "streams_norm: %d streams (1 to %d)", S, BLM_MAX_STREAMS);
  BLM_REQUIRE(y == nullptr || (scale_y && mix && outw && n_planes >= 1 && n_planes <= 64 && plane_stride >= 0),
              "streams_norm: a pending result needs its scale, mixing matrix and write coefficients");
  BLM_REQUIRE(stash == nullptr || (carry && token_seq && cu_seqlens && seq_slots && positions && rows == nullptr),
              "streams_norm: the stash needs the step's index arrays and all rows");
  const int yd = y ? y_dtype : BLM_F32;
#define BLM_SN(TD, TO)                                                                                                  \
  return launch_streams_norm<TD, TO>(x, S, y, n_planes, plane_stride, scale_y, mix, outw, readw, gamma, beta, out, rows, \
                                     n_out, D, eps, out_scale, write_x, carry, stash, token_seq, cu_seqlens, seq_slots,  \
                                     positions, stream)
  if (yd == BLM_F32 && out_dtype == BLM_F32) BLM_SN(float, float);
  if (yd == BLM_F32 && out_dtype == BLM_BF16) BLM_SN(float, bf16);
  if (yd == BLM_BF16 && out_dtype == BLM_F32) BLM_SN(bf16, float);
  if (yd == BLM_BF16 && out_dtype == BLM_BF16) BLM_SN(bf16, bf16);
#undef BLM_SN
  return blm_fail("streams_norm: unsupported dtypes y=%d out=%d", y_dtype, out_dtype);
}

// ---------------------------------------------------------------------------------------
// token shift: out[t] = n[t] + (prev - n[t]) * mu, prev = n[t - 1] inside the step, else the stash of
// the token's sequence; the last token of a sequence leaves n[t] as the sequence's carry.
// ---------------------------------------------------------------------------------------
template <typename TO>
__global__ void token_shift_kernel(const float* __restrict__ n, const float* __restrict__ mu,
                                   const float* __restrict__ stash, float* __restrict__ carry, TO* __restrict__ out,
                                   const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                                   const int* __restrict__ seq_slots, int D) {
  const int t = blockIdx.x;
  const int b = token_seq[t];
  TO* o = out + (size_t)t * D;
  if (b < 0) {
    for (int d = threadIdx.x; d < D; d += blockDim.x) o[d] = from_float<TO>(0.f);
    return;
  }
  const float* cur = n + (size_t)t * D;
  const float* prev = cu_seqlens[b] == t ? stash + (size_t)b * D : cur - D;
  const int slot = seq_slots[b];
  const bool last = cu_seqlens[b + 1] - 1 == t && slot >= 0;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float c = cur[d];
    o[d] = from_float<TO>(c + (prev[d] - c) * mu[d]);
    if (last) carry[(size_t)slot * D + d] = c;
  }
}

extern "C" int blm_token_shift(const float* n, const float* mu, const float* stash, float* carry, void* out,
                               int out_dtype, const int* token_seq, const int* cu_seqlens, const int* seq_slots, int T,
                               int D, hipStream_t stream) {
  BLM_REQUIRE(T > 0 && D > 0, "token_shift: bad sizes T=%d D=%d", T, D);
  if (out_dtype == BLM_F32)
    hipLaunchKernelGGL(token_shift_kernel<float>, dim3(T), dim3(256), 0, stream, n, mu, stash, carry, (float*)out,
                       token_seq, cu_seqlens, seq_slots, D);
  else if (out_dtype == BLM_BF16)
    hipLaunchKernelGGL(token_shift_kernel<bf16>, dim3(T), dim3(256), 0, stream, n, mu, stash, carry, (bf16*)out,
                       token_seq, cu_seqlens, seq_slots, D);
  else
    return blm_fail("token_shift: unsupported dtype %d", out_dtype);
  BLM_LAUNCH_CHECK("token_shift");
  return 0;
}

// ---------------------------------------------------------------------------------------
// xIELU: z > 0: a_pos z^2 + z / 2;  z <= 0: a_neg (exp(z) - 1 - z) + z / 2
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void xielu_kernel(const TA* in, TA* out, long long n, float a_pos, float a_neg) {   // out may be in
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float z = to_float(in[i]);
    const float v = z > 0.f ? fmaf(a_pos * z, z, 0.5f * z) : fmaf(a_neg, expm1f(z) - z, 0.5f * z);
    out[i] = from_float<TA>(v);
  }
}

extern "C" int blm_xielu(const void* in, void* out, int dtype, long long n, float a_pos, float a_neg, hipStream_t stream) {
  BLM_REQUIRE(n > 0, "xielu: nothing to do");
  const long long want = (n + 255) / 256;
  const int blocks = (int)(want < 8192 ? want : 8192);
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(xielu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)in, (float*)out, n, a_pos, a_neg);
  else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(xielu_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)in, (bf16*)out, n, a_pos, a_neg);
  else
    return blm_fail("xielu: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("xielu");
  return 0;
}
