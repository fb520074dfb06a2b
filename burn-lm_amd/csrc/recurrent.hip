// Recurrent mixers whose state is a matrix [key channels][value channels] per head and sequence, kept in
// float in the cache's state tensors: a gated linear recurrence whose forget gate also weighs the write
// (HGRN2), and a delta rule with one decay per key channel.  One block per (sequence, head) walks the
// sequence's tokens of the step in order; thread j owns column j of the state (all key channels of one
// value channel) in registers, so a token costs each thread two passes over its column and the block one
// reduction for the norm of the head's result.  Columns are independent of each other; what a token needs
// of the key side (gates, keys, queries: one value per key channel) is prepared by the block's threads
// together in shared memory.  The same kernels serve prompts and decoding (a sequence then brings one token).
//
// Also here: the short causal convolution in front of the delta rule with its per-sequence history.
#include "common.h"

__device__ __forceinline__ float blm_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float blm_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float blm_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// ---------------------------------------------------------------------------------------
// HGRN2.  proj [T][ld]: q at column 0 (H*dk), forget-gate logits at H*dk (H*dk), values at 2*H*dk (H*dv).
//   f = low + (1 - low) * sigmoid(logit + bias);  S = diag(f) S + (1 - f) v^T;  o = S^T silu(q)
//   out = o / sqrt(mean(o^2) + eps) * norm_w      (per head, over its dv lanes)
// state [slots][H][dk][dv] float.
// ---------------------------------------------------------------------------------------
template <typename TA, int DK>
__global__ void hgrn2_scan_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ f_bias,
                                  const float* __restrict__ low, const float* __restrict__ norm_w, float eps,
                                  float* __restrict__ state, TA* __restrict__ out, const int* __restrict__ cu_seqlens,
                                  const int* __restrict__ seq_slots, int H, int dk, int dv) {
  extern __shared__ float sm[];          // two buffers of [f (dk) | q (dk)]
  __shared__ float red[17];
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int slot = seq_slots[b];
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (slot < 0 || t1 <= t0) return;
  float* S_g = state + (((size_t)slot * H + h) * dk) * dv;
  float S[DK];
  const bool own = j < dv;
#pragma unroll
  for (int i = 0; i < DK; ++i) S[i] = (own && i < dk) ? S_g[(size_t)i * dv + j] : 0.f;
  const float nw = own ? norm_w[j] : 0.f;
  for (int t = t0; t < t1; ++t) {
    float* fq = sm + (size_t)((t - t0) & 1) * 2 * dk;
    const TA* row = proj + (size_t)t * ld;
    for (int i = j; i < dk; i += blockDim.x) {
      const float lo = low[h * dk + i];
      fq[i] = lo + (1.f - lo) * blm_sigmoid(to_float(row[(size_t)H * dk + h * dk + i]) + f_bias[h * dk + i]);
      fq[dk + i] = blm_silu(to_float(row[h * dk + i]));
    }
    const float v = own ? to_float(row[(size_t)2 * H * dk + h * dv + j]) : 0.f;
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      if (i < dk) {
        const float f = fq[i];
        S[i] = fmaf(f, S[i], (1.f - f) * v);
        o = fmaf(S[i], fq[dk + i], o);
      }
    }
    const float ss = block_sum(own ? o * o : 0.f, red);
    if (own) out[(size_t)t * H * dv + h * dv + j] = from_float<TA>(o * (1.0f / sqrtf(ss / (float)dv + eps)) * nw);
  }
  if (own) {
#pragma unroll
    for (int i = 0; i < DK; ++i)
      if (i < dk) S_g[(size_t)i * dv + j] = S[i];
  }
}

#define BLM_SCAN_PICK(CALL)                  \
  do {                                       \
    if (dk <= 16) { CALL(16); }              \
    else if (dk <= 32) { CALL(32); }         \
    else if (dk <= 64) { CALL(64); }         \
    else if (dk <= 128) { CALL(128); }       \
    else { CALL(256); }                      \
  } while (0)

extern "C" int blm_hgrn2_scan(const void* proj, int dtype, int ld, const float* f_bias, const float* low,
                              const float* norm_w, float eps, float* state, void* out, const int* cu_seqlens,
                              const int* seq_slots, int B, int H, int dk, int dv, hipStream_t stream) {
  BLM_REQUIRE(B > 0 && H > 0 && H <= 65535, "hgrn2_scan: bad sizes B=%d H=%d", B, H);
  BLM_REQUIRE(dk >= 1 && dk <= 256 && dv >= 1 && dv <= 1024, "hgrn2_scan: a head of %d x %d is not supported (up to 256 x 1024)", dk, dv);
  BLM_REQUIRE(ld >= 2 * H * dk + H * dv, "hgrn2_scan: rows of %d are too short", ld);
  const int threads = (dv + BLM_WAVE - 1) / BLM_WAVE * BLM_WAVE;
  const size_t smem = (size_t)4 * dk * sizeof(float);
  dim3 grid(B, H), block(threads);
#define BLM_HG(DK)                                                                                                       \
  if (dtype == BLM_F32)                                                                                                  \
    hipLaunchKernelGGL((hgrn2_scan_kernel<float, DK>), grid, block, smem, stream, (const float*)proj, ld, f_bias, low,   \
                       norm_w, eps, state, (float*)out, cu_seqlens, seq_slots, H, dk, dv);                               \
  else                                                                                                                   \
    hipLaunchKernelGGL((hgrn2_scan_kernel<bf16, DK>), grid, block, smem, stream, (const bf16*)proj, ld, f_bias, low,     \
                       norm_w, eps, state, (bf16*)out, cu_seqlens, seq_slots, H, dk, dv)
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "hgrn2_scan: unsupported dtype %d", dtype);
  BLM_SCAN_PICK(BLM_HG);
#undef BLM_HG
  BLM_LAUNCH_CHECK("hgrn2_scan");
  return 0;
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
  extern __shared__ float y[];
  const int t = blockIdx.x;
  const int b = token_seq[t];
  float* o = out + (size_t)t * C;
  if (b < 0) {
    for (int c = threadIdx.x; c < C; c += blockDim.x) o[c] = 0.f;
    return;
  }
  const int start = cu_seqlens[b], slot = seq_slots[b];
  const int off = t - start;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float a = 0.f;
    for (int k = 0; k < taps; ++k) {
      const int src = off - (taps - 1) + k;      // offset in the step of the input under tap k
      float x;
      if (src >= 0) x = to_float(proj[(size_t)(start + src) * ld + c]);
      else x = slot >= 0 ? hist[((size_t)slot * (taps - 1) + (taps - 1 + src)) * C + c] : 0.f;
      a = fmaf(taps_w[(size_t)c * taps + k], x, a);
    }
    y[c] = blm_silu(a);
  }
  __syncthreads();
  const int n_qk = 2 * G * dk;
  const float q_scale = 1.0f / sqrtf((float)dk);
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float v = y[c];
    if (c < n_qk) {
      const float* head = y + (c / dk) * dk;
      float ss = 0.f;
      for (int i = 0; i < dk; ++i) ss = fmaf(head[i], head[i], ss);
      v = v / sqrtf(ss + 1e-6f) * (c < G * dk ? q_scale : 1.f);
    }
    o[c] = v;
  }
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
  BLM_REQUIRE(G >= 0 && dk >= 1 && 2 * G * dk <= C && (size_t)C * sizeof(float) <= 64 * 1024, "conv_prepare: bad head geometry");
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "conv_prepare: unsupported dtype %d", dtype);
  const size_t smem = (size_t)C * sizeof(float);
  const unsigned ycols = (unsigned)((C + 255) / 256);
  if (dtype == BLM_F32) {
    hipLaunchKernelGGL(conv_prepare_kernel<float>, dim3(T), dim3(256), smem, stream, (const float*)proj, ld, taps_w, taps,
                       hist, out, token_seq, cu_seqlens, seq_slots, C, G, dk);
    if (taps > 1)
      hipLaunchKernelGGL(conv_history_kernel<float>, dim3(B, ycols), dim3(256), 0, stream, (const float*)proj, ld, taps, hist,
                         cu_seqlens, seq_slots, C);
  } else {
    hipLaunchKernelGGL(conv_prepare_kernel<bf16>, dim3(T), dim3(256), smem, stream, (const bf16*)proj, ld, taps_w, taps,
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
//   out = o / sqrt(mean(o^2) + eps) * norm_w * sigmoid(gate_in[t][h*dv+j])
// beta_logit: column `beta_col` of rows of `ld_beta` elements; decay_in, gate_in: [T][H*dk], [T][H*dv].
// ---------------------------------------------------------------------------------------
template <typename TA, int DK>
__global__ void delta_scan_kernel(const float* __restrict__ qkv, int C, const TA* __restrict__ beta_src, int ld_beta,
                                  int beta_col, const TA* __restrict__ decay_in, const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, const TA* __restrict__ gate_in,
                                  const float* __restrict__ norm_w, float eps, float* __restrict__ state,
                                  TA* __restrict__ out, const int* __restrict__ cu_seqlens,
                                  const int* __restrict__ seq_slots, int H, int G, int dk, int dv) {
  extern __shared__ float sm[];          // two buffers of [decay (dk) | k (dk) | q (dk) | beta (1)]
  __shared__ float red[17];
  const int b = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int slot = seq_slots[b];
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (slot < 0 || t1 <= t0) return;
  const int g = h / (H / G);
  float* S_g = state + (((size_t)slot * H + h) * dk) * dv;
  float S[DK];
  const bool own = j < dv;
#pragma unroll
  for (int i = 0; i < DK; ++i) S[i] = (own && i < dk) ? S_g[(size_t)i * dv + j] : 0.f;
  const float nw = own ? norm_w[j] : 0.f;
  const float rate = expf(a_log[h]);
  const int stride = 3 * dk + 1;
  for (int t = t0; t < t1; ++t) {
    float* buf = sm + (size_t)((t - t0) & 1) * stride;
    const float* row = qkv + (size_t)t * C;
    for (int i = j; i < dk; i += blockDim.x) {
      buf[i] = expf(-rate * blm_softplus(to_float(decay_in[(size_t)t * H * dk + h * dk + i]) + dt_bias[h * dk + i]));
      buf[dk + i] = row[(size_t)G * dk + g * dk + i];
      buf[2 * dk + i] = row[g * dk + i];
    }
    if (j == 0) buf[3 * dk] = blm_sigmoid(to_float(beta_src[(size_t)t * ld_beta + beta_col + h]));
    const float v = own ? row[(size_t)2 * G * dk + h * dv + j] : 0.f;
    const float gate = own ? blm_sigmoid(to_float(gate_in[(size_t)t * H * dv + h * dv + j])) : 0.f;
    __syncthreads();
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      if (i < dk) {
        S[i] *= buf[i];
        dot = fmaf(S[i], buf[dk + i], dot);
      }
    }
    const float u = buf[3 * dk] * (v - dot);
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      if (i < dk) {
        S[i] = fmaf(buf[dk + i], u, S[i]);
        o = fmaf(S[i], buf[2 * dk + i], o);
      }
    }
    const float ss = block_sum(own ? o * o : 0.f, red);
    if (own) out[(size_t)t * H * dv + h * dv + j] = from_float<TA>(o * (1.0f / sqrtf(ss / (float)dv + eps)) * nw * gate);
  }
  if (own) {
#pragma unroll
    for (int i = 0; i < DK; ++i)
      if (i < dk) S_g[(size_t)i * dv + j] = S[i];
  }
}

extern "C" int blm_delta_scan(const float* qkv, int C, const void* beta_src, int dtype, int ld_beta, int beta_col,
                              const void* decay_in, const float* dt_bias, const float* a_log, const void* gate_in,
                              const float* norm_w, float eps, float* state, void* out, const int* cu_seqlens,
                              const int* seq_slots, int B, int H, int G, int dk, int dv, hipStream_t stream) {
  BLM_REQUIRE(B > 0 && H > 0 && H <= 65535 && G > 0 && H % G == 0, "delta_scan: bad sizes B=%d H=%d G=%d", B, H, G);
  BLM_REQUIRE(dk >= 1 && dk <= 256 && dv >= 1 && dv <= 1024, "delta_scan: a head of %d x %d is not supported (up to 256 x 1024)", dk, dv);
  BLM_REQUIRE(C >= 2 * G * dk + H * dv, "delta_scan: rows of %d are too short", C);
  BLM_REQUIRE(dtype == BLM_F32 || dtype == BLM_BF16, "delta_scan: unsupported dtype %d", dtype);
  const int threads = (dv + BLM_WAVE - 1) / BLM_WAVE * BLM_WAVE;
  const size_t smem = (size_t)2 * (3 * dk + 1) * sizeof(float);
  dim3 grid(B, H), block(threads);
#define BLM_DS(DK)                                                                                                        \
  if (dtype == BLM_F32)                                                                                                   \
    hipLaunchKernelGGL((delta_scan_kernel<float, DK>), grid, block, smem, stream, qkv, C, (const float*)beta_src, ld_beta, \
                       beta_col, (const float*)decay_in, dt_bias, a_log, (const float*)gate_in, norm_w, eps, state,       \
                       (float*)out, cu_seqlens, seq_slots, H, G, dk, dv);                                                 \
  else                                                                                                                    \
    hipLaunchKernelGGL((delta_scan_kernel<bf16, DK>), grid, block, smem, stream, qkv, C, (const bf16*)beta_src, ld_beta,   \
                       beta_col, (const bf16*)decay_in, dt_bias, a_log, (const bf16*)gate_in, norm_w, eps, state,         \
                       (bf16*)out, cu_seqlens, seq_slots, H, G, dk, dv)
  BLM_SCAN_PICK(BLM_DS);
#undef BLM_DS
  BLM_LAUNCH_CHECK("delta_scan");
  return 0;
}
