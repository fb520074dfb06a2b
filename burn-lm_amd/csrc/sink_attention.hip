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
// bias [H*dk (+ G*dk + G*dv)] float or null.  cos_sin [positions][rot/2][2] float.
// ---------------------------------------------------------------------------------------
template <typename TA>
__global__ void qkv_prepare_kernel(TA* __restrict__ qkv, int ld, const float* __restrict__ bias,
                                   const float* __restrict__ cos_sin, int rot, const int* __restrict__ positions,
                                   const int* __restrict__ token_seq, const int* __restrict__ block_table, int table_width,
                                   TA* __restrict__ kcache, TA* __restrict__ vcache, int page_size, int H, int G, int dk,
                                   int dv, int write_kv) {
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
    if (i < half) {
      float u = to_float(row[col + i]), v = to_float(row[col + i + half]);
      if (bias) { u += bias[col + i]; v += bias[col + i + half]; }
      const float c = cs[2 * i], s = cs[2 * i + 1];
      const float ru = u * c - v * s, rv = v * c + u * s;
      if (krow) { krow[i] = from_float<TA>(ru); krow[i + half] = from_float<TA>(rv); }
      else { row[col + i] = from_float<TA>(ru); row[col + i + half] = from_float<TA>(rv); }
    } else {
      const int lane = rot + (i - half);
      float u = to_float(row[col + lane]);
      if (bias) u += bias[col + lane];
      if (krow) krow[lane] = from_float<TA>(u);
      else row[col + lane] = from_float<TA>(u);
    }
  }
  if (write_kv) {
    const int v0 = (H + G) * dk;
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
                               hipStream_t stream) {
  BLM_REQUIRE(T > 0 && H > 0 && G > 0 && dk > 0 && dv > 0, "qkv_prepare: bad sizes T=%d H=%d G=%d dk=%d dv=%d", T, H, G, dk, dv);
  BLM_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk, "qkv_prepare: %d turning lanes of %d (even, at most the head size)", rot, dk);
  BLM_REQUIRE(ld >= H * dk + (write_kv ? G * (dk + dv) : 0), "qkv_prepare: rows of %d are too short", ld);
  BLM_REQUIRE(!write_kv || (kcache && vcache && block_table && page_size > 0 && table_width > 0), "qkv_prepare: the pages are missing");
  BLM_REQUIRE(rot == 0 || cos_sin, "qkv_prepare: the table of angles is missing");
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(qkv_prepare_kernel<float>, dim3(T), dim3(256), 0, stream, (float*)qkv, ld, bias, cos_sin, rot, positions,
                       token_seq, block_table, table_width, (float*)kcache, (float*)vcache, page_size, H, G, dk, dv, write_kv);
  else if (dtype == BLM_BF16)
    hipLaunchKernelGGL(qkv_prepare_kernel<bf16>, dim3(T), dim3(256), 0, stream, (bf16*)qkv, ld, bias, cos_sin, rot, positions,
                       token_seq, block_table, table_width, (bf16*)kcache, (bf16*)vcache, page_size, H, G, dk, dv, write_kv);
  else
    return blm_fail("qkv_prepare: unsupported dtype %d", dtype);
  BLM_LAUNCH_CHECK("qkv_prepare");
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

// out[t][h][d] = sum_g mix[h][g] * A[t][g][c(h)][d]  (mix null: A has one slot per head and is only converted)
template <typename TA>
__global__ void talk_mix_kernel(const float* __restrict__ A, const float* __restrict__ mix, TA* __restrict__ out, int H,
                                int G, int dv) {
  const int t = blockIdx.x;
  const int n_slots = mix ? G : 1;
  const float* a = A + (size_t)t * H * n_slots * dv;
  for (int e = threadIdx.x; e < H * dv; e += blockDim.x) {
    const int h = e / dv, d = e - h * dv;
    float v;
    if (mix) {
      const int c = h / (H / G);
      v = 0.f;
      for (int g = 0; g < H; ++g) v = fmaf(mix[h * H + g], a[((size_t)g * G + c) * dv + d], v);
    } else {
      v = a[(size_t)h * dv + d];
    }
    out[(size_t)t * H * dv + e] = from_float<TA>(v);
  }
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
  const int threads = H * dv >= 1024 ? 512 : 256;
  if (dtype == BLM_F32)
    hipLaunchKernelGGL(talk_mix_kernel<float>, dim3(T), dim3(threads), 0, stream, A, mix, (float*)out, H, G, dv);
  else
    hipLaunchKernelGGL(talk_mix_kernel<bf16>, dim3(T), dim3(threads), 0, stream, A, mix, (bf16*)out, H, G, dv);
  BLM_LAUNCH_CHECK("talk_mix");
  return 0;
}
