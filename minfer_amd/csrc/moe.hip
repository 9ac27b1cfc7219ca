// Mixture of experts: the router's choice and the experts' activation.
//
// Router: logits = Wr x in 32-bit, scores = their softmax over all experts; the experts form `n_groups`
// equal groups of neighbours, a group's score is its best expert's, only experts of the `keep` best
// groups can be chosen; the `top` best of those are chosen (ties go to the lower index) and weighted
// by their scores over the sum of the chosen scores (+ 1e-20).  One wave per token.
//
// A router may add a bias per expert to its logits.  With one group, all of it kept, the weights are the
// softmax over the chosen logits alone (the scores' common divisor cancels).
// Further options: the scores are sigmoid(logits) instead of the softmax; a correction per expert joins the
// scores for the choice of groups and experts only (the weights take the scores themselves); a group's score is
// the sum of its `group_top` best (corrected) scores instead of its best; the weights are multiplied by a scale.
//
// Expert: g = min(gate, limit), u = clamp(up, -limit, limit), y = g sigmoid(1.702 g) (u + 1); or, with
// `act` 1, the plain gated form y = silu(gate) up.
// `moe_act_kernel` applies it to the gate|up sums of every expert and multiplies by the token's
// weight for that expert (0 where it was not chosen), so that one product with the experts' down
// matrices side by side gives the weighted sum of the chosen experts' outputs.
// `moe_sparse_*`: for steps of few tokens, only the chosen experts' matrices are read: a wave per
// output row of a (token, choice) pair.
#include "common.h"

#define MF_MOE_MAX_EXPERTS 1024

#define MF_MOE_SCORE_SOFTMAX 0
#define MF_MOE_SCORE_SIGMOID 1

// index of the largest value among a wave's candidates; ties go to the lower index
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, MF_WAVE);
    const int oi = __shfl_xor(idx, o, MF_WAVE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
}

// what one wave needs to see its own earlier LDS writes (the deciding part runs in one wave)
#define MF_WAVE_SYNC()                                     \
  do {                                                     \
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront"); \
    __builtin_amdgcn_wave_barrier();                       \
  } while (0)

__device__ __forceinline__ void load4(const bf16* __restrict__ p, float (&d)[4]) {
  alignas(8) bf16 raw[4];
  *(uint2*)raw = *(const uint2*)p;
#pragma unroll
  for (int i = 0; i < 4; ++i) d[i] = (float)raw[i];
}
__device__ __forceinline__ void load4(const float* __restrict__ p, float (&d)[4]) {
  const float4 v = *(const float4*)p;
  d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
}

// x [tokens][K] in the run type, router [E][K] float32: a workgroup per token; its four waves form the E
// logits (a wave an expert at a time, lanes over K in runs of 4, sums in 32-bit), then the first wave decides.
template <typename XT>
__global__ __launch_bounds__(256) void moe_route_kernel(const XT* __restrict__ x, const float* __restrict__ router,
                                                       const float* __restrict__ bias, int K,
                                                       float* __restrict__ dense, int* __restrict__ chosen,
                                                       float* __restrict__ weights, int E, int n_groups, int keep,
                                                       int top, int score_kind, const float* __restrict__ correction,
                                                       int group_top, float weight_scale) {
  __shared__ float s[MF_MOE_MAX_EXPERTS], ms[MF_MOE_MAX_EXPERTS], gs[MF_MOE_MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const XT* xr = x + (size_t)t * K;
  for (int e = wv; e < E; e += 4) {
    const float* wr = router + (size_t)e * K;
    float a = 0.f;
    if (K % 4 == 0) {
#pragma unroll 8
      for (int i = lane * 4; i < K; i += 256) {
        float w4[4], x4[4];
        load4(wr + i, w4);
        load4(xr + i, x4);
#pragma unroll
        for (int q = 0; q < 4; ++q) a = fmaf(w4[q], x4[q], a);
      }
    } else {
      for (int i = lane; i < K; i += 64) a = fmaf(wr[i], to_f32(xr[i]), a);
    }
    a = wave_sum(a);
    if (lane == 0) s[e] = bias ? a + bias[e] : a;
  }
  __syncthreads();
  if (wv != 0) return;              // from here on one wave: MF_WAVE_SYNC where the block form has a barrier
  if (score_kind == MF_MOE_SCORE_SIGMOID) {
    for (int e = lane; e < E; e += 64) s[e] = 1.0f / (1.0f + expf(-s[e]));
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, s[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) { const float v = expf(s[e] - mx); s[e] = v; sum += v; }
    sum = wave_sum(sum);
    MF_WAVE_SYNC();
    for (int e = lane; e < E; e += 64) s[e] = s[e] / sum;
  }
  for (int e = lane; e < E; e += 64)
    if (dense) dense[(size_t)t * E + e] = 0.f;
  MF_WAVE_SYNC();
  // an expert is chosen by its score plus the correction (the weights take the score alone); what cannot be
  // chosen counts as minus infinity, since corrected scores may be negative
  const int per = E / n_groups;
  for (int g = lane; g < n_groups; g += 64) {
    // the group's `group_top` largest choice scores, summed: each pass takes the best that comes behind the last
    // one taken in the order (larger first, lower index first)
    float total = 0.f, last_v = INFINITY;
    int last_i = -1;
    for (int n = 0; n < group_top && n < per; ++n) {
      float b = -INFINITY;
      int bi = -1;
      for (int i = 0; i < per; ++i) {
        const float v = s[g * per + i] + (correction ? correction[g * per + i] : 0.f);
        const bool behind = v < last_v || (v == last_v && i > last_i);
        if (behind && (bi < 0 || v > b)) { b = v; bi = i; }
      }
      if (bi < 0) break;
      total += b;
      last_v = b;
      last_i = bi;
    }
    gs[g] = total;
  }
  for (int e = lane; e < E; e += 64) ms[e] = -INFINITY;
  MF_WAVE_SYNC();
  for (int k = 0; k < keep; ++k) {
    float b = -INFINITY;
    int bi = 0x7fffffff;
    for (int g = lane; g < n_groups; g += 64)
      if (gs[g] > b) { b = gs[g]; bi = g; }
    wave_argmax(b, bi);
    bi = min(bi, n_groups - 1);       // (nothing finite left: scores that are not numbers)
    MF_WAVE_SYNC();
    if (lane == 0) gs[bi] = -INFINITY;
    for (int i = lane; i < per; i += 64) ms[bi * per + i] = s[bi * per + i] + (correction ? correction[bi * per + i] : 0.f);
    MF_WAVE_SYNC();
  }
  float wsum = 0.f;
  int mine = -1;          // lane k keeps the k-th choice (top <= 64)
  for (int k = 0; k < top; ++k) {
    float b = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (ms[e] > b) { b = ms[e]; bi = e; }
    wave_argmax(b, bi);
    bi = min(bi, E - 1);
    MF_WAVE_SYNC();
    if (lane == 0) ms[bi] = -INFINITY;
    if (lane == k) mine = bi;
    wsum += s[bi];
    MF_WAVE_SYNC();
  }
  if (lane < top) {
    const float wgt = s[mine] / (wsum + 1e-20f) * weight_scale;
    if (dense) dense[(size_t)t * E + mine] = wgt;
    chosen[(size_t)t * top + lane] = mine;
    weights[(size_t)t * top + lane] = wgt;
  }
}

#define MF_MOE_ACT_CLAMPED 0
#define MF_MOE_ACT_SILU 1

__device__ __forceinline__ float expert_act(float g, float u, float limit, int act) {
  if (act == MF_MOE_ACT_SILU) return g * (1.0f / (1.0f + expf(-g))) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * (1.0f / (1.0f + expf(-1.702f * g))) * (u + 1.0f);
}

// gu [tokens][E][2 F] (an expert's gate sums, then its up sums); dense [tokens][E]; y [tokens][E F]
template <typename OT>
__global__ __launch_bounds__(256) void moe_act_kernel(const float* __restrict__ gu, const float* __restrict__ dense,
                                                      OT* __restrict__ y, int E, int F, float limit, int act) {
  const int t = blockIdx.x;
  const float* row = gu + (size_t)t * E * 2 * F;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < E * F; i += gridDim.y * 256) {
    const int e = i / F, f = i % F;
    const float wgt = dense[(size_t)t * E + e];
    float v = 0.f;
    if (wgt != 0.f) v = wgt * expert_act(row[(size_t)e * 2 * F + f], row[(size_t)e * 2 * F + F + f], limit, act);
    y[(size_t)t * E * F + i] = from_f32<OT>(v);
  }
}

// ------------------------------------------------------------------ few tokens: the chosen experts only
// Every chosen expert's matrices are read once, however many of the step's tokens chose it.  The step's
// (token, choice) pairs, at most MF_MOE_SPARSE_PAIRS of at most MF_MOE_SPARSE_TOKENS tokens, are found by
// the waves themselves: lane i holds the expert of pair i (and of pair i + 64), and a ballot gives the pairs
// of an expert as a bit mask.  An expert has at most one pair per token.
#define MF_MOE_SPARSE_PAIRS 128
#define MF_MOE_SPARSE_TOKENS 16

__device__ __forceinline__ void load8(const bf16* __restrict__ p, bool vec, int left, float (&dst)[8]) {
  if (vec && left >= 8) {
    alignas(16) bf16 raw[8];
    *(uint4*)raw = *(const uint4*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = (float)raw[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = i < left ? (float)p[i] : 0.f;
  }
}
__device__ __forceinline__ void load8(const float* __restrict__ p, bool vec, int left, float (&dst)[8]) {
  if (vec && left >= 8) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    dst[0] = a.x; dst[1] = a.y; dst[2] = a.z; dst[3] = a.w; dst[4] = b.x; dst[5] = b.y; dst[6] = b.z; dst[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = i < left ? p[i] : 0.f;
  }
}

// the lowest pair of the masks, taken off them
__device__ __forceinline__ int next_pair(unsigned long long& m0, unsigned long long& m1) {
  if (m0) { const int i = __builtin_ctzll(m0); m0 &= m0 - 1; return i; }
  const int i = __builtin_ctzll(m1); m1 &= m1 - 1; return 64 + i;
}

// gate_up [E][2 F][K], x [tokens][K] -> y [tokens][top][F] (activation applied, not weighted).
// A wave owns (expert, f): lanes over K in runs of 8; the gate row and the up row f are read once and
// meet the x rows of the expert's tokens.
template <typename WT>
__global__ __launch_bounds__(256) void moe_sparse_up_kernel(const WT* __restrict__ x, const WT* __restrict__ gate_up,
                                                            const int* __restrict__ chosen, WT* __restrict__ y,
                                                            int n_pairs, int top, int F, int K, float limit, int act) {
  const int e = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int f = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int c0 = lane < n_pairs ? chosen[lane] : -1, c1 = lane + 64 < n_pairs ? chosen[lane + 64] : -1;
  const unsigned long long mine0 = __ballot(c0 == e), mine1 = __ballot(c1 == e);
  if (!(mine0 | mine1) || f >= F) return;
  const WT* wg = gate_up + ((size_t)e * 2 * F + f) * K;
  const WT* wu = wg + (size_t)F * K;
  const bool vec = (K * sizeof(WT)) % 16 == 0;
  float ag[MF_MOE_SPARSE_TOKENS], au[MF_MOE_SPARSE_TOKENS];
#pragma unroll
  for (int j = 0; j < MF_MOE_SPARSE_TOKENS; ++j) ag[j] = au[j] = 0.f;
  for (int k = lane * 8; k < K; k += 512) {
    float g[8], u[8];
    load8(wg + k, vec, K - k, g);
    load8(wu + k, vec, K - k, u);
    unsigned long long m0 = mine0, m1 = mine1;
#pragma unroll
    for (int j = 0; j < MF_MOE_SPARSE_TOKENS; ++j) {
      if (m0 | m1) {
        const int pr = next_pair(m0, m1);
        float xv[8];
        load8(x + (size_t)(pr / top) * K + k, vec, K - k, xv);
#pragma unroll
        for (int i = 0; i < 8; ++i) { ag[j] = fmaf(g[i], xv[i], ag[j]); au[j] = fmaf(u[i], xv[i], au[j]); }
      }
    }
  }
  unsigned long long m0 = mine0, m1 = mine1;
#pragma unroll
  for (int j = 0; j < MF_MOE_SPARSE_TOKENS; ++j) {
    if (m0 | m1) {
      const int pr = next_pair(m0, m1);
      const float g = wave_sum(ag[j]), u = wave_sum(au[j]);
      if (lane == 0) y[(size_t)pr * F + f] = from_f32<WT>(expert_act(g, u, limit, act));
    }
  }
}

// down [E][N][F], y [tokens][top][F] -> rows[pair][N]: the pairs' outputs, not yet weighted.  A wave owns
// (expert, n): the expert's row n is read once and meets the y rows of the expert's pairs.  The tokens' sums
// are formed behind it (`moe_combine_kernel`, a token's choices in their order).
template <typename WT>
__global__ __launch_bounds__(256) void moe_sparse_down_kernel(const WT* __restrict__ y, const WT* __restrict__ down,
                                                              const int* __restrict__ chosen, float* __restrict__ rows,
                                                              int n_pairs, int F, int N) {
  const int e = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int c0 = lane < n_pairs ? chosen[lane] : -1, c1 = lane + 64 < n_pairs ? chosen[lane + 64] : -1;
  const unsigned long long mine0 = __ballot(c0 == e), mine1 = __ballot(c1 == e);
  if (!(mine0 | mine1) || n >= N) return;
  const WT* wr = down + ((size_t)e * N + n) * F;
  const bool vec = (F * sizeof(WT)) % 16 == 0;
  float acc[MF_MOE_SPARSE_TOKENS];
#pragma unroll
  for (int j = 0; j < MF_MOE_SPARSE_TOKENS; ++j) acc[j] = 0.f;
  for (int k = lane * 8; k < F; k += 512) {
    float wv[8];
    load8(wr + k, vec, F - k, wv);
    unsigned long long m0 = mine0, m1 = mine1;
#pragma unroll
    for (int j = 0; j < MF_MOE_SPARSE_TOKENS; ++j) {
      if (m0 | m1) {
        const int pr = next_pair(m0, m1);
        float yv[8];
        load8(y + (size_t)pr * F + k, vec, F - k, yv);
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[j] = fmaf(wv[q], yv[q], acc[j]);
      }
    }
  }
  unsigned long long m0 = mine0, m1 = mine1;
#pragma unroll
  for (int j = 0; j < MF_MOE_SPARSE_TOKENS; ++j) {
    if (m0 | m1) {
      const int pr = next_pair(m0, m1);
      const float v = wave_sum(acc[j]);
      if (lane == 0) rows[(size_t)pr * N + n] = v;
    }
  }
}

// ------------------------------------------------------------------ many tokens: the tokens of an expert together
// `moe_group_kernel`: a workgroup per expert walks the step's (token, choice) pairs in order and gives
// every pair of its expert its rank among them; counts[e] is their number.  With the experts' offsets
// (the running sum of the counts, formed by the host) pair p stands in row offsets[chosen[p]] + rank[p] of the
// buffers that hold the experts' tokens one expert after the other.
__global__ __launch_bounds__(256) void moe_group_kernel(const int* __restrict__ chosen, int n_pairs, int* __restrict__ rank,
                                                        int* __restrict__ counts) {
  __shared__ int wave_count[4];
  const int e = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int before = 0;
  for (int p0 = 0; p0 < n_pairs; p0 += 256) {
    const int p = p0 + threadIdx.x;
    const bool mine = p < n_pairs && chosen[p] == e;
    const unsigned long long m = __ballot(mine);
    __syncthreads();
    if (lane == 0) wave_count[w] = __popcll(m);
    __syncthreads();
    int ahead = before;
    for (int i = 0; i < w; ++i) ahead += wave_count[i];
    if (mine) rank[p] = ahead + __popcll(m & ((1ull << lane) - 1));
    before += wave_count[0] + wave_count[1] + wave_count[2] + wave_count[3];
  }
  if (threadIdx.x == 0) counts[e] = before;
}

// xs[row(p)][:] = x[p / top][:]
template <typename T>
__global__ __launch_bounds__(256) void moe_gather_kernel(const T* __restrict__ x, const int* __restrict__ chosen,
                                                         const int* __restrict__ rank, const int* __restrict__ offsets,
                                                         T* __restrict__ xs, int top, int K) {
  const int p = blockIdx.x;
  const T* src = x + (size_t)(p / top) * K;
  T* dst = xs + (size_t)(offsets[chosen[p]] + rank[p]) * K;
  for (int i = threadIdx.x; i < K; i += 256) dst[i] = src[i];
}

// out[t][:] (+)= sum_k w[t][k] rows[row(t top + k)][:], the choices in their order
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ rows, const int* __restrict__ chosen,
                                                          const int* __restrict__ rank, const int* __restrict__ offsets,
                                                          const float* __restrict__ weights, float* __restrict__ out,
                                                          int top, int N, int add) {
  const int t = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= N) return;
  float a = add ? out[(size_t)t * N + i] : 0.f;
  for (int k = 0; k < top; ++k) {
    const int p = t * top + k;
    const int row = offsets ? offsets[chosen[p]] + rank[p] : p;      // without offsets: pair p's row is row p
    a = fmaf(weights[p], rows[(size_t)row * N + i], a);
  }
  out[(size_t)t * N + i] = a;
}

// ------------------------------------------------------------------ entry points
MF_API int mf_moe_route(const void* x, int x_is_bf16, const float* router, const float* bias, int K, float* dense, int* chosen,
                        float* weights, int n_tok, int E, int n_groups, int keep, int top, int score_kind,
                        const float* correction, int group_top, float weight_scale, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (K <= 0 || E <= 0 || E > MF_MOE_MAX_EXPERTS || n_groups <= 0 || E % n_groups || keep <= 0 || keep > n_groups || top <= 0 ||
      top > 64 || top > keep * (E / n_groups) || group_top < 1 ||
      (score_kind != MF_MOE_SCORE_SOFTMAX && score_kind != MF_MOE_SCORE_SIGMOID))
    return (int)hipErrorInvalidValue;
  if (x_is_bf16)
    moe_route_kernel<bf16><<<n_tok, 256, 0, stream>>>((const bf16*)x, router, bias, K, dense, chosen, weights, E, n_groups, keep, top,
                                                      score_kind, correction, group_top, weight_scale);
  else
    moe_route_kernel<float><<<n_tok, 256, 0, stream>>>((const float*)x, router, bias, K, dense, chosen, weights, E, n_groups, keep, top,
                                                      score_kind, correction, group_top, weight_scale);
  return mf_launch_status();
}

MF_API int mf_moe_act(const float* gu, const float* dense, void* y, int y_is_bf16, int n_tok, int E, int F, float limit,
                      int act, hipStream_t stream) {
  if (n_tok <= 0 || E <= 0 || F <= 0) return 0;
  if (act != MF_MOE_ACT_CLAMPED && act != MF_MOE_ACT_SILU) return (int)hipErrorInvalidValue;
  int by = (E * F + 255) / 256;
  if (by > 64) by = 64;
  dim3 grid(n_tok, by);
  if (y_is_bf16)
    moe_act_kernel<bf16><<<grid, 256, 0, stream>>>(gu, dense, (bf16*)y, E, F, limit, act);
  else
    moe_act_kernel<float><<<grid, 256, 0, stream>>>(gu, dense, (float*)y, E, F, limit, act);
  return mf_launch_status();
}

MF_API int mf_moe_sparse(const void* x, const void* gate_up, const void* down, const int* chosen, const float* weights,
                         void* y, float* rows, float* out, int is_bf16, int n_tok, int top, int E, int F, int K, int N,
                         float limit, int act, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (act != MF_MOE_ACT_CLAMPED && act != MF_MOE_ACT_SILU) return (int)hipErrorInvalidValue;
  if (top <= 0 || E <= 0 || F <= 0 || K <= 0 || N <= 0 || n_tok > MF_MOE_SPARSE_TOKENS || n_tok * top > MF_MOE_SPARSE_PAIRS ||
      !y || !rows)
    return (int)hipErrorInvalidValue;
  dim3 g1(E, (F + 3) / 4), g2(E, (N + 3) / 4);
  const int pairs = n_tok * top;
  if (is_bf16) {
    moe_sparse_up_kernel<bf16><<<g1, 256, 0, stream>>>((const bf16*)x, (const bf16*)gate_up, chosen, (bf16*)y, pairs, top, F, K, limit, act);
    int rc = mf_launch_status();
    if (rc) return rc;
    moe_sparse_down_kernel<bf16><<<g2, 256, 0, stream>>>((const bf16*)y, (const bf16*)down, chosen, rows, pairs, F, N);
  } else {
    moe_sparse_up_kernel<float><<<g1, 256, 0, stream>>>((const float*)x, (const float*)gate_up, chosen, (float*)y, pairs, top, F, K, limit, act);
    int rc = mf_launch_status();
    if (rc) return rc;
    moe_sparse_down_kernel<float><<<g2, 256, 0, stream>>>((const float*)y, (const float*)down, chosen, rows, pairs, F, N);
  }
  int rc = mf_launch_status();
  if (rc) return rc;
  moe_combine_kernel<<<dim3(n_tok, (N + 255) / 256), 256, 0, stream>>>(rows, chosen, nullptr, nullptr, weights, out, top, N, 1);
  return mf_launch_status();
}

MF_API int mf_moe_group(const int* chosen, int n_pairs, int E, int* rank, int* counts, hipStream_t stream) {
  if (n_pairs <= 0 || E <= 0) return 0;
  moe_group_kernel<<<E, 256, 0, stream>>>(chosen, n_pairs, rank, counts);
  return mf_launch_status();
}

MF_API int mf_moe_gather(const void* x, int is_bf16, const int* chosen, const int* rank, const int* offsets, void* xs,
                         int n_pairs, int top, int K, hipStream_t stream) {
  if (n_pairs <= 0) return 0;
  if (is_bf16)
    moe_gather_kernel<bf16><<<n_pairs, 256, 0, stream>>>((const bf16*)x, chosen, rank, offsets, (bf16*)xs, top, K);
  else
    moe_gather_kernel<float><<<n_pairs, 256, 0, stream>>>((const float*)x, chosen, rank, offsets, (float*)xs, top, K);
  return mf_launch_status();
}

MF_API int mf_moe_combine(const float* rows, const int* chosen, const int* rank, const int* offsets, const float* weights,
                          float* out, int n_tok, int top, int N, int add, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  moe_combine_kernel<<<dim3(n_tok, (N + 255) / 256), 256, 0, stream>>>(rows, chosen, rank, offsets, weights, out, top, N, add);
  return mf_launch_status();
}
