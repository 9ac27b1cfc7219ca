// Attention over a shared low-rank latent ("latent attention"), in the form that never builds
// per-head keys and values.
//
// A token leaves one row in the cache: [c (R values) | k_rot (DR values)], c the normed latent and
// k_rot one rotated key part that all heads share.  With per-head matrices Wuk_h [DN][R] and
// Wuv_h [DV][R] the keys and values of head h would be Wuk_h c_j and Wuv_h c_j.  Since
//   q_plain . (Wuk_h c_j) = (Wuk_h^T q_plain) . c_j      and
//   sum_j p_j (Wuv_h c_j) = Wuv_h (sum_j p_j c_j),
// every head becomes a query of width DK = R + DR against the cached rows themselves, and the
// values are the first R columns of the same rows: one "kv head" that all H heads share.
//   s_j = ([Wuk_h^T q_plain | q_rot] . row_j) * scale,  p = softmax over j <= position,
//   o_lat = sum_j p_j row_j[0:R],  out_h = gate_h * (Wuv_h o_lat).
// Scores, softmax statistics and accumulators are 32-bit.
//
// Kernels here: `latent_prep_kernel` (norm of the latent, rotation in pairs (2i, 2i+1) of the
// first `rd` values of the rotated parts, cache write, sigmoid of the head gates),
// `headwise_linear_kernel` (a small matrix per head applied to every token's slice of that head:
// the two absorptions above), `latent_attn_kernel` (any sizes, both precisions, keys split over
// blocks) with `latent_combine_kernel`.
#include "common.h"

// ------------------------------------------------------------------ preparation
// proj: 32-bit rows [dkv: R + DR | gate: H gate_w] at the given offsets of a row of `ld` floats; the queries
// [H (DN + DR)] are rows of `ldq` floats of `q_rows` (the same buffer where one product made them all, or the
// result of a product of their own where the queries pass a latent first).  gate_w: 1 where a head has one gate,
// the width of a head's values where every value has its own.  Two blocks per token: one for the cached row,
// one for the queries and gates.  WIDE: the queries are rows of their own or a head has more than one gate; without
// it the kernel is the one-product, one-gate-a-head form, instruction for instruction.
template <typename OT, bool WIDE>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    const float* __restrict__ proj, int ld, int off_dkv, int off_gate, int gate_w, const float* __restrict__ q_rows,
    int ldq, const float* __restrict__ cw, float eps,
    const float* __restrict__ cs, const float* __restrict__ sn, int rd, const int* __restrict__ positions,
    const int* __restrict__ seq_of_tok, const int* __restrict__ page_table, int pt_stride, OT* __restrict__ cache,
    OT* __restrict__ q_plain, OT* __restrict__ q_abs, float* __restrict__ gate, int H, int DN, int DR, int R,
    int write_cache) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const float* row = proj + (size_t)t * ld;
  const int DK = R + DR, half = rd >> 1;
  const float* c_t = cs + (size_t)pos * half;
  const float* s_t = sn + (size_t)pos * half;
  if (blockIdx.y == 0) {
    if (!write_cache) return;
    // the latent: x / sqrt(mean(x^2) + eps) * w
    const float* dkv = row + off_dkv;
    float ss = 0.f;
    for (int i = threadIdx.x; i < R; i += 256) ss = fmaf(dkv[i], dkv[i], ss);
    ss = block_sum<256>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)R + eps);
    const int page = page_table[(size_t)seq_of_tok[t] * pt_stride + pos / MF_PAGE];
    OT* dst = cache + ((size_t)page * MF_PAGE + pos % MF_PAGE) * DK;
    for (int i = threadIdx.x; i < R; i += 256) dst[i] = from_f32<OT>(dkv[i] * inv * cw[i]);
    const float* kr = dkv + R;
    for (int i = threadIdx.x; i < DR; i += 256) {
      float v;
      if (i < rd) {
        const int pr = i >> 1;
        const float a = kr[i & ~1], b = kr[i | 1];
        v = (i & 1) ? b * c_t[pr] + a * s_t[pr] : a * c_t[pr] - b * s_t[pr];
      } else {
        v = kr[i];
      }
      dst[R + i] = from_f32<OT>(v);
    }
    return;
  }
  // queries: plain part as it is, rotated part behind the R columns the absorption will fill
  const int DQ = DN + DR;
  for (int i = threadIdx.x; i < H * DQ; i += 256) {
    const int h = i / DQ, e = i % DQ;
    const float* qh = WIDE ? q_rows + (size_t)t * ldq + (size_t)h * DQ : row + (size_t)h * DQ;
    if (e < DN) {
      q_plain[((size_t)t * H + h) * DN + e] = from_f32<OT>(qh[e]);
    } else {
      const int j = e - DN;
      float v;
      if (j < rd) {
        const int pr = j >> 1;
        const float a = qh[DN + (j & ~1)], b = qh[DN + (j | 1)];
        v = (j & 1) ? b * c_t[pr] + a * s_t[pr] : a * c_t[pr] - b * s_t[pr];
      } else {
        v = qh[e];
      }
      q_abs[((size_t)t * H + h) * DK + R + j] = from_f32<OT>(v);
    }
  }
  if (WIDE) {
    if (gate)
      for (int i = threadIdx.x; i < H * gate_w; i += 256)
        gate[(size_t)t * H * gate_w + i] = 1.0f / (1.0f + expf(-row[off_gate + i]));
  } else {
    for (int h = threadIdx.x; h < H; h += 256) gate[(size_t)t * H + h] = 1.0f / (1.0f + expf(-row[off_gate + h]));
  }
}

MF_API int mf_latent_prep(const float* proj, int ld, int off_dkv, int off_gate, int gate_w, const float* q_rows,
                          int ldq, const float* cw, float eps,
                          const float* cs, const float* sn, int rd, const int* positions, const int* seq_of_tok,
                          const int* page_table, int pt_stride, void* cache, void* q_plain, void* q_abs,
                          float* gate, int is_bf16, int n_tok, int H, int DN, int DR, int R, int write_cache,
                          hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (rd < 0 || rd > DR || (rd & 1) || H < 1 || DN < 1 || R < 1 || gate_w < 1 || !q_rows) return (int)hipErrorInvalidValue;
  const bool wide = gate_w != 1 || q_rows != proj || ldq != ld || !gate;
#define MF_PREP(OT, WIDE)                                                                                              \
  latent_prep_kernel<OT, WIDE><<<dim3(n_tok, 2), 256, 0, stream>>>(proj, ld, off_dkv, off_gate, gate_w, q_rows, ldq, cw, eps, \
                                                                   cs, sn, rd, positions, seq_of_tok, page_table,      \
                                                                   pt_stride, (OT*)cache, (OT*)q_plain, (OT*)q_abs,   \
                                                                   gate, H, DN, DR, R, write_cache)
  if (is_bf16) {
    if (wide) MF_PREP(bf16, true);
    else MF_PREP(bf16, false);
  } else {
    if (wide) MF_PREP(float, true);
    else MF_PREP(float, false);
  }
#undef MF_PREP
  return mf_launch_status();
}

// ------------------------------------------------------------------ a matrix per head
// out[t][h][0:NO] = (gate[t][h] *) sum_i wt[h][i][0:NO] in[t][h][i]; wt is the head's matrix
// stored input-major ([NI][NO]) so that neighbouring threads read neighbouring outputs.  Rows of
// `in` and `out` are H slices of `in_stride` / `out_stride` values.  A block takes TT tokens of one
// head; sums in 32-bit in the order of i.
#define MF_HW_TT 8
template <typename T, bool GV>          // GV: a gate for every value of a head (gate_w = NO) instead of one a head
__global__ __launch_bounds__(256) void headwise_linear_kernel(const T* __restrict__ in, int in_stride,
                                                              const T* __restrict__ wt, T* __restrict__ out,
                                                              int out_stride, const float* __restrict__ gate,
                                                              int gate_w, int n_tok, int H, int NI, int NO) {
  extern __shared__ float xs[];          // [TT][NI]
  const int h = blockIdx.y;
  const int t0 = blockIdx.x * MF_HW_TT;
  const int nt = min(MF_HW_TT, n_tok - t0);
  for (int i = threadIdx.x; i < MF_HW_TT * NI; i += 256) {
    const int tt = i / NI, e = i % NI;
    xs[i] = tt < nt ? to_f32(in[((size_t)(t0 + tt) * H + h) * in_stride + e]) : 0.f;
  }
  __syncthreads();
  const T* w = wt + (size_t)h * NI * NO;
  for (int o = blockIdx.z * 256 + threadIdx.x; o < NO; o += 256 * gridDim.z) {
    float acc[MF_HW_TT];
#pragma unroll
    for (int tt = 0; tt < MF_HW_TT; ++tt) acc[tt] = 0.f;
    for (int i = 0; i < NI; ++i) {
      const float wv = to_f32(w[(size_t)i * NO + o]);
#pragma unroll
      for (int tt = 0; tt < MF_HW_TT; ++tt) acc[tt] = fmaf(wv, xs[tt * NI + i], acc[tt]);
    }
#pragma unroll
    for (int tt = 0; tt < MF_HW_TT; ++tt)
      if (tt < nt) {
        const float g = gate ? (GV ? gate[((size_t)(t0 + tt) * H + h) * gate_w + o] : gate[(size_t)(t0 + tt) * H + h]) : 1.0f;
        out[((size_t)(t0 + tt) * H + h) * out_stride + o] = from_f32<T>(acc[tt] * g);
      }
  }
}

MF_API int mf_headwise_linear(const void* in, int in_stride, const void* wt, void* out, int out_stride,
                              const float* gate, int gate_w, int is_bf16, int n_tok, int H, int NI, int NO,
                              hipStream_t stream) {
  if (n_tok <= 0) return 0;
  const size_t lds = (size_t)MF_HW_TT * NI * sizeof(float);
  if (H < 1 || NI < 1 || NO < 1 || lds > 64 * 1024 || (gate && gate_w != 1 && gate_w != NO)) return (int)hipErrorInvalidValue;
  dim3 grid((n_tok + MF_HW_TT - 1) / MF_HW_TT, H, (NO + 255) / 256);
  const bool gv = gate && gate_w > 1;
#define MF_HW(T, GV)                                                                                                  \
  headwise_linear_kernel<T, GV><<<grid, 256, lds, stream>>>((const T*)in, in_stride, (const T*)wt, (T*)out, out_stride, gate, \
                                                            gate_w, n_tok, H, NI, NO)
  if (is_bf16) {
    if (gv) MF_HW(bf16, true);
    else MF_HW(bf16, false);
  } else {
    if (gv) MF_HW(float, true);
    else MF_HW(float, false);
  }
#undef MF_HW
  return mf_launch_status();
}

// The same on the matrix cores (bfloat16, NI a multiple of 8): `wo` holds each head's matrix
// output-major ([NO][NI]).  A wave takes 16 tokens x 16 MT outputs of one head (MT = 4; 1 where a
// step has at most 16 tokens, so that there are waves enough to have the matrices' bytes in flight) and forms
// D^T = W X^T with 16x16x32 MFMA, operands straight from memory (a lane's 8 consecutive inputs are
// 16 bytes of a row in both), so that a lane ends up with four neighbouring outputs of one token.
// Tasks are numbered head, output tile, token tile (fastest): the four waves of a block share a
// head's rows of W where the step has tokens enough, and spread over the outputs where not.
typedef unsigned int hw_u32x4 __attribute__((ext_vector_type(4)));

template <int MT, bool GV>
__global__ __launch_bounds__(256) void headwise_mfma_kernel(const bf16* __restrict__ in, int in_stride,
                                                            const bf16* __restrict__ wo, bf16* __restrict__ out,
                                                            int out_stride, const float* __restrict__ gate, int gate_w,
                                                            int n_tok, int H, int NI, int NO, int n_ttiles, int n_otiles) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int task = blockIdx.x * 4 + wv;
  if (task >= H * n_otiles * n_ttiles) return;
  const int tt = task % n_ttiles, ot = (task / n_ttiles) % n_otiles, h = task / (n_ttiles * n_otiles);
  const int r16 = lane & 15, q4 = lane >> 4;
  const int t = tt * 16 + r16;
  const bool tok_ok = t < n_tok;
  const bf16* xrow = in + ((size_t)(tok_ok ? t : 0) * H + h) * in_stride;
  const bf16* wrow[MT];
  bool o_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int o = ot * (16 * MT) + mt * 16 + r16;
    o_ok[mt] = o < NO;
    wrow[mt] = wo + ((size_t)h * NO + (o_ok[mt] ? o : 0)) * NI;
  }
  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k0 = 0; k0 < NI; k0 += 32) {
    const int i = k0 + 8 * q4;
    const bool i_ok = i < NI;
    hw_u32x4 xb = {0u, 0u, 0u, 0u};
    if (tok_ok && i_ok) xb = *reinterpret_cast<const hw_u32x4*>(xrow + i);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      hw_u32x4 wa = {0u, 0u, 0u, 0u};
      if (o_ok[mt] && i_ok) wa = *reinterpret_cast<const hw_u32x4*>(wrow[mt] + i);
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wa), __builtin_bit_cast(bf16x8, xb),
                                                        acc[mt], 0, 0, 0);
    }
  }
  if (!tok_ok) return;
  const float* grow = (GV && gate) ? gate + ((size_t)t * H + h) * gate_w : nullptr;
  const float g = (!GV && gate) ? gate[(size_t)t * H + h] : 1.0f;
  bf16* orow = out + ((size_t)t * H + h) * out_stride;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int o0 = ot * (16 * MT) + mt * 16 + 4 * q4;
    if (o0 + 3 < NO && (out_stride & 3) == 0) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (bf16)(acc[mt][i] * (GV ? grow[o0 + i] : g));
      *reinterpret_cast<bf16x4*>(orow + o0) = v;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (o0 + i < NO) orow[o0 + i] = (bf16)(acc[mt][i] * (GV ? grow[o0 + i] : g));
    }
  }
}

// Prompts: a head's whole matrix (NO x NI, at most 150 KB with its padding) is staged in LDS once by
// a workgroup of 8 waves, which then takes 128 tokens: a wave holds its 16 tokens' inputs in
// registers (NI <= 512) and walks the outputs 16 at a time with the matrix's fragments from LDS
// (rows 16 bytes apart in the banks).  The matrix is read from memory once per 128 tokens
// instead of once per 16.
#define MF_HW_KS_MAX 16
template <bool GV>
__global__ __launch_bounds__(512) void headwise_lds_kernel(const bf16* __restrict__ in, int in_stride,
                                                           const bf16* __restrict__ wo, bf16* __restrict__ out,
                                                           int out_stride, const float* __restrict__ gate, int gate_w,
                                                           int n_tok, int H, int NI, int NO) {
  extern __shared__ __attribute__((aligned(16))) unsigned char hw_smem[];
  bf16* Ws = reinterpret_cast<bf16*>(hw_smem);
  const int WSTR = NI + 8;
  const int h = blockIdx.y;
  const int chunks = NI / 8;
  const int NO16 = (NO + 15) / 16 * 16;
  for (int idx = threadIdx.x; idx < NO16 * chunks; idx += 512) {
    const int o = idx / chunks, c = idx % chunks;
    hw_u32x4 v = {0u, 0u, 0u, 0u};
    if (o < NO) v = *reinterpret_cast<const hw_u32x4*>(wo + ((size_t)h * NO + o) * NI + c * 8);
    *reinterpret_cast<hw_u32x4*>(Ws + (size_t)o * WSTR + c * 8) = v;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int t = blockIdx.x * 128 + wv * 16 + r16;
  const bool tok_ok = t < n_tok;
  const bf16* xrow = in + ((size_t)(tok_ok ? t : 0) * H + h) * in_stride;
  const int nks = (NI + 31) / 32;
  hw_u32x4 xb[MF_HW_KS_MAX];
#pragma unroll
  for (int ks = 0; ks < MF_HW_KS_MAX; ++ks) {
    const int i = 32 * ks + 8 * q4;
    xb[ks] = hw_u32x4{0u, 0u, 0u, 0u};
    if (ks < nks && tok_ok && i < NI) xb[ks] = *reinterpret_cast<const hw_u32x4*>(xrow + i);
  }
  if (blockIdx.x * 128 + wv * 16 >= n_tok) return;      // (after the barrier; uniform over the wave)
  const float* grow = (GV && gate && tok_ok) ? gate + ((size_t)t * H + h) * gate_w : nullptr;
  const float g = (!GV && gate && tok_ok) ? gate[(size_t)t * H + h] : 1.0f;
  bf16* orow = out + ((size_t)(tok_ok ? t : 0) * H + h) * out_stride;
  for (int mt = 0; mt < NO16 / 16; ++mt) {
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    const bf16* wrow = Ws + (size_t)(mt * 16 + r16) * WSTR + 8 * q4;
#pragma unroll
    for (int ks = 0; ks < MF_HW_KS_MAX; ++ks) {
      if (ks < nks) {
        hw_u32x4 wa = {0u, 0u, 0u, 0u};
        if (32 * ks + 8 * q4 < NI) wa = *reinterpret_cast<const hw_u32x4*>(wrow + 32 * ks);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wa), __builtin_bit_cast(bf16x8, xb[ks]),
                                                      acc, 0, 0, 0);
      }
    }
    if (!tok_ok) continue;
    const int o0 = mt * 16 + 4 * q4;
    if (o0 + 3 < NO && (out_stride & 3) == 0) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (bf16)(acc[i] * (GV ? grow[o0 + i] : g));
      *reinterpret_cast<bf16x4*>(orow + o0) = v;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (o0 + i < NO) orow[o0 + i] = (bf16)(acc[i] * (GV ? grow[o0 + i] : g));
    }
  }
}

MF_API int mf_headwise_mfma(const void* in, int in_stride, const void* wo, void* out, int out_stride,
                            const float* gate, int gate_w, int n_tok, int H, int NI, int NO, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (H < 1 || NI < 1 || NO < 1 || NI % 8 || in_stride % 8 || (uintptr_t)in % 16 || (uintptr_t)wo % 16 ||
      (uintptr_t)out % 8 || (gate && gate_w != 1 && gate_w != NO))
    return (int)hipErrorInvalidValue;
  const int n_ttiles = (n_tok + 15) / 16;
  const size_t lds = (size_t)((NO + 15) / 16 * 16) * (NI + 8) * 2;
  const bool gv = gate && gate_w > 1;
  if (n_tok >= 256 && NI <= 32 * MF_HW_KS_MAX && lds <= 150 * 1024) {
    static bool raised = false;
    if (!raised) {
      for (const void* fn : {reinterpret_cast<const void*>(headwise_lds_kernel<false>),
                             reinterpret_cast<const void*>(headwise_lds_kernel<true>)}) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
        if (e != hipSuccess) return (int)e;
      }
      raised = true;
    }
    const dim3 grid((n_tok + 127) / 128, H);
    if (gv)
      headwise_lds_kernel<true><<<grid, 512, lds, stream>>>((const bf16*)in, in_stride, (const bf16*)wo, (bf16*)out, out_stride,
                                                           gate, gate_w, n_tok, H, NI, NO);
    else
      headwise_lds_kernel<false><<<grid, 512, lds, stream>>>((const bf16*)in, in_stride, (const bf16*)wo, (bf16*)out, out_stride,
                                                            gate, gate_w, n_tok, H, NI, NO);
    return mf_launch_status();
  }
#define MF_HWM(MT, GV)                                                                                                     \
  headwise_mfma_kernel<MT, GV><<<(unsigned)((tasks + 3) / 4), 256, 0, stream>>>(                                           \
      (const bf16*)in, in_stride, (const bf16*)wo, (bf16*)out, out_stride, gate, gate_w, n_tok, H, NI, NO, n_ttiles, n_otiles)
  if (n_tok <= 16) {
    const int n_otiles = (NO + 15) / 16;
    const long long tasks = (long long)H * n_otiles * n_ttiles;
    if (gv) MF_HWM(1, true);
    else MF_HWM(1, false);
  } else {
    const int n_otiles = (NO + 63) / 64;
    const long long tasks = (long long)H * n_otiles * n_ttiles;
    if (gv) MF_HWM(4, true);
    else MF_HWM(4, false);
  }
#undef MF_HWM
  return mf_launch_status();
}

// ------------------------------------------------------------------ attention, any sizes
// A block owns (token, chunk of up to GC heads, key split) and walks the keys lo..hi of its split
// in steps of 256: thread j takes key j of the step and forms its scores for the chunk's heads
// (the row is read once for all of them); the step's maxima and sums are taken over the block;
// then thread e takes value column e (and e + 256, ...) and adds the step's weighted rows.  The
// running maximum, sum and accumulator are rescaled per step (online softmax).  A token's result
// depends on its own keys and on the split length only.
#define MF_LAT_GC 4
#define MF_LAT_EPT 4      // value columns per thread: R <= 256 * MF_LAT_EPT

template <typename T> __device__ __forceinline__ float lat_exp(float x);
template <> __device__ __forceinline__ float lat_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ float lat_exp<bf16>(float x) { return __expf(x); }

template <typename T>
__global__ __launch_bounds__(256) void latent_attn_kernel(
    const T* __restrict__ q_abs, const T* __restrict__ cache, const int* __restrict__ page_table, int pt_stride,
    const int* __restrict__ positions, const int* __restrict__ seq_of_tok, T* __restrict__ out,
    float* __restrict__ part, int H, int R, int DK, float scale, int window, int n_splits, int split_len) {
  extern __shared__ float sm[];
  float* qs = sm;                        // [GC][DK]
  float* ps = qs + MF_LAT_GC * DK;       // [GC][256]
  float* red = ps + MF_LAT_GC * 256;     // [4]
  const int t = blockIdx.x;
  const int h0 = blockIdx.y * MF_LAT_GC;
  const int gcount = min(MF_LAT_GC, H - h0);
  const int split = blockIdx.z;
  const int p = positions[t];
  const int* pt = page_table + (size_t)seq_of_tok[t] * pt_stride;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int j_begin = max(lo, split * split_len);
  const int j_end = min(p + 1, (split + 1) * split_len);

  for (int i = threadIdx.x; i < MF_LAT_GC * DK; i += 256) {
    const int g = i / DK, e = i % DK;
    qs[i] = g < gcount ? to_f32(q_abs[((size_t)t * H + h0 + g) * DK + e]) : 0.f;
  }
  float m[MF_LAT_GC], l[MF_LAT_GC], acc[MF_LAT_GC][MF_LAT_EPT];
#pragma unroll
  for (int g = 0; g < MF_LAT_GC; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int c = 0; c < MF_LAT_EPT; ++c) acc[g][c] = 0.f;
  }
  __syncthreads();

  for (int j0 = j_begin; j0 < j_end; j0 += 256) {
    const int j = j0 + threadIdx.x;
    const bool valid = j < j_end;
    float s[MF_LAT_GC];
#pragma unroll
    for (int g = 0; g < MF_LAT_GC; ++g) s[g] = 0.f;
    if (valid) {
      const T* kr = cache + ((size_t)pt[j / MF_PAGE] * MF_PAGE + j % MF_PAGE) * DK;
      for (int e = 0; e < DK; ++e) {
        const float kv = to_f32(kr[e]);
#pragma unroll
        for (int g = 0; g < MF_LAT_GC; ++g) s[g] = fmaf(qs[g * DK + e], kv, s[g]);
      }
    }
    float corr[MF_LAT_GC];
#pragma unroll
    for (int g = 0; g < MF_LAT_GC; ++g) {
      const float sv = valid ? s[g] * scale : -INFINITY;
      const float m_new = fmaxf(m[g], block_max<256>(sv, red));
      const float pe = valid ? lat_exp<T>(sv - m_new) : 0.f;
      corr[g] = (m[g] == -INFINITY) ? 0.f : lat_exp<T>(m[g] - m_new);
      l[g] = l[g] * corr[g] + block_sum<256>(pe, red);
      m[g] = m_new;
      ps[g * 256 + threadIdx.x] = pe;
    }
    __syncthreads();
    const int n_here = min(256, j_end - j0);
#pragma unroll
    for (int g = 0; g < MF_LAT_GC; ++g)
#pragma unroll
      for (int c = 0; c < MF_LAT_EPT; ++c) acc[g][c] *= corr[g];
    for (int jj = 0; jj < n_here; ++jj) {
      const int jk = j0 + jj;
      const T* kr = cache + ((size_t)pt[jk / MF_PAGE] * MF_PAGE + jk % MF_PAGE) * DK;
#pragma unroll
      for (int c = 0; c < MF_LAT_EPT; ++c) {
        const int e = c * 256 + threadIdx.x;
        if (e < R) {
          const float kv = to_f32(kr[e]);
#pragma unroll
          for (int g = 0; g < MF_LAT_GC; ++g) acc[g][c] = fmaf(ps[g * 256 + jj], kv, acc[g][c]);
        }
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int g = 0; g < MF_LAT_GC; ++g) {
    if (g >= gcount) break;
    const size_t th = (size_t)t * H + h0 + g;
    if (n_splits == 1) {
      const float inv = l[g] > 0.f ? 1.0f / l[g] : 0.f;
#pragma unroll
      for (int c = 0; c < MF_LAT_EPT; ++c) {
        const int e = c * 256 + threadIdx.x;
        if (e < R) out[th * R + e] = from_f32<T>(acc[g][c] * inv);
      }
    } else {
      float* o = part + (th * n_splits + split) * (size_t)(R + 2);
#pragma unroll
      for (int c = 0; c < MF_LAT_EPT; ++c) {
        const int e = c * 256 + threadIdx.x;
        if (e < R) o[e] = acc[g][c];
      }
      if (threadIdx.x == 0) { o[R] = m[g]; o[R + 1] = l[g]; }
    }
  }
}

// out[th][e] = sum_s acc_s[e] exp(m_s - M) / sum_s l_s exp(m_s - M), splits added in their order
template <typename T>
__global__ __launch_bounds__(256) void latent_combine_kernel(const float* __restrict__ part, T* __restrict__ out,
                                                             int R, int n_splits) {
  const size_t th = blockIdx.x;
  const float* base = part + th * n_splits * (size_t)(R + 2);
  float M = -INFINITY;
  for (int s = 0; s < n_splits; ++s) M = fmaxf(M, base[(size_t)s * (R + 2) + R]);
  float L = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float ms = base[(size_t)s * (R + 2) + R];
    if (ms != -INFINITY) L += base[(size_t)s * (R + 2) + R + 1] * lat_exp<T>(ms - M);
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  for (int e = threadIdx.x; e < R; e += 256) {
    float a = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float ms = base[(size_t)s * (R + 2) + R];
      if (ms != -INFINITY) a += base[(size_t)s * (R + 2) + e] * lat_exp<T>(ms - M);
    }
    out[th * R + e] = from_f32<T>(a * inv);
  }
}

MF_API int mf_latent_attn(const void* q_abs, const void* cache, const int* page_table, int pt_stride,
                          const int* positions, const int* seq_of_tok, void* out, float* part, int is_bf16,
                          int n_tok, int H, int R, int DK, float scale, int window, int n_splits, int split_len,
                          hipStream_t stream) {
  if (n_tok <= 0) return 0;
  const size_t lds = ((size_t)MF_LAT_GC * DK + MF_LAT_GC * 256 + 4) * sizeof(float);
  if (H < 1 || R < 1 || R > 256 * MF_LAT_EPT || DK < R || lds > 64 * 1024 || n_splits < 1 ||
      split_len < 1 || (n_splits > 1 && part == nullptr))
    return (int)hipErrorInvalidValue;
  dim3 grid(n_tok, (H + MF_LAT_GC - 1) / MF_LAT_GC, n_splits);
  if (is_bf16)
    latent_attn_kernel<bf16><<<grid, 256, lds, stream>>>((const bf16*)q_abs, (const bf16*)cache, page_table, pt_stride,
                                                          positions, seq_of_tok, (bf16*)out, part, H, R, DK, scale,
                                                          window, n_splits, split_len);
  else
    latent_attn_kernel<float><<<grid, 256, lds, stream>>>((const float*)q_abs, (const float*)cache, page_table,
                                                           pt_stride, positions, seq_of_tok, (float*)out, part, H, R,
                                                           DK, scale, window, n_splits, split_len);
  int rc = mf_launch_status();
  if (rc == 0 && n_splits > 1) {
    if (is_bf16)
      latent_combine_kernel<bf16><<<n_tok * H, 256, 0, stream>>>(part, (bf16*)out, R, n_splits);
    else
      latent_combine_kernel<float><<<n_tok * H, 256, 0, stream>>>(part, (float*)out, R, n_splits);
    rc = mf_launch_status();
  }
  return rc;
}
