// Windowed, capped attention for many query tokens per sequence (prompts and their portions), bfloat16, on
// the gfx950 matrix cores, for keys of MF_CAPM_D and values of MF_CAPM_V values (multiples of 16, given at
// compile time: the library is built for a model's sizes).  Semantics as `capped_attn_kernel`:
// s = cap tanh(q . k scale temp[h] / cap), keys j with 0 <= p - j < window, softmax, o = sum p_j v_j; with
// `chunk`, a token sees the keys of its own chunk of that many positions only; with `far_a`, `far_b`,
// s -= far_a[h] ln(1 + far_b[h] (p - j)); with `bias`, s += bias[h][min(p - j, n_bias - 1)]; with a window and
// `keep_first`, every token also sees the sequence's first `keep_first` keys: the wave of split 0 walks their
// half pages first and then jumps to the half page of its window's first key.
//
// A wave (a workgroup of its own) owns 16 consecutive new tokens of one sequence times RB query heads of one kv
// head and walks the tokens' keys 32 at a time (half a page), with no LDS and no barrier; the key rows of a
// step are asked for a step ahead, the value rows before the step's scores are formed:
//   S^T[key][token] = K Q^T      16x16x32 MFMA, A = 16 key rows straight from the cache, B = Q kept in registers
//   a lane holds, for its token (lane % 16), the scores of keys 4 (lane / 16) + i of both key tiles:
//   the softmax statistics are per lane, shared by the four lanes of a token through two shuffles
//   O^T[d][token] += V^T P^T     A = rows of V^T straight from the cache, which stores a page's values
//   transposed in halves of 32 keys; B = P^T, the scores' own register layout.  The k index of this product
//   is permuted the same way on both operands: slot 8 g + j stands for key 4 g + j (j < 4) and 16 + 4 g + j - 4.
// The RB heads share every K and V fragment.  Sums, maxima and outputs are 32-bit; probabilities are rounded
// to bfloat16 for the second product.  Keys not yet written (behind the sequence's end) may hold anything:
// their scores are masked and their value columns are zeroed before the product.
// Steps of few tokens (decode) split a tile's keys over several waves, which leave their sums, maxima and
// weights for `attn_combine_kernel` to merge in the order of the splits.
#include "attn_tokens_impl.h"

#ifndef MF_CAPM_D
#define MF_CAPM_D 128
#endif
#ifndef MF_CAPM_V
#define MF_CAPM_V 128
#endif

namespace {

constexpr int D = MF_CAPM_D, V = MF_CAPM_V;
constexpr int DKS = (D + 31) / 32;     // k steps of the first product
constexpr int NVT = V / 16;            // output tiles
static_assert(D % 16 == 0 && V % 16 == 0 && D <= 256 && V <= 256, "sizes the kernel takes");

typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));      // four floats from any float's address

// out[j] = row[clamp(d0 - j, 0, n - 1)], j < 4: the numbers a head's row holds for four neighbouring keys' distances,
// fetched as one run of four floats (the run is moved inside the row at its ends, and every value picked by its
// place in the run)
__device__ __forceinline__ void bias_run(const float* __restrict__ row, int n, int d0, float (&out)[4]) {
  if (__all(d0 >= 3 && d0 < n)) {        // every lane's run lies inside its row: the values as they come, last first
    const float4u v = *(const float4u*)(row + d0 - 3);
    out[0] = v[3];
    out[1] = v[2];
    out[2] = v[1];
    out[3] = v[0];
  } else if (n >= 4) {
    const int start = min(max(d0 - 3, 0), n - 4);
    const float4u v = *(const float4u*)(row + start);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int o = min(max(d0 - j, 0), n - 1) - start;
      out[j] = o == 0 ? v[0] : (o == 1 ? v[1] : (o == 2 ? v[2] : v[3]));
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = row[min(max(d0 - j, 0), n - 1)];
  }
}

__device__ __forceinline__ float fast_tanh(float y) {
  // 1 - 2 / (e^(2y) + 1), exact at both ends
  const float e = __expf(2.0f * y);
  return 1.0f - 2.0f / (e + 1.0f);
}

template <int RB>
__global__ __launch_bounds__(64) void capped_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ page_table, int pt_stride, const int* __restrict__ cu_seqlens,
    const int* __restrict__ start_pos, const int* __restrict__ tile_seq, const int* __restrict__ tile_q0, int n_tiles,
    const float* __restrict__ temp, bf16* __restrict__ out, float* __restrict__ part, int n_splits, int split_len,
    int nh, int nk, float scale, float cap, int window, int chunk, const float* __restrict__ far_a,
    const float* __restrict__ far_b, int keep_first, const float* __restrict__ bias, int n_bias) {
  const int lane = threadIdx.x & 63;
  const int tile = blockIdx.x;                    // a workgroup is one wave: the waves drift apart freely
  if (tile >= n_tiles) return;
  const int G = nh / nk;
  const int n_hc = G / RB;
  const int hk = blockIdx.y / n_hc;
  const int h0 = hk * G + (blockIdx.y % n_hc) * RB;
  const int col = lane & 15, g = lane >> 4;

  const int b = tile_seq[tile], q0 = tile_q0[tile];
  const int t_first = cu_seqlens[b] + q0;
  const int n_new = cu_seqlens[b + 1] - cu_seqlens[b];
  const int rows = min(16, n_new - q0);
  const int p0 = start_pos[b] + q0;               // position of the tile's first token
  const int p_last = p0 + rows - 1;
  const int seq_end = start_pos[b] + n_new;       // keys from here on were never written
  const int p_mine = p0 + col;                    // this lane's token (rows beyond `rows` are masked out)
  const bool row_ok = col < rows;
  const int* pt = page_table + (size_t)b * pt_stride;
  int lo = window > 0 ? max(0, p0 - window + 1) : 0;
  if (chunk > 0) lo = max(lo, p0 / chunk * chunk);          // the first token's chunk starts first
  const int chunk_lo = chunk > 0 ? p_mine / chunk * chunk : 0;
  // with key splits (steps of few tokens), this wave takes the keys [k_first, k_stop) of the tile's, counted
  // in half pages from the one that holds the first key
  const int split = blockIdx.z;
  const int k_first = (lo & ~31) + split * split_len;
  const int k_stop = n_splits > 1 ? min(p_last + 1, k_first + split_len) : p_last + 1;
  // the kept first keys, in half pages [0, kept_stop), where they lie before the first half page of the window;
  // the keys between them and the window are seen by none of the tile's tokens
  const int kept_stop = (keep_first > 0 && split == 0) ? min((keep_first + 31) & ~31, k_first) : 0;
  auto next_step = [&](int kb) { return (kb < kept_stop && kb + 32 >= kept_stop) ? k_first : kb + 32; };

  // Q fragments: token `col`, values 32 ks + 8 g .. + 8 of head h0 + r
  bf16x8 qf[RB][DKS];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int ks = 0; ks < DKS; ++ks) {
      const int d = ks * 32 + g * 8;
      bf16x8 v = {};
      if (row_ok && d < D) v = *(const bf16x8*)(q + ((size_t)(t_first + col) * nh + h0 + r) * D + d);
      qf[r][ks] = v;
    }
  float sc[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) sc[r] = scale * temp[h0 + r];
  float fa[RB], fb[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    fa[r] = far_a ? far_a[h0 + r] : 0.f;
    fb[r] = far_a ? far_b[h0 + r] : 0.f;
  }
  const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;

  floatx4 oacc[RB][NVT];
  float m[RB], l[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NVT; ++c) oacc[r][c] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // K fragments of both key tiles of the 32 keys from kb: key row `col` (+ 16), values 32 ks + 8 g .. + 8;
  // they are asked for one step ahead
  bf16x8 kn[2][DKS];
  auto ask_k = [&](int kb) {
    const int page = pt[kb / MF_PAGE];
    const bf16* kbase = kc + (((size_t)page * nk + hk) * MF_PAGE + kb % MF_PAGE + col) * D + g * 8;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int ks = 0; ks < DKS; ++ks) {
        bf16x8 v = {};
        if (ks * 32 + g * 8 < D) v = *(const bf16x8*)(kbase + (size_t)a * 16 * D + ks * 32);
        kn[a][ks] = v;
      }
  };
  const int kb_first = kept_stop > 0 ? 0 : k_first;
  if (kb_first < k_stop) ask_k(kb_first);
  for (int kb = kb_first; kb < k_stop; kb = next_step(kb)) {
    const int page = pt[kb / MF_PAGE];
    const int in_page = kb % MF_PAGE;              // 0 or 32
    bf16x8 kf[2][DKS];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int ks = 0; ks < DKS; ++ks) kf[a][ks] = kn[a][ks];
    if (next_step(kb) < k_stop) ask_k(next_step(kb));
    // V^T fragments: value row 16 c + col, keys 4 g .. + 4 and 16 + 4 g .. + 4 of this half page, asked for
    // before the scores are formed
    const bf16* vbase = vc + ((((size_t)page * nk + hk) * 2 + in_page / 32) * V + col) * 32 + 4 * g;
    short4v vlo[NVT], vhi[NVT];
#pragma unroll
    for (int c = 0; c < NVT; ++c) {
      vlo[c] = *(const short4v*)(vbase + (size_t)c * 16 * 32);
      vhi[c] = *(const short4v*)(vbase + (size_t)c * 16 * 32 + 16);
    }
    // which of this lane's 8 keys its token sees: slot j < 4: key kb + 4 g + j, else kb + 16 + 4 g + j - 4
    bool seen[8];
    float dist[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = kb + (j < 4 ? 4 * g + j : 16 + 4 * g + j - 4);
      seen[j] = row_ok && key <= p_mine && (window <= 0 || p_mine - key < window || key < keep_first) && key >= chunk_lo;
      dist[j] = (float)max(0, p_mine - key);
    }
    bf16x8 pf[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DKS; ++ks) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][ks], qf[r][ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][ks], qf[r][ks], s1, 0, 0, 0);
      }
      float x[8];
      float mx = -INFINITY;
      float add_lo[4] = {0.f, 0.f, 0.f, 0.f}, add_hi[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias) {        // this lane's keys are two runs of four neighbours, 16 keys apart
        const float* brow = bias + (size_t)(h0 + r) * n_bias;
        bias_run(brow, n_bias, p_mine - (kb + 4 * g), add_lo);
        bias_run(brow, n_bias, p_mine - (kb + 16 + 4 * g), add_hi);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float y = (j < 4 ? s0[j] : s1[j - 4]) * sc[r];
        if (cap > 0.f) y = cap * fast_tanh(y * inv_cap);
        if (far_a) y -= fa[r] * __logf(1.0f + fb[r] * dist[j]);
        if (bias) y += j < 4 ? add_lo[j] : add_hi[j - 4];
        x[j] = seen[j] ? y : -INFINITY;
        mx = fmaxf(mx, x[j]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, MF_WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, MF_WAVE));
      const float m_new = fmaxf(m[r], mx);
      const float corr = m[r] == -INFINITY ? 1.f : __expf(m[r] - m_new);
      float sum = 0.f;
      bf16x8 p;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float pe = seen[j] ? __expf(x[j] - m_new) : 0.f;
        sum += pe;
        p[j] = (bf16)pe;
      }
      pf[r] = p;
      l[r] = l[r] * corr + sum;
      m[r] = m_new;
#pragma unroll
      for (int c = 0; c < NVT; ++c) oacc[r][c] *= corr;
    }
    const bool tail = kb + 32 > seq_end;           // some of these keys were never written
#pragma unroll
    for (int c = 0; c < NVT; ++c) {
      short4v lo4 = vlo[c], hi4 = vhi[c];
      if (tail) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (kb + 4 * g + j >= seq_end) lo4[j] = 0;
          if (kb + 16 + 4 * g + j >= seq_end) hi4[j] = 0;
        }
      }
      typedef short short8v __attribute__((ext_vector_type(8)));
      const short8v both = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
      const bf16x8 vf = __builtin_bit_cast(bf16x8, both);
#pragma unroll
      for (int r = 0; r < RB; ++r) oacc[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[r], oacc[r][c], 0, 0, 0);
    }
  }

  // O^T[d = 16 c + 4 g + i][token col] -> out[token][head][d]
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    float L = l[r];
    L += __shfl_xor(L, 16, MF_WAVE);
    L += __shfl_xor(L, 32, MF_WAVE);
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    if (n_splits > 1) {
      // this split's sums, maximum and weight, for `attn_combine_kernel`: [tokens heads][splits][V + 2]
      if (row_ok) {
        float* o = part + (((size_t)(t_first + col) * nh + h0 + r) * n_splits + split) * (V + 2);
#pragma unroll
        for (int c = 0; c < NVT; ++c)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[c * 16 + 4 * g + i] = oacc[r][c][i];
        if (g == 0) { o[V] = m[r]; o[V + 1] = L; }
      }
      continue;
    }
    if (row_ok) {
      bf16* o = out + ((size_t)(t_first + col) * nh + h0 + r) * V + 4 * g;
#pragma unroll
      for (int c = 0; c < NVT; ++c) {
        bf16x4 v4;
#pragma unroll
        for (int i = 0; i < 4; ++i) v4[i] = (bf16)(oacc[r][c][i] * inv);
        *(bf16x4*)(o + c * 16) = v4;
      }
    }
  }
}

}  // namespace

MF_API int mf_capped_mfma_sizes(int* d, int* v) {
  *d = D;
  *v = V;
  return 0;
}

// tiles: blocks of 16 consecutive new tokens of a sequence (tile_seq, tile_q0), n_tiles of them
MF_API int mf_capped_mfma(const void* q, const void* kc, const void* vc, const int* page_table, int pt_stride,
                          const int* cu_seqlens, const int* start_pos, const int* tile_seq, const int* tile_q0,
                          int n_tiles, const float* temp, void* out, float* part, int n_splits, int split_len, int n_tok,
                          int nh, int nk, int d, int v, float scale, float cap, int window, int chunk, const float* far_a,
                          const float* far_b, int keep_first, const float* bias, int n_bias, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (d != D || v != V || nk <= 0 || nh % nk || !temp || n_splits < 1 || n_splits > 64 ||
      (n_splits > 1 && (!part || split_len < 32 || split_len % 32)) || chunk < 0 ||
      (far_a != nullptr) != (far_b != nullptr) || keep_first < 0 || (keep_first > 0 && chunk > 0) || (bias && n_bias < 1))
    return (int)hipErrorInvalidValue;
  if (!bias) n_bias = 1;
  const int G = nh / nk;
  // heads of a kv head a wave takes together: four where that still leaves waves for all SIMDs
  int rb = G % 2 == 0 ? 2 : 1;
  if (G % 4 == 0 && (long long)n_tiles * nk * (G / 4) >= 4096) rb = 4;
  dim3 grid(n_tiles, nk * (G / rb), n_splits);
#define MF_GO(RB)                                                                                                          \
  capped_mfma_kernel<RB><<<grid, 64, 0, stream>>>((const bf16*)q, (const bf16*)kc, (const bf16*)vc, page_table, pt_stride, \
                                                   cu_seqlens, start_pos, tile_seq, tile_q0, n_tiles, temp, (bf16*)out, part, \
                                                   n_splits, split_len, nh, nk, scale, cap, window, chunk, far_a, far_b, \
                                                   keep_first, bias, n_bias)
  if (rb == 4) MF_GO(4);
  else if (rb == 2) MF_GO(2);
  else MF_GO(1);
#undef MF_GO
  int rc = mf_launch_status();
  if (rc == 0 && n_splits > 1) {
    attn_tokens::attn_combine_kernel<bf16><<<n_tok * nh, 64 * ((V + 63) / 64), 0, stream>>>(part, (bf16*)out, V, n_splits);
    rc = mf_launch_status();
  }
  return rc;
}
