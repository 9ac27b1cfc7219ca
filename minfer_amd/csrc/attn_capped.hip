// Windowed softmax attention whose keys and values have widths of their own, with a short causal
// convolution behind the projections, a half-split rotation over the first values of a head, a
// temperature per head, capped scores and values blended with those of an earlier layer.
//
//   u = conv(W x): y_t[c] = sum_j w[c][j] u_(t - taps + 1 + j)[c], zeros before the sequence's start
//                  (the last taps - 1 projected rows of a sequence are its state);
//   q, k: value i < rot/2 of a head is turned with value i + rot/2 by the token's angle (tables), the
//         values from `rot` on pass;
//   v <- (1 - lambda) v + lambda v_first, where a layer blends;
//   s_j = cap tanh((q . k_j) scale temp[h] / cap), keys j with 0 <= p - j < window, ordinary softmax,
//   o = sum_j p_j v_j.
// The attention kernels also take a mask in chunks (a token sees the keys of its own chunk of `chunk`
// positions counted from 0, up to itself), a penalty on distance, s_j -= a[h] ln(1 + b[h] (p - j)), a number per
// head and distance that joins the score, s_j += bias[h][min(p - j, n_bias - 1)] (a table the host lays out by
// distance, whatever rule groups the distances), and, with a window, the sequence's first `keep_first`
// positions, which every later token goes on seeing (split 0 walks them before its own keys).
//
// `qkv_conv_prep_kernel`: one workgroup per (token, head of q, k or v); convolution of the head's channels
// into LDS, then rotation, blending, the cache write and q rounded to the run type.
// `conv_state_update_kernel`: behind it, the sequences' new last rows.
// `capped_attn_kernel`: a workgroup owns (token, kv head, up to 8 query heads of its group, key
// split) and walks the token's keys 256 at a time, from the half page of its first key on: a thread forms
// the scores of one key for all the heads (phase 1), a wave takes the maximum, the exponentials and their
// sum of a head (phase 2), and the threads, as (key residue, value column) pairs, add the weighted value
// rows (phase 3; in bfloat16 a thread takes a column's 32 keys of a half page with four 16-byte loads).  Every
// size is a run-time number; all sums are 32-bit and their order is fixed.
#include "attn_tokens_impl.h"

#define MF_CAP_GC 8          // query heads of a kv group a workgroup handles together
#define MF_CAP_KEYS 256      // keys per round
#define MF_CONV_MAX_TAPS 16

// ------------------------------------------------------------------ preparation
// A workgroup owns (token, head): a query head, a key head or a value head of the q|k|v row.
template <typename T>
__global__ __launch_bounds__(128) void qkv_conv_prep_kernel(
    const float* __restrict__ qkv, const float* __restrict__ conv_w, int taps, const float* __restrict__ conv_state,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_of_tok, const int* __restrict__ slot_ids,
    const int* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
    float lambda, const float* __restrict__ v_first, float* __restrict__ v_own, const int* __restrict__ page_table,
    int pt_stride, T* __restrict__ q_out, T* __restrict__ kc, T* __restrict__ vc, int H, int G, int D, int V,
    int write_cache) {
  extern __shared__ float y[];      // the head's convolved values
  const int t = blockIdx.x, unit = blockIdx.y;
  const int C = H * D + G * D + G * V;
  const int kind = unit < H ? 0 : (unit < H + G ? 1 : 2);       // query, key, value
  const int head = kind == 0 ? unit : (kind == 1 ? unit - H : unit - H - G);
  const int width = kind == 2 ? V : D;
  const int c0 = kind == 0 ? head * D : (kind == 1 ? H * D + head * D : H * D + G * D + head * V);
  const int b = seq_of_tok[t];
  const int i = t - cu_seqlens[b];  // index of the token inside its sequence's part of the step
  const float* row = qkv + (size_t)t * C + c0;
  if (conv_w) {
    const float* st = taps > 1 ? conv_state + (size_t)slot_ids[b] * (taps - 1) * C + c0 : nullptr;
    for (int e = threadIdx.x; e < width; e += 128) {
      float a = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;          // this tap reads the row `back` tokens before the token
        const float u = back <= i ? row[e - (ptrdiff_t)back * C] : st[(size_t)(i + j) * C + e];
        a = fmaf(conv_w[(size_t)(c0 + e) * taps + j], u, a);
      }
      y[e] = a;
    }
  } else {
    for (int e = threadIdx.x; e < width; e += 128) y[e] = row[e];
  }
  __syncthreads();
  const int p = positions[t];
  const int page = write_cache ? page_table[(size_t)b * pt_stride + p / MF_PAGE] : 0;
  const int in_page = p % MF_PAGE;
  if (kind < 2) {
    const int half = rot / 2;
    const float* cs = cos_t + (size_t)p * half;
    const float* sn = sin_t + (size_t)p * half;
    for (int e = threadIdx.x; e < D; e += 128) {
      float v = y[e];
      if (e < half) v = v * cs[e] - y[e + half] * sn[e];
      else if (e < rot) v = v * cs[e - half] + y[e - half] * sn[e - half];
      if (kind == 0) q_out[(size_t)t * H * D + head * D + e] = from_f32<T>(v);
      else if (write_cache) kc[(((size_t)page * G + head) * MF_PAGE + in_page) * D + e] = from_f32<T>(v);
    }
    return;
  }
  for (int e = threadIdx.x; e < V; e += 128) {
    const int c = head * V + e;
    float v = y[e];
    if (v_own) v_own[(size_t)t * G * V + c] = v;
    if (v_first) v = (1.0f - lambda) * v + lambda * v_first[(size_t)t * G * V + c];
    if (write_cache) {
      if (sizeof(T) == 2)      // bfloat16 pages keep V transposed in two halves of 32 keys
        vc[((((size_t)page * G + head) * 2 + in_page / 32) * V + e) * 32 + in_page % 32] = from_f32<T>(v);
      else
        vc[(((size_t)page * G + head) * MF_PAGE + in_page) * V + e] = from_f32<T>(v);
    }
  }
}

// state[slot][s][c], s < taps - 1, holds the projected row taps - 1 - s tokens before the sequence's next one
__global__ __launch_bounds__(256) void conv_state_update_kernel(const float* __restrict__ qkv, int taps,
                                                                float* __restrict__ conv_state,
                                                                const int* __restrict__ cu_seqlens,
                                                                const int* __restrict__ slot_ids, int C) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = cu_seqlens[b], n = cu_seqlens[b + 1] - r0;
  const int K = taps - 1;
  float* st = conv_state + (size_t)slot_ids[b] * K * C + c;
  float keep[MF_CONV_MAX_TAPS];
  for (int s = 0; s < K; ++s) {
    const int i = n + s - K;      // index inside the step's part, negative: an older row
    keep[s] = i >= 0 ? qkv[(size_t)(r0 + i) * C + c] : st[(size_t)(s + n) * C];
  }
  for (int s = 0; s < K; ++s) st[(size_t)s * C] = keep[s];
}

// ------------------------------------------------------------------ attention
template <typename T>
__device__ __forceinline__ float v_elem(const T* __restrict__ vc, int page, int nk, int hk, int in_page, int V, int e) {
  if (sizeof(T) == 2)
    return to_f32(vc[((((size_t)page * nk + hk) * 2 + in_page / 32) * V + e) * 32 + in_page % 32]);
  return to_f32(vc[(((size_t)page * nk + hk) * MF_PAGE + in_page) * V + e]);
}

template <typename T>
__global__ __launch_bounds__(256) void capped_attn_kernel(
    const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc, const int* __restrict__ page_table,
    int pt_stride, const int* __restrict__ positions, const int* __restrict__ seq_of_tok,
    const float* __restrict__ temp, T* __restrict__ out, float* __restrict__ part, int nh, int nk, int D, int V,
    int VP, float scale, float cap, int window, int chunk, const float* __restrict__ far_a,
    const float* __restrict__ far_b, int keep_first, const float* __restrict__ bias, int n_bias, int n_splits,
    int split_len) {
  extern __shared__ float lds[];
  float* sq = lds;                              // [GC][D]
  float* sc = sq + MF_CAP_GC * D;               // [GC][KEYS]
  float* red = sc + MF_CAP_GC * MF_CAP_KEYS;    // [256 / VP][GC][VP] == [GC * 256]
  __shared__ float sm_m[MF_CAP_GC], sm_l[MF_CAP_GC], sm_corr[MF_CAP_GC];

  const int t = blockIdx.x;
  const int G = nh / nk;
  const int n_gc = (G + MF_CAP_GC - 1) / MF_CAP_GC;
  const int hk = blockIdx.y / n_gc;
  const int g0 = (blockIdx.y % n_gc) * MF_CAP_GC;
  const int gcount = min(MF_CAP_GC, G - g0);
  const int h0 = hk * G + g0;
  const int split = blockIdx.z;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;

  const int p = positions[t];
  const int* pt = page_table + (size_t)seq_of_tok[t] * pt_stride;
  int lo = window > 0 ? max(0, p - window + 1) : 0;
  if (chunk > 0) lo = max(lo, p / chunk * chunk);
  // a windowed token's splits start at its window's first key, so that all of them have keys
  const int main_begin = lo + split * split_len;
  const int main_end = min(p + 1, main_begin + split_len);

  for (int i = threadIdx.x; i < gcount * D; i += 256)
    sq[i] = to_f32(q[((size_t)t * nh + h0) * D + i]);
  if (threadIdx.x < MF_CAP_GC) { sm_m[threadIdx.x] = -INFINITY; sm_l[threadIdx.x] = 0.f; sm_corr[threadIdx.x] = 1.f; }
  const int v = threadIdx.x % VP, ks = threadIdx.x / VP, KS = 256 / VP;
  float acc[MF_CAP_GC];
#pragma unroll
  for (int g = 0; g < MF_CAP_GC; ++g) acc[g] = 0.f;
  float tm[MF_CAP_GC];
#pragma unroll
  for (int g = 0; g < MF_CAP_GC; ++g) tm[g] = g < gcount ? scale * temp[h0 + g] : 0.f;
  float fa[MF_CAP_GC], fb[MF_CAP_GC];      // the penalty on distance, per head
#pragma unroll
  for (int g = 0; g < MF_CAP_GC; ++g) {
    fa[g] = (far_a && g < gcount) ? far_a[h0 + g] : 0.f;
    fb[g] = (far_a && g < gcount) ? far_b[h0 + g] : 0.f;
  }
  const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
  __syncthreads();

  // rounds of 256 keys from the half page of the first key on: a round's 32-key groups are half pages.  The walk
  // runs once over the sequence's kept first keys, where they lie before the window (split 0), and once over the
  // split's own keys; both calls are uniform over the workgroup.
  auto walk = [&](const int j_begin, const int j_end) {
  for (int cb = j_begin < j_end ? (j_begin & ~31) : j_end; cb < j_end; cb += MF_CAP_KEYS) {       // (a split may be empty)
    // phase 1: the scores of key cb + thread (-inf outside the token's keys)
    {
      const int j = cb + threadIdx.x;
      const bool valid = j >= j_begin && j < j_end;
      float s[MF_CAP_GC];
#pragma unroll
      for (int g = 0; g < MF_CAP_GC; ++g) s[g] = 0.f;
      if (valid) {
        const T* krow = kc + (((size_t)pt[j / MF_PAGE] * nk + hk) * MF_PAGE + j % MF_PAGE) * D;
        if ((D * sizeof(T)) % 16 == 0) {
          constexpr int PER = 16 / sizeof(T);
          for (int d = 0; d < D; d += PER) {
            alignas(16) T kv[PER];
            *(uint4*)kv = *(const uint4*)(krow + d);
#pragma unroll
            for (int e = 0; e < PER; ++e) {
              const float kf = to_f32(kv[e]);
#pragma unroll
              for (int g = 0; g < MF_CAP_GC; ++g) s[g] = fmaf(sq[g * D + d + e], kf, s[g]);
            }
          }
        } else {
          for (int d = 0; d < D; ++d) {
            const float kf = to_f32(krow[d]);
#pragma unroll
            for (int g = 0; g < MF_CAP_GC; ++g) s[g] = fmaf(sq[g * D + d], kf, s[g]);
          }
        }
      }
#pragma unroll
      for (int g = 0; g < MF_CAP_GC; ++g) {
        float x = s[g] * tm[g];
        if (cap > 0.f) x = cap * tanhf(x * inv_cap);
        if (far_a && valid) x -= fa[g] * log1pf(fb[g] * (float)(p - j));
        if (bias && valid && g < gcount) x += bias[(size_t)(h0 + g) * n_bias + min(p - j, n_bias - 1)];
        sc[g * MF_CAP_KEYS + threadIdx.x] = valid ? x : -INFINITY;
      }
    }
    __syncthreads();
    // phase 2: wave w takes the heads w, w + 4; every round holds at least one of the token's keys
    for (int g = w; g < gcount; g += 4) {
      float x[MF_CAP_KEYS / 64];
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < MF_CAP_KEYS / 64; ++r) {
        x[r] = sc[g * MF_CAP_KEYS + lane + 64 * r];
        mx = fmaxf(mx, x[r]);
      }
      mx = wave_max(mx);
      const float m_old = sm_m[g];
      const float m_new = fmaxf(m_old, mx);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < MF_CAP_KEYS / 64; ++r) {
        const float pe = x[r] == -INFINITY ? 0.f : attn_tokens::exp_for<T>(x[r] - m_new);
        sc[g * MF_CAP_KEYS + lane + 64 * r] = pe;
        sum += pe;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float corr = m_old == -INFINITY ? 1.f : attn_tokens::exp_for<T>(m_old - m_new);
        sm_corr[g] = corr;
        sm_l[g] = sm_l[g] * corr + sum;
        sm_m[g] = m_new;
      }
    }
    __syncthreads();
    // phase 3: thread (ks, v) adds the value rows.  bfloat16 pages keep a value column's 32 keys of a half
    // page side by side: a thread takes whole half pages, 16 bytes a load; 32-bit pages are read key by key.
    if (v < V) {
#pragma unroll
      for (int g = 0; g < MF_CAP_GC; ++g) acc[g] *= sm_corr[g];
      if (sizeof(T) == 2) {
        for (int gi = ks; gi < MF_CAP_KEYS / 32; gi += KS) {
          const int jb = cb + 32 * gi;
          if (jb >= j_end || jb + 32 <= j_begin) continue;
          const T* vrow = vc + ((((size_t)pt[jb / MF_PAGE] * nk + hk) * 2 + (jb / 32 & 1)) * V + v) * 32;
          alignas(16) T vals[32];
#pragma unroll
          for (int c = 0; c < 4; ++c) *(uint4*)(vals + 8 * c) = *(const uint4*)(vrow + 8 * c);
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            const int j = jb + i;
            const float vv = (j >= j_begin && j < j_end) ? to_f32(vals[i]) : 0.f;      // unwritten keys may hold anything
#pragma unroll
            for (int g = 0; g < MF_CAP_GC; ++g) acc[g] = fmaf(sc[g * MF_CAP_KEYS + 32 * gi + i], vv, acc[g]);
          }
        }
      } else {
        for (int i = ks; i < MF_CAP_KEYS; i += KS) {
          const int j = cb + i;
          if (j < j_begin || j >= j_end) continue;
          const float vv = v_elem<T>(vc, pt[j / MF_PAGE], nk, hk, j % MF_PAGE, V, v);
#pragma unroll
          for (int g = 0; g < MF_CAP_GC; ++g) acc[g] = fmaf(sc[g * MF_CAP_KEYS + i], vv, acc[g]);
        }
      }
    }
    __syncthreads();
  }
  };
  if (keep_first > 0 && split == 0 && lo > 0) walk(0, min(keep_first, lo));
  walk(main_begin, main_end);

  // add the key residues, in their order
#pragma unroll
  for (int g = 0; g < MF_CAP_GC; ++g) red[(ks * MF_CAP_GC + g) * VP + v] = acc[g];
  __syncthreads();
  for (int i = threadIdx.x; i < gcount * V; i += 256) {
    const int g = i / V, e = i % V;
    float a = 0.f;
    for (int k = 0; k < KS; ++k) a += red[(k * MF_CAP_GC + g) * VP + e];
    const int h = h0 + g;
    const float L = sm_l[g];
    if (n_splits == 1) {
      out[((size_t)t * nh + h) * V + e] = from_f32<T>(L > 0.f ? a / L : 0.f);
    } else {
      float* o = part + (((size_t)t * nh + h) * n_splits + split) * (V + 2);
      o[e] = a;
      if (e == 0) { o[V] = sm_m[g]; o[V + 1] = L; }
    }
  }
}

// ------------------------------------------------------------------ the half-split rotation alone
// rows [tokens][n_heads_total][head_dim] float32, in place, on the first n_rot_heads heads
__global__ __launch_bounds__(256) void rope_half_inplace_kernel(float* __restrict__ rows, const float* __restrict__ cos_t,
                                                                const float* __restrict__ sin_t,
                                                                const int* __restrict__ positions, int n_rot_heads,
                                                                int n_heads_total, int head_dim, int rot) {
  const int t = blockIdx.x;
  const int half = rot / 2;
  const float* cs = cos_t + (size_t)positions[t] * half;
  const float* sn = sin_t + (size_t)positions[t] * half;
  float* row = rows + (size_t)t * n_heads_total * head_dim;
  for (int i = threadIdx.x; i < n_rot_heads * half; i += 256) {
    const int h = i / half, e = i % half;
    float* a = row + (size_t)h * head_dim + e;
    const float x = a[0], z = a[half];
    a[0] = x * cs[e] - z * sn[e];
    a[half] = z * cs[e] + x * sn[e];
  }
}

// ------------------------------------------------------------------ entry points
MF_API int mf_qkv_conv_prep(const float* qkv, const float* conv_w, int taps, float* conv_state, const int* cu_seqlens,
                            const int* seq_of_tok, const int* slot_ids, const int* positions, const float* cos_t,
                            const float* sin_t, int rot, float lambda, const float* v_first, float* v_own,
                            const int* page_table, int pt_stride, void* q_out, void* kc, void* vc, int is_bf16, int n_tok,
                            int n_seqs, int H, int G, int D, int V, int write_cache, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  const int C = H * D + G * D + G * V;
  if (H <= 0 || G <= 0 || D <= 0 || V <= 0 || rot < 0 || rot % 2 || rot > D || taps < 1 || taps > MF_CONV_MAX_TAPS ||
      (taps > 1 && (!conv_w || !conv_state)) || D > 8192 || V > 8192)
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(D > V ? D : V) * sizeof(float);
  const dim3 grid(n_tok, H + 2 * G);
  int rc;
  if (is_bf16) {
    qkv_conv_prep_kernel<bf16><<<grid, 128, lds, stream>>>(qkv, conv_w, taps, conv_state, cu_seqlens, seq_of_tok, slot_ids,
                                                            positions, cos_t, sin_t, rot, lambda, v_first, v_own, page_table,
                                                            pt_stride, (bf16*)q_out, (bf16*)kc, (bf16*)vc, H, G, D, V,
                                                            write_cache);
  } else {
    qkv_conv_prep_kernel<float><<<grid, 128, lds, stream>>>(qkv, conv_w, taps, conv_state, cu_seqlens, seq_of_tok, slot_ids,
                                                             positions, cos_t, sin_t, rot, lambda, v_first, v_own, page_table,
                                                             pt_stride, (float*)q_out, (float*)kc, (float*)vc, H, G, D, V,
                                                             write_cache);
  }
  rc = mf_launch_status();
  if (rc || taps <= 1 || !write_cache) return rc;
  conv_state_update_kernel<<<dim3((C + 255) / 256, n_seqs), 256, 0, stream>>>(qkv, taps, conv_state, cu_seqlens, slot_ids, C);
  return mf_launch_status();
}

MF_API int mf_capped_attn(const void* q, const void* kc, const void* vc, const int* page_table, int pt_stride,
                          const int* positions, const int* seq_of_tok, const float* temp, void* out, float* part,
                          int is_bf16, int n_tok, int nh, int nk, int D, int V, float scale, float cap, int window,
                          int chunk, const float* far_a, const float* far_b, int keep_first, const float* bias,
                          int n_bias, int n_splits, int split_len, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (nk <= 0 || nh % nk || D <= 0 || D > 512 || V <= 0 || V > 256 || n_splits < 1 || n_splits > 64 ||
      split_len < 1 || (n_splits > 1 && !part) || !temp || chunk < 0 || (far_a != nullptr) != (far_b != nullptr) ||
      keep_first < 0 || (keep_first > 0 && chunk > 0) || (bias && n_bias < 1))
    return (int)hipErrorInvalidValue;
  int VP = 1;
  while (VP < V) VP *= 2;
  const int G = nh / nk;
  dim3 grid(n_tok, nk * ((G + MF_CAP_GC - 1) / MF_CAP_GC), n_splits);
  const size_t lds = sizeof(float) * ((size_t)MF_CAP_GC * D + MF_CAP_GC * MF_CAP_KEYS + MF_CAP_GC * 256);
  int rc;
  if (is_bf16) {
    capped_attn_kernel<bf16><<<grid, 256, lds, stream>>>((const bf16*)q, (const bf16*)kc, (const bf16*)vc, page_table,
                                                         pt_stride, positions, seq_of_tok, temp, (bf16*)out, part, nh, nk,
                                                         D, V, VP, scale, cap, window, chunk, far_a, far_b, keep_first, bias, n_bias, n_splits,
                                                         split_len);
    rc = mf_launch_status();
    if (rc == 0 && n_splits > 1) {
      attn_tokens::attn_combine_kernel<bf16><<<n_tok * nh, 64 * ((V + 63) / 64), 0, stream>>>(part, (bf16*)out, V, n_splits);
      rc = mf_launch_status();
    }
  } else {
    capped_attn_kernel<float><<<grid, 256, lds, stream>>>((const float*)q, (const float*)kc, (const float*)vc, page_table,
                                                          pt_stride, positions, seq_of_tok, temp, (float*)out, part, nh,
                                                          nk, D, V, VP, scale, cap, window, chunk, far_a, far_b, keep_first, bias, n_bias, n_splits,
                                                         split_len);
    rc = mf_launch_status();
    if (rc == 0 && n_splits > 1) {
      attn_tokens::attn_combine_kernel<float><<<n_tok * nh, 64 * ((V + 63) / 64), 0, stream>>>(part, (float*)out, V, n_splits);
      rc = mf_launch_status();
    }
  }
  return rc;
}

MF_API int mf_rope_half_inplace(float* rows, const float* cos_t, const float* sin_t, const int* positions, int n_tok,
                                int n_rot_heads, int n_heads_total, int head_dim, int rot, hipStream_t stream) {
  if (n_tok <= 0 || rot <= 0) return 0;
  if (rot % 2 || rot > head_dim || n_rot_heads > n_heads_total) return (int)hipErrorInvalidValue;
  rope_half_inplace_kernel<<<n_tok, 256, 0, stream>>>(rows, cos_t, sin_t, positions, n_rot_heads, n_heads_total, head_dim, rot);
  return mf_launch_status();
}
