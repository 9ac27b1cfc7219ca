// Preparation of queries, keys and values for an attention whose queries and keys are RMS-normed per
// head, whose rotation turns neighbouring pairs, and whose values may be the keys as projected and may
// be rotated themselves; and the turn back of the attention's result.
//
//   q, k (per head): x / sqrt(mean(x^2) + eps) (or no norm at all), times a gain vector shared by the heads
//         where one is given; then values 2i and 2i + 1, i < rot / 2, turn by the token's angle i (tables
//         [positions][rot / 2]), or, in the half-split layout, value i turns with value i + rot / 2; the
//         values from `rot` on pass.  A design that norms behind the rotation, without gains, gets the same
//         numbers: a rotation leaves a head's sum of squares as it is, and a common factor passes through it;
//   a layer that reads another layer's keys and values (`q_only`) has query heads only;
//   v:    its own projection, or (`v_from_k`) the key head as projected, before the norm; with value
//         tables [positions][V / 2] its pairs (2m, 2m + 1) turn by the token's angle m on the way into the
//         cache;
//   the attention's result per head is rotated back by the query token's angles (`unrotate_kernel`),
//   multiplied by a scale and rounded to the run type.
//
// `qk_norm_prep_kernel`: a workgroup per (token, head of q, k or v): the head in LDS, the sum of squares
// over the workgroup, then norm, rotation, the cache write (pages as every attention kernel reads them)
// and q rounded to the run type.  All arithmetic is 32-bit.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(128) void qk_norm_prep_kernel(
    const float* __restrict__ qkv, int C, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    int normed, const int* __restrict__ seq_of_tok, const int* __restrict__ positions, const float* __restrict__ cos_r,
    const float* __restrict__ sin_r, int rot, int halves, const float* __restrict__ cos_v,
    const float* __restrict__ sin_v, int v_from_k, const int* __restrict__ page_table, int pt_stride, T* __restrict__ q_out, T* __restrict__ kc,
    T* __restrict__ vc, int H, int G, int D, int V, int write_cache) {
  extern __shared__ float y[];
  __shared__ float scratch[2];
  const int t = blockIdx.x, unit = blockIdx.y;
  const int kind = unit < H ? 0 : (unit < H + G ? 1 : 2);       // query, key, value
  const int head = kind == 0 ? unit : (kind == 1 ? unit - H : unit - H - G);
  const int width = kind == 2 ? V : D;
  const int c0 = kind == 0 ? head * D : (kind == 1 ? H * D + head * D : H * D + G * D + head * V);
  const float* row = qkv + (size_t)t * C + c0;
  float ss = 0.f;
  for (int e = threadIdx.x; e < width; e += 128) {
    const float v = row[e];
    y[e] = v;
    ss = fmaf(v, v, ss);
  }
  const int p = positions[t];
  const int page = write_cache ? page_table[(size_t)seq_of_tok[t] * pt_stride + p / MF_PAGE] : 0;
  const int in_page = p % MF_PAGE;
  ss = block_sum<128>(ss, scratch);          // (its barriers also publish y)

  // the value: its own head, or the key head as it was projected
  if (write_cache && (kind == 2 || (kind == 1 && v_from_k))) {
    const float* cs = cos_v ? cos_v + (size_t)p * (V / 2) : nullptr;
    const float* sn = cos_v ? sin_v + (size_t)p * (V / 2) : nullptr;
    for (int e = threadIdx.x; e < V; e += 128) {
      float v = y[e];
      if (cs) {
        const int m = e >> 1;
        v = (e & 1) ? v * cs[m] + y[e - 1] * sn[m] : v * cs[m] - y[e + 1] * sn[m];
      }
      if (sizeof(T) == 2)      // bfloat16 pages keep V transposed in two halves of 32 keys
        vc[((((size_t)page * G + head) * 2 + in_page / 32) * V + e) * 32 + in_page % 32] = from_f32<T>(v);
      else
        vc[(((size_t)page * G + head) * MF_PAGE + in_page) * V + e] = from_f32<T>(v);
    }
  }
  if (kind == 2) return;

  const float inv = normed ? 1.0f / sqrtf(ss / (float)D + eps) : 1.0f;
  const float* gain = kind == 0 ? q_gain : k_gain;
  const int half = rot / 2;
  const float* cs = cos_r + (size_t)p * half;
  const float* sn = sin_r + (size_t)p * half;
  for (int e = threadIdx.x; e < D; e += 128) {
    float v = y[e] * inv * (gain ? gain[e] : 1.0f);
    if (e < rot) {
      // the value's partner and whether the value is the pair's second: neighbours, or half a rotation apart
      const int o = halves ? (e < half ? e + half : e - half) : (e ^ 1);
      const bool second = halves ? e >= half : (e & 1);
      const int i = halves ? (second ? e - half : e) : (e >> 1);
      const float w = y[o] * inv * (gain ? gain[o] : 1.0f);
      v = second ? v * cs[i] + w * sn[i] : v * cs[i] - w * sn[i];
    }
    if (kind == 0) q_out[((size_t)t * H + head) * D + e] = from_f32<T>(v);
    else if (write_cache) kc[(((size_t)page * G + head) * MF_PAGE + in_page) * D + e] = from_f32<T>(v);
  }
}

// rows [tokens][heads][V] of the run type, in place: pair m of every head turns by minus the token's angle m,
// and everything is multiplied by `scale`
template <typename T>
__global__ __launch_bounds__(256) void unrotate_kernel(T* __restrict__ rows, const float* __restrict__ cos_v,
                                                       const float* __restrict__ sin_v, const int* __restrict__ positions,
                                                       int H, int V, float scale) {
  const int t = blockIdx.x;
  const int half = V / 2;
  const float* cs = cos_v ? cos_v + (size_t)positions[t] * half : nullptr;
  const float* sn = cos_v ? sin_v + (size_t)positions[t] * half : nullptr;
  T* row = rows + (size_t)t * H * V;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < H * half; i += gridDim.y * 256) {
    const int h = i / half, m = i % half;
    T* a = row + (size_t)h * V + 2 * m;
    const float u = to_f32(a[0]), v = to_f32(a[1]);
    const float c = cs ? cs[m] : 1.0f, s = cs ? sn[m] : 0.0f;
    a[0] = from_f32<T>((u * c + v * s) * scale);
    a[1] = from_f32<T>((v * c - u * s) * scale);
  }
}

MF_API int mf_qk_norm_prep(const float* qkv, const float* q_gain, const float* k_gain, float eps, int normed,
                           const int* seq_of_tok, const int* positions, const float* cos_r, const float* sin_r, int rot,
                           int halves, int q_only, const float* cos_v, const float* sin_v, int v_from_k, const int* page_table, int pt_stride,
                           void* q_out, void* kc, void* vc, int is_bf16, int n_tok, int H, int G, int D, int V,
                           int write_cache, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (H <= 0 || G <= 0 || D <= 0 || V <= 0 || rot < 0 || rot % 2 || rot > D || (rot > 0 && (!cos_r || !sin_r)) ||
      (cos_v != nullptr) != (sin_v != nullptr) || (cos_v && V % 2) || (v_from_k && V != D) || D > 8192 || V > 8192)
    return (int)hipErrorInvalidValue;
  // with q_only the rows hold the query heads alone and only they are prepared: nothing is written to the cache
  const int C = q_only ? H * D : H * D + G * D + (v_from_k ? 0 : G * V);
  const size_t lds = (size_t)(D > V ? D : V) * sizeof(float);
  const dim3 grid(n_tok, q_only ? H : H + G + (v_from_k ? 0 : G));
  if (q_only) write_cache = 0;
  if (is_bf16)
    qk_norm_prep_kernel<bf16><<<grid, 128, lds, stream>>>(qkv, C, q_gain, k_gain, eps, normed, seq_of_tok, positions, cos_r,
                                                           sin_r, rot, halves, cos_v, sin_v, v_from_k, page_table, pt_stride,
                                                           (bf16*)q_out, (bf16*)kc, (bf16*)vc, H, G, D, V, write_cache);
  else
    qk_norm_prep_kernel<float><<<grid, 128, lds, stream>>>(qkv, C, q_gain, k_gain, eps, normed, seq_of_tok, positions, cos_r,
                                                            sin_r, rot, halves, cos_v, sin_v, v_from_k, page_table, pt_stride,
                                                            (float*)q_out, (float*)kc, (float*)vc, H, G, D, V, write_cache);
  return mf_launch_status();
}

MF_API int mf_unrotate(void* rows, int is_bf16, const float* cos_v, const float* sin_v, const int* positions, int n_tok,
                       int H, int V, float scale, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (H <= 0 || V <= 0 || V % 2 || (cos_v != nullptr) != (sin_v != nullptr)) return (int)hipErrorInvalidValue;
  int by = (H * (V / 2) + 255) / 256;
  if (by > 16) by = 16;
  const dim3 grid(n_tok, by);
  if (is_bf16)
    unrotate_kernel<bf16><<<grid, 256, 0, stream>>>((bf16*)rows, cos_v, sin_v, positions, H, V, scale);
  else
    unrotate_kernel<float><<<grid, 256, 0, stream>>>((float*)rows, cos_v, sin_v, positions, H, V, scale);
  return mf_launch_status();
}
