// Linear attention whose forget gate, one per key channel and token, sets the input gate as well
// (the HGRN2 recurrence), over the ragged batch of a step, state in 32-bit per sequence slot.
//
// Per head, with q_t = silu(q projection) (dim values), v_t the value projection (vdim values) and
//   a_t = l + (1 - l) sigmoid(f projection + bias)      (dim values, l the learned lower bounds),
//   S_t = diag(a_t) S_(t-1) + (1 - a_t) v_t^T           (dim x vdim),      o_t = S_t^T q_t.
// Every head's o_t is then RMS-normed over its vdim values with a gain vector shared by the heads,
// multiplied by a scale and rounded once (`head_rmsnorm_kernel`).  q | f | v arrive as one 32-bit row per
// token (the bias already added); gates, state, products and sums are 32-bit throughout.
//
// `gated_scan_kernel`: a workgroup owns (segment, head, 64 value columns) and walks the segment's
// tokens in order; its 256 threads are 4 slices of the key dimension times 64 columns, a thread keeping its
// slice of its column of S in registers.  A segment is a sequence's part of the step (decode steps, short
// portions), or a chunk of MF_GR_CHUNK tokens of it.  The recurrence is linear in the state,
// S_out = diag(A) S_in + B with A the product of the chunk's gates and B what the chunk leaves from a zero
// state, so prompts run in three passes: every chunk's (A, B) side by side; the fold along each sequence,
// which leaves every chunk its S_in; every chunk again from its S_in, side by side, writing the outputs (the
// last chunk of a sequence leaves the new state).  The order of a position's additions depends on where the
// chunk edges fall inside the step, never on the batch.
#include "common.h"

#define MF_GR_CHUNK 64
#define MF_GR_TT 8     // tokens whose q and gates are staged together

__device__ __forceinline__ float gr_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

#define MF_GR_SEQUENCES 0
#define MF_GR_REDUCE 1
#define MF_GR_APPLY 2

// proj row: q [H D] | f [H D] | v [H V].  chunk table: int32 [4][n_chunks] = first token, tokens, sequence, last of
// its sequence or not.
template <int DS, int MODE>
__global__ __launch_bounds__(256) void gated_scan_kernel(const float* __restrict__ proj, int row_len,
                                                         const float* __restrict__ lower,
                                                         const int* __restrict__ cu_seqlens,
                                                         const int* __restrict__ chunks, int n_chunks,
                                                         const int* __restrict__ slot_ids, float* __restrict__ state,
                                                         float* __restrict__ ws, float* __restrict__ ws_a,
                                                         float* __restrict__ out, int H, int D, int V) {
  __shared__ float sq[MF_GR_TT][4 * DS], sa[MF_GR_TT][4 * DS];
  __shared__ float partial[MF_GR_TT][4][64];
  const int seg = blockIdx.x, h = blockIdx.y;
  const int col = blockIdx.z * 64 + (threadIdx.x & 63), slice = threadIdx.x >> 6;
  const bool live = col < V;
  int t0, t1, seq;
  bool leaves_state = true;
  if (MODE == MF_GR_SEQUENCES) {
    seq = seg;
    t0 = cu_seqlens[seq];
    t1 = cu_seqlens[seq + 1];
  } else {
    t0 = chunks[seg];
    t1 = t0 + chunks[n_chunks + seg];
    seq = chunks[2 * n_chunks + seg];
    leaves_state = chunks[3 * n_chunks + seg] != 0;
  }
  float* st = state + (((size_t)slot_ids[seq] * H + h) * D) * V + col;
  float* mine = ws + (((size_t)seg * H + h) * D) * V + col;          // the chunk's B, then its S_in
  float S[DS], A[DS];
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = slice * DS + i;
    A[i] = 1.f;
    if (MODE == MF_GR_REDUCE) S[i] = 0.f;
    else if (MODE == MF_GR_APPLY) S[i] = (live && d < D) ? mine[(size_t)d * V] : 0.f;
    else S[i] = (live && d < D) ? st[(size_t)d * V] : 0.f;
  }
  const int off_f = H * D, off_v = 2 * H * D;
  for (int tb = t0; tb < t1; tb += MF_GR_TT) {
    const int nt = min(MF_GR_TT, t1 - tb);
    __syncthreads();
    for (int i = threadIdx.x; i < nt * 4 * DS; i += 256) {
      const int tt = i / (4 * DS), d = i % (4 * DS);
      const float* row = proj + (size_t)(tb + tt) * row_len + h * D + d;
      float qv = 0.f, av = 1.f;
      if (d < D) {
        const float l = lower[h * D + d];
        av = l + (1.0f - l) * gr_sigmoid(row[off_f]);
        if (MODE != MF_GR_REDUCE) { const float z = row[0]; qv = z * gr_sigmoid(z); }
      }
      sq[tt][d] = qv;
      sa[tt][d] = av;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = live ? proj[(size_t)(tb + tt) * row_len + off_v + h * V + col] : 0.f;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        const int d = slice * DS + i;
        const float a = sa[tt][d];
        S[i] = fmaf(a, S[i], (1.0f - a) * vv);
        if (MODE == MF_GR_REDUCE) A[i] *= a;
        else o = fmaf(S[i], sq[tt][d], o);
      }
      if (MODE != MF_GR_REDUCE) partial[tt][slice][threadIdx.x & 63] = o;
    }
    if (MODE == MF_GR_REDUCE) continue;
    __syncthreads();
    for (int i = threadIdx.x; i < nt * 64; i += 256) {
      const int tt = i >> 6, c = i & 63;
      const int cc = blockIdx.z * 64 + c;
      if (cc < V)
        out[(size_t)(tb + tt) * H * V + h * V + cc] =
            ((partial[tt][0][c] + partial[tt][1][c]) + partial[tt][2][c]) + partial[tt][3][c];
    }
  }
  if (MODE == MF_GR_REDUCE) {
#pragma unroll
    for (int i = 0; i < DS; ++i) {
      const int d = slice * DS + i;
      if (live && d < D) mine[(size_t)d * V] = S[i];
      if (d < D && blockIdx.z == 0 && (threadIdx.x & 63) == 0) ws_a[((size_t)seg * H + h) * D + d] = A[i];
    }
    return;
  }
  if (live && leaves_state) {
#pragma unroll
    for (int i = 0; i < DS; ++i) {
      const int d = slice * DS + i;
      if (d < D) st[(size_t)d * V] = S[i];
    }
  }
}

// the fold along each sequence: a thread owns one element of a head's state; ws[c] goes from the chunk's B to
// the state the chunk starts from
__global__ __launch_bounds__(256) void gated_fold_kernel(const int* __restrict__ seq_first_chunk,
                                                         const int* __restrict__ slot_ids,
                                                         const float* __restrict__ state, float* __restrict__ ws,
                                                         const float* __restrict__ ws_a, int H, int D, int V) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= D * V) return;
  const int d = e / V;
  float S = state[((size_t)slot_ids[seq] * H + h) * D * V + e];
  for (int c = seq_first_chunk[seq]; c < seq_first_chunk[seq + 1]; ++c) {
    float* w = ws + ((size_t)c * H + h) * D * V + e;
    const float B = *w;
    *w = S;
    S = fmaf(ws_a[((size_t)c * H + h) * D + d], S, B);
  }
}

// y[t][h][:] = o[t][h][:] / sqrt(mean(o[t][h][:]^2) + eps) * w[:] * scale, a wave per head
template <typename OT>
__global__ __launch_bounds__(256) void head_rmsnorm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                           OT* __restrict__ y, int H, int V, float eps, float scale) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  for (int h = threadIdx.x >> 6; h < H; h += 4) {
    const float* row = o + ((size_t)t * H + h) * V;
    float ss = 0.f;
    for (int i = lane; i < V; i += 64) ss = fmaf(row[i], row[i], ss);
    ss = wave_sum(ss);
    const float inv = scale / sqrtf(ss / (float)V + eps);
    for (int i = lane; i < V; i += 64) y[((size_t)t * H + h) * V + i] = from_f32<OT>(row[i] * inv * (w ? w[i] : 1.0f));
  }
}

#define MF_GR_DISPATCH(CALL)  \
  if (D <= 32) { CALL(8) }    \
  else if (D <= 64) { CALL(16) } \
  else if (D <= 128) { CALL(32) } \
  else { CALL(64) }

MF_API int mf_gr_chunk(void) { return MF_GR_CHUNK; }

// proj float32 [tokens][2 H D + H V]; lower float32 [H D]; state float32 [slots][H][D][V]; out float32 [tokens][H V]
MF_API int mf_gated_scan(const float* proj, const float* lower, const int* cu_seqlens, const int* slot_ids, float* state,
                         float* out, int n_seqs, int H, int D, int V, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (H <= 0 || D <= 0 || V <= 0 || D > 256) return (int)hipErrorInvalidValue;
  const int row_len = 2 * H * D + H * V;
  dim3 grid(n_seqs, H, (V + 63) / 64);
#define MF_CALL(DS)                                                                                                    \
  gated_scan_kernel<DS, MF_GR_SEQUENCES><<<grid, 256, 0, stream>>>(proj, row_len, lower, cu_seqlens, nullptr, 0, slot_ids, \
                                                                    state, nullptr, nullptr, out, H, D, V);
  MF_GR_DISPATCH(MF_CALL)
#undef MF_CALL
  return mf_launch_status();
}

// chunks int32 [4][n_chunks]; seq_first_chunk int32 [n_seqs + 1]; ws float32 [n_chunks][H][D][V] and ws_a
// float32 [n_chunks][H][D], both scratch
MF_API int mf_gated_scan_chunked(const float* proj, const float* lower, const int* chunks, int n_chunks,
                                 const int* seq_first_chunk, const int* slot_ids, float* state, float* ws, float* ws_a,
                                 float* out, int n_seqs, int H, int D, int V, hipStream_t stream) {
  if (n_seqs <= 0 || n_chunks <= 0) return 0;
  if (H <= 0 || D <= 0 || V <= 0 || D > 256 || !ws || !ws_a) return (int)hipErrorInvalidValue;
  const int row_len = 2 * H * D + H * V;
  dim3 grid(n_chunks, H, (V + 63) / 64);
#define MF_CALL(DS)                                                                                                    \
  gated_scan_kernel<DS, MF_GR_REDUCE><<<grid, 256, 0, stream>>>(proj, row_len, lower, nullptr, chunks, n_chunks, slot_ids, \
                                                                 state, ws, ws_a, nullptr, H, D, V);
  MF_GR_DISPATCH(MF_CALL)
#undef MF_CALL
  int rc = mf_launch_status();
  if (rc) return rc;
  gated_fold_kernel<<<dim3(n_seqs, H, (D * V + 255) / 256), 256, 0, stream>>>(seq_first_chunk, slot_ids, state, ws, ws_a, H,
                                                                              D, V);
  rc = mf_launch_status();
  if (rc) return rc;
#define MF_CALL(DS)                                                                                                    \
  gated_scan_kernel<DS, MF_GR_APPLY><<<grid, 256, 0, stream>>>(proj, row_len, lower, nullptr, chunks, n_chunks, slot_ids, \
                                                                state, ws, ws_a, out, H, D, V);
  MF_GR_DISPATCH(MF_CALL)
#undef MF_CALL
  return mf_launch_status();
}

MF_API int mf_head_rmsnorm(const float* o, const float* w, void* y, int y_is_bf16, int rows, int H, int V, float eps,
                           float scale, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || V <= 0) return (int)hipErrorInvalidValue;
  if (y_is_bf16)
    head_rmsnorm_kernel<bf16><<<rows, 256, 0, stream>>>(o, w, (bf16*)y, H, V, eps, scale);
  else
    head_rmsnorm_kernel<float><<<rows, 256, 0, stream>>>(o, w, (float*)y, H, V, eps, scale);
  return mf_launch_status();
}
