// Gated linear recurrences over the ragged batch of a step, state in 32-bit per sequence slot.
//
// minGRU: the gates read only the current token, so with z_t = sigmoid(zp_t) and the candidate
// c_t = up_t + 1/2 (up_t >= 0), sigmoid(up_t) (up_t < 0) the state obeys, element by element,
//   S_t = (1 - z_t) S_(t-1) + z_t c_t,
// a first-order linear recurrence S_t = a_t S_(t-1) + b_t.  The mixer's output row is
// S_t silu(g_t).  zp | up | g arrive as one 32-bit row [3 W] per token (biases added by the
// product that made them); everything here is 32-bit, the output is rounded once.
//
// Two forms.  `mingru_scan_kernel`: a thread per (sequence, channel) walks the sequence's new
// tokens in order (decode steps, short portions).  The chunked form for prompts: the tokens of a
// sequence are cut into chunks of MF_SCAN_CHUNK; pass 1 reduces every chunk to the pair (A, B)
// with S_out = A S_in + B; pass 2 gives each chunk its S_in by folding the pairs of the chunks
// before it, in order, onto the sequence's stored state, and walks the chunk once more to write
// the outputs.  The additions of a position happen in an order that depends only on where the
// chunk edges fall inside the step, never on what else is in the batch.
#include "common.h"

#define MF_SCAN_CHUNK 32

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ void mingru_coeffs(float zp, float up, float& a, float& b) {
  const float z = sigmoid_f(zp);
  const float c = up >= 0.f ? up + 0.5f : sigmoid_f(up);
  a = 1.0f - z;
  b = z * c;
}

template <typename OT>
__global__ __launch_bounds__(256) void mingru_scan_kernel(const float* __restrict__ zug,
                                                          const int* __restrict__ cu_seqlens,
                                                          const int* __restrict__ slot_ids,
                                                          float* __restrict__ state, OT* __restrict__ out,
                                                          int W) {
  const int seq = blockIdx.y;
  const int ch = blockIdx.x * 256 + threadIdx.x;
  if (ch >= W) return;
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
  float* st = state + (size_t)slot_ids[seq] * W + ch;
  float S = *st;
  for (int t = t0; t < t1; ++t) {
    const float* row = zug + (size_t)t * 3 * W + ch;
    float a, b;
    mingru_coeffs(row[0], row[W], a, b);
    S = a * S + b;
    const float g = row[2 * W];
    out[(size_t)t * W + ch] = from_f32<OT>(S * (g * sigmoid_f(g)));
  }
  *st = S;
}

// pass 1: chunk c (tokens chunk_t0[c] .. chunk_t0[c] + chunk_n[c]) -> AB[c][0][ch], AB[c][1][ch]
__global__ __launch_bounds__(256) void mingru_chunk_reduce_kernel(const float* __restrict__ zug,
                                                                  const int* __restrict__ chunk_t0,
                                                                  const int* __restrict__ chunk_n,
                                                                  float* __restrict__ ab, int W) {
  const int c = blockIdx.y;
  const int ch = blockIdx.x * 256 + threadIdx.x;
  if (ch >= W) return;
  const int t0 = chunk_t0[c], n = chunk_n[c];
  float A = 1.f, B = 0.f;
#pragma unroll 4
  for (int i = 0; i < n; ++i) {
    const float* row = zug + (size_t)(t0 + i) * 3 * W + ch;
    float a, b;
    mingru_coeffs(row[0], row[W], a, b);
    A *= a;
    B = a * B + b;
  }
  ab[((size_t)c * 2) * W + ch] = A;
  ab[((size_t)c * 2 + 1) * W + ch] = B;
}

// pass 2: chunk_first[c] is the index of the first chunk of c's sequence, chunk_seq[c] the
// sequence; the last chunk of a sequence (chunk_last[c] != 0) stores the state.  The state that
// the chunks of a sequence start from was copied to `state_in[seq]` beforehand (the stored state
// is overwritten by the sequence's last chunk while others may still read).
template <typename OT>
__global__ __launch_bounds__(256) void mingru_chunk_apply_kernel(
    const float* __restrict__ zug, const int* __restrict__ chunk_t0, const int* __restrict__ chunk_n,
    const int* __restrict__ chunk_seq, const int* __restrict__ chunk_first, const int* __restrict__ chunk_last,
    const float* __restrict__ ab, const float* __restrict__ state_in, const int* __restrict__ slot_ids,
    float* __restrict__ state, OT* __restrict__ out, int W) {
  const int c = blockIdx.y;
  const int ch = blockIdx.x * 256 + threadIdx.x;
  if (ch >= W) return;
  const int seq = chunk_seq[c];
  float S = state_in[(size_t)seq * W + ch];
#pragma unroll 4
  for (int k = chunk_first[c]; k < c; ++k)
    S = ab[((size_t)k * 2) * W + ch] * S + ab[((size_t)k * 2 + 1) * W + ch];
  const int t0 = chunk_t0[c], n = chunk_n[c];
#pragma unroll 4
  for (int i = 0; i < n; ++i) {
    const float* row = zug + (size_t)(t0 + i) * 3 * W + ch;
    float a, b;
    mingru_coeffs(row[0], row[W], a, b);
    S = a * S + b;
    const float g = row[2 * W];
    out[(size_t)(t0 + i) * W + ch] = from_f32<OT>(S * (g * sigmoid_f(g)));
  }
  if (chunk_last[c]) state[(size_t)slot_ids[seq] * W + ch] = S;
}

__global__ __launch_bounds__(256) void state_snapshot_kernel(const float* __restrict__ state,
                                                             const int* __restrict__ slot_ids,
                                                             float* __restrict__ state_in, int W) {
  const int seq = blockIdx.y;
  const int ch = blockIdx.x * 256 + threadIdx.x;
  if (ch < W) state_in[(size_t)seq * W + ch] = state[(size_t)slot_ids[seq] * W + ch];
}

MF_API int mf_mingru_scan(const float* zug, const int* cu_seqlens, const int* slot_ids, float* state, void* out,
                          int out_is_bf16, int n_seqs, int W, hipStream_t stream) {
  if (n_seqs <= 0 || W <= 0) return 0;
  dim3 grid((W + 255) / 256, n_seqs);
  if (out_is_bf16)
    mingru_scan_kernel<bf16><<<grid, 256, 0, stream>>>(zug, cu_seqlens, slot_ids, state, (bf16*)out, W);
  else
    mingru_scan_kernel<float><<<grid, 256, 0, stream>>>(zug, cu_seqlens, slot_ids, state, (float*)out, W);
  return mf_launch_status();
}

// chunks: int32 [5][n_chunks] = t0, n, seq, first, last; ab: 2 n_chunks W floats; state_in: n_seqs W
MF_API int mf_mingru_scan_chunked(const float* zug, const int* chunks, int n_chunks, const int* slot_ids,
                                  float* state, float* ab, float* state_in, void* out, int out_is_bf16,
                                  int n_seqs, int W, hipStream_t stream) {
  if (n_seqs <= 0 || W <= 0 || n_chunks <= 0) return 0;
  const int* t0 = chunks;
  const int* n = chunks + n_chunks;
  const int* seq = chunks + 2 * (size_t)n_chunks;
  const int* first = chunks + 3 * (size_t)n_chunks;
  const int* last = chunks + 4 * (size_t)n_chunks;
  state_snapshot_kernel<<<dim3((W + 255) / 256, n_seqs), 256, 0, stream>>>(state, slot_ids, state_in, W);
  int rc = mf_launch_status();
  if (rc) return rc;
  dim3 grid((W + 255) / 256, n_chunks);
  mingru_chunk_reduce_kernel<<<grid, 256, 0, stream>>>(zug, t0, n, ab, W);
  rc = mf_launch_status();
  if (rc) return rc;
  if (out_is_bf16)
    mingru_chunk_apply_kernel<bf16><<<grid, 256, 0, stream>>>(zug, t0, n, seq, first, last, ab, state_in, slot_ids,
                                                               state, (bf16*)out, W);
  else
    mingru_chunk_apply_kernel<float><<<grid, 256, 0, stream>>>(zug, t0, n, seq, first, last, ab, state_in, slot_ids,
                                                                state, (float*)out, W);
  return mf_launch_status();
}

MF_API int mf_scan_chunk(void) { return MF_SCAN_CHUNK; }
