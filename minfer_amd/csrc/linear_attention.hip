// Linear attention with a per-head decay over the ragged batch of a step, state in 32-bit per
// sequence slot.
//
// Per head, with q_t, k_t (dim values) and v_t (vdim values) the silu of their projections:
//   S_t = decay S_(t-1) + k_t v_t^T        (dim x vdim),      o_t = S_t^T q_t.
// The heads of a token side by side are then RMS-normed with a gain vector, multiplied by the
// sigmoid of a gate projection and rounded once (`gated_rmsnorm_kernel`).  q | k | v | gate arrive as
// one 32-bit row per token; state, decays, products and sums are 32-bit throughout.
//
// `lightning_scan_kernel`: a workgroup owns (sequence, head, 64 value columns) and walks the
// sequence's new tokens in order; its 256 threads are 4 slices of the key dimension times 64
// columns, a thread keeping its slice of its column of S in registers.  Decode steps and short
// portions use it alone.
//
// Prompts: the tokens of a sequence are cut into chunks of MF_LA_CHUNK.  Unrolling the recurrence
// inside a chunk that starts at token c0 from the state S_in,
//   o_t = decay^(t - c0 + 1) S_in^T q_t + sum_{c0 <= s <= t} decay^(t - s) (q_t . k_s) v_s,
//   S_out = decay^n S_in + sum_s decay^(c0 + n - 1 - s) k_s v_s^T,
// so pass 1 reduces every chunk to its own sum B_c (all chunks side by side), pass 2 folds
// S_in(c + 1) = decay^n S_in(c) + B_c along each sequence, and pass 3 writes every chunk's outputs
// from its S_in and its own tokens (all chunks side by side again).  The order of a position's
// additions depends on where the chunk edges fall inside the step, never on the batch.
#include "common.h"

#define MF_LA_CHUNK 64
#define MF_LA_TT 8     // tokens whose q and k are staged together in the sequential kernel

__device__ __forceinline__ float la_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float la_silu(float x) { return x * la_sigmoid(x); }

// proj row: q [H D] | k [H D] | v [H V] | gate [H V]
template <int DS>      // registers of a thread: its slice of the key dimension (dim <= 4 DS)
__global__ __launch_bounds__(256) void lightning_scan_kernel(const float* __restrict__ proj, int row_len,
                                                             const int* __restrict__ cu_seqlens,
                                                             const int* __restrict__ slot_ids,
                                                             const float* __restrict__ decays,
                                                             float* __restrict__ state, float* __restrict__ out,
                                                             int H, int D, int V) {
  __shared__ float sq[MF_LA_TT][4 * DS], sk[MF_LA_TT][4 * DS];
  __shared__ float partial[MF_LA_TT][4][64];
  const int seq = blockIdx.x, h = blockIdx.y;
  const int col = blockIdx.z * 64 + (threadIdx.x & 63), slice = threadIdx.x >> 6;
  const bool live = col < V;
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
  const float decay = decays[h];
  float* st = state + (((size_t)slot_ids[seq] * H + h) * D) * V + col;
  float S[DS];
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = slice * DS + i;
    S[i] = (live && d < D) ? st[(size_t)d * V] : 0.f;
  }
  const int off_k = H * D, off_v = 2 * H * D;
  for (int tb = t0; tb < t1; tb += MF_LA_TT) {
    const int nt = min(MF_LA_TT, t1 - tb);
    __syncthreads();
    for (int i = threadIdx.x; i < nt * 4 * DS; i += 256) {
      const int tt = i / (4 * DS), d = i % (4 * DS);
      const float* row = proj + (size_t)(tb + tt) * row_len + h * D + d;
      sq[tt][d] = d < D ? la_silu(row[0]) : 0.f;
      sk[tt][d] = d < D ? la_silu(row[off_k]) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = live ? la_silu(proj[(size_t)(tb + tt) * row_len + off_v + h * V + col]) : 0.f;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        const int d = slice * DS + i;
        S[i] = fmaf(decay, S[i], sk[tt][d] * vv);
        o = fmaf(S[i], sq[tt][d], o);
      }
      partial[tt][slice][threadIdx.x & 63] = o;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * 64; i += 256) {
      const int tt = i >> 6, c = i & 63;
      const int cc = blockIdx.z * 64 + c;
      if (cc < V)
        out[(size_t)(tb + tt) * H * V + h * V + cc] =
            ((partial[tt][0][c] + partial[tt][1][c]) + partial[tt][2][c]) + partial[tt][3][c];
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DS; ++i) {
      const int d = slice * DS + i;
      if (d < D) st[(size_t)d * V] = S[i];
    }
  }
}

// ------------------------------------------------------------------ the chunked form
// chunk table: int32 [2][n_chunks] = first token, tokens; then [n_seqs + 1] first chunks of the sequences
//
// The products of the chunked form run on the matrix cores in 32-bit (16x16x4 MFMA with float operands: the
// same multiply-adds as the plain form, no rounding of an operand): a lane gives A[i = lane % 16][k = lane / 16]
// and B[k = lane / 16][j = lane % 16] and holds D[i = 4 (lane / 16) + r][j = lane % 16], r < 4.  Operands are
// staged in LDS with rows 4 floats longer than they are, which spreads a fragment's 64 reads over the banks.
#define MF_LA_VS (64 + 4)     // row stride of tiles of 64 columns

// Staging of a [MF_LA_CHUNK][W] tile of 32-bit rows into LDS, silu applied or not: rows tt >= n and
// columns beyond `valid` are zero.  With `vec` (every row start and `valid` multiples of 4 floats) a thread's
// loads are 16 bytes each and all issued before the first is used.
template <int WP, bool SILU>
__device__ __forceinline__ void stage_tile(float* __restrict__ dst, int dst_stride, const float* __restrict__ src,
                                           size_t src_stride, int n_rows, int n, int valid, bool vec) {
  constexpr int W4 = WP / 4;
  if (vec) {
    for (int base = 0; base < n_rows * W4; base += 256 * 8) {
      float4 tmp[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = base + u * 256 + threadIdx.x;
        const int tt = i / W4, c4 = (i % W4) * 4;
        tmp[u] = (i < n_rows * W4 && tt < n && c4 < valid) ? *(const float4*)(src + (size_t)tt * src_stride + c4)
                                                             : float4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = base + u * 256 + threadIdx.x;
        if (i >= n_rows * W4) continue;
        const int tt = i / W4, c4 = (i % W4) * 4;
        float4 v = tmp[u];
        if (SILU) { v.x = la_silu(v.x); v.y = la_silu(v.y); v.z = la_silu(v.z); v.w = la_silu(v.w); }
        *(float4*)(dst + tt * dst_stride + c4) = v;
      }
    }
  } else {
    for (int i = threadIdx.x; i < n_rows * WP; i += 256) {
      const int tt = i / WP, cc = i % WP;
      const float v = (tt < n && cc < valid) ? src[(size_t)tt * src_stride + cc] : 0.f;
      dst[tt * dst_stride + cc] = SILU ? la_silu(v) : v;
    }
  }
}

// pass 1: B_c[d][v] = sum_s decay^(n - 1 - s) k_s[d] v_s[v] = K'^T V; a workgroup owns (chunk, head, 64
// columns), a wave 16 of the columns.
template <int DS>
__global__ __launch_bounds__(256) void lightning_chunk_sum_kernel(const float* __restrict__ proj, int row_len,
                                                                  const int* __restrict__ chunk_t0,
                                                                  const int* __restrict__ chunk_n,
                                                                  const float* __restrict__ decays,
                                                                  float* __restrict__ bsum, int H, int D, int V) {
  constexpr int DP = 4 * DS, DPS = DP + 4;
  extern __shared__ float lds[];
  float* sk = lds;                          // [CHUNK][DPS]
  float* sv = sk + MF_LA_CHUNK * DPS;       // [CHUNK][VS]
  const int c = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * 64;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t0 = chunk_t0[c], n = chunk_n[c];
  const float decay = decays[h];
  const int off_k = H * D, off_v = 2 * H * D;
  const bool vec = D % 4 == 0 && V % 4 == 0;
  const float* rows = proj + (size_t)t0 * row_len;
  stage_tile<DP, true>(sk, DPS, rows + off_k + h * D, row_len, MF_LA_CHUNK, n, D, vec);
  stage_tile<64, true>(sv, MF_LA_VS, rows + off_v + h * V + v0, row_len, MF_LA_CHUNK, n, min(64, V - v0), vec);
  __shared__ float to_end[MF_LA_CHUNK];          // decay^(n - 1 - s): what a token's k v^T is worth at the chunk's end
  if (threadIdx.x < MF_LA_CHUNK) to_end[threadIdx.x] = threadIdx.x < n ? powf(decay, (float)(n - 1 - threadIdx.x)) : 0.f;
  __syncthreads();
  const int col = lane & 15, g = lane >> 4;
  for (int di = 0; di < DP / 16; ++di) {
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int kk = 0; kk < MF_LA_CHUNK / 4; ++kk) {
      const int srow = 4 * kk + g;
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sk[srow * DPS + 16 * di + col] * to_end[srow], sv[srow * MF_LA_VS + 16 * w + col], acc,
                                                 0, 0, 0);
    }
    const int cc = v0 + 16 * w + col;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int dd = 16 * di + 4 * g + r;
      if (dd < D && cc < V) bsum[(((size_t)c * H + h) * D + dd) * V + cc] = acc[r];
    }
  }
}

// pass 2: along each sequence, S_in(first) = stored state, S_in(c + 1) = decay^n(c) S_in(c) + B_c, the
// last one stored back as the sequence's state.  B_c is replaced by S_in(c) in place.  One thread per
// element of the state; grid (sequence, head, elements / 256).
__global__ __launch_bounds__(256) void lightning_chunk_fold_kernel(const int* __restrict__ chunk_n,
                                                                   const int* __restrict__ seq_first_chunk,
                                                                   const int* __restrict__ slot_ids,
                                                                   const float* __restrict__ decays,
                                                                   float* __restrict__ bsum, float* __restrict__ state,
                                                                   int H, int DV) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= DV) return;
  const int c0 = seq_first_chunk[seq], c1 = seq_first_chunk[seq + 1];
  const float decay = decays[h];
  float* st = state + ((size_t)slot_ids[seq] * H + h) * DV + e;
  float S = *st;
  for (int c = c0; c < c1; ++c) {
    float* b = bsum + ((size_t)c * H + h) * DV + e;
    const float B = *b;
    *b = S;
    S = fmaf(powf(decay, (float)chunk_n[c]), S, B);
  }
  *st = S;
}

// pass 3: the outputs of a chunk from S_in and its own tokens.  A workgroup owns (chunk, head, 64 columns).
// First the decayed scores a[t][s] = decay^(t - s) (q_t . k_s), s <= t, tile by tile (the tiles above the
// diagonal are neither formed nor read), then for every 16 tokens x 16 columns
// o = decay^(t + 1) (Q S_in) + a V: the first product's sums are scaled row by row before the second
// product adds onto them.
template <int DS>
__global__ __launch_bounds__(256) void lightning_chunk_out_kernel(const float* __restrict__ proj, int row_len,
                                                                  const int* __restrict__ chunk_t0,
                                                                  const int* __restrict__ chunk_n,
                                                                  const float* __restrict__ decays,
                                                                  const float* __restrict__ s_in,
                                                                  float* __restrict__ out, int H, int D, int V) {
  constexpr int DP = 4 * DS, DPS = DP + 4;
  extern __shared__ float lds[];
  float* sq = lds;                                   // [CHUNK][DPS]
  float* sk = sq + MF_LA_CHUNK * DPS;                 // [CHUNK][DPS]
  float* sa = sk + MF_LA_CHUNK * DPS;                 // [CHUNK][VS]: decayed scores
  float* sv = sa + MF_LA_CHUNK * MF_LA_VS;            // [CHUNK][VS]
  float* ss = sv + MF_LA_CHUNK * MF_LA_VS;            // [DP][VS]: S_in of this head and these columns
  float* dpow = ss + DP * MF_LA_VS;                   // [CHUNK + 1]: decay^i
  const int c = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * 64;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t0 = chunk_t0[c], n = chunk_n[c];
  const float decay = decays[h];
  const int off_k = H * D, off_v = 2 * H * D;
  const bool vec = D % 4 == 0 && V % 4 == 0;
  const float* rows = proj + (size_t)t0 * row_len;
  stage_tile<DP, true>(sq, DPS, rows + h * D, row_len, MF_LA_CHUNK, n, D, vec);
  stage_tile<DP, true>(sk, DPS, rows + off_k + h * D, row_len, MF_LA_CHUNK, n, D, vec);
  stage_tile<64, true>(sv, MF_LA_VS, rows + off_v + h * V + v0, row_len, MF_LA_CHUNK, n, min(64, V - v0), vec);
  stage_tile<64, false>(ss, MF_LA_VS, s_in + (((size_t)c * H + h) * D) * V + v0, V, DP, D, min(64, V - v0), vec);
  if (threadIdx.x <= MF_LA_CHUNK) dpow[threadIdx.x] = powf(decay, (float)threadIdx.x);
  __syncthreads();
  const int col = lane & 15, g = lane >> 4;
  // the ten score tiles on and below the diagonal, in turn over the waves
  for (int tile = w; tile < 10; tile += 4) {
    int ti = 0, rest = tile;
    while (rest > ti) { rest -= ti + 1; ++ti; }       // tile -> (ti, sj = rest), sj <= ti
    const int sj = rest;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int kk = 0; kk < DP / 4; ++kk)
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sq[(16 * ti + col) * DPS + 4 * kk + g], sk[(16 * sj + col) * DPS + 4 * kk + g],
                                                 acc, 0, 0, 0);
    const int sidx = 16 * sj + col;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int t = 16 * ti + 4 * g + r;
      sa[t * MF_LA_VS + sidx] = sidx <= t ? acc[r] * dpow[t - sidx] : 0.f;
    }
  }
  __syncthreads();
  const int cc = v0 + 16 * w + col;
  for (int ti = 0; ti < MF_LA_CHUNK / 16 && 16 * ti < n; ++ti) {
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int kk = 0; kk < DP / 4; ++kk)
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sq[(16 * ti + col) * DPS + 4 * kk + g], ss[(4 * kk + g) * MF_LA_VS + 16 * w + col],
                                                 acc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] *= dpow[16 * ti + 4 * g + r + 1];
#pragma unroll 4
    for (int kk = 0; kk < 4 * (ti + 1); ++kk)
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sa[(16 * ti + col) * MF_LA_VS + 4 * kk + g], sv[(4 * kk + g) * MF_LA_VS + 16 * w + col],
                                                 acc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int t = 16 * ti + 4 * g + r;
      if (t < n && cc < V) out[(size_t)(t0 + t) * H * V + h * V + cc] = acc[r];
    }
  }
}

// ------------------------------------------------------------------ norm of the heads together, and the gate
// y[t][:] = o[t][:] / sqrt(mean(o[t]^2) + eps) * w * sigmoid(gate[t][:]); gate is a column range of the
// projection row.  One workgroup per token.
template <typename OT>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                                            int gate_stride, const float* __restrict__ w,
                                                            OT* __restrict__ y, int n, float eps) {
  __shared__ float scratch[4];
  const float* row = o + (size_t)blockIdx.x * n;
  const float* g = gate + (size_t)blockIdx.x * gate_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(row[i], row[i], ss);
  ss = block_sum<256>(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += 256)
    y[(size_t)blockIdx.x * n + i] = from_f32<OT>(row[i] * r * w[i] * la_sigmoid(g[i]));
}

// ------------------------------------------------------------------ entry points
#define MF_LA_DISPATCH(CALL)                   \
  if (D <= 32) { CALL(8) }                     \
  else if (D <= 64) { CALL(16) }               \
  else if (D <= 128) { CALL(32) }              \
  else { CALL(64) }

MF_API int mf_la_chunk(void) { return MF_LA_CHUNK; }

// proj float32 [tokens][2 H D + 2 H V]; state float32 [slots][H][D][V]; out float32 [tokens][H V]
MF_API int mf_lightning_scan(const float* proj, const int* cu_seqlens, const int* slot_ids, const float* decays,
                             float* state, float* out, int n_seqs, int H, int D, int V, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (H <= 0 || D <= 0 || V <= 0 || D > 256) return (int)hipErrorInvalidValue;
  const int row_len = 2 * H * D + 2 * H * V;
  dim3 grid(n_seqs, H, (V + 63) / 64);
#define MF_CALL(DS) lightning_scan_kernel<DS><<<grid, 256, 0, stream>>>(proj, row_len, cu_seqlens, slot_ids, decays, state, out, H, D, V);
  MF_LA_DISPATCH(MF_CALL)
#undef MF_CALL
  return mf_launch_status();
}

// chunks int32 [5][n_chunks]; seq_first_chunk int32 [n_seqs + 1]; bsum float32 [n_chunks][H][D][V] scratch
MF_API int mf_lightning_scan_chunked(const float* proj, const int* chunks, int n_chunks, const int* seq_first_chunk,
                                     const int* slot_ids, const float* decays, float* state, float* bsum, float* out,
                                     int n_seqs, int H, int D, int V, hipStream_t stream) {
  if (n_seqs <= 0 || n_chunks <= 0) return 0;
  if (H <= 0 || D <= 0 || V <= 0 || D > 128 || !bsum) return (int)hipErrorInvalidValue;
  const int row_len = 2 * H * D + 2 * H * V;
  const int* t0 = chunks;
  const int* n = chunks + n_chunks;
  dim3 grid(n_chunks, H, (V + 63) / 64);
  int rc = 0;
#define MF_CALL(DS)                                                                                                   \
  {                                                                                                                   \
    const size_t lds = sizeof(float) * (MF_LA_CHUNK * (4 * DS + 4) + MF_LA_CHUNK * MF_LA_VS);                         \
    static bool raised = false;                                                                                       \
    if (!raised && lds > 48 * 1024) {                                                                                 \
      rc = (int)hipFuncSetAttribute((const void*)lightning_chunk_sum_kernel<DS>,                                      \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                            \
      if (rc) return rc;                                                                                              \
      raised = true;                                                                                                  \
    }                                                                                                                 \
    lightning_chunk_sum_kernel<DS><<<grid, 256, lds, stream>>>(proj, row_len, t0, n, decays, bsum, H, D, V);          \
  }
  MF_LA_DISPATCH(MF_CALL)
#undef MF_CALL
  rc = mf_launch_status();
  if (rc) return rc;
  lightning_chunk_fold_kernel<<<dim3(n_seqs, H, (D * V + 255) / 256), 256, 0, stream>>>(n, seq_first_chunk, slot_ids, decays,
                                                                                        bsum, state, H, D * V);
  rc = mf_launch_status();
  if (rc) return rc;
#define MF_CALL(DS)                                                                                                   \
  {                                                                                                                   \
    const size_t lds = sizeof(float) * (2 * MF_LA_CHUNK * (4 * DS + 4) + 2 * MF_LA_CHUNK * MF_LA_VS +                 \
                                        4 * DS * MF_LA_VS + MF_LA_CHUNK + 1);                                         \
    static bool raised = false;                                                                                       \
    if (!raised && lds > 48 * 1024) {                                                                                 \
      rc = (int)hipFuncSetAttribute((const void*)lightning_chunk_out_kernel<DS>,                                      \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                            \
      if (rc) return rc;                                                                                              \
      raised = true;                                                                                                  \
    }                                                                                                                 \
    lightning_chunk_out_kernel<DS><<<grid, 256, lds, stream>>>(proj, row_len, t0, n, decays, bsum, out, H, D, V);     \
  }
  MF_LA_DISPATCH(MF_CALL)
#undef MF_CALL
  return mf_launch_status();
}

MF_API int mf_gated_rmsnorm(const float* o, const float* gate, int gate_stride, const float* w, void* y, int y_is_bf16,
                            int rows, int n, float eps, hipStream_t stream) {
  if (rows <= 0 || n <= 0) return 0;
  if (y_is_bf16)
    gated_rmsnorm_kernel<bf16><<<rows, 256, 0, stream>>>(o, gate, gate_stride, w, (bf16*)y, n, eps);
  else
    gated_rmsnorm_kernel<float><<<rows, 256, 0, stream>>>(o, gate, gate_stride, w, (float*)y, n, eps);
  return mf_launch_status();
}
