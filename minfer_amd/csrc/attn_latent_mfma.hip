// Latent attention on the matrix cores, bfloat16, for prompts and for decode steps alike.
//
// The problem (see attn_latent.hip): rows are (token, head) pairs with queries of DK values against
// the cached rows [c (R) | k_rot] of the token's sequence; the values are the first R columns of
// the same rows.  All heads of a token, and neighbouring tokens of a sequence, read the same rows,
// so a workgroup takes 64 rows = TQ consecutive new tokens x HC heads and every cached row it
// brings in serves all of them.
//
// The library is compiled for one pair of padded sizes (MF_LAT_DKP, MF_LAT_RP: DK and R rounded
// up to multiples of 32), so queries and accumulators live in registers; the host asks for the
// variant a model needs the first time it runs.
//
// A workgroup of 4 waves walks the keys in tiles of 32.  A tile is loaded into registers a tile
// ahead, then written to LDS twice: as it is ([key][d], for q . k) and transposed ([column][key],
// for p . v: the matrix cores want the contracted index contiguous in both operands; the
// transposition is 8 x 8 blocks turned in registers).  Wave (wr, wk) forms the scores of row half
// wr against key half wk as S^T = K Q^T, so that a lane ends up with four keys of one row; the
// two key halves exchange their row maxima through LDS; the probabilities go to LDS in bfloat16;
// wave (wr, wc) then adds P V for row half wr and column half wc as O^T = V^T P^T, where a lane
// again owns one row, so the running maximum, the rescaling and the sum stay in the lane.
// 16x16x32 MFMA throughout; scores, statistics and accumulators 32-bit.
//
// Keys behind a sequence's last position (the rest of its last page) are written to LDS as zeros:
// their probabilities are zero, and zero times whatever a page held before must not be NaN.
#include "common.h"

#ifndef MF_LAT_DKP
#define MF_LAT_DKP 576
#endif
#ifndef MF_LAT_RP
#define MF_LAT_RP 512
#endif

namespace latm {

constexpr int DKP = MF_LAT_DKP, RP = MF_LAT_RP;
constexpr int KS = DKP / 32;          // k steps of a score product
constexpr int CT = RP / 32;           // 16-column tiles of a wave's column half
constexpr int M = 64, TK = 32;        // rows of a workgroup, keys of a tile
constexpr int KSTR = DKP + 8;         // LDS row strides in elements (16 bytes of padding)
constexpr int VSTR = TK + 8;
// a transposed row (one value column, TK keys) starts 16 bytes further for every 8 columns: the 64
// lanes of a staging write hold 64 neighbouring blocks of 8 columns, and without the shift their
// rows, a multiple of 128 bytes apart, would all fall on the same banks
__device__ __forceinline__ int vt_at(int col) { return col * VSTR + (col >> 3) * 8; }
constexpr int PSTR = TK + 8;
constexpr int NB8 = (DKP / 8) * (TK / 8);          // 8 x 8 blocks of a tile
constexpr int ROUNDS = (NB8 + 255) / 256;
constexpr size_t LDS_BYTES = ((size_t)TK * KSTR + (size_t)RP * VSTR + (RP / 8) * 8 + (size_t)M * PSTR) * 2 + (2 * M + M + M) * 4;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

__global__ __launch_bounds__(256) void latent_mfma_kernel(
    const bf16* __restrict__ q_abs, const bf16* __restrict__ cache, const int* __restrict__ page_table, int pt_stride,
    const int* __restrict__ positions, const int* __restrict__ cu_seqlens, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, bf16* __restrict__ out, float* __restrict__ part, int H, int R, int DK, int HC,
    int TQ, float scale, int window, int n_splits, int split_len) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* Kt = reinterpret_cast<bf16*>(smem);                 // [TK][KSTR]
  bf16* Vt = Kt + TK * KSTR;                                // [RP][VSTR]
  bf16* Ps = Vt + RP * VSTR + (RP / 8) * 8;                 // [M][PSTR]
  float* smax = reinterpret_cast<float*>(Ps + M * PSTR);    // [2][M]
  float* ssum = smax + 2 * M;                               // [M]   sums of key half 1, at the end
  float* spare = ssum + M;                                  // [M]

  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wr = w >> 1, wk = w & 1;
  const int r16 = lane & 15, q4 = lane >> 4;

  const int b = tile_seq ? tile_seq[blockIdx.x] : (int)blockIdx.x;
  const int q0 = tile_q0 ? tile_q0[blockIdx.x] : 0;
  const int h0 = blockIdx.y * HC;
  const int hcount = min(HC, H - h0);
  const int split = blockIdx.z;
  const int t_first = cu_seqlens[b] + q0;
  const int n_here = min(TQ, cu_seqlens[b + 1] - t_first);
  const int* pt = page_table + (size_t)b * pt_stride;
  const int first_pos = positions[t_first];
  const int last_pos = first_pos + n_here - 1;              // new tokens of a sequence are consecutive
  const int lo_all = window > 0 ? max(0, first_pos - window + 1) : 0;
  const int j_begin = max(lo_all, split * split_len);
  const int j_end = min(last_pos + 1, (split + 1) * split_len);

  // this lane's two rows (one per row tile), their positions and queries
  int row_pos[2], row_lo[2];
  size_t row_th[2];
  bool row_ok[2];
  bf16x8 qf[2][KS];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int r = 32 * wr + 16 * rt + r16;
    const int tq = r / HC, hh = r % HC;
    row_ok[rt] = tq < n_here && hh < hcount;
    const int t = t_first + (row_ok[rt] ? tq : 0);
    row_pos[rt] = row_ok[rt] ? first_pos + tq : -1;
    row_lo[rt] = window > 0 ? max(0, row_pos[rt] - window + 1) : 0;
    row_th[rt] = (size_t)t * H + h0 + (row_ok[rt] ? hh : 0);
    const bf16* qrow = q_abs + row_th[rt] * DK;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 32 * ks + 8 * q4;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok[rt] && d < DK) v = *reinterpret_cast<const u32x4*>(qrow + d);
      qf[rt][ks] = as_bf16x8(v);
    }
  }

  floatx4 o[2][CT];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int c = 0; c < CT; ++c) o[rt][c] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};

  // a tile ahead, in registers: 8 x 8 blocks (8 keys x 8 columns), block `blk` of a round is
  // column chunk blk % (DKP/8) of key group blk / (DKP/8)
  u32x4 pre[ROUNDS][8];
  auto fetch = [&](int j0) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int blk = rd * 256 + (int)threadIdx.x;
      const int cc = blk % (DKP / 8), kg = blk / (DKP / 8);
      const int jg = j0 + kg * 8;                  // the block's 8 keys lie in one page
      const bool live = blk < NB8 && jg <= last_pos && cc * 8 < DK;
      const bf16* src = cache + ((size_t)(live ? pt[jg / MF_PAGE] : 0) * MF_PAGE + jg % MF_PAGE) * DK + cc * 8;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        u32x4 v = {0u, 0u, 0u, 0u};
        if (live && jg + k <= last_pos) v = *reinterpret_cast<const u32x4*>(src + (size_t)k * DK);
        pre[rd][k] = v;
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int blk = rd * 256 + (int)threadIdx.x;
      if (blk >= NB8) continue;
      const int cc = blk % (DKP / 8), kg = blk / (DKP / 8);
#pragma unroll
      for (int k = 0; k < 8; ++k)
        *reinterpret_cast<u32x4*>(Kt + (size_t)(kg * 8 + k) * KSTR + cc * 8) = pre[rd][k];
      if (cc * 8 < RP) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {           // column c of the block: element c of each of the 8 keys
          u32x4 tv;
#pragma unroll
          for (int j2 = 0; j2 < 4; ++j2) {
            const unsigned a = pre[rd][2 * j2][c >> 1], bb = pre[rd][2 * j2 + 1][c >> 1];
            tv[j2] = (c & 1) ? ((a >> 16) | (bb & 0xffff0000u)) : ((a & 0xffffu) | (bb << 16));
          }
          *reinterpret_cast<u32x4*>(Vt + vt_at(cc * 8 + c) + kg * 8) = tv;
        }
      }
    }
  };

  const int tile0 = j_begin & ~(TK - 1);
  if (tile0 < j_end) fetch(tile0);
  for (int j0 = tile0; j0 < j_end; j0 += TK) {
    __syncthreads();                       // the tile before is no longer read
    stage();
    if (j0 + TK < j_end) fetch(j0 + TK);
    __syncthreads();

    // scores: S^T (keys x rows) for key half wk, row half wr
    floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 kf = as_bf16x8(*reinterpret_cast<const u32x4*>(Kt + (size_t)(16 * wk + r16) * KSTR + 32 * ks + 8 * q4));
      s[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[0][ks], s[0], 0, 0, 0);
      s[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[1][ks], s[1], 0, 0, 0);
    }
    // lane (r16, q4): row 32 wr + 16 rt + r16, keys j0 + 16 wk + 4 q4 + i
    float mloc[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = j0 + 16 * wk + 4 * q4 + i;
        const bool ok = row_ok[rt] && j >= j_begin && j < j_end && j <= row_pos[rt] && j >= row_lo[rt];
        s[rt][i] = ok ? s[rt][i] * scale : -INFINITY;
        mx = fmaxf(mx, s[rt][i]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, MF_WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, MF_WAVE));
      mloc[rt] = mx;
      if (q4 == 0) smax[wk * M + 32 * wr + 16 * rt + r16] = mx;
    }
    __syncthreads();
    float corr[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const int r = 32 * wr + 16 * rt + r16;
      const float m_new = fmaxf(m_run[rt], fmaxf(mloc[rt], smax[(wk ^ 1) * M + r]));
      corr[rt] = (m_new == -INFINITY) ? 1.f : __expf(m_run[rt] - m_new);
      float ps = 0.f;
      bf16x4 pv;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pe = (s[rt][i] == -INFINITY) ? 0.f : __expf(s[rt][i] - m_new);
        ps += pe;
        pv[i] = (bf16)pe;
      }
      ps += __shfl_xor(ps, 16, MF_WAVE);
      ps += __shfl_xor(ps, 32, MF_WAVE);
      l_run[rt] = l_run[rt] * corr[rt] + ps;       // of this wave's key half only; the halves meet at the end
      m_run[rt] = m_new;
      *reinterpret_cast<bf16x4*>(Ps + (size_t)r * PSTR + 16 * wk + 4 * q4) = pv;
    }
    __syncthreads();

    // O^T (columns x rows) += V^T P^T for row half wr, column half wc = wk
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int c = 0; c < CT; ++c) o[rt][c] *= corr[rt];
    bf16x8 pf[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
      pf[rt] = as_bf16x8(*reinterpret_cast<const u32x4*>(Ps + (size_t)(32 * wr + 16 * rt + r16) * PSTR + 8 * q4));
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const int col = wk * (RP / 2) + 16 * c + r16;
      const bf16x8 vf = as_bf16x8(*reinterpret_cast<const u32x4*>(Vt + vt_at(col) + 8 * q4));
      o[0][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[0], o[0][c], 0, 0, 0);
      o[1][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[1], o[1][c], 0, 0, 0);
    }
  }

  // the two key halves' sums meet: wave (wr, 1) hands its sums to (wr, 0) and back
  __syncthreads();
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
    if (q4 == 0) (wk ? ssum : spare)[32 * wr + 16 * rt + r16] = l_run[rt];
  __syncthreads();
  // lane (r16, q4) of wave (wr, wc = wk): row 32 wr + 16 rt + r16, columns wc RP/2 + 16 c + 4 q4 + i
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    if (!row_ok[rt]) continue;
    const int r = 32 * wr + 16 * rt + r16;
    const float L = ssum[r] + spare[r];
    if (n_splits == 1) {
      const float inv = L > 0.f ? 1.0f / L : 0.f;
      bf16* orow = out + row_th[rt] * R;
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const int col = wk * (RP / 2) + 16 * c + 4 * q4;
        if (col < R) {                      // R is a multiple of 8: the four columns go together
          bf16x4 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = (bf16)(o[rt][c][i] * inv);
          *reinterpret_cast<bf16x4*>(orow + col) = v;
        }
      }
    } else {
      float* prow = part + (row_th[rt] * n_splits + split) * (size_t)(R + 2);
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const int col = wk * (RP / 2) + 16 * c + 4 * q4;
        if (col < R) {
#pragma unroll
          for (int i = 0; i < 4; ++i) prow[col + i] = o[rt][c][i];
        }
      }
      if (wk == 0 && q4 == 0) { prow[R] = m_run[rt]; prow[R + 1] = L; }
    }
  }
}

// out[th][e] = sum_s acc_s[e] exp(m_s - M) / sum_s l_s exp(m_s - M), the splits in their order
__global__ __launch_bounds__(256) void latent_mfma_combine_kernel(const float* __restrict__ part,
                                                                  bf16* __restrict__ out, int R, int n_splits) {
  const size_t th = blockIdx.x;
  const float* base = part + th * n_splits * (size_t)(R + 2);
  float Mx = -INFINITY;
  for (int s = 0; s < n_splits; ++s) Mx = fmaxf(Mx, base[(size_t)s * (R + 2) + R]);
  float L = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float ms = base[(size_t)s * (R + 2) + R];
    if (ms != -INFINITY) L += base[(size_t)s * (R + 2) + R + 1] * __expf(ms - Mx);
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  for (int e = threadIdx.x; e < R; e += 256) {
    float a = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float ms = base[(size_t)s * (R + 2) + R];
      if (ms != -INFINITY) a += base[(size_t)s * (R + 2) + e] * __expf(ms - Mx);
    }
    out[th * R + e] = (bf16)(a * inv);
  }
}

}  // namespace latm

MF_API int mf_latent_mfma_sizes(int* dkp, int* rp) {
  *dkp = latm::DKP;
  *rp = latm::RP;
  return 0;
}

// tile_seq / tile_q0: the workgroups' (sequence, first new token) pairs, n_tiles of them; null for
// a step in which every sequence brings one token (tile i is sequence i).
MF_API int mf_latent_mfma(const void* q_abs, const void* cache, const int* page_table, int pt_stride,
                          const int* positions, const int* cu_seqlens, const int* tile_seq, const int* tile_q0,
                          int n_tiles, void* out, float* part, int n_tok, int H, int R, int DK, int HC, int TQ,
                          float scale, int window, int n_splits, int split_len, hipStream_t stream) {
  using namespace latm;
  if (n_tiles <= 0) return 0;
  if (DK > DKP || DK + 31 < DKP || R > RP || R + 31 < RP || R % 8 || DK % 8 || R > DK || HC < 1 || TQ < 1 ||
      HC * TQ > M || n_splits < 1 || split_len < TK || split_len % TK || (n_splits > 1 && !part) ||
      (uintptr_t)q_abs % 16 || (uintptr_t)cache % 16 || (uintptr_t)out % 8)
    return (int)hipErrorInvalidValue;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(latent_mfma_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES);
    if (e != hipSuccess) return (int)e;
    raised = true;
  }
  dim3 grid(n_tiles, (H + HC - 1) / HC, n_splits);
  latent_mfma_kernel<<<grid, 256, LDS_BYTES, stream>>>(
      (const bf16*)q_abs, (const bf16*)cache, page_table, pt_stride, positions, cu_seqlens, tile_seq, tile_q0,
      (bf16*)out, part, H, R, DK, HC, TQ, scale, window, n_splits, split_len);
  int rc = mf_launch_status();
  if (rc == 0 && n_splits > 1) {
    latent_mfma_combine_kernel<<<n_tok * H, 256, 0, stream>>>(part, (bf16*)out, R, n_splits);
    rc = mf_launch_status();
  }
  return rc;
}
