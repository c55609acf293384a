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
// A workgroup of 8 waves walks the keys in tiles of 32 (two tiles ahead of the products, their rows
// are on their way from the cache into registers); waves 2 r and 2 r + 1 own rows 16 r .. 16 r + 15,
// one for each half of the value columns (both form the rows' scores: that is the smaller of the two
// products, and two waves on a SIMD hide each other's waits for LDS and memory).  A tile
// is written to LDS twice: as it is ([key][d], for
// q . k) and transposed ([column][key], for p . v: the matrix cores want the contracted index
// contiguous in both operands; the transposition is 8 x 8 blocks turned in registers).  A wave
// forms its rows' scores against the tile as S^T = K Q^T (two products of 16 keys), so that lane
// (r, q) ends up with keys 4 q .. 4 q + 3 and 16 + 4 q .. 16 + 4 q + 3 of row r: the softmax of a
// row stays inside its wave, and the eight probabilities of a lane are, as they lie, its share of
// the second product's operand, O^T = V^T P^T; the transposed tile keeps its keys in that same
// order (`key_slot`), so a lane's eight values of a column are 16 contiguous bytes.  Nothing but the tile passes through LDS, and a tile costs two barriers.
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
constexpr int CT = RP / 32;           // 16-column tiles of a wave's half of the values
constexpr int NTHR = 512;
constexpr int M = 64, TK = 32;        // rows of a workgroup, keys of a tile
constexpr int KSTR = DKP + 8;         // LDS row strides in elements (16 bytes of padding)
constexpr int VSTR = TK + 8;
// a transposed row (one value column, TK keys) starts 16 bytes further for every 8 columns: the 64
// lanes of a staging write hold 64 neighbouring blocks of 8 columns, and without the shift their
// rows, a multiple of 128 bytes apart, would all fall on the same banks
__device__ __forceinline__ int vt_at(int col) { return col * VSTR + (col >> 3) * 8; }
constexpr int NB8 = (DKP / 8) * (TK / 8);          // 8 x 8 blocks of a tile
constexpr int ROUNDS = (NB8 + NTHR - 1) / NTHR;
constexpr size_t LDS_BYTES = ((size_t)TK * KSTR + (size_t)RP * VSTR + (RP / 8) * 8) * 2;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

__global__ __launch_bounds__(512) void latent_mfma_kernel(
    const bf16* __restrict__ q_abs, const bf16* __restrict__ cache, const int* __restrict__ page_table, int pt_stride,
    const int* __restrict__ positions, const int* __restrict__ cu_seqlens, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, bf16* __restrict__ out, float* __restrict__ part, int H, int R, int DK, int HC,
    int TQ, float scale, int window, int n_splits, int split_len) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* Kt = reinterpret_cast<bf16*>(smem);                 // [TK][KSTR]
  bf16* Vt = Kt + TK * KSTR;                                // [RP][VSTR]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int w = wave >> 1, cw = wave & 1;         // row tile, column half
  const int r16 = lane & 15, q4 = lane >> 4;

  // Without `cu_seqlens` every sequence brings one token (tile i is token i of sequence i): the
  // token's position and its queries are asked for at once.
  const bool single = cu_seqlens == nullptr;
  const int b = tile_seq ? tile_seq[blockIdx.x] : (int)blockIdx.x;
  const int q0 = tile_q0 ? tile_q0[blockIdx.x] : 0;
  const int h0 = blockIdx.y * HC;
  const int hcount = min(HC, H - h0);
  const int split = blockIdx.z;
  const int* pt = page_table + (size_t)b * pt_stride;
  const int early = split * split_len;                      // the split's first key, unless a window cuts it
  const int t_first = single ? b : cu_seqlens[b] + q0;
  const int n_here = single ? 1 : min(TQ, cu_seqlens[b + 1] - t_first);
  const int first_pos = positions[t_first];
  const int last_pos = first_pos + n_here - 1;              // new tokens of a sequence are consecutive
  const int lo_all = window > 0 ? max(0, first_pos - window + 1) : 0;
  const int j_begin = max(lo_all, early);
  const int j_end = min(last_pos + 1, (split + 1) * split_len);

  // this lane's row, its position and query
  const int r = 16 * w + r16;
  const int tq = r / HC, hh = r % HC;
  const bool row_ok = tq < n_here && hh < hcount;
  const int row_pos = row_ok ? first_pos + tq : -1;
  const int row_lo = window > 0 ? max(0, row_pos - window + 1) : 0;
  const size_t row_th = (size_t)(t_first + (row_ok ? tq : 0)) * H + h0 + (row_ok ? hh : 0);
  const bool wave_live = 16 * w < n_here * HC;        // some row of this wave exists
  bf16x8 qf[KS];
  {
    const bf16* qrow = q_abs + row_th * DK;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 32 * ks + 8 * q4;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok && d < DK) v = *reinterpret_cast<const u32x4*>(qrow + d);
      qf[ks] = as_bf16x8(v);
    }
  }
  floatx4 o[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) o[c] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  // two tiles ahead, in registers: 8 x 8 blocks (8 keys x 8 columns), block `blk` of a round is
  // column chunk blk % (DKP/8) of key group blk / (DKP/8).  A tile of 32 keys lies in one page.
  u32x4 pre_a[ROUNDS][8], pre_b[ROUNDS][8];
  auto fetch = [&](u32x4 (&pre)[ROUNDS][8], int j0) {
    const int page = j0 <= last_pos ? pt[j0 / MF_PAGE] : 0;
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int blk = rd * NTHR + (int)threadIdx.x;
      const int cc = blk % (DKP / 8), kg = blk / (DKP / 8);
      const int jg = j0 + kg * 8;
      const bool live = blk < NB8 && jg <= last_pos && cc * 8 < DK;
      const bf16* src = cache + ((size_t)(live ? page : 0) * MF_PAGE + jg % MF_PAGE) * DK + cc * 8;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        u32x4 v = {0u, 0u, 0u, 0u};
        if (live && jg + k <= last_pos) v = *reinterpret_cast<const u32x4*>(src + (size_t)k * DK);
        pre[rd][k] = v;
      }
    }
  };
  auto stage = [&](const u32x4 (&pre)[ROUNDS][8]) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int blk = rd * NTHR + (int)threadIdx.x;
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
          // keys 8 kg .. + 3 and 8 kg + 4 .. + 7 go to the slots of two neighbouring lanes' shares
          typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
          bf16* vrow = Vt + vt_at(cc * 8 + c) + (kg >> 1) * 4 + (kg & 1) * 16;
          *reinterpret_cast<u32x2*>(vrow) = u32x2{tv[0], tv[1]};
          *reinterpret_cast<u32x2*>(vrow + 8) = u32x2{tv[2], tv[3]};
        }
      }
    }
  };

  auto compute = [&](int j0) {
    if (!wave_live) return;              // (uniform over the wave)
    // scores: S^T (keys x rows), keys 0..15 and 16..31 of the tile
    floatx4 s2[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 k0f = as_bf16x8(*reinterpret_cast<const u32x4*>(Kt + (size_t)r16 * KSTR + 32 * ks + 8 * q4));
      const bf16x8 k1f = as_bf16x8(*reinterpret_cast<const u32x4*>(Kt + (size_t)(16 + r16) * KSTR + 32 * ks + 8 * q4));
      s2[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0f, qf[ks], s2[0], 0, 0, 0);
      s2[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1f, qf[ks], s2[1], 0, 0, 0);
    }
    // lane (r16, q4): row 16 w + r16, keys j0 + 16 kt + 4 q4 + i
    float mx = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = j0 + 16 * kt + 4 * q4 + i;
        const bool ok = row_ok && j >= j_begin && j < j_end && j <= row_pos && j >= row_lo;
        s2[kt][i] = ok ? s2[kt][i] * scale : -INFINITY;
        mx = fmaxf(mx, s2[kt][i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, MF_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, MF_WAVE));
    const float m_new = fmaxf(m_run, mx);
    const float corr = (m_new == -INFINITY) ? 1.f : __expf(m_run - m_new);
    float ps = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pe = (s2[kt][i] == -INFINITY) ? 0.f : __expf(s2[kt][i] - m_new);
        ps += pe;
        pf[4 * kt + i] = (bf16)pe;
      }
    ps += __shfl_xor(ps, 16, MF_WAVE);
    ps += __shfl_xor(ps, 32, MF_WAVE);
    l_run = l_run * corr + ps;
    m_run = m_new;
    // O^T (columns x rows) += V^T P^T; the lane's eight keys, 4 q4 .. + 3 and 16 + 4 q4 .. + 3, lie
    // together in the transposed rows.  The accumulators are rescaled only when some row's maximum moved.
    if (__any(corr != 1.f)) {
#pragma unroll
      for (int c = 0; c < CT; ++c) o[c] *= corr;
    }
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const bf16x8 vf = as_bf16x8(*reinterpret_cast<const u32x4*>(Vt + vt_at(cw * (RP / 2) + 16 * c + r16) + 8 * q4));
      o[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[c], 0, 0, 0);
    }
  };

  const int tile0 = j_begin & ~(TK - 1);
  if (tile0 < j_end) fetch(pre_a, tile0);
  if (tile0 + TK < j_end) fetch(pre_b, tile0 + TK);
  for (int j0 = tile0; j0 < j_end; j0 += 2 * TK) {
    __syncthreads();                       // the tile before is no longer read
    stage(pre_a);
    if (j0 + 2 * TK < j_end) fetch(pre_a, j0 + 2 * TK);
    __syncthreads();
    compute(j0);
    if (j0 + TK < j_end) {                 // (uniform over the workgroup)
      __syncthreads();
      stage(pre_b);
      if (j0 + 3 * TK < j_end) fetch(pre_b, j0 + 3 * TK);
      __syncthreads();
      compute(j0 + TK);
    }
  }

  // lane (r16, q4): row 16 w + r16, columns cw RP/2 + 16 c + 4 q4 + i
  if (!row_ok) return;
  if (n_splits == 1) {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    bf16* orow = out + row_th * R;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const int col = cw * (RP / 2) + 16 * c + 4 * q4;
      if (col < R) {                        // R is a multiple of 8: the four columns go together
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (bf16)(o[c][i] * inv);
        *reinterpret_cast<bf16x4*>(orow + col) = v;
      }
    }
  } else {
    float* prow = part + (row_th * n_splits + split) * (size_t)(R + 2);
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const int col = cw * (RP / 2) + 16 * c + 4 * q4;
      if (col < R) {
#pragma unroll
        for (int i = 0; i < 4; ++i) prow[col + i] = o[c][i];
      }
    }
    if (q4 == 0 && cw == 0) { prow[R] = m_run; prow[R + 1] = l_run; }
  }
}

// out[th][e] = sum_s acc_s[e] exp(m_s - M) / sum_s l_s exp(m_s - M), the splits in their order (at
// most 64).  Lane s weighs split s (every wave for itself); a thread then adds its columns' weighted
// sums over the splits that had keys, eight loads in flight.
__global__ __launch_bounds__(256) void latent_mfma_combine_kernel(const float* __restrict__ part,
                                                                  bf16* __restrict__ out, int R, int n_splits) {
  const size_t th = blockIdx.x;
  const float* base = part + th * n_splits * (size_t)(R + 2);
  const int lane = threadIdx.x & 63;
  const float ms = lane < n_splits ? base[(size_t)lane * (R + 2) + R] : -INFINITY;
  const float ls = lane < n_splits ? base[(size_t)lane * (R + 2) + R + 1] : 0.f;
  const float Mx = wave_max(ms);
  const float wv = (ms == -INFINITY) ? 0.f : __expf(ms - Mx);
  const unsigned long long with_keys = __ballot(ms != -INFINITY);
  const int n_used = with_keys ? 64 - __clzll((long long)with_keys) : 0;
  auto of_split = [](float x, int s) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), s)); };
  float L = 0.f;
  for (int s = 0; s < n_used; ++s) L += of_split(ls, s) * of_split(wv, s);
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  for (int e = threadIdx.x; e < R; e += 256) {
    float a = 0.f;
    for (int s0 = 0; s0 < n_used; s0 += 8) {
      float wgt[8], v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        wgt[j] = s0 + j < 64 ? of_split(wv, (s0 + j) & 63) : 0.f;
        v[j] = base[(wgt[j] != 0.f ? (size_t)(s0 + j) * (R + 2) : 0) + e];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) a += (wgt[j] != 0.f ? v[j] : 0.f) * wgt[j];
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

// tile_seq / tile_q0: the workgroups' (sequence, first new token) pairs, n_tiles of them; null, and
// cu_seqlens null as well, for a step in which every sequence brings one token (tile i is sequence i).
MF_API int mf_latent_mfma(const void* q_abs, const void* cache, const int* page_table, int pt_stride,
                          const int* positions, const int* cu_seqlens, const int* tile_seq, const int* tile_q0,
                          int n_tiles, void* out, float* part, int n_tok, int H, int R, int DK, int HC, int TQ,
                          float scale, int window, int n_splits, int split_len, hipStream_t stream) {
  using namespace latm;
  if (n_tiles <= 0) return 0;
  if (DK > DKP || DK + 31 < DKP || R > RP || R + 31 < RP || R % 8 || DK % 8 || R > DK || HC < 1 || TQ < 1 ||
      HC * TQ > M || n_splits < 1 || n_splits > 64 || split_len < TK || split_len % TK || (n_splits > 1 && !part) ||
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
  latent_mfma_kernel<<<grid, NTHR, LDS_BYTES, stream>>>(
      (const bf16*)q_abs, (const bf16*)cache, page_table, pt_stride, positions, cu_seqlens, tile_seq, tile_q0,
      (bf16*)out, part, H, R, DK, HC, TQ, scale, window, n_splits, split_len);
  int rc = mf_launch_status();
  if (rc == 0 && n_splits > 1) {
    latent_mfma_combine_kernel<<<n_tok * H, 256, 0, stream>>>(part, (bf16*)out, R, n_splits);
    rc = mf_launch_status();
  }
  return rc;
}
