// Local (chunked / windowed) paged attention for prompt pieces on the MFMA
// matrix cores: bf16 activations, page size 32, flash-style online softmax.
//
// Same geometry as the dense model's prefill kernel (one workgroup per tile
// of 32 query rows and kv head, one wave per query head of the group, scores
// = mfma(A = K page, B = Q), softmax in fp32 lane pairs, O += mfma(A = P,
// B = V^T staged transposed in LDS) with mfma_f32_32x32x16_bf16), extended by
//   - separate key and value sizes (dk <= DKP, dv <= DVP, zero padded in LDS),
//   - a per-row lower key bound lo(p) = max(chunk ? p/chunk*chunk : 0,
//     window ? p - window + 1 : 0): pages wholly below the bound of the
//     tile's first row are never read; masked scores contribute exactly 0,
//   - an optional per-head distance bias r1 * ln(1 + r2 * (p - j)) taken off
//     the scaled score,
//   - score scale from the caller, per-head sigmoid output gate and output
//     scale in the epilogue, output written into a column section of the
//     merged output-projection input.
//
// Fragment layouts (gfx950 v_mfma_f32_32x32x16_bf16):
//   A[32,16]: lane l holds A[l%32][(l/32)*8 + j], j = 0..7
//   B[16,32]: lane l holds B[(l/32)*8 + j][l%32]
//   C/D     : lane l holds D[(r&3) + 8*(r>>2) + 4*(l/32)][l%32], r = 0..15
#include "mix_common.h"

#define PG 32        // page size (keys per tile)
#define QT 32        // query rows per tile
#define VPAD 40      // padded row length of the transposed V tile and of P

typedef s16x8 bfrag;

__device__ __forceinline__ f32x16 mfma32(bfrag a, bfrag b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ int drow(int r, int hi) {
  return (r & 3) + 8 * (r >> 2) + 4 * hi;
}
// XOR swizzle of a [32][DKP] bf16 tile: 16-byte chunk index ^= row bits
template <int DKP>
__device__ __forceinline__ int kswz(int row, int byte_in_row) {
  constexpr int mask = DKP / 8 - 1;  // chunks per row - 1 (DKP power of two)
  return row * (2 * DKP) + (byte_in_row ^ ((row & mask & 15) << 4));
}

// Wide tiles (DKP + DVP > 256) keep 128 accumulator and 64 query registers a
// lane: they run with at most 4 waves a workgroup so that a wave may use the
// whole register file of its SIMD.
template <int DKP, int DVP>
__global__ void __launch_bounds__(DKP + DVP > 256 ? 256 : 1024)
local_attention_mfma_kernel(
    u16* __restrict__ out, long ldo, int out_off, const u16* __restrict__ q,
    const u16* __restrict__ k_cache, const u16* __restrict__ v_cache,
    const int* __restrict__ bt, int bt_stride, const int* __restrict__ seq_lens,
    const int* __restrict__ qlocs, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, float scale, int chunk, int window,
    const u16* __restrict__ proj, long ld, int gate_off, float out_scale,
    const float* __restrict__ bias_r1, const float* __restrict__ bias_r2,
    int sink, int keep_first, int H, int Hk, int dk, int dv, int parts) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int w = threadIdx.x / WAVE;
  const int G = blockDim.x / WAVE;        // query heads of this workgroup
  // the query heads of one kv head are spread over `parts` workgroups
  const int kh = blockIdx.y / parts;
  const int hq = (kh * parts + blockIdx.y % parts) * G + w;
  const int s = tile_seq[blockIdx.x];
  const int q0 = tile_q0[blockIdx.x];
  const int row_base = qlocs[s] + q0;
  const int nq_total = qlocs[s + 1] - qlocs[s];
  const int nq = min(QT, nq_total - q0);
  const int L = seq_lens[s];
  const int p0 = L - nq_total + q0;       // position of the tile's first row
  const int kv_end = p0 + nq;             // causal bound (exclusive)

  extern __shared__ __attribute__((aligned(16))) char smem[];
  u16* ktile = (u16*)smem;                          // [PG][DKP] swizzled
  u16* vt = ktile + PG * DKP;                       // [DVP][VPAD]
  u16* p_lds = vt + DVP * VPAD + (long)w * QT * VPAD;
  float* stat = (float*)(vt + DVP * VPAD + (long)G * QT * VPAD) + w * 2 * QT;
  float* alpha_lds = stat;                          // [32]
  float* fin_lds = stat + QT;                       // [32]

  const int my_q = lane & 31;
  const int hi = lane >> 5;
  const int my_p = p0 + my_q;             // position of this lane's query row
  int lo_row = 0;
  if (chunk > 0) lo_row = (my_p / chunk) * chunk;
  const int clo_row = lo_row;             // kept first keys: [clo_row, keep_first)
  if (window > 0) lo_row = max(lo_row, my_p - window + 1);
  int lo_tile = 0;                        // bound of the tile's first row
  if (chunk > 0) lo_tile = (p0 / chunk) * chunk;
  const int clo_tile = lo_tile;
  if (window > 0) lo_tile = max(lo_tile, p0 - window + 1);

  bfrag qb[DKP / 16];
  {
    const int qrow = row_base + (my_q < nq ? my_q : 0);
    const u16* qp = q + ((long)qrow * H + hq) * dk;
#pragma unroll
    for (int kk = 0; kk < DKP / 16; ++kk) {
      const int c = kk * 16 + hi * 8;
      qb[kk] = c < dk ? *(const s16x8*)(qp + c) : (s16x8)(0);
    }
  }
  f32x16 acc[DVP / 32];
#pragma unroll
  for (int b = 0; b < DVP / 32; ++b) acc[b] = (f32x16)(0.f);
  // a sink (a key of score 0 without a value) starts the running maximum at
  // 0 and the running sum at its weight
  float m_run = sink ? 0.f : -1e30f, l_run = sink ? 1.f : 0.f;
  // distance bias of this wave's head: r1 * ln(1 + r2 * (p - j))
  const float r1 = bias_r1 ? bias_r1[hq] : 0.f;
  const float r2 = bias_r1 ? bias_r2[hq] : 0.f;

  const int kt0 = lo_tile / PG, kt1 = (kv_end + PG - 1) / PG;
  // pages of kept first keys that lie wholly before the window's pages
  const int kf0 = clo_tile / PG;
  const int n_kept = max(min(kt0, (keep_first + PG - 1) / PG) - kf0, 0);
  for (int it = 0; it < n_kept + kt1 - kt0; ++it) {
    const int kt = it < n_kept ? kf0 + it : kt0 + (it - n_kept);
    const int blk = bt[(long)s * bt_stride + kt];
    const u16* kp = k_cache + (((long)blk * Hk + kh) * PG) * dk;
    const u16* vp = v_cache + (((long)blk * Hk + kh) * PG) * dv;
    const int kv0 = kt * PG;
    {
      const int tid = threadIdx.x, nthr = blockDim.x;
      constexpr int KS = DKP / 8, VS = DVP / 8;
      for (int it = tid; it < PG * KS; it += nthr) {
        const int row = it / KS, slot = it % KS;
        u16x8 kx = (u16x8)(0);
        if (slot * 8 < dk) kx = *(const u16x8*)(kp + row * dk + slot * 8);
        *(u16x8*)((char*)ktile + kswz<DKP>(row, slot * 16)) = kx;
      }
      for (int it = tid; it < PG * VS; it += nthr) {
        const int kv = it % PG, d0 = (it / PG) * 8;
        u16x8 vx = (u16x8)(0);
        if (d0 < dv) vx = *(const u16x8*)(vp + kv * dv + d0);
#pragma unroll
        for (int j = 0; j < 8; ++j) vt[(d0 + j) * VPAD + kv] = vx[j];
      }
    }
    __syncthreads();

    f32x16 d1 = (f32x16)(0.f);
#pragma unroll
    for (int kk = 0; kk < DKP / 16; ++kk) {
      bfrag ka = *(const s16x8*)((char*)ktile +
                                 kswz<DKP>(lane & 31, (kk * 16 + hi * 8) * 2));
      d1 = mfma32(ka, qb[kk], d1);
    }

    float sc[16];
    bool vis[16];
    float tmax = -1e30f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kvpos = kv0 + drow(r, hi);
      vis[r] = kvpos <= my_p &&
               (kvpos >= lo_row || (kvpos < keep_first && kvpos >= clo_row));
      float sv = d1[r] * scale;
      if (bias_r1) sv -= r1 * logf(1.f + r2 * (float)max(my_p - kvpos, 0));
      sc[r] = vis[r] ? sv : -1e30f;
      tmax = fmaxf(tmax, sc[r]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);
    const float alpha = __expf(m_run - m_new);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float p = vis[r] ? __expf(sc[r] - m_new) : 0.f;
      sc[r] = p;
      psum += p;
    }
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      p_lds[my_q * VPAD + drow(r, hi)] = f2bf(sc[r]);
    if (hi == 0) alpha_lds[my_q] = alpha;

    float al[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) al[r] = alpha_lds[drow(r, hi)];
#pragma unroll
    for (int b = 0; b < DVP / 32; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[b][r] *= al[r];

    bfrag pa[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
      pa[kk] = *(const s16x8*)(p_lds + (lane & 31) * VPAD + kk * 16 + hi * 8);
#pragma unroll
    for (int b = 0; b < DVP / 32; ++b) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        bfrag vb = *(const s16x8*)(vt + (b * 32 + (lane & 31)) * VPAD +
                                   kk * 16 + hi * 8);
        acc[b] = mfma32(pa[kk], vb, acc[b]);
      }
    }
    __syncthreads();
  }

  // epilogue: out = acc / l * out_scale * sigmoid(gate logit of (row, head))
  if (hi == 0) {
    float f = l_run > 0.f ? out_scale / l_run : 0.f;
    if (gate_off >= 0 && my_q < nq)
      f *= sigmoid_f(bf2f(proj[(long)(row_base + my_q) * ld + gate_off + hq]));
    fin_lds[my_q] = f;
  }
  float fin[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) fin[r] = fin_lds[drow(r, hi)];
  const int dcol = lane & 31;
#pragma unroll
  for (int b = 0; b < DVP / 32; ++b) {
    const int col = b * 32 + dcol;
    if (col < dv) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int qrow = drow(r, hi);
        if (qrow < nq)
          out[(long)(row_base + qrow) * ldo + out_off + (long)hq * dv + col] =
              f2bf(acc[b][r] * fin[r]);
      }
    }
  }
}

// returns 0 when the shape is not covered (caller uses the generic kernel)
extern "C" int mix_local_attention_mfma(
    void* out, long ldo, int out_off, const void* q, const void* k_cache,
    const void* v_cache, const int* bt, int bt_stride, const int* seq_lens,
    const int* qlocs, const int* tile_seq, const int* tile_q0, int n_tiles,
    float scale, int chunk, int window, const void* proj, long ld,
    int gate_off, float out_scale, const float* bias_r1, const float* bias_r2,
    int sink, int keep_first, int H, int Hk, int dk, int dv, int page,
    hipStream_t s) {
  if (page != PG || dk % 8 || dv % 8 || dk > 256 || dv > 256 || H % Hk)
    return 0;
  const int DKP = dk <= 64 ? 64 : (dk <= 128 ? 128 : 256);
  const int DVP = dv <= 64 ? 64 : (dv <= 128 ? 128 : 256);
  // one wave a query head; many query heads on one kv head (one shared
  // latent, say) are split over several workgroups so that the tiles fit LDS
  int G = H / Hk, parts = 1;
  size_t smem = 0;
  for (;; ++parts) {
    if (parts > H / Hk) return 0;
    if ((H / Hk) % parts) continue;
    G = H / Hk / parts;
    smem = (size_t)PG * DKP * 2 + (size_t)DVP * VPAD * 2 +
           (size_t)G * QT * VPAD * 2 + (size_t)G * 2 * QT * 4;
    if (G <= (DKP + DVP > 256 ? 4 : 8) && smem <= 64 * 1024) break;
  }
  if (n_tiles == 0) return 1;
#define LAUNCH_M(KP, VP)                                                      \
  hipLaunchKernelGGL((local_attention_mfma_kernel<KP, VP>),                   \
                     dim3(n_tiles, Hk * parts), dim3(G * WAVE), smem, s,      \
                     (u16*)out,                                               \
                     ldo, out_off, (const u16*)q, (const u16*)k_cache,        \
                     (const u16*)v_cache, bt, bt_stride, seq_lens, qlocs,     \
                     tile_seq, tile_q0, scale, chunk, window,                 \
                     (const u16*)proj, ld, gate_off, out_scale, bias_r1,     \
                     bias_r2, sink, keep_first, H, Hk, dk, dv, parts)
  if (DKP == 64) {
    if (DVP == 64) LAUNCH_M(64, 64);
    else if (DVP == 128) LAUNCH_M(64, 128);
    else LAUNCH_M(64, 256);
  } else if (DKP == 128) {
    if (DVP == 64) LAUNCH_M(128, 64);
    else if (DVP == 128) LAUNCH_M(128, 128);
    else LAUNCH_M(128, 256);
  } else {
    if (DVP == 64) LAUNCH_M(256, 64);
    else if (DVP == 128) LAUNCH_M(256, 128);
    else LAUNCH_M(256, 256);
  }
#undef LAUNCH_M
  return 1;
}
