// Local (chunked / windowed) paged attention with split key and value sizes.
//
//   attn_prep        per-head RMS norm of q and k, rotation of a prefix of
//                    each head (rotate-half pairing; cos and sin of the fp32
//                    angle position * inv_freq[i] come in a [T, 2*half] table
//                    made once per step), K/V scatter into the paged caches,
//                    q out.
//   local_attention  softmax attention of every new token over the cached
//                    keys its mask lets it see, times a per-head sigmoid gate;
//                    optionally r1[h] * ln(1 + r2[h] * distance) is taken off
//                    every score (per-head logarithmic distance bias).
//
// Cache layout per layer: K [blocks, G, page, dk], V [blocks, G, page, dv].
// Mask of a query at position p: keys j in [lo, p],
//   lo = max(chunk ? (p / chunk) * chunk : 0, window ? p - window + 1 : 0).
// Positions count from the start of the sequence, so a chunk edge does not
// move when a prompt is processed in pieces.
//
// attn_prep and the general local_attention kernel use one wave per (token,
// head); shapes made of 16-byte vectors take the row-split kernel further
// down. All math fp32.
#include "mix_common.h"

#define WPB 4  // waves per block

#define UPW 4   // (token, head) units per wave
#define DPL 4   // elements per lane and unit (head sizes up to 64 * DPL)

// A wave handles UPW consecutive units (a unit = one q, k or v head of one
// token): the global loads of all its units are issued before any of them is
// reduced, so their latencies overlap. The normalised head passes through a
// wave-private LDS row to bring rotation partners (i, i + half) together;
// LDS operations of one wave execute in order, so no barrier is needed.
template <typename A>
__global__ void attn_prep_kernel(
    A* __restrict__ q_out, const A* __restrict__ proj, long ld, int q_off,
    int k_off, int v_off, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps,
    const float* __restrict__ cos_sin, int half,
    const long* __restrict__ slots, A* __restrict__ k_cache,
    A* __restrict__ v_cache, const A* __restrict__ vfirst, long ldvf,
    const float* __restrict__ vlam, long T, int H, int G, int dk, int dv,
    int page) {
  extern __shared__ float sm[];  // WPB * dmax floats
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int dmax = dk > dv ? dk : dv;
  float* buf = sm + wid * dmax;
  const int units = H + 2 * G;
  const long total = T * units;
  const long u0 = ((long)blockIdx.x * WPB + wid) * UPW;

  float x[UPW][DPL];
#pragma unroll
  for (int n = 0; n < UPW; ++n) {
    const long u = u0 + n;
    const long t = u < total ? u / units : 0;
    const int j = u < total ? (int)(u - t * units) : 0;
    const int kind = j < H ? 0 : (j < H + G ? 1 : 2);
    const int head = kind == 0 ? j : (kind == 1 ? j - H : j - H - G);
    const int d = kind == 2 ? dv : dk;
    const A* src = proj + t * ld +
                   (kind == 0 ? q_off : (kind == 1 ? k_off : v_off)) +
                   (long)head * d;
#pragma unroll
    for (int k = 0; k < DPL; ++k) {
      const int i = lane + k * (int)WAVE;
      x[n][k] = i < d ? ldf<A>(src + i) : 0.f;
    }
    if (vfirst && kind == 2) {
      // cached value = (1 - lambda) v + lambda * (another layer's value)
      const float lam = vlam[0];
      const A* vf = vfirst + t * ldvf + (long)head * d;
#pragma unroll
      for (int k = 0; k < DPL; ++k) {
        const int i = lane + k * (int)WAVE;
        if (i < d) x[n][k] = (1.f - lam) * x[n][k] + lam * ldf<A>(vf + i);
      }
    }
  }
#pragma unroll
  for (int n = 0; n < UPW; ++n) {
    const long u = u0 + n;
    if (u >= total) break;  // wave-uniform
    const long t = u / units;
    const int j = (int)(u - t * units);
    const int kind = j < H ? 0 : (j < H + G ? 1 : 2);
    const int head = kind == 0 ? j : (kind == 1 ? j - H : j - H - G);
    const int d = kind == 2 ? dv : dk;
    const float* w = kind == 0 ? q_w : (kind == 1 ? k_w : nullptr);
    float ssq = 0.f;
#pragma unroll
    for (int k = 0; k < DPL; ++k) ssq += x[n][k] * x[n][k];
    ssq = wave_sum_f32(ssq);
    const float inv = w ? 1.f / sqrtf(ssq / (float)d + eps) : 1.f;
#pragma unroll
    for (int k = 0; k < DPL; ++k) {
      const int i = lane + k * (int)WAVE;
      if (i < d) {
        x[n][k] *= inv * (w ? w[i] : 1.f);
        buf[i] = x[n][k];
      }
    }
    __builtin_amdgcn_wave_barrier();
    const int hf = kind == 2 ? 0 : half;
    const float* cs = cos_sin + t * 2L * half;  // row t: cos[half] | sin[half]
    A* dst;
    if (kind == 0) {
      dst = q_out + (t * H + head) * (long)dk;
    } else {
      const long slot = slots[t];
      const long blk = slot / page, off = slot - blk * page;
      dst = (kind == 1 ? k_cache : v_cache) +
            ((blk * G + head) * page + off) * (long)d;
    }
#pragma unroll
    for (int k = 0; k < DPL; ++k) {
      const int i = lane + k * (int)WAVE;
      if (i >= d) continue;
      float v = x[n][k];
      if (i < 2 * hf) {
        const int fi = i < hf ? i : i - hf;
        const float y = buf[i < hf ? i + hf : i - hf];
        const float c = cs[fi], sn = cs[half + fi];
        v = i < hf ? v * c - y * sn : v * c + y * sn;
      }
      stf<A>(dst + i, v);
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// bf16 fast path of attn_prep: a group of GS lanes owns one unit, lane gl its
// 8-element chunk gl (one 16-byte load and store a lane). The norm reduces
// over the group by xor-shuffles; the rotation partner chunk (gl +- half/8)
// arrives by lane shuffles. Needs dk, dv, half and all offsets to be multiples
// of 8; other shapes and fp32 take the generic kernel above.
template <int GS>
__global__ void attn_prep_vec_kernel(
    u16* __restrict__ q_out, const u16* __restrict__ proj, long ld, int q_off,
    int k_off, int v_off, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps,
    const float* __restrict__ cos_sin, int half,
    const long* __restrict__ slots, u16* __restrict__ k_cache,
    u16* __restrict__ v_cache, const u16* __restrict__ vfirst, long ldvf,
    const float* __restrict__ vlam, long T, int H, int G, int dk, int dv,
    int page) {
  constexpr int UPWV = 64 / GS;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int gi = lane / GS, gl = lane % GS;
  const int units = H + 2 * G;
  const long total = T * units;
  const long u = ((long)blockIdx.x * WPB + wid) * UPWV + gi;
  const bool valid = u < total;
  const long t = valid ? u / units : 0;
  const int j = valid ? (int)(u - t * units) : 0;
  const int kind = j < H ? 0 : (j < H + G ? 1 : 2);
  const int head = kind == 0 ? j : (kind == 1 ? j - H : j - H - G);
  const int d = kind == 2 ? dv : dk;
  const int c0 = gl * 8;
  const bool act = valid && c0 < d;
  const u16* src = proj + t * ld +
                   (kind == 0 ? q_off : (kind == 1 ? k_off : v_off)) +
                   (long)head * d + c0;
  float x[8];
  {
    u16x8 raw = (u16x8)(0);
    if (act) raw = *(const u16x8*)src;
    bf8_to_f32(raw, x);
    if (vfirst && kind == 2 && act) {
      const float lam = vlam[0];
      float y[8];
      bf8_to_f32(*(const u16x8*)(vfirst + t * ldvf + (long)head * d + c0), y);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = (1.f - lam) * x[e] + lam * y[e];
    }
  }
  float ssq = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ssq += x[e] * x[e];
#pragma unroll
  for (int off = GS / 2; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, WAVE);
  const float* w = kind == 0 ? q_w : (kind == 1 ? k_w : nullptr);
  if (w && act) {
    const float inv = 1.f / sqrtf(ssq / (float)d + eps);
    const f32x4 w0 = *(const f32x4*)(w + c0), w1 = *(const f32x4*)(w + c0 + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      x[e] *= inv * w0[e];
      x[e + 4] *= inv * w1[e];
    }
  }
  const int hc = half / 8;  // chunks in half of the rotated prefix
  if (hc > 0) {             // uniform: every lane takes part in the shuffles
    const bool rot = kind != 2 && c0 < 2 * half;
    const bool first = c0 < half;
    const int partner = rot ? (first ? lane + hc : lane - hc) : lane;
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = __shfl(x[e], partner, WAVE);
    if (rot && act) {
      const float* cs = cos_sin + t * 2L * half + (first ? c0 : c0 - half);
      const f32x4 ca = *(const f32x4*)cs, cb = *(const f32x4*)(cs + 4);
      const f32x4 sa = *(const f32x4*)(cs + half),
                  sb = *(const f32x4*)(cs + half + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float c = e < 4 ? ca[e & 3] : cb[e & 3];
        const float sn = e < 4 ? sa[e & 3] : sb[e & 3];
        x[e] = first ? x[e] * c - y[e] * sn : x[e] * c + y[e] * sn;
      }
    }
  }
  if (!act) return;
  u16* dst;
  if (kind == 0) {
    dst = q_out + (t * H + head) * (long)dk + c0;
  } else {
    const long slot = slots[t];
    const long blk = slot / page, off = slot - blk * page;
    dst = (kind == 1 ? k_cache : v_cache) +
          ((blk * G + head) * page + off) * (long)d + c0;
  }
  u16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = f2bf(x[e]);
  *(u16x8*)dst = o;
}

// NV = value columns per lane (dv <= 64 * NV)
template <typename A, int NV>
__global__ void local_attention_kernel(
    A* __restrict__ out, long ldo, int out_off, const A* __restrict__ q,
    const A* __restrict__ k_cache, const A* __restrict__ v_cache,
    const int* __restrict__ bt, int bt_stride, const int* __restrict__ seq_lens,
    const int* __restrict__ qlocs, const int* __restrict__ token_seq,
    float scale, int chunk, int window, const A* __restrict__ proj, long ld,
    int gate_off, float out_scale, const float* __restrict__ bias_r1,
    const float* __restrict__ bias_r2, int sink, int keep_first, long t0, long T, int H, int G,
    int dk, int dv, int page) {
  extern __shared__ float sm[];  // WPB * dk floats: the wave's query
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  float* qs = sm + wid * dk;
  const long u = (long)blockIdx.x * WPB + wid;
  const bool valid = u < T * H;
  const long t = t0 + (valid ? u / H : 0);  // rows [t0, t0 + T)
  const int h = valid ? (int)(u % H) : 0;
  const int g = h / (H / G);
  for (int i = lane; i < dk; i += WAVE)
    qs[i] = ldf<A>(q + (t * H + h) * (long)dk + i);
  __syncthreads();
  if (!valid) return;

  const int s = token_seq[t];
  const int p = seq_lens[s] - (qlocs[s + 1] - (int)t);  // position of token t
  int lo = 0;
  if (chunk > 0) lo = (p / chunk) * chunk;
  const int clo = lo;
  if (window > 0 && p - window + 1 > lo) lo = p - window + 1;
  // kept first keys [clo, min(keep_first, lo)) come before the window: the
  // loop runs over virtual indices vlo..p, the first nk of which are kept keys
  const int nk = max(min(keep_first, lo) - clo, 0);
  const int vlo = lo - nk;
  const int* table = bt + (long)s * bt_stride;
  // distance bias: r1 * ln(1 + r2 * (p - j)) is taken off the score
  const float r1 = bias_r1 ? bias_r1[h] : 0.f;
  const float r2 = bias_r1 ? bias_r2[h] : 0.f;

  // a sink is a key of score 0 without a value that is always visible
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) acc[c] = 0.f;

  for (int base = vlo; base <= p; base += WAVE) {
    const int jv = base + lane;
    const bool live = jv <= p;
    const int j = jv - vlo < nk ? clo + (jv - vlo) : jv;
    int row = 0;  // blk * page + offset of key j
    float sc = -INFINITY;
    if (live) {
      row = table[j / page] * page + j % page;
      const long blk = row / page, off = row - blk * page;
      const A* kr = k_cache + ((blk * G + g) * page + off) * (long)dk;
      float dot = 0.f;
      for (int i = 0; i < dk; ++i) dot += qs[i] * ldf<A>(kr + i);
      sc = dot * scale;
      if (bias_r1) sc -= r1 * logf(1.f + r2 * (float)(p - j));
    }
    const float m_new = fmaxf(m, wave_max_f32(sc));
    const float pj = live ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf on the first tile -> 0
    l = l * corr + wave_sum_f32(pj);
#pragma unroll
    for (int c = 0; c < NV; ++c) acc[c] *= corr;
    m = m_new;
    const int n = (p - base + 1) < (int)WAVE ? (p - base + 1) : (int)WAVE;
    for (int jj = 0; jj < n; ++jj) {
      const float pw = __shfl(pj, jj, WAVE);
      const int r = __shfl(row, jj, WAVE);
      const long blk = r / page, off = r - blk * page;
      const A* vr = v_cache + ((blk * G + g) * page + off) * (long)dv;
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        const int col = lane + c * (int)WAVE;
        if (col < dv) acc[c] += pw * ldf<A>(vr + col);
      }
    }
  }
  float gate = out_scale;
  if (gate_off >= 0) gate *= sigmoid_f(ldf<A>(proj + t * ld + gate_off + h));
  const float f = gate / l;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int col = lane + c * (int)WAVE;
    if (col < dv)
      stf<A>(out + t * ldo + out_off + (long)h * dv + col, acc[c] * f);
  }
}


// ---- row-split kernel ------------------------------------------------------
// One 4-wave block per (token, head); the visible keys are cut into tiles that
// the waves take in turn, and the four partial (max, sum, accumulator)
// triples meet in LDS. Inside a wave, LPR adjacent lanes own one cached row
// (16 bytes a lane: 8 bf16 or 4 fp32), so one load instruction fetches whole
// rows of 64 / LPR keys, fully coalesced; the partial dot products are summed
// over the LPR lanes by xor-shuffles, which leaves every lane of a row group
// with its key's score, and the same lanes then weight their 16-byte chunk of
// the value row. This is the kernel of single-token (decode) rows: with a
// window of W keys a row costs W / (4 * 64 / LPR) dependent steps instead of
// W. Needs dk and dv to be multiples of the 16-byte vector and at most
// 64 vectors long; other shapes take the one-wave kernel above. NW waves a
// workgroup: 4 when there are rows enough to fill the chip, 16 when few rows
// face long contexts (a decode step of a small batch), so that every SIMD
// still holds several waves with loads in flight.
template <typename A> struct Vec16;
template <> struct Vec16<u16> { typedef u16x8 type; };
template <> struct Vec16<float> { typedef f32x4 type; };

template <typename A, int LPR, int NW>
__global__ void __launch_bounds__(NW * 64) local_attention_rows_kernel(
    A* __restrict__ out, long ldo, int out_off, const A* __restrict__ q,
    const A* __restrict__ k_cache, const A* __restrict__ v_cache,
    const int* __restrict__ bt, int bt_stride, const int* __restrict__ seq_lens,
    const int* __restrict__ qlocs, const int* __restrict__ token_seq,
    float scale, int chunk, int window, const A* __restrict__ proj, long ld,
    int gate_off, float out_scale, const float* __restrict__ bias_r1,
    const float* __restrict__ bias_r2, int sink, int keep_first, long t0, int H, int G, int dk,
    int dv, int page) {
  typedef typename Vec16<A>::type vec_t;
  constexpr int EPL = 16 / sizeof(A);     // elements per lane
  constexpr int KPI = 64 / LPR;           // keys per load instruction
  constexpr int TS = LPR < 16 ? LPR : 16; // steps per tile
  constexpr int TK = TS * KPI;            // keys per tile
  constexpr int DP = LPR * EPL;           // padded row length
  constexpr int CS = 2 + DP;              // floats a wave leaves in LDS
  __shared__ float qs[DP];
  __shared__ float comb[NW * CS];
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int kg = lane / LPR, c0 = (lane % LPR) * EPL;
  const long u = blockIdx.x;
  const long t = t0 + u / H;
  const int h = (int)(u % H);
  const int g = h / (H / G);
  for (int i = threadIdx.x; i < DP; i += blockDim.x)
    qs[i] = i < dk ? ldf<A>(q + (t * H + h) * (long)dk + i) : 0.f;
  __syncthreads();
  float qr[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) qr[e] = qs[c0 + e];

  const int s = token_seq[t];
  const int p = seq_lens[s] - (qlocs[s + 1] - (int)t);  // position of token t
  int lo = 0;
  if (chunk > 0) lo = (p / chunk) * chunk;
  const int clo = lo;
  if (window > 0 && p - window + 1 > lo) lo = p - window + 1;
  // kept first keys [clo, min(keep_first, lo)) take the first nk virtual
  // indices of vlo..p
  const int nk = max(min(keep_first, lo) - clo, 0);
  const int vlo = lo - nk;
  const int* table = bt + (long)s * bt_stride;
  const float r1 = bias_r1 ? bias_r1[h] : 0.f;
  const float r2 = bias_r1 ? bias_r2[h] : 0.f;
  const bool kact = c0 < dk, vact = c0 < dv;

  float m = -INFINITY, l = 0.f;
  float acc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc[e] = 0.f;

  const int n_tiles = (p - vlo) / TK + 1;
  for (int tile = wid; tile < n_tiles; tile += NW) {
    const int base = vlo + tile * TK;
    float sc[TS];
    long vrow[TS];
    float tmax = -INFINITY;
#pragma unroll
    for (int st = 0; st < TS; ++st) {
      const int jv = base + st * KPI + kg;
      const bool live = jv <= p;
      const int j = jv - vlo < nk ? clo + (jv - vlo) : jv;
      float dot = 0.f;
      long cell = 0;  // (blk * G + g) * page + off
      if (live) {
        const int blk = table[j / page];
        cell = ((long)blk * G + g) * page + j % page;
        if (kact) {
          const vec_t kx = *(const vec_t*)(k_cache + cell * dk + c0);
#pragma unroll
          for (int e = 0; e < EPL; ++e) {
            A ke = kx[e];
            dot += qr[e] * ldf<A>(&ke);
          }
        }
      }
#pragma unroll
      for (int o = LPR / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o, WAVE);
      float sv = -INFINITY;
      if (live) {
        sv = dot * scale;
        if (bias_r1) sv -= r1 * logf(1.f + r2 * (float)(p - j));
      }
      sc[st] = sv;
      vrow[st] = cell;
      tmax = fmaxf(tmax, sv);
    }
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1)
      tmax = fmaxf(tmax, __shfl_xor(tmax, o, WAVE));
    const float m_new = fmaxf(m, tmax);   // finite: key `base` is visible
    const float corr = expf(m - m_new);   // m = -inf on the first tile -> 0
    l *= corr;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] *= corr;
    m = m_new;
#pragma unroll
    for (int st = 0; st < TS; ++st) {
      if (sc[st] == -INFINITY) continue;
      const float pj = expf(sc[st] - m_new);
      l += pj;
      if (vact) {
        const vec_t vx = *(const vec_t*)(v_cache + vrow[st] * dv + c0);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          A ve = vx[e];
          acc[e] += pj * ldf<A>(&ve);
        }
      }
    }
  }
  // key groups of the wave
#pragma unroll
  for (int o = LPR; o < 64; o <<= 1) {
    l += __shfl_xor(l, o, WAVE);
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] += __shfl_xor(acc[e], o, WAVE);
  }
  float* mine = comb + wid * CS;
  if (lane < LPR) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) mine[2 + c0 + e] = acc[e];
    if (lane == 0) {
      mine[0] = m;
      mine[1] = l;
    }
  }
  __syncthreads();
  float mx = comb[0];  // wave 0 always has a tile
#pragma unroll
  for (int w = 1; w < NW; ++w) mx = fmaxf(mx, comb[w * CS]);
  // a sink (score 0, no value) joins the normalisation here, once per row
  if (sink) mx = fmaxf(mx, 0.f);
  float wgt[NW], lsum = sink ? expf(-mx) : 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    wgt[w] = expf(comb[w * CS] - mx);   // a wave without tiles: exp(-inf) = 0
    lsum += wgt[w] * comb[w * CS + 1];
  }
  float gate = out_scale;
  if (gate_off >= 0) gate *= sigmoid_f(ldf<A>(proj + t * ld + gate_off + h));
  const float f = gate / lsum;
  for (int c = threadIdx.x; c < dv; c += blockDim.x) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) o += wgt[w] * comb[w * CS + 2 + c];
    stf<A>(out + t * ldo + out_off + (long)h * dv + c, o * f);
  }
}

extern "C" void mix_attn_prep(void* q_out, const void* proj, long ld,
                              int q_off, int k_off, int v_off,
                              const float* q_w, const float* k_w, float eps,
                              const float* cos_sin, int half,
                              const long* slots, void* k_cache, void* v_cache,
                              const void* vfirst, long ldvf,
                              const float* vlam,
                              long T, int H, int G, int dk, int dv, int page,
                              int f32, hipStream_t s) {
  const long units = (T * (H + 2 * G) + UPW - 1) / UPW;
  const int grid = (int)((units + WPB - 1) / WPB);
  const int dmax = dk > dv ? dk : dv;
  const size_t smem = (size_t)WPB * dmax * sizeof(float);
  if (grid == 0) return;
  const int dm8 = (dmax + 7) / 8;
  // vfirst points at the first value column: 16-byte loads need it aligned
  if (!f32 && dk % 8 == 0 && dv % 8 == 0 && half % 8 == 0 && ld % 8 == 0 &&
      (!vfirst || (ldvf % 8 == 0 && ((size_t)vfirst & 15) == 0)) &&
      q_off % 8 == 0 && k_off % 8 == 0 && v_off % 8 == 0 && dm8 <= 32) {
    const int GS = dm8 <= 4 ? 4 : (dm8 <= 8 ? 8 : (dm8 <= 16 ? 16 : 32));
    const long tot = T * (H + 2 * G);
    const long waves = (tot + 64 / GS - 1) / (64 / GS);
    const int vgrid = (int)((waves + WPB - 1) / WPB);
#define LAUNCH_PV(GG)                                                         \
  hipLaunchKernelGGL(attn_prep_vec_kernel<GG>, dim3(vgrid), dim3(WPB * WAVE), \
                     0, s, (u16*)q_out, (const u16*)proj, ld, q_off, k_off,   \
                     v_off, q_w, k_w, eps, cos_sin, half, slots,              \
                     (u16*)k_cache, (u16*)v_cache, (const u16*)vfirst, ldvf,  \
                     vlam, T, H, G, dk, dv, page)
    if (GS == 4) LAUNCH_PV(4);
    else if (GS == 8) LAUNCH_PV(8);
    else if (GS == 16) LAUNCH_PV(16);
    else LAUNCH_PV(32);
#undef LAUNCH_PV
    return;
  }
  if (f32)
    hipLaunchKernelGGL(attn_prep_kernel<float>, dim3(grid), dim3(WPB * WAVE),
                       smem, s, (float*)q_out, (const float*)proj, ld, q_off,
                       k_off, v_off, q_w, k_w, eps, cos_sin, half, slots,
                       (float*)k_cache, (float*)v_cache, (const float*)vfirst,
                       ldvf, vlam, T, H, G, dk, dv, page);
  else
    hipLaunchKernelGGL(attn_prep_kernel<u16>, dim3(grid), dim3(WPB * WAVE),
                       smem, s, (u16*)q_out, (const u16*)proj, ld, q_off,
                       k_off, v_off, q_w, k_w, eps, cos_sin, half, slots,
                       (u16*)k_cache, (u16*)v_cache, (const u16*)vfirst, ldvf,
                       vlam, T, H, G, dk, dv, page);
}

template <typename A>
static void launch_local_attention(
    void* out, long ldo, int out_off, const void* q, const void* k_cache,
    const void* v_cache, const int* bt, int bt_stride, const int* seq_lens,
    const int* qlocs, const int* token_seq, float scale, int chunk,
    int window, const void* proj, long ld, int gate_off, float out_scale,
    const float* bias_r1, const float* bias_r2, int sink, int keep_first,
    long t0, long T,
    int H, int G, int dk, int dv, int page, hipStream_t s) {
  const long units = T * H;
  const int grid = (int)((units + WPB - 1) / WPB);
  if (grid == 0) return;
  {
    constexpr int EPL = 16 / (int)sizeof(A);
    const int dmax = dk > dv ? dk : dv;
    if (dk % EPL == 0 && dv % EPL == 0 && dmax <= 64 * EPL) {
      int lpr = 2;
      while (lpr * EPL < dmax) lpr <<= 1;
      // few rows over long tables (the table width bounds the context)
      const bool wide = units <= 512 && (long)bt_stride * page >= 512;
#define LAUNCH_LR(LL)                                                         \
  do {                                                                        \
    if (wide) LAUNCH_LRN(LL, 16);                                             \
    else LAUNCH_LRN(LL, 4);                                                   \
  } while (0)
#define LAUNCH_LRN(LL, NN)                                                    \
  hipLaunchKernelGGL((local_attention_rows_kernel<A, LL, NN>),                \
                     dim3((unsigned)units), dim3(NN * WAVE), 0, s, (A*)out,   \
                     ldo, out_off, (const A*)q, (const A*)k_cache,            \
                     (const A*)v_cache, bt, bt_stride, seq_lens, qlocs,       \
                     token_seq, scale, chunk, window, (const A*)proj, ld,     \
                     gate_off, out_scale, bias_r1, bias_r2, sink, keep_first, t0, H, G,   \
                     dk, dv, page)
      if (lpr == 2) LAUNCH_LR(2);
      else if (lpr == 4) LAUNCH_LR(4);
      else if (lpr == 8) LAUNCH_LR(8);
      else if (lpr == 16) LAUNCH_LR(16);
      else if (lpr == 32) LAUNCH_LR(32);
      else LAUNCH_LR(64);
#undef LAUNCH_LR
#undef LAUNCH_LRN
      return;
    }
  }
  const size_t smem = (size_t)WPB * dk * sizeof(float);
#define LAUNCH_LA(NV)                                                        \
  hipLaunchKernelGGL((local_attention_kernel<A, NV>), dim3(grid),            \
                     dim3(WPB * WAVE), smem, s, (A*)out, ldo, out_off,       \
                     (const A*)q, (const A*)k_cache, (const A*)v_cache, bt,  \
                     bt_stride, seq_lens, qlocs, token_seq, scale, chunk,    \
                     window, (const A*)proj, ld, gate_off, out_scale,        \
                     bias_r1, bias_r2, sink, keep_first, t0, T, H, G, dk, dv, page)
  if (dv <= 64) LAUNCH_LA(1);
  else if (dv <= 128) LAUNCH_LA(2);
  else if (dv <= 256) LAUNCH_LA(4);
  else LAUNCH_LA(8);
#undef LAUNCH_LA
}

extern "C" void mix_local_attention(
    void* out, long ldo, int out_off, const void* q, const void* k_cache,
    const void* v_cache, const int* bt, int bt_stride, const int* seq_lens,
    const int* qlocs, const int* token_seq, float scale, int chunk,
    int window, const void* proj, long ld, int gate_off, float out_scale,
    const float* bias_r1, const float* bias_r2, int sink, int keep_first,
    long t0, long T,
    int H, int G, int dk, int dv, int page, int f32, hipStream_t s) {
  if (f32)
    launch_local_attention<float>(out, ldo, out_off, q, k_cache, v_cache, bt,
                                  bt_stride, seq_lens, qlocs, token_seq, scale,
                                  chunk, window, proj, ld, gate_off, out_scale,
                                  bias_r1, bias_r2, sink, keep_first, t0, T, H, G, dk, dv,
                                  page, s);
  else
    launch_local_attention<u16>(out, ldo, out_off, q, k_cache, v_cache, bt,
                                bt_stride, seq_lens, qlocs, token_seq, scale,
                                chunk, window, proj, ld, gate_off, out_scale,
                                bias_r1, bias_r2, sink, keep_first, t0, T, H, G, dk, dv,
                                page, s);
}
