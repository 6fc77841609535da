// Decay recurrences of layer-list decoders (fixed-decay linear attention,
// Mamba-2), everything in fp32:
//
//   ssd_prep           short causal depthwise filter with bias + silu on the
//                      x|B|C channels of the Mamba-2 projection (history from
//                      the state slot), step dt = softplus(dt + bias), decay
//                      = exp(-exp(A_log) dt)
//   ssd_conv_update    keeps the last taps-1 raw filter inputs per sequence
//   decay_scan         S <- a S + b k v^T, o = S^T q + skip v, token by token,
//                      S [dk, dv] fp32 per sequence and head
//
// A sequence whose first token (position 0) is in the batch starts from zero
// filter history and zero S, whatever its state slot held before.
//
// decay_scan maps the state onto lanes by COLUMN: the dv columns of S never
// interact, so a column is owned by R adjacent lanes holding RPT rows each in
// registers; one token costs one R-lane sum (DPP moves) and broadcast reads
// of the staged k and q rows. Blocks cover (sequence, head, group of columns).
#include "mix_common.h"

template <typename A>
__global__ void __launch_bounds__(256) ssd_prep_kernel(
    float* __restrict__ xbc, float* __restrict__ decay, float* __restrict__ dt,
    const A* __restrict__ proj, long ld, int xbc_off, int dt_off,
    const float* __restrict__ conv_wt, const float* __restrict__ conv_b,
    int taps, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ conv_state,
    const int* __restrict__ state_slots, const int* __restrict__ qlocs,
    const int* __restrict__ seq_lens, const int* __restrict__ token_seq, long T,
    int C, int H) {
  const int cols = C + H;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * cols) return;
  const long t = i / cols;
  const int c = (int)(i - t * cols);
  if (c >= C) {
    const int h = c - C;
    const float d = softplus_f(ldf<A>(proj + t * ld + dt_off + h) + dt_bias[h]);
    dt[t * H + h] = d;
    decay[t * H + h] = expf(-expf(a_log[h]) * d);
    return;
  }
  const int s = token_seq[t];
  const int q0 = qlocs[s], n = qlocs[s + 1] - q0;
  const int start = seq_lens[s] - n;
  const int loc = (int)t - q0;
  const float* hist = conv_state + (long)state_slots[s] * (taps - 1) * C + c;
  float acc = conv_b[c];
  for (int j = 0; j < taps; ++j) {
    const int tau = loc - (taps - 1 - j);   // chunk-local time of this tap
    float x = 0.f;
    if (tau >= 0)
      x = ldf<A>(proj + (long)(q0 + tau) * ld + xbc_off + c);
    else if (start > 0)
      x = hist[(long)(taps - 1 + tau) * C];
    acc += conv_wt[(long)j * C + c] * x;
  }
  xbc[t * C + c] = acc * sigmoid_f(acc);
}

// bf16 fast path: a thread filters 8 consecutive channels of one token (one
// 16-byte load a tap, two 16-byte stores); the steps and decays of a token are
// made by the threads past the channel work. Needs C, the section start and
// the row length to be multiples of 8.
__global__ void __launch_bounds__(256) ssd_prep_vec_kernel(
    float* __restrict__ xbc, float* __restrict__ decay, float* __restrict__ dt,
    const u16* __restrict__ proj, long ld, int xbc_off, int dt_off,
    const float* __restrict__ conv_wt, const float* __restrict__ conv_b,
    int taps, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ conv_state,
    const int* __restrict__ state_slots, const int* __restrict__ qlocs,
    const int* __restrict__ seq_lens, const int* __restrict__ token_seq, long T,
    int C, int H) {
  const int C8 = C / 8;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * C8) {
    const long j = i - T * C8;
    if (j >= T * H) return;
    const long t = j / H;
    const int h = (int)(j - t * H);
    const float d = softplus_f(bf2f(proj[t * ld + dt_off + h]) + dt_bias[h]);
    dt[j] = d;
    decay[j] = expf(-expf(a_log[h]) * d);
    return;
  }
  const long t = i / C8;
  const int c = (int)(i - t * C8) * 8;
  const int s = token_seq[t];
  const int q0 = qlocs[s], n = qlocs[s + 1] - q0;
  const int start = seq_lens[s] - n;
  const int loc = (int)t - q0;
  const float* hist = conv_state + (long)state_slots[s] * (taps - 1) * C + c;
  float acc[8];
  {
    const f32x4 b0 = *(const f32x4*)(conv_b + c), b1 = *(const f32x4*)(conv_b + c + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { acc[e] = b0[e]; acc[e + 4] = b1[e]; }
  }
  for (int j = 0; j < taps; ++j) {
    const int tau = loc - (taps - 1 - j);
    float x[8];
    if (tau >= 0) {
      bf8_to_f32(*(const u16x8*)(proj + (long)(q0 + tau) * ld + xbc_off + c), x);
    } else if (start > 0) {
      const float* hr = hist + (long)(taps - 1 + tau) * C;
      const f32x4 h0 = *(const f32x4*)hr, h1 = *(const f32x4*)(hr + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] = h0[e]; x[e + 4] = h1[e]; }
    } else {
      continue;
    }
    const float* wr = conv_wt + (long)j * C + c;
    const f32x4 w0 = *(const f32x4*)wr, w1 = *(const f32x4*)(wr + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[e] += w0[e] * x[e];
      acc[e + 4] += w1[e] * x[e + 4];
    }
  }
  f32x4 o0, o1;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o0[e] = acc[e] * sigmoid_f(acc[e]);
    o1[e] = acc[e + 4] * sigmoid_f(acc[e + 4]);
  }
  *(f32x4*)(xbc + t * C + c) = o0;
  *(f32x4*)(xbc + t * C + c + 4) = o1;
}

// one thread per (sequence, channel): new history = last taps-1 raw inputs
template <typename A>
__global__ void __launch_bounds__(256) ssd_conv_update_kernel(
    float* __restrict__ conv_state, const A* __restrict__ proj, long ld,
    int xbc_off, int taps, const int* __restrict__ state_slots,
    const int* __restrict__ qlocs, const int* __restrict__ seq_lens, int S,
    int C) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)S * C) return;
  const int s = (int)(idx / C), c = (int)(idx - (long)s * C);
  const int q0 = qlocs[s], n = qlocs[s + 1] - q0;
  if (n <= 0) return;
  const int start = seq_lens[s] - n;
  float* hist = conv_state + (long)state_slots[s] * (taps - 1) * C + c;
  for (int i = 0; i < taps - 1; ++i) {
    const int tau = n - (taps - 1) + i;  // chunk-local time of history row i
    float x = 0.f;
    if (tau >= 0)
      x = ldf<A>(proj + (long)(q0 + tau) * ld + xbc_off + c);
    else if (start > 0 && i + n <= taps - 2)
      x = hist[(long)(i + n) * C];       // read before row i+n is rewritten
    hist[(long)i * C] = x;
  }
}

extern "C" void mix_ssd_prep(float* xbc, float* decay, float* dt,
                             const void* proj, long ld, int xbc_off,
                             int dt_off, const float* conv_wt,
                             const float* conv_b, int taps,
                             const float* dt_bias, const float* a_log,
                             float* conv_state, const int* state_slots,
                             const int* qlocs, const int* seq_lens,
                             const int* token_seq, long T, int S, int C, int H,
                             int f32, hipStream_t s) {
  if (T == 0) return;
  const unsigned grid = (unsigned)((T * (C + H) + 255) / 256);
  const unsigned sgrid = (unsigned)(((long)S * C + 255) / 256);
  if (f32) {
    hipLaunchKernelGGL(ssd_prep_kernel<float>, dim3(grid), dim3(256), 0, s, xbc,
                       decay, dt, (const float*)proj, ld, xbc_off, dt_off,
                       conv_wt, conv_b, taps, dt_bias, a_log, conv_state,
                       state_slots, qlocs, seq_lens, token_seq, T, C, H);
    if (taps > 1)
      hipLaunchKernelGGL(ssd_conv_update_kernel<float>, dim3(sgrid), dim3(256),
                         0, s, conv_state, (const float*)proj, ld, xbc_off,
                         taps, state_slots, qlocs, seq_lens, S, C);
  } else {
    if (C % 8 == 0 && xbc_off % 8 == 0 && ld % 8 == 0) {
      const unsigned vgrid = (unsigned)((T * (C / 8) + T * H + 255) / 256);
      hipLaunchKernelGGL(ssd_prep_vec_kernel, dim3(vgrid), dim3(256), 0, s, xbc,
                         decay, dt, (const u16*)proj, ld, xbc_off, dt_off,
                         conv_wt, conv_b, taps, dt_bias, a_log, conv_state,
                         state_slots, qlocs, seq_lens, token_seq, T, C, H);
    } else
    hipLaunchKernelGGL(ssd_prep_kernel<u16>, dim3(grid), dim3(256), 0, s, xbc,
                       decay, dt, (const u16*)proj, ld, xbc_off, dt_off,
                       conv_wt, conv_b, taps, dt_bias, a_log, conv_state,
                       state_slots, qlocs, seq_lens, token_seq, T, C, H);
    if (taps > 1)
      hipLaunchKernelGGL(ssd_conv_update_kernel<u16>, dim3(sgrid), dim3(256), 0,
                         s, conv_state, (const u16*)proj, ld, xbc_off, taps,
                         state_slots, qlocs, seq_lens, S, C);
  }
}

// ---- decay_scan ------------------------------------------------------------
#define DTB 8   // tokens staged per step

// Block = (sequence, head, group of 256/R columns); lane (col, r) keeps rows
// {((n/4)*R + r)*4 + n%4 : n < RPT} of its column of S in registers (rows
// past dk stay zero: their k and q are staged as 0). k, q, v, decay and gain
// of DTB tokens at a time are staged through a double-buffered LDS tile: the
// global loads of tile s+1 are issued before the arithmetic of tile s and
// parked in registers. With this row mapping the R lanes of a column read
// consecutive float4s of a staged row, and all columns read the same
// addresses (LDS broadcast).
template <int R, int RPT>
__global__ void __launch_bounds__(256) decay_scan_kernel(
    float* __restrict__ o, const float* __restrict__ q, long ldq,
    const float* __restrict__ k, long ldk, const float* __restrict__ v,
    long ldv, const float* __restrict__ decay, long lda,
    const float* __restrict__ gain, const float* __restrict__ skip,
    float* __restrict__ state, const int* __restrict__ state_slots,
    const int* __restrict__ qlocs, const int* __restrict__ seq_lens, int H,
    int G, int dk, int dv, int col_groups) {
  constexpr int DKP = R * RPT;
  constexpr int CPB = 256 / R;             // columns per block
  constexpr int NK = 2 * DTB * DKP / 256;  // staged k|q floats per lane
  constexpr int NV = DTB * CPB / 256 > 0 ? DTB * CPB / 256 : 1;
  constexpr int TILE = 2 * DTB * DKP + DTB * CPB + 2 * DTB;
  __shared__ __attribute__((aligned(16))) float lds[2][TILE];

  int b = blockIdx.x;
  const int cg = b % col_groups;
  b /= col_groups;
  const int h = b % H;
  const int s = b / H;
  const int q0 = qlocs[s], n = qlocs[s + 1] - q0;
  if (n <= 0) return;
  const int start = seq_lens[s] - n;
  const int g = h / (H / G);
  const int tid = threadIdx.x;
  const int r = tid % R;
  const int col = cg * CPB + tid / R;
  const bool cact = col < dv;
  float* Sg = state + (((long)state_slots[s] * H + h) * dk) * dv;

  float S[RPT];
#pragma unroll
  for (int m = 0; m < RPT; ++m) {
    const int row = ((m / 4) * R + r) * 4 + m % 4;
    S[m] = (start > 0 && cact && row < dk) ? Sg[(long)row * dv + col] : 0.f;
  }
  const float sk = skip ? skip[h] : 0.f;

  float pk[NK], pv[NV], pa = 0.f, pb = 0.f;
  // issue the loads of tile `base` into registers
  auto fetch = [&](int base) {
#pragma unroll
    for (int m = 0; m < NK; ++m) {
      const int e = tid + m * 256;          // [which(2)][token][DKP]
      const int which = e / (DTB * DKP);
      const int rem = e - which * DTB * DKP;
      const int tt = rem / DKP, d = rem - tt * DKP;
      const long tok = q0 + base + tt;
      float x = 0.f;
      if (base + tt < n && d < dk)
        x = which == 0 ? k[tok * ldk + (long)g * dk + d]
                       : q[tok * ldq + (long)g * dk + d];
      pk[m] = x;
    }
#pragma unroll
    for (int m = 0; m < NV; ++m) {
      const int e = tid + m * 256;          // [token][CPB]
      const int tt = e / CPB, cc = e - tt * CPB;
      float x = 0.f;
      if (e < DTB * CPB && base + tt < n && cg * CPB + cc < dv)
        x = v[(long)(q0 + base + tt) * ldv + (long)h * dv + cg * CPB + cc];
      pv[m] = x;
    }
    if (tid < DTB) {
      const bool in = base + tid < n;
      pa = in ? decay[(long)(q0 + base + tid) * lda + h] : 1.f;
      pb = in ? (gain ? gain[(long)(q0 + base + tid) * H + h] : 1.f) : 0.f;
    }
  };
  auto park = [&](float* tile) {
#pragma unroll
    for (int m = 0; m < NK; ++m) tile[tid + m * 256] = pk[m];
#pragma unroll
    for (int m = 0; m < NV; ++m)
      if (tid + m * 256 < DTB * CPB)
        tile[2 * DTB * DKP + tid + m * 256] = pv[m];
    if (tid < DTB) {
      tile[2 * DTB * DKP + DTB * CPB + tid] = pa;
      tile[2 * DTB * DKP + DTB * CPB + DTB + tid] = pb;
    }
  };

  fetch(0);
  park(lds[0]);
  __syncthreads();
  int buf = 0;
  for (int base = 0; base < n; base += DTB) {
    const bool more = base + DTB < n;
    if (more) fetch(base + DTB);
    const float* tile = lds[buf];
    const int lim = n - base < DTB ? n - base : DTB;
    for (int tt = 0; tt < lim; ++tt) {
      const float a = tile[2 * DTB * DKP + DTB * CPB + tt];
      const float bb = tile[2 * DTB * DKP + DTB * CPB + DTB + tt];
      const float vv = tile[2 * DTB * DKP + tt * CPB + tid / R];
      const float bv = bb * vv;
      const f32x4* kr = (const f32x4*)(tile + tt * DKP);
      const f32x4* qr = (const f32x4*)(tile + DTB * DKP + tt * DKP);
      float part = 0.f;
#pragma unroll
      for (int f = 0; f < RPT / 4; ++f) {
        const f32x4 kk = kr[f * R + r];
        const f32x4 qq = qr[f * R + r];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[f * 4 + e] = a * S[f * 4 + e] + kk[e] * bv;
          part += S[f * 4 + e] * qq[e];
        }
      }
      part = group_sum<R>(part);
      if (r == 0 && cact)
        o[((long)(q0 + base + tt) * H + h) * dv + col] = part + sk * vv;
    }
    if (more) park(lds[buf ^ 1]);
    __syncthreads();
    buf ^= 1;
  }
  if (cact) {
#pragma unroll
    for (int m = 0; m < RPT; ++m) {
      const int row = ((m / 4) * R + r) * 4 + m % 4;
      if (row < dk) Sg[(long)row * dv + col] = S[m];
    }
  }
}

extern "C" int mix_decay_scan(float* o, const float* q, long ldq,
                              const float* k, long ldk, const float* v,
                              long ldv, const float* decay, long lda,
                              const float* gain, const float* skip,
                              float* state, const int* state_slots,
                              const int* qlocs, const int* seq_lens, int S,
                              int H, int G, int dk, int dv, hipStream_t s) {
  if (S == 0) return 1;
#define LAUNCH_DS(RR, PP)                                                    \
  do {                                                                       \
    const int cgs = (dv + 256 / RR - 1) / (256 / RR);                        \
    hipLaunchKernelGGL((decay_scan_kernel<RR, PP>), dim3(S * H * cgs),       \
                       dim3(256), 0, s, o, q, ldq, k, ldk, v, ldv, decay,    \
                       lda, gain, skip, state, state_slots, qlocs, seq_lens, \
                       H, G, dk, dv, cgs);                                   \
  } while (0)
  if (dk <= 16) LAUNCH_DS(4, 4);
  else if (dk <= 32) LAUNCH_DS(4, 8);
  else if (dk <= 64) LAUNCH_DS(8, 8);
  else if (dk <= 128) LAUNCH_DS(8, 16);
  else if (dk <= 256) LAUNCH_DS(16, 16);
  else return 0;
#undef LAUNCH_DS
  return 1;
}
