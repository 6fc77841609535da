// Parallel layers under a Dynamic-Tanh norm, and routed experts:
//   dyt_residual   x += ls1 * y1 + ls2 * (y2 | sum_j w[t,j] * rows[pp[t,j]]);
//                  h = tanh(alpha * x) * nw + nb. Every part optional: the
//                  same kernel serves the first layer's norm (no update), a
//                  layer without experts and the final norm.
//   moe_route      sigmoid scores, group-limited choice (a group is worth the
//                  sum of its `rank` largest scores, the `keep` best groups
//                  stay), the `top` best experts and their normalised weights
//   moe_dispatch   (token, choice) pairs -> per-expert segments padded to the
//                  GEMM tile height: row -> token table, segment starts,
//                  counts, pair -> row table. One workgroup, LDS counters.
//   expert_gemm    plain tiled GEMM over those segments for shapes or types
//                  the matrix-core kernel (grouped_gemm.hip) does not take:
//                  fp32 FMA, optional squared-ReLU epilogue
//   softcap        c * tanh(z / c) in fp32
// The stream x, norm parameters, layer scales, router scores and weights are
// fp32; `A` is the activation type (u16 = bf16 bits, or float).
#include "mix_common.h"

// ---- dyt_residual ----------------------------------------------------------
// One 256-thread block a row, V columns a thread and turn (V = 4 when the
// width allows 16-byte fp32 accesses, else 1).
template <typename A, int V>
__global__ void __launch_bounds__(256) dyt_residual_kernel(
    float* __restrict__ x, const A* __restrict__ y1,
    const float* __restrict__ ls1, const A* __restrict__ y2,
    const float* __restrict__ ls2, const A* __restrict__ rows,
    const int* __restrict__ padpos, const float* __restrict__ wts, int k,
    const float* __restrict__ alpha, const float* __restrict__ nw,
    const float* __restrict__ nb, A* __restrict__ h_out, int W) {
  const long t = blockIdx.x;
  float* xr = x + t * W;
  const float a = alpha ? alpha[0] : 0.f;
  for (int c = threadIdx.x * V; c < W; c += 256 * V) {
    float xv[V];
#pragma unroll
    for (int e = 0; e < V; ++e) xv[e] = xr[c + e];
    if (y1) {
#pragma unroll
      for (int e = 0; e < V; ++e)
        xv[e] += ls1[c + e] * ldf<A>(y1 + t * W + c + e);
      if (y2) {
#pragma unroll
        for (int e = 0; e < V; ++e)
          xv[e] += ls2[c + e] * ldf<A>(y2 + t * W + c + e);
      } else if (rows) {
        float acc[V];
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = 0.f;
        for (int j = 0; j < k; ++j) {
          const float wj = wts[t * k + j];
          const A* rr = rows + (long)padpos[t * k + j] * W + c;
#pragma unroll
          for (int e = 0; e < V; ++e) acc[e] += wj * ldf<A>(rr + e);
        }
#pragma unroll
        for (int e = 0; e < V; ++e) xv[e] += ls2[c + e] * acc[e];
      }
#pragma unroll
      for (int e = 0; e < V; ++e) xr[c + e] = xv[e];
    }
    if (h_out) {
#pragma unroll
      for (int e = 0; e < V; ++e)
        stf<A>(h_out + t * W + c + e,
               tanhf(a * xv[e]) * nw[c + e] + nb[c + e]);
    }
  }
}

extern "C" void mix_dyt_residual(float* x, const void* y1, const float* ls1,
                                 const void* y2, const float* ls2,
                                 const void* rows, const int* padpos,
                                 const float* wts, int k, const float* alpha,
                                 const float* nw, const float* nb, void* h_out,
                                 long T, int W, int f32, hipStream_t s) {
  if (T == 0) return;
#define LAUNCH_DY(AA, VV)                                                    \
  hipLaunchKernelGGL((dyt_residual_kernel<AA, VV>), dim3((unsigned)T),       \
                     dim3(256), 0, s, x, (const AA*)y1, ls1, (const AA*)y2,  \
                     ls2, (const AA*)rows, padpos, wts, k, alpha, nw, nb,    \
                     (AA*)h_out, W)
  if (W % 4 == 0) {
    if (f32) LAUNCH_DY(float, 4); else LAUNCH_DY(u16, 4);
  } else {
    if (f32) LAUNCH_DY(float, 1); else LAUNCH_DY(u16, 1);
  }
#undef LAUNCH_DY
}

// ---- moe_route -------------------------------------------------------------
// One wave a token, 4 waves a block. LDS per wave: E scores, then G group
// worths. Order everywhere: larger value first, lower index on ties.
__device__ __forceinline__ bool before(float va, int ia, float vb, int ib) {
  return va > vb || (va == vb && ia < ib);
}

__global__ void __launch_bounds__(256) moe_route_kernel(
    int* __restrict__ idx, float* __restrict__ wts,
    const float* __restrict__ logits, long T, int E, int top, int G, int keep,
    int rank) {
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  float* sc = sm + wid * (E + G);
  float* worth = sc + E;
  const long t0 = (long)blockIdx.x * 4 + wid;
  const bool valid = t0 < T;
  const long t = valid ? t0 : 0;
  const int size = E / G;
  for (int e = lane; e < E; e += 64) sc[e] = sigmoid_f(logits[t * E + e]);
  __syncthreads();
  if (G > 1) {
    for (int g = lane; g < G; g += 64) {
      const float* part = sc + g * size;
      float pv = INFINITY, sum = 0.f;
      int pi = -1;
      const int r = rank < size ? rank : size;
      for (int n = 0; n < r; ++n) {
        float bv = -1.f;
        int bi = -1;
        for (int i = 0; i < size; ++i) {
          const float v = part[i];
          // after the previous pick in the order, and first among those
          if (before(pv, pi, v, i) && (bi < 0 || before(v, i, bv, bi))) {
            bv = v;
            bi = i;
          }
        }
        sum += bv;
        pv = bv;
        pi = bi;
      }
      worth[g] = sum;
    }
    __syncthreads();
    // a group stays when fewer than `keep` groups come before it
    bool drop[16];  // groups of this lane: G <= 1024
#pragma unroll
    for (int n = 0; n < 16; ++n) {
      const int g = lane + n * 64;
      drop[n] = false;
      if (g < G) {
        int ahead = 0;
        for (int o = 0; o < G; ++o)
          ahead += before(worth[o], o, worth[g], g) ? 1 : 0;
        drop[n] = ahead >= keep;
      }
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < 16; ++n) {
      const int g = lane + n * 64;
      if (g < G) worth[g] = drop[n] ? 1.f : 0.f;
    }
    __syncthreads();
  }
  // the `top` best of the allowed experts, one a turn; `taken` scores are
  // marked in LDS with -2 after their value went into a register
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    float bv = -3.f;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      float v = sc[e];
      if (G > 1 && v >= 0.f && worth[e / size] != 0.f) v = -1.f;
      if (before(v, e, bv, bi)) {
        bv = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (before(ov, oi, bv, bi)) {
        bv = ov;
        bi = oi;
      }
    }
    const float s = sc[bi];          // the raw score (bv is it too)
    __syncthreads();
    if (lane == 0) sc[bi] = -2.f;
    __syncthreads();
    total += s;
    if (valid && lane == 0) {
      idx[t * top + j] = bi;
      wts[t * top + j] = s;
    }
  }
  __syncthreads();
  if (valid) {
    const float inv = 1.f / (total + 1e-20f);
    for (int j = lane; j < top; j += 64) wts[t * top + j] *= inv;
  }
}

extern "C" void mix_moe_route(int* idx, float* wts, const float* logits, long T,
                              int E, int top, int G, int keep, int rank,
                              hipStream_t s) {
  if (T == 0) return;
  const size_t smem = (size_t)4 * (E + G) * sizeof(float);
  hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)((T + 3) / 4)), dim3(256),
                     smem, s, idx, wts, logits, T, E, top, G, keep, rank);
}

// ---- moe_dispatch ----------------------------------------------------------
// One 1024-thread workgroup. The place of a pair inside its expert's segment
// comes from an LDS counter, so it depends on timing; a row's result does not
// depend on its place, and every pair finds its row through padpos.
__global__ void __launch_bounds__(1024) moe_dispatch_kernel(
    int* __restrict__ row_tok, int* __restrict__ tile_off,
    int* __restrict__ counts, int* __restrict__ padpos,
    const int* __restrict__ idx, long n_pairs, int k, int E, int bm,
    long n_rows) {
  extern __shared__ int smi[];
  int* cnt = smi;          // [E] pairs per expert, then a running cursor
  int* start = smi + E;    // [E + 1] first padded row of each segment
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (long i = tid; i < n_pairs; i += 1024) atomicAdd(&cnt[idx[i]], 1);
  for (long i = tid; i < n_rows; i += 1024) row_tok[i] = -1;
  __syncthreads();
  if (tid == 0) {
    int off = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = off;
      off += (cnt[e] + bm - 1) / bm * bm;
    }
    start[E] = off;
  }
  __syncthreads();
  for (int e = tid; e <= E; e += 1024) {
    tile_off[e] = start[e] / bm;
    if (e < E) counts[e] = cnt[e];
  }
  __syncthreads();
  for (int e = tid; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (long i = tid; i < n_pairs; i += 1024) {
    const int e = idx[i];
    const int r = start[e] + atomicAdd(&cnt[e], 1);
    row_tok[r] = (int)(i / k);
    padpos[i] = r;
  }
}

extern "C" void mix_moe_dispatch(int* row_tok, int* tile_off, int* counts,
                                 int* padpos, const int* idx, long n_pairs,
                                 int k, int E, int bm, long n_rows,
                                 hipStream_t s) {
  const size_t smem = (size_t)(2 * E + 1) * sizeof(int);
  hipLaunchKernelGGL(moe_dispatch_kernel, dim3(1), dim3(1024), smem, s, row_tok,
                     tile_off, counts, padpos, idx, n_pairs, k, E, bm, n_rows);
}

// ---- expert_gemm (plain) ---------------------------------------------------
// out[r, n] = act(sum_k a[tok(r), k] * w[e, n, k]) over 64-row tiles of the
// padded segments; 256 threads as 16 x 16, 4 x 4 outputs a thread, K staged
// 16 at a time through LDS. Rows past a segment's live count are not stored.
// act 1: relu(x)^2. act 2: w holds N gate rows then N up rows per expert and
// out[r, n] = g sigmoid(1.702 g) (u + 1), g = min(gate, limit), u = clamp(up).
template <typename A>
__global__ void __launch_bounds__(256) expert_gemm_plain_kernel(
    A* __restrict__ out, const A* __restrict__ a, const A* __restrict__ w,
    const int* __restrict__ row_tok, const int* __restrict__ tile_off,
    const int* __restrict__ counts, int E, int N, int K, int bm, int act,
    float limit) {
  __shared__ float As[16][65];
  __shared__ float Bs[16][65];
  __shared__ float Us[16][65];
  const bool glu = act == 2;
  const int tiles_per = bm / 64;
  const int t64 = blockIdx.x;              // 64-row tile over all segments
  const int t = t64 / tiles_per;           // bm-row tile
  if (t >= tile_off[E]) return;
  int lo = 0, hi = E - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (tile_off[mid] <= t) lo = mid; else hi = mid - 1;
  }
  const int e = lo;
  const int m0 = (t - tile_off[e]) * bm + (t64 % tiles_per) * 64;
  const int live = counts[e] - m0;         // live rows of this tile
  if (live <= 0) return;
  const long seg = (long)tile_off[e] * bm + m0;
  const int n0 = blockIdx.y * 64;
  const A* we = w + (long)e * (glu ? 2 : 1) * N * K;
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  float acc[4][4], accu[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = accu[i][j] = 0.f;
  // staging: thread -> (row = tid / 4, 4 consecutive k)
  const int sr = tid >> 2, sk = (tid & 3) * 4;
  long arow = -1;
  if (sr < live) arow = row_tok ? (long)row_tok[seg + sr] : seg + sr;
  const int bn = n0 + sr;
  for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int kk = k0 + sk + q;
      As[sk + q][sr] = (arow >= 0 && kk < K) ? ldf<A>(a + arow * K + kk) : 0.f;
      Bs[sk + q][sr] = (bn < N && kk < K) ? ldf<A>(we + (long)bn * K + kk) : 0.f;
      if (glu)
        Us[sk + q][sr] =
            (bn < N && kk < K) ? ldf<A>(we + (long)(N + bn) * K + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
      if (glu) {
#pragma unroll
        for (int j = 0; j < 4; ++j) bv[j] = Us[kk][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) accu[i][j] += av[i] * bv[j];
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= live) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (act == 1) {
        v = v > 0.f ? v : 0.f;
        v *= v;
      } else if (glu) {
        const float g = fminf(v, limit);
        const float u = fminf(fmaxf(accu[i][j], -limit), limit);
        v = g * sigmoid_f(1.702f * g) * (u + 1.f);
      }
      stf<A>(out + (seg + r) * N + n, v);
    }
  }
}

extern "C" void mix_expert_gemm_plain(void* out, const void* a, const void* w,
                                      const int* row_tok, const int* tile_off,
                                      const int* counts, int E, int N, int K,
                                      int bm, long n_rows, int act, float limit,
                                      int f32, hipStream_t s) {
  const long tiles = n_rows / 64;
  if (tiles == 0) return;
  const dim3 grid((unsigned)tiles, (unsigned)((N + 63) / 64));
  if (f32)
    hipLaunchKernelGGL(expert_gemm_plain_kernel<float>, grid, dim3(256), 0, s,
                       (float*)out, (const float*)a, (const float*)w, row_tok,
                       tile_off, counts, E, N, K, bm, act, limit);
  else
    hipLaunchKernelGGL(expert_gemm_plain_kernel<u16>, grid, dim3(256), 0, s,
                       (u16*)out, (const u16*)a, (const u16*)w, row_tok,
                       tile_off, counts, E, N, K, bm, act, limit);
}

// ---- softcap ---------------------------------------------------------------
template <typename A>
__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ out,
                                                      const A* __restrict__ z,
                                                      float cap, long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = cap * tanhf(ldf<A>(z + i) / cap);
}

extern "C" void mix_softcap(float* out, const void* z, float cap, long n,
                            int f32, hipStream_t s) {
  if (n == 0) return;
  const unsigned grid = (unsigned)((n + 255) / 256);
  if (f32)
    hipLaunchKernelGGL(softcap_kernel<float>, dim3(grid), dim3(256), 0, s, out,
                       (const float*)z, cap, n);
  else
    hipLaunchKernelGGL(softcap_kernel<u16>, dim3(grid), dim3(256), 0, s, out,
                       (const u16*)z, cap, n);
}
