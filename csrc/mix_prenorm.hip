// Kernels of pre-norm layer-list decoders with weighted RMS norms:
//
//   add_rmsnorm        x += y + sum_j w_j rows[padpos_j] + idw * h_in
//                      + sigmoid(sg) * y2 in fp32, then the NEXT sublayer's
//                      input h = x / rms(x) * weight: residual sum, gather of a
//                      token's expert rows, identity experts, gated shared
//                      expert and norm in one pass
//   glu_mul            act(gate) * up over two sections of a merged projection:
//                      tanh-GELU, silu, or the clamped unit g sigmoid(1.702 g)
//                      (u + 1) with g = min(gate, limit), u = clamp(up)
//   moe_route_softmax  softmax scores, choice = score + correction, groups
//                      worth their largest choice, the best `keep` groups, the
//                      `top` best allowed outputs, identity experts folded
//                      into one weight per token
//   silu_sections      fp32 silu of up to three sections of a projection
//   gated_group_norm   read-out of a recurrence against its gate: gate first
//                      (y silu(z), then normed in equal parts) or norm first
//                      (normed, weight, sigmoid gate)
#include "mix_common.h"

// ---- add_rmsnorm -----------------------------------------------------------
// One 256-thread block a row, V columns a thread and turn. A thread reads back
// only the columns it wrote, so h_out may be the buffer h_in is read from.
template <typename A, int V>
__global__ void __launch_bounds__(256) add_rmsnorm_kernel(
    float* __restrict__ x, const A* __restrict__ y, const A* __restrict__ rows,
    const int* __restrict__ padpos, const float* __restrict__ wts, int k,
    const float* __restrict__ idw, const A* h_in, const A* __restrict__ y2,
    const A* __restrict__ proj2, long ld2, int sg_off,
    const float* __restrict__ nw, float eps, A* h_out, int W) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  const bool upd = y || rows || idw || y2;
  float sgate = 1.f;
  if (y2 && sg_off >= 0) sgate = sigmoid_f(ldf<A>(proj2 + t * ld2 + sg_off));
  const float iw = idw ? idw[t] : 0.f;
  float ssq = 0.f;
  for (int c = threadIdx.x * V; c < W; c += 256 * V) {
    float xv[V];
#pragma unroll
    for (int e = 0; e < V; ++e) xv[e] = xr[c + e];
    if (y) {
#pragma unroll
      for (int e = 0; e < V; ++e) xv[e] += ldf<A>(y + t * W + c + e);
    }
    if (rows) {
      float acc[V];
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = 0.f;
      for (int j = 0; j < k; ++j) {
        const float wj = wts[t * k + j];
        if (wj == 0.f) continue;  // a pair without a row (identity expert)
        const A* rr = rows + (long)padpos[t * k + j] * W + c;
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] += wj * ldf<A>(rr + e);
      }
#pragma unroll
      for (int e = 0; e < V; ++e) xv[e] += acc[e];
    }
    if (idw) {
#pragma unroll
      for (int e = 0; e < V; ++e) xv[e] += iw * ldf<A>(h_in + t * W + c + e);
    }
    if (y2) {
#pragma unroll
      for (int e = 0; e < V; ++e) xv[e] += sgate * ldf<A>(y2 + t * W + c + e);
    }
    if (upd) {
#pragma unroll
      for (int e = 0; e < V; ++e) xr[c + e] = xv[e];
    }
#pragma unroll
    for (int e = 0; e < V; ++e) ssq += xv[e] * xv[e];
  }
  if (!h_out) return;
  const float tot = block_sum_256(ssq, red);
  const float inv = 1.f / sqrtf(tot / (float)W + eps);
  for (int c = threadIdx.x * V; c < W; c += 256 * V) {
#pragma unroll
    for (int e = 0; e < V; ++e)
      stf<A>(h_out + t * W + c + e, xr[c + e] * inv * nw[c + e]);
  }
}

extern "C" void mix_add_rmsnorm(float* x, const void* y, const void* rows,
                                const int* padpos, const float* wts, int k,
                                const float* idw, const void* h_in,
                                const void* y2, const void* proj2, long ld2,
                                int sg_off, const float* nw, float eps,
                                void* h_out, long T, int W, int f32,
                                hipStream_t s) {
  if (T == 0) return;
#define LAUNCH_AR(AA, VV)                                                     \
  hipLaunchKernelGGL((add_rmsnorm_kernel<AA, VV>), dim3((unsigned)T),         \
                     dim3(256), 0, s, x, (const AA*)y, (const AA*)rows,       \
                     padpos, wts, k, idw, (const AA*)h_in, (const AA*)y2,     \
                     (const AA*)proj2, ld2, sg_off, nw, eps, (AA*)h_out, W)
  if (W % 4 == 0) {
    if (f32) LAUNCH_AR(float, 4); else LAUNCH_AR(u16, 4);
  } else {
    if (f32) LAUNCH_AR(float, 1); else LAUNCH_AR(u16, 1);
  }
#undef LAUNCH_AR
}

// ---- glu_mul ---------------------------------------------------------------
__device__ __forceinline__ float glu_unit(float g, float u, int act,
                                          float limit) {
  if (act == 0) {
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return 0.5f * g * (1.f + tanhf(z)) * u;
  }
  if (act == 1) return g * sigmoid_f(g) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sigmoid_f(1.702f * g) * (u + 1.f);
}

template <typename A>
__global__ void __launch_bounds__(256) glu_mul_kernel(
    A* __restrict__ out, const A* __restrict__ proj, long ld, int gate_off,
    int up_off, long T, int F, int act, float limit) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * F) return;
  const long t = i / F;
  const int c = (int)(i - t * F);
  const A* row = proj + t * ld;
  stf<A>(out + i, glu_unit(ldf<A>(row + gate_off + c), ldf<A>(row + up_off + c),
                           act, limit));
}

// bf16, 8 columns (16 bytes) a thread
__global__ void __launch_bounds__(256) glu_mul_vec_kernel(
    u16* __restrict__ out, const u16* __restrict__ proj, long ld, int gate_off,
    int up_off, long T, int F8, int act, float limit) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * F8) return;
  const long t = i / F8;
  const int c = (int)(i - t * F8) * 8;
  const u16* row = proj + t * ld;
  float g[8], u[8];
  bf8_to_f32(*(const u16x8*)(row + gate_off + c), g);
  bf8_to_f32(*(const u16x8*)(row + up_off + c), u);
  u16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = f2bf(glu_unit(g[e], u[e], act, limit));
  *(u16x8*)(out + t * (long)F8 * 8 + c) = o;
}

extern "C" void mix_glu_mul(void* out, const void* proj, long ld, int gate_off,
                            int up_off, long T, int F, int act, float limit,
                            int f32, hipStream_t s) {
  if (T * F == 0) return;
  if (!f32 && F % 8 == 0 && gate_off % 8 == 0 && up_off % 8 == 0 &&
      ld % 8 == 0) {
    const long n = T * (F / 8);
    hipLaunchKernelGGL(glu_mul_vec_kernel, dim3((unsigned)((n + 255) / 256)),
                       dim3(256), 0, s, (u16*)out, (const u16*)proj, ld,
                       gate_off, up_off, T, F / 8, act, limit);
    return;
  }
  const unsigned grid = (unsigned)((T * F + 255) / 256);
  if (f32)
    hipLaunchKernelGGL(glu_mul_kernel<float>, dim3(grid), dim3(256), 0, s,
                       (float*)out, (const float*)proj, ld, gate_off, up_off,
                       T, F, act, limit);
  else
    hipLaunchKernelGGL(glu_mul_kernel<u16>, dim3(grid), dim3(256), 0, s,
                       (u16*)out, (const u16*)proj, ld, gate_off, up_off, T, F,
                       act, limit);
}

// ---- moe_route_softmax -----------------------------------------------------
// One wave a token, 4 waves a block. LDS per wave: n scores, n choice scores,
// G group worths. Order everywhere: larger value first, lower index on ties.
__device__ __forceinline__ bool ahead_of(float va, int ia, float vb, int ib) {
  return va > vb || (va == vb && ia < ib);
}

__global__ void __launch_bounds__(256) moe_route_softmax_kernel(
    int* __restrict__ idx, float* __restrict__ wts, float* __restrict__ idw,
    const float* __restrict__ logits, const float* __restrict__ corr, long T,
    int n, int n_real, int top, int G, int keep, float scale) {
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  float* sc = sm + wid * (2 * n + G);
  float* ch = sc + n;
  float* worth = ch + n;
  const long t0 = (long)blockIdx.x * 4 + wid;
  const bool valid = t0 < T;
  const long t = valid ? t0 : 0;
  const int size = n / G;
  float mx = -INFINITY;
  for (int e = lane; e < n; e += 64) mx = fmaxf(mx, logits[t * n + e]);
  mx = wave_max_f32(mx);
  float sum = 0.f;
  for (int e = lane; e < n; e += 64) {
    const float v = expf(logits[t * n + e] - mx);
    sc[e] = v;
    sum += v;
  }
  sum = wave_sum_f32(sum);
  const float inv = 1.f / sum;
  for (int e = lane; e < n; e += 64) {
    const float v = sc[e] * inv;
    sc[e] = v;
    ch[e] = v + (corr ? corr[e] : 0.f);
  }
  __syncthreads();
  if (G > 1) {
    for (int g = lane; g < G; g += 64) {
      float w = -INFINITY;
      for (int i = 0; i < size; ++i) w = fmaxf(w, ch[g * size + i]);
      worth[g] = w;
    }
    __syncthreads();
    // a group stays when fewer than `keep` groups come before it
    bool drop[16];  // groups of this lane: G <= 1024
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int g = lane + m * 64;
      drop[m] = false;
      if (g < G) {
        int before = 0;
        for (int o = 0; o < G; ++o)
          before += ahead_of(worth[o], o, worth[g], g) ? 1 : 0;
        drop[m] = before >= keep;
      }
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int g = lane + m * 64;
      if (g < G && drop[m])
        for (int i = 0; i < size; ++i) ch[g * size + i] = -INFINITY;
    }
    __syncthreads();
  }
  // the `top` best allowed outputs, one a turn; a taken one drops to -inf
  float ident = 0.f;
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < n; e += 64) {
      const float v = ch[e];
      if (ahead_of(v, e, bv, bi)) {
        bv = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ahead_of(ov, oi, bv, bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi >= n) bi = 0;  // unreachable with finite logits
    const float w = sc[bi] * scale;
    __syncthreads();
    if (lane == 0) ch[bi] = -INFINITY;
    __syncthreads();
    const bool is_ident = bi >= n_real;
    if (is_ident) ident += w;
    if (valid && lane == 0) {
      idx[t * top + j] = is_ident ? n_real : bi;
      wts[t * top + j] = is_ident ? 0.f : w;
    }
  }
  if (valid && lane == 0) idw[t] = ident;
}

extern "C" void mix_moe_route_softmax(int* idx, float* wts, float* idw,
                                      const float* logits, const float* corr,
                                      long T, int n, int n_real, int top, int G,
                                      int keep, float scale, hipStream_t s) {
  if (T == 0) return;
  const size_t smem = (size_t)4 * (2 * n + G) * sizeof(float);
  hipLaunchKernelGGL(moe_route_softmax_kernel, dim3((unsigned)((T + 3) / 4)),
                     dim3(256), smem, s, idx, wts, idw, logits, corr, T, n,
                     n_real, top, G, keep, scale);
}

// ---- silu_sections ---------------------------------------------------------
template <typename A>
__global__ void __launch_bounds__(256) silu_sections_kernel(
    float* __restrict__ out, const A* __restrict__ proj, long ld, int o0,
    int n0, int o1, int n1, int o2, int n2, long T) {
  const int tot = n0 + n1 + n2;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * tot) return;
  const long t = i / tot;
  const int c = (int)(i - t * tot);
  const int col = c < n0 ? o0 + c : (c < n0 + n1 ? o1 + c - n0 : o2 + c - n0 - n1);
  const float z = ldf<A>(proj + t * ld + col);
  out[i] = z * sigmoid_f(z);
}

// bf16, 8 columns (16 bytes in, 32 bytes out) a thread
__global__ void __launch_bounds__(256) silu_sections_vec_kernel(
    float* __restrict__ out, const u16* __restrict__ proj, long ld, int o0,
    int n0, int o1, int n1, int o2, int n2, long T) {
  const int tot = n0 + n1 + n2, tot8 = tot / 8;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * tot8) return;
  const long t = i / tot8;
  const int c = (int)(i - t * tot8) * 8;
  const int col = c < n0 ? o0 + c : (c < n0 + n1 ? o1 + c - n0 : o2 + c - n0 - n1);
  float z[8];
  bf8_to_f32(*(const u16x8*)(proj + t * ld + col), z);
  f32x4 a, b;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    a[e] = z[e] * sigmoid_f(z[e]);
    b[e] = z[e + 4] * sigmoid_f(z[e + 4]);
  }
  *(f32x4*)(out + t * tot + c) = a;
  *(f32x4*)(out + t * tot + c + 4) = b;
}

extern "C" void mix_silu_sections(float* out, const void* proj, long ld, int o0,
                                  int n0, int o1, int n1, int o2, int n2,
                                  long T, int f32, hipStream_t s) {
  const long n = T * (n0 + n1 + n2);
  if (n == 0) return;
  if (!f32 && ld % 8 == 0 && o0 % 8 == 0 && n0 % 8 == 0 && o1 % 8 == 0 &&
      n1 % 8 == 0 && o2 % 8 == 0 && n2 % 8 == 0) {
    hipLaunchKernelGGL(silu_sections_vec_kernel,
                       dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, s,
                       out, (const u16*)proj, ld, o0, n0, o1, n1, o2, n2, T);
    return;
  }
  const unsigned grid = (unsigned)((n + 255) / 256);
  if (f32)
    hipLaunchKernelGGL(silu_sections_kernel<float>, dim3(grid), dim3(256), 0, s,
                       out, (const float*)proj, ld, o0, n0, o1, n1, o2, n2, T);
  else
    hipLaunchKernelGGL(silu_sections_kernel<u16>, dim3(grid), dim3(256), 0, s,
                       out, (const u16*)proj, ld, o0, n0, o1, n1, o2, n2, T);
}

// ---- gated_group_norm ------------------------------------------------------
// One 256-thread block per (token, part of the row).
template <typename A>
__global__ void __launch_bounds__(256) gated_group_norm_kernel(
    A* __restrict__ out, long ldo, int out_off, const float* __restrict__ o,
    const A* __restrict__ proj, long ld, int g_off,
    const float* __restrict__ nw, float eps, int n, int parts,
    int gate_first) {
  __shared__ float red[4];
  const long t = blockIdx.x / parts;
  const int part = blockIdx.x % parts;
  const int m = n / parts, c0 = part * m;
  const float* orow = o + t * n + c0;
  const A* grow = proj + t * ld + g_off + c0;
  float ssq = 0.f;
  for (int c = threadIdx.x; c < m; c += 256) {
    float v = orow[c];
    if (gate_first) {
      const float z = ldf<A>(grow + c);
      v *= z * sigmoid_f(z);
    }
    ssq += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum_256(ssq, red) / (float)m + eps);
  A* dst = out + t * ldo + out_off + c0;
  for (int c = threadIdx.x; c < m; c += 256) {
    const float z = ldf<A>(grow + c);
    float v = orow[c];
    if (gate_first) v *= z * sigmoid_f(z);
    v *= inv * nw[c0 + c];
    if (!gate_first) v *= sigmoid_f(z);
    stf<A>(dst + c, v);
  }
}

extern "C" void mix_gated_group_norm(void* out, long ldo, int out_off,
                                     const float* o, const void* proj, long ld,
                                     int g_off, const float* nw, float eps,
                                     long T, int n, int parts, int gate_first,
                                     int f32, hipStream_t s) {
  if (T == 0) return;
  const unsigned grid = (unsigned)(T * parts);
  if (f32)
    hipLaunchKernelGGL(gated_group_norm_kernel<float>, dim3(grid), dim3(256), 0,
                       s, (float*)out, ldo, out_off, o, (const float*)proj, ld,
                       g_off, nw, eps, n, parts, gate_first);
  else
    hipLaunchKernelGGL(gated_group_norm_kernel<u16>, dim3(grid), dim3(256), 0,
                       s, (u16*)out, ldo, out_off, o, (const u16*)proj, ld,
                       g_off, nw, eps, n, parts, gate_first);
}
