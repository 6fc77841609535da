// Row-wise pieces of layer-list decoders that keep every layer's result:
//   token_embed       X0 = scale * token row + hashed-bigram row + position
//                     sinusoid
//   weighted_rmsnorm  h = n(x) * w
//   norm_residual     r = x_in + n(y) * w_post -> x_out; optionally the
//                     depth-weighted sum z = sum_j d[j] * X_j over the kept
//                     layer results (the newest of which is r) -> mix_out;
//                     optionally the next sublayer's input h = n(z) * w_next
//   poly_act          a n(z) + b n(z^2) + c n(z^3) + e  (PolyNorm)
// n(z) = z / sqrt(mean(z^2) + eps) over a row. All sums, norms and the
// streams are fp32; `A` is the activation type. One 256-thread block a row;
// a thread touches the same columns in every pass, so a pass may read back
// what the pass before it wrote (also when buffers alias) without a barrier
// of its own. Second passes hit cache.
#include "mix_common.h"

template <typename A>
__global__ void token_embed_kernel(
    float* __restrict__ out, const long* __restrict__ ids,
    const long* __restrict__ prev, const long* __restrict__ pos,
    const A* __restrict__ embed, const A* __restrict__ bigram, long buckets,
    long mul_prev, long mul_cur, const float* __restrict__ inv_freq,
    float scale, int W) {
  const long t = blockIdx.x;
  const long id = ids[t];
  const A* er = embed + id * W;
  const A* br = nullptr;
  if (bigram) {
    const long pv = prev[t];
    const long row = pv < 0 ? buckets : (pv * mul_prev + id * mul_cur) % buckets;
    br = bigram + row * W;
  }
  const float p = (float)pos[t];
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float x = ldf<A>(er + c) * scale;
    if (br) x += ldf<A>(br + c);
    if (inv_freq) {
      const float ang = p * inv_freq[c >> 1];
      x += (c & 1) ? cosf(ang) : sinf(ang);
    }
    out[t * W + c] = x;
  }
}

template <typename A>
__global__ void weighted_rmsnorm_kernel(A* __restrict__ out,
                                        const float* __restrict__ x,
                                        const float* __restrict__ w, float eps,
                                        int W) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const float* xr = x + row * W;
  float ssq = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) ssq += xr[c] * xr[c];
  const float inv = 1.f / sqrtf(block_sum_256(ssq, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    stf<A>(out + row * W + c, xr[c] * inv * w[c]);
}

template <typename A>
__global__ void norm_residual_kernel(
    const float* x_in, const A* __restrict__ y,
    const float* __restrict__ w_post, float eps, float* x_out,
    const float* stack, long stack_stride, const float* __restrict__ depth_w,
    int n_depth, float* mix_out, const float* __restrict__ next_w,
    A* __restrict__ h_out, int W) {
  __shared__ float red[8];
  const long row = blockIdx.x;
  const A* yr = y + row * W;
  float ssq = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = ldf<A>(yr + c);
    ssq += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum_256(ssq, red) / (float)W + eps);
  const float dlast = n_depth > 0 ? depth_w[n_depth - 1] : 1.f;
  float ssz = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float r = x_in[row * W + c] + ldf<A>(yr + c) * inv * w_post[c];
    x_out[row * W + c] = r;
    float z = r;
    if (n_depth > 0) {
      z = 0.f;
      for (int j = 0; j + 1 < n_depth; ++j)
        z += depth_w[j] * stack[j * stack_stride + row * W + c];
      z += dlast * r;
      mix_out[row * W + c] = z;
    }
    ssz += z * z;
  }
  if (!next_w) return;
  const float invz = 1.f / sqrtf(block_sum_256(ssz, red + 4) / (float)W + eps);
  const float* zr = (n_depth > 0 ? mix_out : x_out) + row * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    stf<A>(h_out + row * W + c, zr[c] * invz * next_w[c]);
}

template <typename A>
__global__ void poly_act_kernel(A* __restrict__ out, const A* __restrict__ z,
                                const float* __restrict__ coef, float eps,
                                int F) {
  __shared__ float red[12];
  const long row = blockIdx.x;
  const A* zr = z + row * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += blockDim.x) {
    const float v = ldf<A>(zr + c);
    const float v2 = v * v, v3 = v2 * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v3 * v3;
  }
  s1 = block_sum_256(s1, red);
  s2 = block_sum_256(s2, red + 4);
  s3 = block_sum_256(s3, red + 8);
  const float i1 = coef[0] / sqrtf(s1 / (float)F + eps);
  const float i2 = coef[1] / sqrtf(s2 / (float)F + eps);
  const float i3 = coef[2] / sqrtf(s3 / (float)F + eps);
  const float e = coef[3];
  for (int c = threadIdx.x; c < F; c += blockDim.x) {
    const float v = ldf<A>(zr + c);
    const float v2 = v * v;
    stf<A>(out + row * F + c, v * i1 + v2 * i2 + v2 * v * i3 + e);
  }
}


// ---- vector forms: a thread keeps its share of the row in registers --------
// NCH chunks of V elements a thread (chunk k of thread t starts at column
// (t + 256 k) V), so a row is read from memory once and every access is a
// 16-byte (or, for 4 bf16, 8-byte) vector. Rows must be a multiple of V long
// and at most 256 * V * NCH; other rows take the plain kernels above.
template <typename A, int V> struct VecOf {
  typedef A type __attribute__((ext_vector_type(V)));
};

template <typename A, int NCH>
__global__ void __launch_bounds__(256) norm_residual_vec_kernel(
    const float* x_in, const A* __restrict__ y,
    const float* __restrict__ w_post, float eps, float* x_out,
    const float* stack, long stack_stride, const float* __restrict__ depth_w,
    int n_depth, float* mix_out, const float* __restrict__ next_w,
    A* __restrict__ h_out, int W) {
  typedef typename VecOf<A, 4>::type avec;
  __shared__ float red[8];
  const long row = blockIdx.x;
  const long base = row * W;
  float yv[NCH][4];
  float ssq = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + 256 * k) * 4;
    if (c < W) {
      const avec v = *(const avec*)(y + base + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        A ve = v[e];
        yv[k][e] = ldf<A>(&ve);
        ssq += yv[k][e] * yv[k][e];
      }
    }
  }
  const float inv = 1.f / sqrtf(block_sum_256(ssq, red) / (float)W + eps);
  const float dlast = n_depth > 0 ? depth_w[n_depth - 1] : 1.f;
  float ssz = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + 256 * k) * 4;
    if (c < W) {
      const f32x4 xi = *(const f32x4*)(x_in + base + c);
      const f32x4 wp = *(const f32x4*)(w_post + c);
      f32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = xi[e] + yv[k][e] * inv * wp[e];
      *(f32x4*)(x_out + base + c) = r;
      f32x4 z = r;
      if (n_depth > 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) z[e] = 0.f;
        for (int j = 0; j + 1 < n_depth; ++j) {
          const f32x4 sj = *(const f32x4*)(stack + j * stack_stride + base + c);
          const float dj = depth_w[j];
#pragma unroll
          for (int e = 0; e < 4; ++e) z[e] += dj * sj[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) z[e] += dlast * r[e];
        *(f32x4*)(mix_out + base + c) = z;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        yv[k][e] = z[e];
        ssz += z[e] * z[e];
      }
    }
  }
  if (!next_w) return;
  const float invz = 1.f / sqrtf(block_sum_256(ssz, red + 4) / (float)W + eps);
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + 256 * k) * 4;
    if (c < W) {
      const f32x4 nw = *(const f32x4*)(next_w + c);
      avec o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        A oe;
        stf<A>(&oe, yv[k][e] * invz * nw[e]);
        o[e] = oe;
      }
      *(avec*)(h_out + base + c) = o;
    }
  }
}

template <typename A, int V, int NCH>
__global__ void __launch_bounds__(256) poly_act_vec_kernel(
    A* __restrict__ out, const A* __restrict__ z,
    const float* __restrict__ coef, float eps, int F) {
  typedef typename VecOf<A, V>::type avec;
  __shared__ float red[12];
  const long base = (long)blockIdx.x * F;
  float zv[NCH][V];
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + 256 * k) * V;
    if (c < F) {
      const avec v = *(const avec*)(z + base + c);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        A ve = v[e];
        const float x = ldf<A>(&ve);
        const float x2 = x * x, x3 = x2 * x;
        zv[k][e] = x;
        s1 += x2;
        s2 += x2 * x2;
        s3 += x3 * x3;
      }
    }
  }
  s1 = block_sum_256(s1, red);
  s2 = block_sum_256(s2, red + 4);
  s3 = block_sum_256(s3, red + 8);
  const float i1 = coef[0] / sqrtf(s1 / (float)F + eps);
  const float i2 = coef[1] / sqrtf(s2 / (float)F + eps);
  const float i3 = coef[2] / sqrtf(s3 / (float)F + eps);
  const float cc = coef[3];
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + 256 * k) * V;
    if (c < F) {
      avec o;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float x = zv[k][e], x2 = x * x;
        A oe;
        stf<A>(&oe, x * i1 + x2 * i2 + x2 * x * i3 + cc);
        o[e] = oe;
      }
      *(avec*)(out + base + c) = o;
    }
  }
}

extern "C" void mix_token_embed(float* out, const long* ids, const long* prev,
                                const long* pos, const void* embed,
                                const void* bigram, long buckets,
                                long mul_prev, long mul_cur,
                                const float* inv_freq, float scale, long T,
                                int W, int f32, hipStream_t s) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL(token_embed_kernel<float>, dim3((unsigned)T), dim3(256),
                       0, s, out, ids, prev, pos, (const float*)embed,
                       (const float*)bigram, buckets, mul_prev, mul_cur,
                       inv_freq, scale, W);
  else
    hipLaunchKernelGGL(token_embed_kernel<u16>, dim3((unsigned)T), dim3(256), 0,
                       s, out, ids, prev, pos, (const u16*)embed,
                       (const u16*)bigram, buckets, mul_prev, mul_cur,
                       inv_freq, scale, W);
}

extern "C" void mix_weighted_rmsnorm(void* out, const float* x, const float* w,
                                     float eps, long T, int W, int f32,
                                     hipStream_t s) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL(weighted_rmsnorm_kernel<float>, dim3((unsigned)T),
                       dim3(256), 0, s, (float*)out, x, w, eps, W);
  else
    hipLaunchKernelGGL(weighted_rmsnorm_kernel<u16>, dim3((unsigned)T),
                       dim3(256), 0, s, (u16*)out, x, w, eps, W);
}

extern "C" void mix_norm_residual(const float* x_in, const void* y,
                                  const float* w_post, float eps, float* x_out,
                                  const float* stack, long stack_stride,
                                  const float* depth_w, int n_depth,
                                  float* mix_out, const float* next_w,
                                  void* h_out, long T, int W, int f32,
                                  hipStream_t s) {
  if (T == 0) return;
  if (W % 4 == 0 && W <= 256 * 4 * 8) {
    const int nch = (W / 4 + 255) / 256;
#define LAUNCH_NR(AA, NN)                                                     \
  hipLaunchKernelGGL((norm_residual_vec_kernel<AA, NN>), dim3((unsigned)T),   \
                     dim3(256), 0, s, x_in, (const AA*)y, w_post, eps, x_out, \
                     stack, stack_stride, depth_w, n_depth, mix_out, next_w,  \
                     (AA*)h_out, W)
#define PICK_NR(AA)                                \
  if (nch <= 1) LAUNCH_NR(AA, 1);                  \
  else if (nch <= 2) LAUNCH_NR(AA, 2);             \
  else if (nch <= 4) LAUNCH_NR(AA, 4);             \
  else LAUNCH_NR(AA, 8);
    if (f32) { PICK_NR(float) } else { PICK_NR(u16) }
#undef PICK_NR
#undef LAUNCH_NR
    return;
  }
  if (f32)
    hipLaunchKernelGGL(norm_residual_kernel<float>, dim3((unsigned)T),
                       dim3(256), 0, s, x_in, (const float*)y, w_post, eps,
                       x_out, stack, stack_stride, depth_w, n_depth, mix_out,
                       next_w, (float*)h_out, W);
  else
    hipLaunchKernelGGL(norm_residual_kernel<u16>, dim3((unsigned)T), dim3(256),
                       0, s, x_in, (const u16*)y, w_post, eps, x_out, stack,
                       stack_stride, depth_w, n_depth, mix_out, next_w,
                       (u16*)h_out, W);
}

extern "C" void mix_poly_act(void* out, const void* z, const float* coef,
                             float eps, long T, int F, int f32, hipStream_t s) {
  if (T == 0) return;
  {
    const int V = f32 ? 4 : 8;
    if (F % V == 0 && F <= 256 * V * 8) {
      const int nch = (F / V + 255) / 256;
#define LAUNCH_PA(AA, VV, NN)                                                \
  hipLaunchKernelGGL((poly_act_vec_kernel<AA, VV, NN>), dim3((unsigned)T),   \
                     dim3(256), 0, s, (AA*)out, (const AA*)z, coef, eps, F)
#define PICK_PA(AA, VV)                            \
  if (nch <= 1) LAUNCH_PA(AA, VV, 1);              \
  else if (nch <= 2) LAUNCH_PA(AA, VV, 2);         \
  else if (nch <= 4) LAUNCH_PA(AA, VV, 4);         \
  else LAUNCH_PA(AA, VV, 8);
      if (f32) { PICK_PA(float, 4) } else { PICK_PA(u16, 8) }
#undef PICK_PA
#undef LAUNCH_PA
      return;
    }
  }
  if (f32)
    hipLaunchKernelGGL(poly_act_kernel<float>, dim3((unsigned)T), dim3(256), 0,
                       s, (float*)out, (const float*)z, coef, eps, F);
  else
    hipLaunchKernelGGL(poly_act_kernel<u16>, dim3((unsigned)T), dim3(256), 0, s,
                       (u16*)out, (const u16*)z, coef, eps, F);
}
