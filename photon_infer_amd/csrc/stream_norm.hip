// Kernels around a residual stream whose sublayers are normalised on the way OUT:
//   x <- x + mult * norm(y; w),   y = a                               (one branch)
//                                 y = (norm(a; wa) + norm(b; wb)) / 2 (two branches side by side)
// with norm(v; w) = v / sqrt(mean(v^2) + eps) * w.  One block per token row does the branch
// norms, their mean, the outer norm, the scaled add into the float32 stream and, when asked,
// the copy of the new stream in the activation type that the next sublayer's products read.
// Sums of squares, roots and the stream are float32 throughout.  Weights are float32 (a weight
// stored around zero is handed over as 1 + w).
#include "common.h"

template <typename TH>
__global__ __launch_bounds__(256) void branch_norm_add_kernel(float* __restrict__ x, TH* __restrict__ h, const float* __restrict__ a,
                                                              const float* __restrict__ wa, const float* __restrict__ b,
                                                              const float* __restrict__ wb, const float* __restrict__ wo,
                                                              float eps, float mult, int D) {
  extern __shared__ float y[];          // D floats
  __shared__ float scratch[16];
  const long row = blockIdx.x;
  const float* ar = a + row * D;
  const float* br = b ? b + row * D : nullptr;
  float sa = 0.f, sb = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float va = ar[d];
    sa = fmaf(va, va, sa);
    if (br) {
      const float vb = br[d];
      sb = fmaf(vb, vb, sb);
    }
  }
  float sy = 0.f;
  if (wa) {
    const float ra = 1.0f / sqrtf(block_sum(sa, scratch) / D + eps);
    const float rb = br ? 1.0f / sqrtf(block_sum(sb, scratch) / D + eps) : 0.f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      float v = ar[d] * ra * wa[d];
      if (br) v = 0.5f * (v + br[d] * rb * wb[d]);
      y[d] = v;
      sy = fmaf(v, v, sy);
    }
  } else {
    for (int d = threadIdx.x; d < D; d += blockDim.x) y[d] = ar[d];
    sy = sa;
  }
  const float ry = 1.0f / sqrtf(block_sum(sy, scratch) / D + eps);
  float* xr = x + row * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = xr[d] + mult * (y[d] * ry * wo[d]);
    xr[d] = v;
    if (h) h[row * D + d] = from_float<TH>(v);
  }
}

// The same for rows of whole 16-byte groups, at most VPT groups per thread: a thread keeps its
// values in registers between the passes, both branches' sums of squares share one reduction,
// and every access is 16 bytes wide.  Few rows (decode steps) are a matter of latency: as many
// threads per row as the row has groups.
template <typename TH, int VPT>
__global__ __launch_bounds__(1024) void branch_norm_add_wide_kernel(float* __restrict__ x, TH* __restrict__ h, const float* __restrict__ a,
                                                                    const float* __restrict__ wa, const float* __restrict__ b,
                                                                    const float* __restrict__ wb, const float* __restrict__ wo,
                                                                    float eps, float mult, int D) {
  __shared__ float scratch[32];
  const long row = blockIdx.x;
  const int groups = D / 4;
  float4 va[VPT], vb[VPT], xo[VPT];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int g = threadIdx.x + v * blockDim.x;
    const bool in = g < groups;
    va[v] = in ? reinterpret_cast<const float4*>(a + row * D)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
    vb[v] = (in && b) ? reinterpret_cast<const float4*>(b + row * D)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
    xo[v] = in ? reinterpret_cast<const float4*>(x + row * D)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
    sa = fmaf(va[v].x, va[v].x, sa); sa = fmaf(va[v].y, va[v].y, sa); sa = fmaf(va[v].z, va[v].z, sa); sa = fmaf(va[v].w, va[v].w, sa);
    sb = fmaf(vb[v].x, vb[v].x, sb); sb = fmaf(vb[v].y, vb[v].y, sb); sb = fmaf(vb[v].z, vb[v].z, sb); sb = fmaf(vb[v].w, vb[v].w, sb);
  }
  float sy = sa, unused = 0.f;
  if (wa) {
    block_sum2(sa, sb, scratch);
    const float ra = 1.0f / sqrtf(sa / D + eps);
    const float rb = b ? 1.0f / sqrtf(sb / D + eps) : 0.f;
    sy = 0.f;
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
      const int g = threadIdx.x + v * blockDim.x;
      if (g >= groups) continue;
      const float4 w1 = reinterpret_cast<const float4*>(wa)[g];
      float y[4] = {va[v].x * ra * w1.x, va[v].y * ra * w1.y, va[v].z * ra * w1.z, va[v].w * ra * w1.w};
      if (b) {
        const float4 w2 = reinterpret_cast<const float4*>(wb)[g];
        y[0] = 0.5f * (y[0] + vb[v].x * rb * w2.x);
        y[1] = 0.5f * (y[1] + vb[v].y * rb * w2.y);
        y[2] = 0.5f * (y[2] + vb[v].z * rb * w2.z);
        y[3] = 0.5f * (y[3] + vb[v].w * rb * w2.w);
      }
      va[v] = make_float4(y[0], y[1], y[2], y[3]);
      sy = fmaf(y[0], y[0], sy); sy = fmaf(y[1], y[1], sy); sy = fmaf(y[2], y[2], sy); sy = fmaf(y[3], y[3], sy);
    }
  }
  block_sum2(sy, unused, scratch);
  const float ry = 1.0f / sqrtf(sy / D + eps);
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int g = threadIdx.x + v * blockDim.x;
    if (g >= groups) continue;
    const float4 w3 = reinterpret_cast<const float4*>(wo)[g];
    const float4 r = make_float4(xo[v].x + mult * (va[v].x * ry * w3.x), xo[v].y + mult * (va[v].y * ry * w3.y),
                                 xo[v].z + mult * (va[v].z * ry * w3.z), xo[v].w + mult * (va[v].w * ry * w3.w));
    reinterpret_cast<float4*>(x + row * D)[g] = r;
    if (h) {
      TH* hp = h + row * D + 4 * (long)g;
      hp[0] = from_float<TH>(r.x); hp[1] = from_float<TH>(r.y); hp[2] = from_float<TH>(r.z); hp[3] = from_float<TH>(r.w);
    }
  }
}

// x (float32 stream) += mult * norm(...); h (optional, h_dtype) = the new stream.
// wa == null: a is taken as it is (one branch, no inner norm); b == null: one branch.
extern "C" int pi_branch_norm_add(float* x, void* h, int h_dtype, const float* a, const float* wa, const float* b,
                                  const float* wb, const float* wo, float eps, float mult, int T, int D, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && D > 0 && D <= 40000, "branch norm: bad sizes T=%d D=%d", T, D);
  PI_REQUIRE(x && a && wo, "branch norm: the stream, a branch and the outer weight are needed");
  PI_REQUIRE(!b || (wa && wb), "branch norm: two branches need both their weights");
  if (T == 0) return 0;
  PI_REQUIRE(!h || h_dtype == PI_BF16 || h_dtype == PI_F32, "branch norm: unsupported activation dtype %d", h_dtype);
  const bool aligned = D % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)a % 16 == 0 && (!b || (uintptr_t)b % 16 == 0) &&
                       (uintptr_t)wo % 16 == 0 && (!wa || (uintptr_t)wa % 16 == 0) && (!wb || (uintptr_t)wb % 16 == 0);
  if (aligned && D / 4 <= 4 * 1024) {
    const int groups = D / 4;
    // few rows: a thread per group (latency); many rows: fewer, fatter threads
    int threads = T <= 512 ? groups : (groups + 3) / 4;
    threads = threads > 1024 ? 1024 : ((threads + PI_WAVE - 1) / PI_WAVE) * PI_WAVE;
    const int vpt = (groups + threads - 1) / threads;
#define BN_GO(TH, V) hipLaunchKernelGGL((branch_norm_add_wide_kernel<TH, V>), dim3(T), dim3(threads), 0, stream, x, (TH*)h, a, wa, b, wb, wo, eps, mult, D)
#define BN_PICK(TH)            \
  do {                         \
    if (vpt <= 1) BN_GO(TH, 1); \
    else if (vpt <= 2) BN_GO(TH, 2); \
    else BN_GO(TH, 4);         \
  } while (0)
    if (h && h_dtype == PI_BF16) BN_PICK(bf16_t);
    else BN_PICK(float);
#undef BN_PICK
#undef BN_GO
    return pi_check_launch("branch_norm_add_wide");
  }
  const size_t lds = (size_t)D * sizeof(float);
  if (h && h_dtype == PI_BF16)
    hipLaunchKernelGGL(branch_norm_add_kernel<bf16_t>, dim3(T), dim3(256), lds, stream, x, (bf16_t*)h, a, wa, b, wb, wo, eps, mult, D);
  else if (!h || h_dtype == PI_F32)
    hipLaunchKernelGGL(branch_norm_add_kernel<float>, dim3(T), dim3(256), lds, stream, x, (float*)h, a, wa, b, wb, wo, eps, mult, D);
  else
    return pi_fail("branch norm: unsupported activation dtype %d", h_dtype);
  return pi_check_launch("branch_norm_add");
}

// ---------------------------------------------------------------- layer norm with weight and bias
// LN(v; w, b) = (v - mean) / sqrt(mean of squared deviations + eps) * w + b, all float32.  The row sits in
// LDS between the passes: the mean first, then the deviations' squares, so that nothing is cancelled.
__device__ inline void layer_norm_stats(const float* row, int D, float eps, float* scratch, float& mean, float& rinv) {
  float s = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) s += row[d];
  mean = block_sum(s, scratch) / D;
  float q = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float dev = row[d] - mean;
    q = fmaf(dev, dev, q);
  }
  rinv = 1.0f / sqrtf(block_sum(q, scratch) / D + eps);
}

// out[m, :] = LN(x[rows[m] or m, :]; w, b) in the activation type
template <typename TO>
__global__ __launch_bounds__(256) void layer_norm_kernel(TO* __restrict__ out, const float* __restrict__ x, const int* __restrict__ rows,
                                                         const float* __restrict__ w, const float* __restrict__ b, float eps, int D,
                                                         int x_rows) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const long m = blockIdx.x;
  const long r = rows ? rows[m] : m;
  const bool ok = r >= 0 && r < x_rows;          // a row outside the stream gives NaN, no fault
  for (int d = threadIdx.x; d < D; d += blockDim.x) row[d] = ok ? x[r * D + d] : NAN;
  __syncthreads();
  float mean, rinv;
  layer_norm_stats(row, D, eps, scratch, mean, rinv);
  for (int d = threadIdx.x; d < D; d += blockDim.x) out[m * D + d] = from_float<TO>((row[d] - mean) * rinv * w[d] + b[d]);
}

// The same for rows of whole 16-byte groups, at most VPT groups per thread: a thread keeps its values in registers
// between the passes and every access is 16 bytes wide.  Few rows (decode steps) are a matter of latency: as many
// threads per row as the row has groups.
__device__ inline float sum4(const float4& v) { return (v.x + v.y) + (v.z + v.w); }
__device__ inline float4 sub4(const float4& v, float m) { return make_float4(v.x - m, v.y - m, v.z - m, v.w - m); }
__device__ inline float dot4(const float4& v) { return fmaf(v.w, v.w, fmaf(v.z, v.z, fmaf(v.y, v.y, v.x * v.x))); }
__device__ inline float4 affine4(const float4& d, float r, const float4& w, const float4& b) {
  return make_float4(fmaf(d.x * r, w.x, b.x), fmaf(d.y * r, w.y, b.y), fmaf(d.z * r, w.z, b.z), fmaf(d.w * r, w.w, b.w));
}
template <typename TO> __device__ inline void store4(TO* p, const float4& v);
template <> __device__ inline void store4<float>(float* p, const float4& v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ inline void store4<bf16_t>(bf16_t* p, const float4& v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(f32x2_to_bf16x2_bits(v.x, v.y), f32x2_to_bf16x2_bits(v.z, v.w));
}

// mean and 1 / sqrt(variance + eps) of a row whose groups sit in v[VPT] (groups beyond the row are zero and not counted);
// v becomes the deviations from the mean
template <int VPT>
__device__ inline float centre_and_scale(float4 (&v)[VPT], int groups, int D, float eps, float* scratch) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) s += sum4(v[i]);
  const float mean = block_sum(s, scratch) / D;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const bool in = (int)(threadIdx.x + i * blockDim.x) < groups;
    v[i] = in ? sub4(v[i], mean) : make_float4(0.f, 0.f, 0.f, 0.f);
    q += dot4(v[i]);
  }
  return 1.0f / sqrtf(block_sum(q, scratch) / D + eps);
}

template <typename TO, int VPT>
__global__ __launch_bounds__(1024) void layer_norm_wide_kernel(TO* __restrict__ out, const float* __restrict__ x, const int* __restrict__ rows,
                                                               const float* __restrict__ w, const float* __restrict__ b, float eps, int D,
                                                               int x_rows) {
  __shared__ float scratch[16];
  const long m = blockIdx.x;
  const long r = rows ? rows[m] : m;
  const bool ok = r >= 0 && r < x_rows;
  const int groups = D / 4;
  float4 v[VPT], wv[VPT], bv[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int g = threadIdx.x + i * blockDim.x;
    const bool in = g < groups;
    v[i] = !in ? make_float4(0.f, 0.f, 0.f, 0.f) : ok ? reinterpret_cast<const float4*>(x + r * D)[g] : make_float4(NAN, NAN, NAN, NAN);
    wv[i] = in ? reinterpret_cast<const float4*>(w)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
    bv[i] = in ? reinterpret_cast<const float4*>(b)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  const float rinv = centre_and_scale<VPT>(v, groups, D, eps, scratch);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int g = threadIdx.x + i * blockDim.x;
    if (g < groups) store4<TO>(out + m * D + 4 * (long)g, affine4(v[i], rinv, wv[i], bv[i]));
  }
}

// threads per row and groups per thread for the wide kernels: few rows, a thread per group (latency); many rows, fewer, fatter threads
static inline bool wide_row_shape(int T, int D, int& threads, int& vpt) {
  if (D % 4) return false;
  const int groups = D / 4;
  threads = T <= 512 ? groups : (groups + 3) / 4;
  threads = threads > 1024 ? 1024 : ((threads + PI_WAVE - 1) / PI_WAVE) * PI_WAVE;
  vpt = (groups + threads - 1) / threads;
  return vpt <= 4;
}

extern "C" int pi_layer_norm(void* out, int out_dtype, const float* x, const int* rows, const float* w, const float* b, float eps,
                             int M, int D, int x_rows, hipStream_t stream) {
  PI_REQUIRE(M >= 0 && D > 0 && D <= 16000 && x_rows >= 0, "layer norm: bad sizes M=%d D=%d", M, D);
  PI_REQUIRE(out && x && w && b, "layer norm: output, input, weight and bias are needed");
  PI_REQUIRE(out_dtype == PI_F32 || out_dtype == PI_BF16, "layer norm: unsupported dtype %d", out_dtype);
  if (M == 0) return 0;
  int wide_threads = 0, vpt = 0;
  const bool aligned = (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)b % 16 == 0 && (uintptr_t)out % 16 == 0;
  if (aligned && wide_row_shape(M, D, wide_threads, vpt)) {
#define LN_GO(TO, V) hipLaunchKernelGGL((layer_norm_wide_kernel<TO, V>), dim3(M), dim3(wide_threads), 0, stream, (TO*)out, x, rows, w, b, eps, D, x_rows)
#define LN_PICK(TO) do { if (vpt <= 1) LN_GO(TO, 1); else if (vpt <= 2) LN_GO(TO, 2); else LN_GO(TO, 4); } while (0)
    if (out_dtype == PI_F32) LN_PICK(float); else LN_PICK(bf16_t);
#undef LN_PICK
#undef LN_GO
    return pi_check_launch("layer_norm_wide");
  }
  const int threads = D >= 1024 ? 256 : (D >= 256 ? 128 : 64);
  const size_t lds = (size_t)D * sizeof(float);
  if (out_dtype == PI_F32)
    hipLaunchKernelGGL(layer_norm_kernel<float>, dim3(M), dim3(threads), lds, stream, (float*)out, x, rows, w, b, eps, D, x_rows);
  else
    hipLaunchKernelGGL(layer_norm_kernel<bf16_t>, dim3(M), dim3(threads), lds, stream, (bf16_t*)out, x, rows, w, b, eps, D, x_rows);
  return pi_check_launch("layer_norm");
}

// A sublayer's result joins the stream through a layer norm, and the next sublayer's input is made on the way:
//   y = a (+ a_bias)                                                      (one branch)
//   y = (rms(a (+ a_bias); wa) + rms(b; wb)) / 2                           (two branches side by side)
//   x <- x + LN(y; pw, pb);   h = LN(x; nw, nb)   (nw null: no h)
// with rms(v; w) = v / sqrt(mean(v^2) + eps) * w.  One block per token; the row stays in LDS throughout.
template <typename TH>
__global__ __launch_bounds__(256) void sandwich_norm_add_kernel(float* __restrict__ x, TH* __restrict__ h, const float* __restrict__ a,
                                                                const float* __restrict__ a_bias, const float* __restrict__ wa,
                                                                const float* __restrict__ b, const float* __restrict__ wb,
                                                                const float* __restrict__ pw, const float* __restrict__ pb,
                                                                const float* __restrict__ nw, const float* __restrict__ nb, float eps,
                                                                int D) {
  extern __shared__ float row[];
  __shared__ float scratch[32];
  const long t = blockIdx.x;
  const float* ar = a + t * D;
  const float* br = b ? b + t * D : nullptr;
  if (wa) {
    float sa = 0.f, sb = 0.f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      const float va = ar[d] + (a_bias ? a_bias[d] : 0.f);
      row[d] = va;
      sa = fmaf(va, va, sa);
      if (br) {
        const float vb = br[d];
        sb = fmaf(vb, vb, sb);
      }
    }
    block_sum2(sa, sb, scratch);
    const float ra = 1.0f / sqrtf(sa / D + eps), rb = br ? 1.0f / sqrtf(sb / D + eps) : 0.f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      float v = row[d] * ra * wa[d];
      if (br) v = 0.5f * (v + br[d] * rb * wb[d]);
      row[d] = v;
    }
  } else {
    for (int d = threadIdx.x; d < D; d += blockDim.x) row[d] = ar[d] + (a_bias ? a_bias[d] : 0.f);
  }
  __syncthreads();
  float mean, rinv;
  layer_norm_stats(row, D, eps, scratch, mean, rinv);
  float* xr = x + t * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = xr[d] + ((row[d] - mean) * rinv * pw[d] + pb[d]);
    xr[d] = v;
    row[d] = v;
  }
  if (!nw) return;
  __syncthreads();
  layer_norm_stats(row, D, eps, scratch, mean, rinv);
  for (int d = threadIdx.x; d < D; d += blockDim.x) h[t * D + d] = from_float<TH>((row[d] - mean) * rinv * nw[d] + nb[d]);
}

// The same with the row in registers and 16-byte accesses (see layer_norm_wide_kernel).
template <typename TH, int VPT>
__global__ __launch_bounds__(1024) void sandwich_norm_add_wide_kernel(float* __restrict__ x, TH* __restrict__ h, const float* __restrict__ a,
                                                                      const float* __restrict__ a_bias, const float* __restrict__ wa,
                                                                      const float* __restrict__ b, const float* __restrict__ wb,
                                                                      const float* __restrict__ pw, const float* __restrict__ pb,
                                                                      const float* __restrict__ nw, const float* __restrict__ nb,
                                                                      float eps, int D) {
  __shared__ float scratch[32];
  const long t = blockIdx.x;
  const int groups = D / 4;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 y[VPT], xo[VPT];
  float sa = 0.f, sb = 0.f;
  {
    float4 vb[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int g = threadIdx.x + i * blockDim.x;
      const bool in = g < groups;
      y[i] = in ? reinterpret_cast<const float4*>(a + t * D)[g] : zero;
      if (in && a_bias) {
        const float4 ab = reinterpret_cast<const float4*>(a_bias)[g];
        y[i] = make_float4(y[i].x + ab.x, y[i].y + ab.y, y[i].z + ab.z, y[i].w + ab.w);
      }
      vb[i] = (in && b) ? reinterpret_cast<const float4*>(b + t * D)[g] : zero;
      xo[i] = in ? reinterpret_cast<const float4*>(x + t * D)[g] : zero;
      sa += dot4(y[i]);
      sb += dot4(vb[i]);
    }
    if (wa) {
      block_sum2(sa, sb, scratch);
      const float ra = 1.0f / sqrtf(sa / D + eps), rb = b ? 1.0f / sqrtf(sb / D + eps) : 0.f;
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int g = threadIdx.x + i * blockDim.x;
        if (g >= groups) continue;
        const float4 w1 = reinterpret_cast<const float4*>(wa)[g];
        float4 v = make_float4(y[i].x * ra * w1.x, y[i].y * ra * w1.y, y[i].z * ra * w1.z, y[i].w * ra * w1.w);
        if (b) {
          const float4 w2 = reinterpret_cast<const float4*>(wb)[g];
          v = make_float4(0.5f * (v.x + vb[i].x * rb * w2.x), 0.5f * (v.y + vb[i].y * rb * w2.y), 0.5f * (v.z + vb[i].z * rb * w2.z),
                          0.5f * (v.w + vb[i].w * rb * w2.w));
        }
        y[i] = v;
      }
    }
  }
  float rinv = centre_and_scale<VPT>(y, groups, D, eps, scratch);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int g = threadIdx.x + i * blockDim.x;
    if (g >= groups) continue;
    const float4 l = affine4(y[i], rinv, reinterpret_cast<const float4*>(pw)[g], reinterpret_cast<const float4*>(pb)[g]);
    xo[i] = make_float4(xo[i].x + l.x, xo[i].y + l.y, xo[i].z + l.z, xo[i].w + l.w);
    reinterpret_cast<float4*>(x + t * D)[g] = xo[i];
  }
  if (!nw) return;
  rinv = centre_and_scale<VPT>(xo, groups, D, eps, scratch);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int g = threadIdx.x + i * blockDim.x;
    if (g < groups)
      store4<TH>(h + t * D + 4 * (long)g, affine4(xo[i], rinv, reinterpret_cast<const float4*>(nw)[g], reinterpret_cast<const float4*>(nb)[g]));
  }
}

extern "C" int pi_sandwich_norm_add(float* x, void* h, int h_dtype, const float* a, const float* a_bias, const float* wa,
                                    const float* b, const float* wb, const float* pw, const float* pb, const float* nw,
                                    const float* nb, float eps, int T, int D, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && D > 0 && D <= 16000, "norm and add: bad sizes T=%d D=%d", T, D);
  PI_REQUIRE(x && a && pw && pb, "norm and add: the stream, a result and the norm's weight and bias are needed");
  PI_REQUIRE(!b || (wa && wb), "norm and add: two branches need both their weights");
  PI_REQUIRE(!nw || (nb && h), "norm and add: the next norm needs its bias and a place for its result");
  PI_REQUIRE(!nw || h_dtype == PI_F32 || h_dtype == PI_BF16, "norm and add: unsupported activation dtype %d", h_dtype);
  if (T == 0) return 0;
  const bool f32 = !nw || h_dtype == PI_F32;
  int wide_threads = 0, vpt = 0;
  bool aligned = true;
  for (const void* p : {(const void*)x, (const void*)h, (const void*)a, (const void*)a_bias, (const void*)wa, (const void*)b, (const void*)wb,
                        (const void*)pw, (const void*)pb, (const void*)nw, (const void*)nb})
    aligned = aligned && (uintptr_t)p % 16 == 0;
  if (aligned && wide_row_shape(T, D, wide_threads, vpt)) {
#define SW_GO(TH, V) hipLaunchKernelGGL((sandwich_norm_add_wide_kernel<TH, V>), dim3(T), dim3(wide_threads), 0, stream, x, (TH*)h, a, a_bias, wa, b, wb, pw, pb, nw, nb, eps, D)
#define SW_PICK(TH) do { if (vpt <= 1) SW_GO(TH, 1); else if (vpt <= 2) SW_GO(TH, 2); else SW_GO(TH, 4); } while (0)
    if (f32) SW_PICK(float); else SW_PICK(bf16_t);
#undef SW_PICK
#undef SW_GO
    return pi_check_launch("sandwich_norm_add_wide");
  }
  const int threads = D >= 1024 ? 256 : (D >= 256 ? 128 : 64);
  const size_t lds = (size_t)D * sizeof(float);
  if (f32)
    hipLaunchKernelGGL(sandwich_norm_add_kernel<float>, dim3(T), dim3(threads), lds, stream, x, (float*)h, a, a_bias, wa, b, wb, pw, pb, nw, nb, eps, D);
  else
    hipLaunchKernelGGL(sandwich_norm_add_kernel<bf16_t>, dim3(T), dim3(threads), lds, stream, x, (bf16_t*)h, a, a_bias, wa, b, wb, pw, pb, nw, nb, eps, D);
  return pi_check_launch("sandwich_norm_add");
}

// ---------------------------------------------------------------- two attention maps into one head
// Differential attention: head n of kv group g holds the results a1 and a2 of two softmax maps over the same
// values.  In `attn` the maps are heads of their own, and a head's value vector may come in `split` equal pieces
// (each attended as a head of its own, so that heads whose values are a multiple of their keys' width fit kernels
// that want both alike): heads are ordered [g][map][piece][head within group], so that piece p of map m of group g
// is kv head (2 g + m) * split + p of the attention.  out[t, n, :] = mult * o / sqrt(mean(o^2) + eps),
// o = a1 - lam * a2, float32; one wave per (token, head).
template <typename TO, typename TI>
__global__ __launch_bounds__(PI_WAVE) void diff_combine_kernel(TO* __restrict__ out, const TI* __restrict__ attn, float lam, float eps,
                                                               float mult, int H, int G, int dv, int split) {
  const long t = blockIdx.x;
  const int n = blockIdx.y, lane = threadIdx.x;
  const int per = H / G, g = n / per, i = n % per, w = dv / split;      // w: a piece's width
  const TI* row = attn + t * 2 * H * dv;
  const long map_step = (long)split * per * w;                          // from map 1 to map 2 of a group
  float ss = 0.f;
  for (int c = lane; c < dv; c += PI_WAVE) {
    const long at = (((long)(2 * g) * split + c / w) * per + i) * w + c % w;
    const float o = fmaf(-lam, to_float(row[at + map_step]), to_float(row[at]));
    ss = fmaf(o, o, ss);
  }
  const float r = mult / sqrtf(wave_sum(ss) / dv + eps);
  for (int c = lane; c < dv; c += PI_WAVE) {
    const long at = (((long)(2 * g) * split + c / w) * per + i) * w + c % w;
    out[(t * H + n) * dv + c] = from_float<TO>(fmaf(-lam, to_float(row[at + map_step]), to_float(row[at])) * r);
  }
}

extern "C" int pi_diff_combine(void* out, int out_dtype, const void* attn, int in_dtype, float lam, float eps, float mult, int T, int H,
                               int G, int dv, int split, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && H > 0 && H <= 65535 && G > 0 && H % G == 0 && dv > 0, "two maps: bad sizes heads=%d kv_heads=%d vdim=%d", H, G, dv);
  PI_REQUIRE(split >= 1 && dv % split == 0, "two maps: values of %d do not come in %d equal pieces", dv, split);
  if (T == 0) return 0;
  const dim3 grid(T, H), block(PI_WAVE);
#define DC_GO(TO, TI) hipLaunchKernelGGL((diff_combine_kernel<TO, TI>), grid, block, 0, stream, (TO*)out, (const TI*)attn, lam, eps, mult, H, G, dv, split)
  if (out_dtype == PI_F32 && in_dtype == PI_F32) DC_GO(float, float);
  else if (out_dtype == PI_BF16 && in_dtype == PI_BF16) DC_GO(bf16_t, bf16_t);
  else if (out_dtype == PI_BF16 && in_dtype == PI_F32) DC_GO(bf16_t, float);
  else return pi_fail("two maps: unsupported dtypes out=%d in=%d", out_dtype, in_dtype);
#undef DC_GO
  return pi_check_launch("diff_combine");
}

template <typename TO>
__global__ void cast_stream_kernel(TO* __restrict__ out, const float* __restrict__ x, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_float<TO>(x[i]);
}

// out = the float32 stream in the activation type (for sublayers that read the stream itself)
extern "C" int pi_cast_stream(void* out, int out_dtype, const float* x, long n, hipStream_t stream) {
  PI_REQUIRE(n >= 0 && out_dtype == PI_BF16, "cast: only float32 -> bfloat16 is a copy worth making (dtype %d)", out_dtype);
  if (n == 0) return 0;
  hipLaunchKernelGGL(cast_stream_kernel<bf16_t>, dim3(ceil_div(n, 256)), dim3(256), 0, stream, (bf16_t*)out, x, n);
  return pi_check_launch("cast_stream");
}

// ---------------------------------------------------------------- queries and keys normalised, then into the cache
// One block per token.  The projection row (float32) holds [q: nh*hd | k: nkv*hd | v: nkv*vd | gate: ng]
// (without the k and v columns when has_kv is 0: a layer that reads another layer's keys and values).
//   per_head 0:  q <- q / sqrt(mean over ALL nh*hd entries + eps) * wq     (wq / wk null: no norm of that projection)
//                k <- k / sqrt(mean over all nkv*hd entries + eps) * wk
//   per_head 1:  every head of q and of k divided by the root mean square of its own hd entries (+ eps inside the
//                root), times wq / wk where they are given
//   q times the token's temperature 1 + coef * ln(floor((p + 1) / every) + 1)           (coef 0: none)
//   k -> key pages [page, kv head, slot, hd];   v -> value pages [page, kv head, vd, slot]
//   gate <- 1 / (1 + exp(-gate))                              -> float32 [T, ng]
// `part` (with `splits` planes of `part_stride` floats, rows of proj_stride columns): the projection as the float32
// pieces of a product split over k, instead of `proj`.
template <typename T>
__global__ __launch_bounds__(1024) void qk_norm_kv_write_kernel(
    T* __restrict__ q_out, long q_stride, float* __restrict__ gate_out, const float* __restrict__ proj, long proj_stride,
    const float* __restrict__ wq, const float* __restrict__ wk, const int* __restrict__ positions, const int* __restrict__ req_of_token,
    float eps, float temp_coef, int temp_every, int nh, int nkv, int hd, int vd, int ng, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int* __restrict__ block_table, int table_width, int page_size, long num_pages,
    const float* __restrict__ part, int splits, long part_stride, int per_head, int has_kv) {
  __shared__ float scratch[32];
  extern __shared__ float staged[];              // the token's row, when it comes in pieces
  const long t = blockIdx.x;
  const float* row = proj + t * proj_stride;
  const int QN = nh * hd, KN = has_kv ? nkv * hd : 0, VN = has_kv ? nkv * vd : 0;
  if (part) {
    // the projection is still split over k: its float32 pieces are added here, in split order, once per element
    for (int i = threadIdx.x; i < QN + KN + VN + ng; i += blockDim.x) staged[i] = split_sum(part, splits, part_stride, t * proj_stride + i);
    __syncthreads();
    row = staged;
  }
  const int p = positions[t];
  const float temp = temp_coef != 0.f ? 1.0f + temp_coef * logf((float)((p + 1) / temp_every) + 1.0f) : 1.0f;
  T* qr = q_out + t * q_stride;
  for (int i = threadIdx.x; i < ng; i += blockDim.x) gate_out[t * ng + i] = 1.0f / (1.0f + expf(-row[QN + KN + VN + i]));
  long page = -1;
  int slot = 0;
  if (k_cache && has_kv) {
    const int blk = p / page_size;
    slot = p % page_size;
    page = blk < table_width ? block_table[(long)req_of_token[t] * table_width + blk] : -1;
    if (page >= num_pages) page = -1;              // no page for this position: nothing is written
  }
  if (per_head) {
    // a wave per head: query heads first, then key heads; the sum of squares runs over the head's own entries
    const int wave = threadIdx.x / PI_WAVE, lane = threadIdx.x % PI_WAVE, nwaves = blockDim.x / PI_WAVE;
    for (int u = wave; u < nh + (has_kv ? nkv : 0); u += nwaves) {
      const bool is_q = u < nh;
      const float* src = row + (is_q ? u * hd : QN + (u - nh) * hd);
      float ss = 0.f;
      for (int d = lane; d < hd; d += PI_WAVE) ss = fmaf(src[d], src[d], ss);
      ss = wave_sum(ss);
      const float r = 1.0f / sqrtf(ss / hd + eps);
      if (is_q) {
        for (int d = lane; d < hd; d += PI_WAVE) {
          float v = src[d] * r;
          if (wq) v *= wq[u * hd + d];
          qr[u * hd + d] = from_float<T>(v * temp);
        }
      } else if (page >= 0) {
        const int g = u - nh;
        for (int d = lane; d < hd; d += PI_WAVE) {
          float v = src[d] * r;
          if (wk) v *= wk[g * hd + d];
          k_cache[((page * nkv + g) * page_size + slot) * hd + d] = from_float<T>(v);
        }
      }
    }
  } else {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < QN; i += blockDim.x) sq = fmaf(row[i], row[i], sq);
    for (int i = threadIdx.x; i < KN; i += blockDim.x) sk = fmaf(row[QN + i], row[QN + i], sk);
    block_sum2(sq, sk, scratch);                   // both sums of squares in one trip through LDS
    const float rq = wq ? 1.0f / sqrtf(sq / QN + eps) : 1.0f;
    const float rk = wk && KN ? 1.0f / sqrtf(sk / KN + eps) : 1.0f;
    for (int i = threadIdx.x; i < QN; i += blockDim.x) {
      float v = row[i];
      if (wq) v = v * rq * wq[i];
      qr[i] = from_float<T>(v * temp);
    }
    if (page >= 0) {
      for (int i = threadIdx.x; i < KN; i += blockDim.x) {
        float v = row[QN + i];
        if (wk) v = v * rk * wk[i];
        const int g = i / hd, d = i % hd;
        k_cache[((page * nkv + g) * page_size + slot) * hd + d] = from_float<T>(v);
      }
    }
  }
  if (page < 0) return;
  for (int i = threadIdx.x; i < VN; i += blockDim.x) {
    const int g = i / vd, d = i % vd;
    v_cache[((page * nkv + g) * vd + d) * page_size + slot] = from_float<T>(row[QN + KN + i]);
  }
}

extern "C" int pi_qk_norm_kv_write(void* q_out, long q_stride, float* gate_out, int dtype, const float* proj, long proj_stride,
                                   const float* wq, const float* wk, const int* positions, const int* req_of_token, float eps,
                                   float temp_coef, int temp_every, int T, int nh, int nkv, int hd, int vd, int ng,
                                   void* k_cache, void* v_cache, const int* block_table, int table_width, int page_size,
                                   long num_pages, const float* part, int splits, long part_stride, int per_head, int has_kv,
                                   hipStream_t stream) {
  PI_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && hd > 0 && vd > 0 && ng >= 0, "qk norm: bad sizes");
  const long row_floats = (long)nh * hd + (has_kv ? (long)nkv * (hd + vd) : 0) + ng;
  PI_REQUIRE(proj_stride >= row_floats, "qk norm: projection rows of %ld hold no q, k, v and gates", proj_stride);
  PI_REQUIRE(temp_coef == 0.f || temp_every > 0, "qk norm: the temperature's period must be positive, got %d", temp_every);
  PI_REQUIRE(!k_cache || (has_kv && v_cache && block_table && req_of_token && table_width > 0 && page_size > 0 && num_pages > 0),
             "qk norm: bad cache geometry");
  PI_REQUIRE(ng == 0 || gate_out, "qk norm: gates without a place for them");
  PI_REQUIRE((proj != nullptr) != (part != nullptr), "qk norm: give the projection as a tensor or as pieces");
  PI_REQUIRE(!part || (splits >= 1 && part_stride >= (long)T * proj_stride), "qk norm: bad pieces (%d planes of %ld floats)", splits, part_stride);
  PI_REQUIRE(!part || row_floats * 4 <= 60000, "qk norm: rows of %ld floats in pieces do not fit the staging memory", row_floats);
  const size_t lds = part ? (size_t)row_floats * sizeof(float) : 0;
  if (T == 0) return 0;
  const int threads = T <= 64 ? 1024 : 256;      // few tokens (decode steps): the row's passes are a matter of latency
#define QKN_GO(TT) hipLaunchKernelGGL(qk_norm_kv_write_kernel<TT>, dim3(T), dim3(threads), lds, stream, (TT*)q_out, q_stride, gate_out, proj, \
                                      proj_stride, wq, wk, positions, req_of_token, eps, temp_coef, temp_every, nh, nkv, hd, vd, ng,  \
                                      (TT*)k_cache, (TT*)v_cache, block_table, table_width, page_size, num_pages, part, splits, part_stride, \
                                      per_head, has_kv)
  if (dtype == PI_F32) QKN_GO(float);
  else if (dtype == PI_BF16) QKN_GO(bf16_t);
  else return pi_fail("qk norm: unsupported dtype %d", dtype);
#undef QKN_GO
  return pi_check_launch("qk_norm_kv_write");
}
