// Attention through a low-rank latent: what stands around the attention kernel itself.
//
// A token's input h goes through one product into [dq: q_rank | dkv: kv_rank | shared rotated key part: rot].
//   c_q = dq / rms(dq) * wq            -> the query latent, which a second product turns into the heads' queries
//   c   = dkv / rms(dkv) * wkv         -> the key/value latent, the only thing kept per token besides
//   k_r = rotate(shared part)             the rotated part, one for all heads
// A head's key is [Wuk_h c | k_r] and its value Wuv_h c.  Neither is ever made: with
//   q_lat_h = [Wuk_h^T q_plain_h | rotate(q_rot_h)]      (kv_rank + rot numbers per head)
// the score <q_plain_h, Wuk_h c> + <q_rot_h, k_r> is <q_lat_h, [c | k_r]>, so every head attends over the
// same cached rows [c | k_r] (one key/value head for all query heads) with c as the value, and
// Wuv_h is applied to the attention's result afterwards (a product per head).
//
// Norms, angles and rotations are float32; rms(v) = sqrt(mean(v^2) + eps).
#include "common.h"

// One block per token.  Row (float32): [q_rank | kv_rank | rot], as a tensor or as the pieces of a product split over k.
// Cache: keys [page, 1, slot, kv_rank + rot] = [c | k_r]; values transposed [page, 1, v_rows, slot], rows 0 .. kv_rank - 1
// = c and, when v_rows = kv_rank + rot (values kept as wide as keys, for kernels that want them so), then k_r.
// table: the step's [T, rot] cosines then sines (rot / 2 each), already scaled; pairs are neighbours (2j, 2j + 1).
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(
    T* __restrict__ cq_out, long cq_stride, const float* __restrict__ proj, long proj_stride, const float* __restrict__ wq,
    const float* __restrict__ wkv, const float* __restrict__ table, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, float eps, int q_rank, int kv_rank, int rot, int v_rows, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int* __restrict__ block_table, int table_width, int page_size, long num_pages,
    const float* __restrict__ part, int splits, long part_stride) {
  __shared__ float scratch[32];
  extern __shared__ float staged[];
  const long t = blockIdx.x;
  const float* row = proj + t * proj_stride;
  const int N = q_rank + kv_rank + rot;
  if (part) {
    for (int i = threadIdx.x; i < N; i += blockDim.x) staged[i] = split_sum(part, splits, part_stride, t * proj_stride + i);
    __syncthreads();
    row = staged;
  }
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) sq = fmaf(row[i], row[i], sq);
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) sk = fmaf(row[q_rank + i], row[q_rank + i], sk);
  block_sum2(sq, sk, scratch);
  const float rq = q_rank ? 1.0f / sqrtf(sq / q_rank + eps) : 0.f;
  const float rk = 1.0f / sqrtf(sk / kv_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) cq_out[t * cq_stride + i] = from_float<T>(row[i] * rq * wq[i]);
  if (!k_cache) return;
  const int p = positions[t];
  const int blk = p / page_size, slot = p % page_size;
  const long page = blk < table_width ? block_table[(long)req_of_token[t] * table_width + blk] : -1;
  if (page < 0 || page >= num_pages) return;      // no page for this position: nothing is written
  const int hd = kv_rank + rot;
  T* kr = k_cache + (page * page_size + slot) * hd;
  T* vr = v_cache + page * (long)v_rows * page_size + slot;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const T c = from_float<T>(row[q_rank + i] * rk * wkv[i]);
    kr[i] = c;
    vr[(long)i * page_size] = c;
  }
  const float* cs = table + t * rot;
  for (int j = threadIdx.x; j < rot / 2; j += blockDim.x) {
    float lo, hi;
    rope_pair(row[q_rank + kv_rank + 2 * j], row[q_rank + kv_rank + 2 * j + 1], cs[j], cs[rot / 2 + j], lo, hi);
    const T a = from_float<T>(lo), b = from_float<T>(hi);
    kr[kv_rank + 2 * j] = a;
    kr[kv_rank + 2 * j + 1] = b;
    if (v_rows > kv_rank) {
      vr[(long)(kv_rank + 2 * j) * page_size] = a;
      vr[(long)(kv_rank + 2 * j + 1) * page_size] = b;
    }
  }
}

extern "C" int pi_latent_kv_write(void* cq_out, long cq_stride, int dtype, const float* proj, long proj_stride, const float* wq,
                                  const float* wkv, const float* table, const int* positions, const int* req_of_token, float eps,
                                  int T, int q_rank, int kv_rank, int rot, int v_rows, void* k_cache, void* v_cache,
                                  const int* block_table, int table_width, int page_size, long num_pages, const float* part,
                                  int splits, long part_stride, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && q_rank >= 0 && kv_rank > 0 && rot >= 0 && rot % 2 == 0, "latent: bad sizes q_rank=%d kv_rank=%d rot=%d", q_rank, kv_rank, rot);
  PI_REQUIRE(v_rows == kv_rank || v_rows == kv_rank + rot, "latent: value rows %d are neither the latent's %d nor the key's %d", v_rows, kv_rank, kv_rank + rot);
  const long row_floats = (long)q_rank + kv_rank + rot;
  PI_REQUIRE(proj_stride >= row_floats, "latent: projection rows of %ld hold no %ld columns", proj_stride, row_floats);
  PI_REQUIRE((proj != nullptr) != (part != nullptr), "latent: give the projection as a tensor or as pieces");
  PI_REQUIRE(!part || (splits >= 1 && part_stride >= (long)T * proj_stride), "latent: bad pieces (%d planes of %ld floats)", splits, part_stride);
  PI_REQUIRE(!part || row_floats * 4 <= 60000, "latent: rows of %ld floats in pieces do not fit the staging memory", row_floats);
  PI_REQUIRE(q_rank == 0 || (cq_out && wq), "latent: a query latent without its weight or a place for it");
  PI_REQUIRE(wkv && (rot == 0 || table), "latent: the key latent's weight or the rotation's table is missing");
  PI_REQUIRE(!k_cache || (v_cache && block_table && positions && req_of_token && table_width > 0 && page_size > 0 && num_pages > 0),
             "latent: bad cache geometry");
  if (T == 0) return 0;
  const size_t lds = part ? (size_t)row_floats * sizeof(float) : 0;
#define LKV_GO(TT) hipLaunchKernelGGL(latent_kv_write_kernel<TT>, dim3(T), dim3(256), lds, stream, (TT*)cq_out, cq_stride, proj, proj_stride, \
                                      wq, wkv, table, positions, req_of_token, eps, q_rank, kv_rank, rot, v_rows, (TT*)k_cache,            \
                                      (TT*)v_cache, block_table, table_width, page_size, num_pages, part, splits, part_stride)
  if (dtype == PI_F32) LKV_GO(float);
  else if (dtype == PI_BF16) LKV_GO(bf16_t);
  else return pi_fail("latent: unsupported dtype %d", dtype);
#undef LKV_GO
  return pi_check_launch("latent_kv_write");
}

// ---------------------------------------------------------------- a product per head
// out[t, h * out_head + n] = sum_k a[t, h * a_head + k] * w[h, k, n]      (w: [heads, K, N])
// and, with `rot` > 0, the rot numbers that follow a head's K inputs are rotated by the token's angles (neighbouring pairs)
// and placed behind the head's N results: [w_h^T a_h | rotate(tail)].  One block per (eight tokens, head, 64 output
// columns): the tokens' inputs sit in LDS and are read four at a time; a lane owns one output column, neighbouring lanes
// read neighbouring weights, sixteen loads in flight; the block's eight waves each take an eighth of k (in whole eights) and
// their float32 sums - each in ascending k - are added in wave order.  A token's result does not depend on the tokens
// beside it.  `skip_product`: only the rotated tails are made (the product comes from another kernel).
#define HG_TOKENS 8
#define HG_WAVES 8
#define HG_LOADS 16        // weights a lane asks for before it waits: a wave's whole share of k at the usual sizes
template <typename T>
__global__ __launch_bounds__(HG_WAVES * PI_WAVE) void head_gemm_kernel(T* __restrict__ out, long out_stride, int out_head,
                                                                       const T* __restrict__ a, long a_stride, int a_head,
                                                                       const T* __restrict__ w, int M, int K, int N, int rot,
                                                                       const float* __restrict__ table, int skip_product) {
  extern __shared__ __attribute__((aligned(16))) float as[];          // [HG_TOKENS][KP], KP = K + rot rounded up to four
  __shared__ float sums[HG_WAVES][HG_TOKENS][PI_WAVE];
  const int h = blockIdx.y, lane = threadIdx.x % PI_WAVE, wave = threadIdx.x / PI_WAVE;
  const long t0 = (long)blockIdx.x * HG_TOKENS;
  const int nt = (M - t0) < HG_TOKENS ? (int)(M - t0) : HG_TOKENS;
  const int KR = K + rot, KP = (KR + 3) & ~3;
  const int k_from = skip_product ? K : 0;
  for (int i = threadIdx.x; i < HG_TOKENS * KP; i += blockDim.x) {
    const int tt = i / KP, k = i % KP;
    as[i] = (tt < nt && k >= k_from && k < KR) ? to_float(a[(t0 + tt) * a_stride + (long)h * a_head + k]) : 0.f;
  }
  __syncthreads();
  if (!skip_product) {
    const int n = blockIdx.z * PI_WAVE + lane;
    const int per = ((K + HG_WAVES - 1) / HG_WAVES + 7) & ~7;          // a wave's share of k, in whole eights
    const int k0 = wave * per, k1 = min(K, k0 + per);
    float acc[HG_TOKENS];
#pragma unroll
    for (int tt = 0; tt < HG_TOKENS; ++tt) acc[tt] = 0.f;
    if (n < N) {
      const T* wh = w + (long)h * K * N + n;
      int k = k0;
      for (; k + HG_LOADS <= k1; k += HG_LOADS) {
        float wv[HG_LOADS];
#pragma unroll
        for (int u = 0; u < HG_LOADS; ++u) wv[u] = to_float(wh[(long)(k + u) * N]);
#pragma unroll
        for (int tt = 0; tt < HG_TOKENS; ++tt) {
#pragma unroll
          for (int u = 0; u < HG_LOADS; u += 4) {
            const float4 a4 = *reinterpret_cast<const float4*>(as + tt * KP + k + u);
            acc[tt] = fmaf(a4.x, wv[u], acc[tt]);
            acc[tt] = fmaf(a4.y, wv[u + 1], acc[tt]);
            acc[tt] = fmaf(a4.z, wv[u + 2], acc[tt]);
            acc[tt] = fmaf(a4.w, wv[u + 3], acc[tt]);
          }
        }
      }
      for (; k + 8 <= k1; k += 8) {
        float wv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) wv[u] = to_float(wh[(long)(k + u) * N]);
#pragma unroll
        for (int tt = 0; tt < HG_TOKENS; ++tt) {
          const float4 a0 = *reinterpret_cast<const float4*>(as + tt * KP + k);
          const float4 a1 = *reinterpret_cast<const float4*>(as + tt * KP + k + 4);
          acc[tt] = fmaf(a0.x, wv[0], acc[tt]);
          acc[tt] = fmaf(a0.y, wv[1], acc[tt]);
          acc[tt] = fmaf(a0.z, wv[2], acc[tt]);
          acc[tt] = fmaf(a0.w, wv[3], acc[tt]);
          acc[tt] = fmaf(a1.x, wv[4], acc[tt]);
          acc[tt] = fmaf(a1.y, wv[5], acc[tt]);
          acc[tt] = fmaf(a1.z, wv[6], acc[tt]);
          acc[tt] = fmaf(a1.w, wv[7], acc[tt]);
        }
      }
      for (; k < k1; ++k) {
        const float wv = to_float(wh[(long)k * N]);
#pragma unroll
        for (int tt = 0; tt < HG_TOKENS; ++tt) acc[tt] = fmaf(as[tt * KP + k], wv, acc[tt]);
      }
    }
#pragma unroll
    for (int tt = 0; tt < HG_TOKENS; ++tt) sums[wave][tt][lane] = acc[tt];
    __syncthreads();
    // wave tt finishes token tt: the waves' shares in wave order
    for (int tt = wave; tt < nt; tt += HG_WAVES) {
      if (n < N) {
        float v = sums[0][tt][lane];
#pragma unroll
        for (int u = 1; u < HG_WAVES; ++u) v += sums[u][tt][lane];
        out[(t0 + tt) * out_stride + (long)h * out_head + n] = from_float<T>(v);
      }
    }
  }
  if (blockIdx.z != 0) return;
  for (int i = threadIdx.x; i < nt * (rot / 2); i += blockDim.x) {
    const int tt = i / (rot / 2), j = i % (rot / 2);
    const float* cs = table + (t0 + tt) * rot;
    float lo, hi;
    rope_pair(as[tt * KP + K + 2 * j], as[tt * KP + K + 2 * j + 1], cs[j], cs[rot / 2 + j], lo, hi);
    T* o = out + (t0 + tt) * out_stride + (long)h * out_head + N;
    o[2 * j] = from_float<T>(lo);
    o[2 * j + 1] = from_float<T>(hi);
  }
}

extern "C" int pi_head_gemm(void* out, long out_stride, int out_head, const void* a, long a_stride, int a_head, const void* w,
                            int dtype, int M, int heads, int K, int N, int rot, const float* table, int skip_product,
                            hipStream_t stream) {
  PI_REQUIRE(M >= 0 && heads > 0 && K > 0 && N > 0 && rot >= 0 && rot % 2 == 0, "head product: bad sizes M=%d heads=%d K=%d N=%d rot=%d", M, heads, K, N, rot);
  PI_REQUIRE(heads <= 65535 && N <= 65535 * PI_WAVE, "head product: too many heads or columns (%d, %d)", heads, N);
  PI_REQUIRE(a_head >= K + rot && out_head >= N + rot, "head product: heads of %d / %d numbers hold no %d / %d", a_head, out_head, K + rot, N + rot);
  PI_REQUIRE(a_stride >= (long)(heads - 1) * a_head + K + rot && out_stride >= (long)(heads - 1) * out_head + N + rot,
             "head product: rows of %ld / %ld numbers hold no %d heads", a_stride, out_stride, heads);
  PI_REQUIRE(rot == 0 || table, "head product: a rotated tail needs the step's table");
  PI_REQUIRE(skip_product || w, "head product: the weights are missing");
  const size_t lds = (size_t)HG_TOKENS * ((K + rot + 3) & ~3) * sizeof(float);
  PI_REQUIRE(lds <= 48000, "head product: %d inputs per head do not fit the staging memory", K + rot);
  if (M == 0 || (skip_product && rot == 0)) return 0;
  const dim3 grid(ceil_div(M, HG_TOKENS), heads, skip_product ? 1 : ceil_div(N, PI_WAVE)), block(HG_WAVES * PI_WAVE);
  if (dtype == PI_F32)
    hipLaunchKernelGGL(head_gemm_kernel<float>, grid, block, lds, stream, (float*)out, out_stride, out_head, (const float*)a, a_stride,
                       a_head, (const float*)w, M, K, N, rot, table, skip_product);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(head_gemm_kernel<bf16_t>, grid, block, lds, stream, (bf16_t*)out, out_stride, out_head, (const bf16_t*)a, a_stride,
                       a_head, (const bf16_t*)w, M, K, N, rot, table, skip_product);
  else
    return pi_fail("head product: unsupported dtype %d", dtype);
  return pi_check_launch("head_gemm");
}
