// Routed experts (mixture of experts): routing, grouping of the step's (token, choice) entries
// by expert, the grouped products, and the weighted sum.  Everything stays on the device: no
// count ever travels to the host, so a step's launches depend on its number of tokens only.
//
// Routing, per token, from float32 router logits z [E]:
//   s = softmax(z) over all experts;
//   experts form `groups` equal groups of neighbours, a group's score is its largest s, and
//   only experts of the `keep` best groups may be chosen (groups <= 1: all may);
//   the `top` allowed experts with the largest s are chosen, weights = their s (as they are,
//   or divided by their sum + renorm_eps when `renorm`).  Equal scores: the lower index wins.
//   With a `correction` [E] the choice (of groups and of experts) goes by s + correction; the
//   weights stay the scores themselves.
// Experts from `num_real` on are identity experts: they have no matrices, make no tiles, and the
// weighted sum takes the token's own activations for them.
#include "common.h"

#define RE_MAX_EXPERTS 1024
#define RE_TILE 64          // rows of a tile of the general grouped product (the most it takes)

// (value, index) arg max over a wave; equal values: the lower index
__device__ inline void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int off = PI_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, PI_WAVE);
    const int oi = __shfl_xor(idx, off, PI_WAVE);
    if (ov > v || (ov == v && oi < idx)) {
      v = ov;
      idx = oi;
    }
  }
}

__global__ __launch_bounds__(PI_WAVE) void route_kernel(int* __restrict__ ids, float* __restrict__ weights, const float* __restrict__ logits,
                                                        long logits_stride, int E, int top, int groups, int keep, int renorm,
                                                        const float* __restrict__ correction, float renorm_eps) {
  __shared__ float s[RE_MAX_EXPERTS];
  __shared__ float c[RE_MAX_EXPERTS];      // what the choice goes by
  __shared__ unsigned char allowed[RE_MAX_EXPERTS];
  __shared__ float gscore[RE_MAX_EXPERTS];
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + t * logits_stride;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += PI_WAVE) mx = fmaxf(mx, z[e]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += PI_WAVE) {
    const float v = expf(z[e] - mx);
    s[e] = v;
    sum += v;
  }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
  for (int e = lane; e < E; e += PI_WAVE) {
    s[e] *= inv;
    c[e] = correction ? s[e] + correction[e] : s[e];
    allowed[e] = (groups <= 1) ? 1 : 0;
  }
  __syncthreads();
  if (groups > 1) {
    const int per = E / groups;
    for (int g = lane; g < groups; g += PI_WAVE) {
      float best = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, c[e]);
      gscore[g] = best;
    }
    __syncthreads();
    for (int j = 0; j < keep; ++j) {
      float v = -INFINITY;
      int idx = 0x7fffffff;
      for (int g = lane; g < groups; g += PI_WAVE)
        if (gscore[g] > v) {
          v = gscore[g];
          idx = g;
        }
      wave_argmax(v, idx);
      if (idx < groups) {
        for (int e = idx * per + lane; e < (idx + 1) * per; e += PI_WAVE) allowed[e] = 1;
        if (lane == 0) gscore[idx] = -INFINITY;
      }
      __syncthreads();
    }
  }
  float wsum = 0.f;
  for (int j = 0; j < top; ++j) {
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int e = lane; e < E; e += PI_WAVE)
      if (allowed[e] && c[e] > v) {
        v = c[e];
        idx = e;
      }
    wave_argmax(v, idx);
    if (idx >= E) {          // fewer allowed experts than choices: the entry counts nothing
      idx = 0;
      v = 0.f;
    } else {
      v = s[idx];
      if (lane == 0) allowed[idx] = 0;
    }
    wsum += v;
    if (lane == 0) {
      ids[t * top + j] = idx;
      weights[t * top + j] = v;
    }
    __syncthreads();
  }
  if (renorm && lane == 0) {
    const float r = 1.0f / (wsum + renorm_eps);
    for (int j = 0; j < top; ++j) weights[t * top + j] *= r;
  }
}

extern "C" int pi_route(int* ids, float* weights, const float* logits, long logits_stride, int T, int E, int top, int groups,
                        int keep, int renorm, const float* correction, float renorm_eps, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && E > 0 && E <= RE_MAX_EXPERTS, "routing: %d experts (at most %d)", E, RE_MAX_EXPERTS);
  PI_REQUIRE(top > 0 && top <= E, "routing: %d choices among %d experts", top, E);
  PI_REQUIRE(groups <= 1 || (E % groups == 0 && keep > 0 && keep <= groups), "routing: %d experts in %d groups, %d kept", E, groups, keep);
  PI_REQUIRE(groups <= 1 || (long)keep * (E / groups) >= top, "routing: %d kept groups of %d experts hold fewer than %d choices", keep, groups > 0 ? E / groups : 0, top);
  if (T == 0) return 0;
  hipLaunchKernelGGL(route_kernel, dim3(T), dim3(PI_WAVE), 0, stream, ids, weights, logits, logits_stride, E, top, groups, keep, renorm, correction, renorm_eps);
  return pi_check_launch("route");
}

// ---------------------------------------------------------------- entries grouped by expert
// N entries (entry = token * top + choice) with their expert ids -> rows in expert order:
//   row_entry[row] = entry, entry_row[entry] = row (entries of one expert keep their order),
//   tiles of up to `tile` rows that never straddle two experts: tile_expert[i] (-1: unused),
//   tile_row0[i], tile_rows[i]; max_tiles = ceil(N / tile) + E bounds their number.
// Entries whose id is not in 0 .. E - 1 (identity experts) own no row: their entry_row is 0, and the rows
// that stay empty behind the last expert's name entry 0, so that whoever walks all N rows stays in bounds.
// One block of 1024 threads; wave w places the experts w, w + 16, ...
__global__ __launch_bounds__(1024) void group_entries_kernel(const int* __restrict__ ids, int N, int E, int* __restrict__ row_entry,
                                                             int* __restrict__ entry_row, int* __restrict__ tile_expert,
                                                             int* __restrict__ tile_row0, int* __restrict__ tile_rows, int max_tiles,
                                                             int tile) {
  __shared__ int count[RE_MAX_EXPERTS];
  __shared__ int start[RE_MAX_EXPERTS + 1];
  __shared__ int tstart[RE_MAX_EXPERTS + 1];
  const int tid = threadIdx.x, lane = tid % PI_WAVE, wave = tid / PI_WAVE;
  for (int e = tid; e < E; e += 1024) count[e] = 0;
  __syncthreads();
  for (int i = tid; i < N; i += 1024) {
    const int e = ids[i];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int acc = 0, tacc = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = acc;
      tstart[e] = tacc;
      acc += count[e];
      tacc += (count[e] + tile - 1) / tile;
    }
    start[E] = acc;
    tstart[E] = tacc;
  }
  __syncthreads();
  for (int i = start[E] + tid; i < N; i += 1024) row_entry[i] = 0;
  for (int i = tid; i < N; i += 1024)
    if (ids[i] < 0 || ids[i] >= E) entry_row[i] = 0;
  for (int i = tstart[E] + tid; i < max_tiles; i += 1024) {
    tile_expert[i] = -1;
    tile_row0[i] = 0;
    tile_rows[i] = 0;
  }
  for (int e = wave; e < E; e += 16) {
    for (int i = lane; i < (count[e] + tile - 1) / tile; i += PI_WAVE) {
      tile_expert[tstart[e] + i] = e;
      tile_row0[tstart[e] + i] = start[e] + i * tile;
      const int left = count[e] - i * tile;
      tile_rows[tstart[e] + i] = left < tile ? left : tile;
    }
    int placed = start[e];
    for (int i0 = 0; i0 < N; i0 += PI_WAVE) {
      const int i = i0 + lane;
      const bool mine = i < N && ids[i] == e;
      const unsigned long long votes = __ballot(mine);
      if (mine) {
        const int row = placed + __popcll(votes & ((1ull << lane) - 1ull));
        row_entry[row] = i;
        entry_row[i] = row;
      }
      placed += __popcll(votes);
    }
  }
}

extern "C" int pi_group_entries(const int* ids, int N, int E, int* row_entry, int* entry_row, int* tile_expert, int* tile_row0,
                                int* tile_rows, int max_tiles, int tile, hipStream_t stream) {
  PI_REQUIRE(N >= 0 && E > 0 && E <= RE_MAX_EXPERTS && tile > 0, "grouping: bad sizes N=%d E=%d tile=%d", N, E, tile);
  PI_REQUIRE(max_tiles >= (N + tile - 1) / tile + E, "grouping: room for %d tiles is too little", max_tiles);
  if (N == 0) return 0;
  hipLaunchKernelGGL(group_entries_kernel, dim3(1), dim3(1024), 0, stream, ids, N, E, row_entry, entry_row, tile_expert, tile_row0,
                     tile_rows, max_tiles, tile);
  return pi_check_launch("group_entries");
}

extern "C" int pi_group_tile_rows() { return RE_TILE; }

// rows[row, :] = src[row_entry[row] / top, :]   (activations copied into expert order)
template <typename T>
__global__ void gather_rows_kernel(T* __restrict__ out, const T* __restrict__ src, const int* __restrict__ row_entry, int top, int D) {
  const long row = blockIdx.x;
  const long t = row_entry[row] / top;
  for (int d = threadIdx.x; d < D; d += blockDim.x) out[row * D + d] = src[t * D + d];
}

extern "C" int pi_gather_rows(void* out, const void* src, int dtype, const int* row_entry, int N, int top, int D, hipStream_t stream) {
  PI_REQUIRE(N >= 0 && top > 0 && D > 0, "gather: bad sizes");
  if (N == 0) return 0;
  if (dtype == PI_F32)
    hipLaunchKernelGGL(gather_rows_kernel<float>, dim3(N), dim3(256), 0, stream, (float*)out, (const float*)src, row_entry, top, D);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(gather_rows_kernel<bf16_t>, dim3(N), dim3(256), 0, stream, (bf16_t*)out, (const bf16_t*)src, row_entry, top, D);
  else
    return pi_fail("gather: unsupported dtype %d", dtype);
  return pi_check_launch("gather_rows");
}

// ---------------------------------------------------------------- grouped product, any size and type
// C[row, :] = A[row, :] . W[expert of row]^T for the rows of every tile; W is [E, N, K].  float32
// multiply-add, each output accumulating over k in ascending order: a row's result does not
// depend on the rows around it.
#define RG_T 64
#define RG_K 16
template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void grouped_gemm_general_kernel(TC* __restrict__ C, long ldc, const TA* __restrict__ A, long lda,
                                                                   const TW* __restrict__ W, long ldw, long w_expert_stride,
                                                                   const int* __restrict__ tile_expert, const int* __restrict__ tile_row0,
                                                                   const int* __restrict__ tile_rows, int N, int K) {
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  __shared__ float As[RG_K][RG_T + 4];
  __shared__ float Ws[RG_K][RG_T + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const long n0 = (long)blockIdx.x * RG_T;
  const TW* We = W + (long)e * w_expert_stride;
  // a tile of more than RG_T rows (lists made for the matrix-core kernel) is walked in pieces
  for (int sub = 0; sub < tile_rows[blockIdx.y]; sub += RG_T) {
    const long m0 = tile_row0[blockIdx.y] + sub;
    const int M = min(RG_T, tile_rows[blockIdx.y] - sub);
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += RG_K) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int idx = tid + i * 256;
        const int row = idx / RG_K, kk = idx % RG_K;
        const long n = n0 + row;
        const int k = k0 + kk;
        As[kk][row] = (row < M && k < K) ? to_float(A[(m0 + row) * lda + k]) : 0.f;
        Ws[kk][row] = (n < N && k < K) ? to_float(We[n * ldw + k]) : 0.f;
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < RG_K; ++kk) {
        float a[4], w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
      }
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = ty * 4 + i;
      if (r >= M) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const long n = n0 + tx * 4 + j;
        if (n < N) C[(m0 + r) * ldc + n] = from_float<TC>(acc[i][j]);
      }
    }
  }
}

extern "C" int pi_grouped_gemm_general(void* C, int c_dtype, long ldc, const void* A, int a_dtype, long lda, const void* W, int w_dtype,
                                       long ldw, long w_expert_stride, const int* tile_expert, const int* tile_row0,
                                       const int* tile_rows, int tiles, int N, int K, hipStream_t stream) {
  PI_REQUIRE(tiles >= 0 && N > 0 && K > 0 && lda >= K && ldw >= K && ldc >= N, "grouped product: bad sizes");
  PI_REQUIRE(tiles <= 65535, "grouped product: too many tiles (%d)", tiles);
  PI_REQUIRE(a_dtype == w_dtype, "grouped product: activations and weights must have one type");
  if (tiles == 0) return 0;
  const dim3 grid(ceil_div(N, RG_T), tiles), block(256);
#define RG_GO(TA, TC) hipLaunchKernelGGL((grouped_gemm_general_kernel<TA, TA, TC>), grid, block, 0, stream, (TC*)C, ldc, (const TA*)A, lda, \
                                         (const TA*)W, ldw, w_expert_stride, tile_expert, tile_row0, tile_rows, N, K)
  if (a_dtype == PI_F32 && c_dtype == PI_F32) RG_GO(float, float);
  else if (a_dtype == PI_BF16 && c_dtype == PI_F32) RG_GO(bf16_t, float);
  else if (a_dtype == PI_BF16 && c_dtype == PI_BF16) RG_GO(bf16_t, bf16_t);
  else return pi_fail("grouped product: unsupported dtypes a=%d c=%d", a_dtype, c_dtype);
#undef RG_GO
  return pi_check_launch("grouped_gemm_general");
}

// out[t, :] (+)= sum_j weights[t, j] * y[entry_row[t * top + j], :], choices in order (float32); a choice whose
// id is num_real or more (ids given) stands for the token's own activations h[t, :] instead
template <typename TH>
__global__ void combine_choices_kernel(float* __restrict__ out, const float* __restrict__ y, const float* __restrict__ weights,
                                       const int* __restrict__ entry_row, int top, int D, int accumulate, const int* __restrict__ ids,
                                       int num_real, const TH* __restrict__ h) {
  const long t = blockIdx.x;
  const int d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  float acc = 0.f;
  for (int j = 0; j < top; ++j) {
    const bool own = ids && ids[t * top + j] >= num_real;
    const float v = own ? to_float(h[t * D + d]) : y[(long)entry_row[t * top + j] * D + d];
    acc = fmaf(weights[t * top + j], v, acc);
  }
  out[t * D + d] = accumulate ? out[t * D + d] + acc : acc;
}

extern "C" int pi_combine_choices(float* out, const float* y, const float* weights, const int* entry_row, int T, int top, int D,
                                  int accumulate, const int* ids, int num_real, const void* h, int h_dtype, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && top > 0 && D > 0, "combine: bad sizes");
  PI_REQUIRE(!ids || h, "combine: identity experts need the tokens' activations");
  if (T == 0) return 0;
  PI_REQUIRE((D + 255) / 256 <= 65535, "combine: rows of %d are too long", D);
  const dim3 grid(T, (D + 255) / 256), block(256);
  if (ids && h_dtype == PI_BF16)
    hipLaunchKernelGGL(combine_choices_kernel<bf16_t>, grid, block, 0, stream, out, y, weights, entry_row, top, D, accumulate, ids, num_real, (const bf16_t*)h);
  else if (!ids || h_dtype == PI_F32)
    hipLaunchKernelGGL(combine_choices_kernel<float>, grid, block, 0, stream, out, y, weights, entry_row, top, D, accumulate, ids, num_real, (const float*)h);
  else
    return pi_fail("combine: unsupported activation dtype %d", h_dtype);
  return pi_check_launch("combine_choices");
}
