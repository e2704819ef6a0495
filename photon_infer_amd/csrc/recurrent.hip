// Mixers whose memory is a state of fixed size per request: the short causal convolution in
// front of them, the state-space recurrence (Mamba-2 form), the gated delta rule with one decay
// per head and key channel or per head, gated linear attention, and the norms behind them.  Everything that enters a recurrence is
// float32 in both compute modes: inputs after the convolution, step sizes, decays, gates, the
// state.  A request's state row lies at state[slots[r]]; a step runs the tokens
// q_start[r] .. q_start[r+1]-1 of request r from that row and leaves the row ready for the next
// step, so a prompt may be cut anywhere.  All sizes are run-time values.
#include "common.h"

#define PI_CONV_MAX_TAPS 8
#define PI_CONV_SEGMENT 64
#define PI_SCAN_COLUMNS 16      // value columns of a block: four walking waves of four columns each
#define PI_SCAN_WAVES 4

__device__ inline float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ inline float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ inline float softplus_f(float v) { return v > 20.0f ? v : log1pf(expf(v)); }

// ------------------------------------------------------------------ causal convolution + silu
// out[t, c] = silu(bias[c] + sum_j w[c, j] * u[t - (taps - 1) + j, c]), the last column of w on the
// token itself; inputs before the step's first token come from the request's state (the last
// taps - 1 inputs of earlier steps, zeros at the start of a sequence), which is brought up to
// date here.  A thread owns a channel of one segment of a request's tokens; the thread of the
// first segment reads the old state before it writes the new one, and nobody else touches it.
template <typename TW>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    float* __restrict__ out, long out_stride, const float* __restrict__ in, long in_stride, const TW* __restrict__ w,
    const TW* __restrict__ bias, int C, int taps, const int* __restrict__ q_start, const int* __restrict__ slots,
    float* __restrict__ state, long state_stride) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r = blockIdx.y, seg = blockIdx.z;
  const int qs = q_start[r], n = q_start[r + 1] - qs;
  const int t0 = seg * PI_CONV_SEGMENT;
  if (t0 >= n) return;
  const int t1 = t0 + PI_CONV_SEGMENT < n ? t0 + PI_CONV_SEGMENT : n;
  float* st = state + (long)slots[r] * state_stride;      // [(taps - 1), C]
  // weights and window aligned at the end of fixed arrays: unused leading taps weigh zero
  float wr[PI_CONV_MAX_TAPS], win[PI_CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < PI_CONV_MAX_TAPS; ++j) {
    const int tap = j - (PI_CONV_MAX_TAPS - taps);
    wr[j] = tap >= 0 ? to_float(w[(long)c * taps + tap]) : 0.f;
    win[j] = 0.f;
    if (tap >= 0 && tap < taps - 1) {
      const int src = t0 - (taps - 1) + tap;
      win[j] = src >= 0 ? in[(long)(qs + src) * in_stride + c] : st[(long)(taps - 1 + src) * C + c];
    }
  }
  float old[PI_CONV_MAX_TAPS - 1];
  if (seg == 0) {
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS - 1; ++j) old[j] = j < taps - 1 ? st[(long)j * C + c] : 0.f;
  }
  const float b = bias ? to_float(bias[c]) : 0.f;
  for (int t = t0; t < t1; ++t) {
    win[PI_CONV_MAX_TAPS - 1] = in[(long)(qs + t) * in_stride + c];
    float acc = b;
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS; ++j) acc = fmaf(wr[j], win[j], acc);
    out[(long)(qs + t) * out_stride + c] = silu_f(acc);
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS - 1; ++j) win[j] = win[j + 1];
  }
  if (seg == 0) {
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS - 1; ++j) {
      if (j < taps - 1) {
        const int src = n - (taps - 1) + j;
        float v;
        if (src >= 0) {
          v = in[(long)(qs + src) * in_stride + c];
        } else {                  // fewer new tokens than the window holds: the old ones move up
          v = 0.f;
#pragma unroll
          for (int o = 0; o < PI_CONV_MAX_TAPS - 1; ++o) v = (o == j + n) ? old[o] : v;
        }
        st[(long)j * C + c] = v;
      }
    }
  }
}

extern "C" int pi_causal_conv_silu(float* out, long out_stride, const float* in, long in_stride, const void* w, const void* bias,
                                   int w_dtype, int C, int taps, const int* q_start, const int* slots, int R, int longest,
                                   float* state, long state_stride, hipStream_t stream) {
  PI_REQUIRE(C > 0 && taps >= 1 && taps <= PI_CONV_MAX_TAPS, "convolution: %d channels with %d taps (at most %d)", C, taps, PI_CONV_MAX_TAPS);
  PI_REQUIRE(R >= 0 && R <= 65535 && longest >= 0, "convolution: bad step shape (%d requests, longest %d)", R, longest);
  PI_REQUIRE(state_stride >= (long)(taps - 1) * C, "convolution: a state row of %ld floats cannot hold %d x %d inputs", state_stride, taps - 1, C);
  if (R == 0 || longest == 0) return 0;
  const int segs = (longest + PI_CONV_SEGMENT - 1) / PI_CONV_SEGMENT;
  PI_REQUIRE(segs <= 65535, "convolution: a request brings too many tokens (%d)", longest);
  const dim3 grid((C + 255) / 256, R, segs), block(256);
  if (w_dtype == PI_F32)
    hipLaunchKernelGGL(causal_conv_silu_kernel<float>, grid, block, 0, stream, out, out_stride, in, in_stride, (const float*)w,
                       (const float*)bias, C, taps, q_start, slots, state, state_stride);
  else if (w_dtype == PI_BF16)
    hipLaunchKernelGGL(causal_conv_silu_kernel<bf16_t>, grid, block, 0, stream, out, out_stride, in, in_stride, (const bf16_t*)w,
                       (const bf16_t*)bias, C, taps, q_start, slots, state, state_stride);
  else
    return pi_fail("convolution: unsupported weight dtype %d", w_dtype);
  return pi_check_launch("causal_conv_silu");
}

// ------------------------------------------------------------------ how a block walks a state
// A block owns 16 value columns of one head of one request.  Four of its five waves keep the
// state, four columns each: a column's state (one value per key channel / state row) is split
// over the sixteen lanes of a row of the wave, lane = 16 * column + part, and a lane keeps the rows
// part * NR .. part * NR + NR - 1 in registers; a sum over a column is four adds through the
// data-parallel primitives (quad_perm, row_ror), no trip through LDS.  Rows beyond the real size
// are zero in every staged vector, so they stay zero in the state and the walk needs no tests.
// The fifth wave stages the tokens' vectors through LDS a chunk ahead of the walk, so that the
// memory's latency lies behind it; everything of a token that does not depend on the state
// (decays, unit vectors, beta) is made beforehand, once per token and head, by a kernel that is
// parallel in the tokens.  The walk itself is multiply-adds on registers and LDS reads.  One
// barrier per chunk hands a buffer over.
//
// In memory a request's state is kept in the walk's own order, [head][slice of four columns][i][lane]
// (NR * 64 floats per slice), so that a wave loads and stores it in whole 256-byte rows.
// Nothing else reads it; a cleared row is a zero state in any order.
template <int CTRL>
__device__ inline float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
// the sum over the 16 lanes of a row, in every lane of the row
__device__ inline float row16_sum(float v) {
  v += dpp_move<0xB1>(v);       // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);       // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x124>(v);      // row_ror 4
  v += dpp_move<0x128>(v);      // row_ror 8
  return v;
}

static inline int scan_rows_per_lane(int rows) {
  for (int nr = 1; nr <= 16; nr *= 2)
    if (16 * nr >= rows) return nr;
  return 0;
}

// Floats of one request's state for `heads` heads of `rows` x `cols` (0: rows beyond 256).
extern "C" long pi_scan_state_floats(int heads, int rows, int cols) {
  const int nr = scan_rows_per_lane(rows);
  return (long)heads * ((cols + PI_SCAN_COLUMNS - 1) / PI_SCAN_COLUMNS) * PI_SCAN_WAVES * nr * PI_WAVE;
}

// SHORT: a step in which no request brings more than two tokens (decoding) is staged two tokens at a time:
// few registers and little LDS, so that many blocks share a compute unit while they wait for their states.
template <int NR, bool SHORT> struct ScanShape {
  static constexpr int W = 16 * NR;                                   // rows of a staged vector
  static constexpr int CH = SHORT ? 2 : (NR >= 16 ? 8 : 16);          // tokens per chunk
};

// `cn` tokens' vectors of `size` floats (token t at src + t * stride) on their way into LDS rows of W floats,
// zeros from `size` on, by one wave.  Fetching and storing are two steps, so that a chunk's fetches are all
// in flight before the first of them is waited for.  `vec`: size % 4 == 0 and 16-byte accesses are allowed;
// otherwise the vectors are copied one float at a time by store().
template <int W, int CH>
struct StagedVectors {
  static constexpr int Q = W / 4, IT = (CH * Q + PI_WAVE - 1) / PI_WAVE;
  float4 v[IT];
  const float* src;
  long stride;
  int cn, size;
  bool vec;
  __device__ inline void fetch(const float* __restrict__ from, long row_stride, int tokens, int floats, bool wide, int lane) {
    src = from; stride = row_stride; cn = tokens; size = floats; vec = wide;
    if (!vec) return;
#pragma unroll
    for (int j = 0; j < IT; ++j) {
      const int i = lane + j * PI_WAVE, tt = i / Q, r = (i - tt * Q) * 4;
      v[j] = (tt < cn && r < size) ? *reinterpret_cast<const float4*>(src + tt * stride + r) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  __device__ inline void store(float* dst, int lane) const {
    if (vec) {
#pragma unroll
      for (int j = 0; j < IT; ++j) {
        const int i = lane + j * PI_WAVE, tt = i / Q, r = (i - tt * Q) * 4;
        if (tt < cn) *reinterpret_cast<float4*>(dst + tt * W + r) = v[j];
      }
    } else {
      for (int i = lane; i < cn * W; i += PI_WAVE) {
        const int tt = i / W, r = i - tt * W;
        dst[i] = r < size ? src[tt * stride + r] : 0.f;
      }
    }
  }
};

// ------------------------------------------------------------------ state-space recurrence
// Per head h with group g = h / (H / G), state S [N, P] (float32, zero at the start):
//   dt = softplus(dt_raw + dt_bias[h]);  S <- exp(-exp(A_log[h]) * dt) S + dt * B_t x_t^T;
//   y_t = S^T C_t + D[h] x_t
// x, B, C are columns of the convolution's output: x at 0, B at H * P, C at H * P + G * N.
template <int NR, bool SHORT>
__global__ __launch_bounds__((PI_SCAN_WAVES + 1) * PI_WAVE) void state_space_scan_kernel(
    float* __restrict__ y, long y_stride, const float* __restrict__ xbc, long xbc_stride, const float* __restrict__ dt_raw,
    long dt_stride, const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dskip,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ state, long state_stride, int H, int P,
    int N, int G, int vec) {
  constexpr int W = ScanShape<NR, SHORT>::W, CH = ScanShape<NR, SHORT>::CH;
  __shared__ __attribute__((aligned(16))) float sB[2][CH * W];
  __shared__ __attribute__((aligned(16))) float sC[2][CH * W];
  __shared__ float sx[2][CH][PI_SCAN_COLUMNS], sdt[2][CH], sa[2][CH];
  const int r = blockIdx.x, h = blockIdx.y, z = blockIdx.z;
  const int wave = threadIdx.x / PI_WAVE, lane = threadIdx.x % PI_WAVE, part = lane % 16;
  const int g = h / (H / G);
  const int qs = q_start[r], n = q_start[r + 1] - qs;
  if (n <= 0) return;
  const int chunks = (n + CH - 1) / CH;
  const long b_col = (long)H * P + (long)g * N, c_col = b_col + (long)G * N, x_col = (long)h * P + z * PI_SCAN_COLUMNS;

  auto fill = [&](int c) {      // the staging wave
    const int buf = c & 1, t0 = c * CH, cn = n - t0 < CH ? n - t0 : CH;
    const float* src = xbc + (long)(qs + t0) * xbc_stride;
    StagedVectors<W, CH> Bs, Cs;
    Bs.fetch(src + b_col, xbc_stride, cn, N, vec != 0, lane);
    Cs.fetch(src + c_col, xbc_stride, cn, N, vec != 0, lane);
    constexpr int XI = (CH * PI_SCAN_COLUMNS + PI_WAVE - 1) / PI_WAVE;
    float xs[XI];
#pragma unroll
    for (int j = 0; j < XI; ++j) {
      const int i = lane + j * PI_WAVE, tt = i / PI_SCAN_COLUMNS, cc = i % PI_SCAN_COLUMNS;
      xs[j] = (tt < cn && z * PI_SCAN_COLUMNS + cc < P) ? src[tt * xbc_stride + x_col + cc] : 0.f;
    }
    const float raw = lane < cn ? dt_raw[(long)(qs + t0 + lane) * dt_stride + h] : 0.f;
    Bs.store(sB[buf], lane);
    Cs.store(sC[buf], lane);
#pragma unroll
    for (int j = 0; j < XI; ++j) {
      const int i = lane + j * PI_WAVE;
      if (i < CH * PI_SCAN_COLUMNS) (&sx[buf][0][0])[i] = xs[j];
    }
    if (lane < cn) {
      const float dt = softplus_f(raw + dt_bias[h]);
      sdt[buf][lane] = dt;
      sa[buf][lane] = expf(-expf(A_log[h]) * dt);
    }
  };

  float s[NR];
  const int cw = wave * 4 + lane / 16;                 // this lane's column within the block
  const int col = z * PI_SCAN_COLUMNS + cw;
  const bool live = col < P;
  float* Sg = state + (long)slots[r] * state_stride + (((long)h * gridDim.z + z) * PI_SCAN_WAVES + (wave & 3)) * NR * PI_WAVE + lane;
  const float skip = Dskip[h];
  if (wave < PI_SCAN_WAVES) {
#pragma unroll
    for (int i = 0; i < NR; ++i) s[i] = Sg[i * PI_WAVE];
  } else {
    fill(0);
  }
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    if (wave == PI_SCAN_WAVES) {
      if (c + 1 < chunks) fill(c + 1);
    } else {
      const int buf = c & 1, cn = n - c * CH < CH ? n - c * CH : CH;
#pragma unroll 2
      for (int tt = 0; tt < cn; ++tt) {
        const float x = sx[buf][tt][cw], a = sa[buf][tt], dx = sdt[buf][tt] * x;
        const float* Bv = &sB[buf][tt * W + part * NR];
        const float* Cv = &sC[buf][tt * W + part * NR];
        float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          s[i] = fmaf(a, s[i], Bv[i] * dx);
          if (i & 1) acc1 = fmaf(s[i], Cv[i], acc1);
          else acc0 = fmaf(s[i], Cv[i], acc0);
        }
        const float acc = row16_sum(acc0 + acc1);
        if (live && part == 0) y[(long)(qs + c * CH + tt) * y_stride + (long)h * P + col] = fmaf(skip, x, acc);
      }
    }
    __syncthreads();
  }
  if (wave < PI_SCAN_WAVES) {
#pragma unroll
    for (int i = 0; i < NR; ++i) Sg[i * PI_WAVE] = s[i];
  }
}

extern "C" int pi_state_space_scan(float* y, long y_stride, const float* xbc, long xbc_stride, const float* dt_raw, long dt_stride,
                                   const float* dt_bias, const float* A_log, const float* Dskip, const int* q_start,
                                   const int* slots, int R, int longest, float* state, long state_stride, int H, int P, int N, int G,
                                   hipStream_t stream) {
  PI_REQUIRE(H > 0 && H <= 65535 && P > 0 && N > 0 && G > 0 && H % G == 0, "state space: bad sizes heads=%d vdim=%d state=%d groups=%d", H, P, N, G);
  const int nr = scan_rows_per_lane(N);
  PI_REQUIRE(nr > 0, "state space: a state of %d rows per head is more than 256", N);
  PI_REQUIRE(R >= 0 && state_stride >= pi_scan_state_floats(H, N, P), "state space: a state row of %ld floats cannot hold %d x %d x %d", state_stride, H, N, P);
  if (R == 0) return 0;
  const int vec = N % 4 == 0 && xbc_stride % 4 == 0 && ((long)H * P) % 4 == 0 && (uintptr_t)xbc % 16 == 0;
  const dim3 grid(R, H, (P + PI_SCAN_COLUMNS - 1) / PI_SCAN_COLUMNS), block((PI_SCAN_WAVES + 1) * PI_WAVE);
#define PI_LAUNCH_SS1(NR_, SHORT_)                                                                                                       \
  hipLaunchKernelGGL((state_space_scan_kernel<NR_, SHORT_>), grid, block, 0, stream, y, y_stride, xbc, xbc_stride, dt_raw, dt_stride, \
                     dt_bias, A_log, Dskip, q_start, slots, state, state_stride, H, P, N, G, vec)
#define PI_LAUNCH_SS(NR_) do { if (longest <= 2) PI_LAUNCH_SS1(NR_, true); else PI_LAUNCH_SS1(NR_, false); } while (0)
  switch (nr) {
    case 1: PI_LAUNCH_SS(1); break;
    case 2: PI_LAUNCH_SS(2); break;
    case 4: PI_LAUNCH_SS(4); break;
    case 8: PI_LAUNCH_SS(8); break;
    default: PI_LAUNCH_SS(16); break;
  }
#undef PI_LAUNCH_SS
#undef PI_LAUNCH_SS1
  return pi_check_launch("state_space_scan");
}

// ------------------------------------------------------------------ gate, then norm in equal parts
// out[t, i] = mult * w[i] * v[i] / sqrt(mean over i's part of v^2 + eps),  v = y * silu(z).
// One block per (token, part).
template <typename TO>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(TO* __restrict__ out, long out_stride, const float* __restrict__ y,
                                                              long y_stride, const float* __restrict__ z, long z_stride,
                                                              const float* __restrict__ w, float eps, float mult, int size) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const int base = blockIdx.y * size;
  const float* yr = y + t * y_stride + base;
  const float* zr = z + t * z_stride + base;
  float ss = 0.f;
  for (int i = threadIdx.x; i < size; i += blockDim.x) {
    const float v = yr[i] * silu_f(zr[i]);
    ss = fmaf(v, v, ss);
  }
  const float rinv = 1.0f / sqrtf(block_sum(ss, scratch) / size + eps);
  for (int i = threadIdx.x; i < size; i += blockDim.x) {
    const float v = yr[i] * silu_f(zr[i]);
    out[t * out_stride + base + i] = from_float<TO>(v * rinv * w[base + i] * mult);
  }
}

extern "C" int pi_gated_group_norm(void* out, int out_dtype, long out_stride, const float* y, long y_stride, const float* z,
                                   long z_stride, const float* w, float eps, float mult, int T, int width, int parts,
                                   hipStream_t stream) {
  PI_REQUIRE(T >= 0 && width > 0 && parts > 0 && parts <= 65535 && width % parts == 0, "gated norm: %d columns in %d parts", width, parts);
  if (T == 0) return 0;
  const int size = width / parts;
  const dim3 grid(T, parts), block(size >= 256 ? 256 : 64);
  if (out_dtype == PI_F32)
    hipLaunchKernelGGL(gated_group_norm_kernel<float>, grid, block, 0, stream, (float*)out, out_stride, y, y_stride, z, z_stride, w, eps, mult, size);
  else if (out_dtype == PI_BF16)
    hipLaunchKernelGGL(gated_group_norm_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, out_stride, y, y_stride, z, z_stride, w, eps, mult, size);
  else
    return pi_fail("gated norm: unsupported dtype %d", out_dtype);
  return pi_check_launch("gated_group_norm");
}

// ------------------------------------------------------------------ walks over a state with decayed key rows
// Per head h with key head g = h / (H / G), state S [d, dv] (float32, zero at the start).  Three kinds:
//   SCAN_CHANNEL_DELTA  the gated delta rule with a decay per head and key channel:
//     q^ = q / sqrt(sum q^2 + unit_eps) * q_scale;  k^ = k / sqrt(sum k^2 + unit_eps);
//     decay[c] = exp(-exp(A_log[h]) * softplus(a[h, c] + dt_bias[h, c]));  beta = sigmoid(b[h]);
//     S <- diag(decay) S;  u = beta * (v - S^T k^);  S <- S + k^ u^T;  o = S^T q^
//   SCAN_HEAD_DELTA     the same with one decay per head: a is [T, H], dt_bias [H],
//     decay = exp(-exp(A_log[h]) * softplus(a[h] + dt_bias[h]));  S <- decay S
//   SCAN_DECAYED_OUTER  gated linear attention, no delta term and no unit vectors:
//     q' = q * q_scale;  decay[c] = sigmoid(a[h, c] + dt_bias[h, c])^(1 / tau);
//     S <- diag(decay) S + k v^T;  o = S^T q'
// q, k, v are columns of one float32 row per token (q at 0, k at G * d, v at 2 * G * d).
//
// First, once per token and head and in place: unit vectors over q and k (or the scaled q), decays
// over a, beta over b.  One wave per (token, key head) and per (token, head).
enum ScanKind : int { SCAN_CHANNEL_DELTA = 0, SCAN_HEAD_DELTA = 1, SCAN_DECAYED_OUTER = 2 };

__global__ __launch_bounds__(PI_WAVE) void delta_prepare_kernel(float* __restrict__ qkv, long qkv_stride, float* __restrict__ a,
                                                               long a_stride, const float* __restrict__ dt_bias,
                                                               const float* __restrict__ A_log, float* __restrict__ b,
                                                               long b_stride, int H, int G, int d, float q_scale, float unit_eps,
                                                               int kind, float inv_tau) {
  const long t = blockIdx.x;
  const int j = blockIdx.y, lane = threadIdx.x;
  if (j < G) {
    float* q = qkv + t * qkv_stride + (long)j * d;
    if (kind == SCAN_DECAYED_OUTER) {
      for (int c = lane; c < d; c += PI_WAVE) q[c] *= q_scale;
      return;
    }
    float* k = q + (long)G * d;
    float q2 = 0.f, k2 = 0.f;
    for (int c = lane; c < d; c += PI_WAVE) {
      q2 = fmaf(q[c], q[c], q2);
      k2 = fmaf(k[c], k[c], k2);
    }
    const float qn = q_scale / sqrtf(wave_sum(q2) + unit_eps), kn = 1.0f / sqrtf(wave_sum(k2) + unit_eps);
    for (int c = lane; c < d; c += PI_WAVE) {
      q[c] *= qn;
      k[c] *= kn;
    }
    return;
  }
  const int h = j - G;
  if (kind == SCAN_DECAYED_OUTER) {
    // sigmoid(z)^(1 / tau) = exp(-softplus(-z) / tau)
    float* ar = a + t * a_stride + (long)h * d;
    for (int c = lane; c < d; c += PI_WAVE) ar[c] = expf(-softplus_f(-(ar[c] + dt_bias[(long)h * d + c])) * inv_tau);
    return;
  }
  const float A = expf(A_log[h]);
  if (kind == SCAN_HEAD_DELTA) {
    if (lane == 0) {
      a[t * a_stride + h] = expf(-A * softplus_f(a[t * a_stride + h] + dt_bias[h]));
      b[t * b_stride + h] = sigmoid_f(b[t * b_stride + h]);
    }
    return;
  }
  float* ar = a + t * a_stride + (long)h * d;
  for (int c = lane; c < d; c += PI_WAVE) ar[c] = expf(-A * softplus_f(ar[c] + dt_bias[(long)h * d + c]));
  if (lane == 0) b[t * b_stride + h] = sigmoid_f(b[t * b_stride + h]);
}

// Then the walk: q^, k^ and v from qkv, decays from a, beta from b.  A column of S never meets another
// column, so a wave walks its four columns alone.
template <int NR, bool SHORT, int KIND>
__global__ __launch_bounds__((PI_SCAN_WAVES + 1) * PI_WAVE) void delta_scan_kernel(
    float* __restrict__ o, long o_stride, const float* __restrict__ qkv, long qkv_stride, const float* __restrict__ decay,
    long decay_stride, const float* __restrict__ beta, long beta_stride, const int* __restrict__ q_start,
    const int* __restrict__ slots, float* __restrict__ state, long state_stride, int H, int G, int d, int dv, int vec) {
  constexpr int W = ScanShape<NR, SHORT>::W, CH = ScanShape<NR, SHORT>::CH;
  __shared__ __attribute__((aligned(16))) float sq[2][CH * W];
  __shared__ __attribute__((aligned(16))) float sk[2][CH * W];
  __shared__ __attribute__((aligned(16))) float sg[2][KIND == SCAN_HEAD_DELTA ? 4 : CH * W];
  __shared__ float sv[2][CH][PI_SCAN_COLUMNS], sbeta[2][CH], sdecay[2][CH];
  const int r = blockIdx.x, h = blockIdx.y, z = blockIdx.z;
  const int wave = threadIdx.x / PI_WAVE, lane = threadIdx.x % PI_WAVE, part = lane % 16;
  const int g = h / (H / G);
  const int qs = q_start[r], n = q_start[r + 1] - qs;
  if (n <= 0) return;
  const int chunks = (n + CH - 1) / CH;
  const long q_col = (long)g * d, k_col = (long)G * d + (long)g * d, v_col = 2L * G * d + (long)h * dv + z * PI_SCAN_COLUMNS;

  auto fill = [&](int c) {      // the staging wave
    const int buf = c & 1, t0 = c * CH, cn = n - t0 < CH ? n - t0 : CH;
    const float* src = qkv + (long)(qs + t0) * qkv_stride;
    StagedVectors<W, CH> qs_, ks_, gs_;
    qs_.fetch(src + q_col, qkv_stride, cn, d, (vec & 1) != 0, lane);
    ks_.fetch(src + k_col, qkv_stride, cn, d, (vec & 1) != 0, lane);
    if constexpr (KIND != SCAN_HEAD_DELTA)
      gs_.fetch(decay + (long)(qs + t0) * decay_stride + (long)h * d, decay_stride, cn, d, (vec & 2) != 0, lane);
    constexpr int XI = (CH * PI_SCAN_COLUMNS + PI_WAVE - 1) / PI_WAVE;
    float vs[XI];
#pragma unroll
    for (int j = 0; j < XI; ++j) {
      const int i = lane + j * PI_WAVE, tt = i / PI_SCAN_COLUMNS, cc = i % PI_SCAN_COLUMNS;
      vs[j] = (tt < cn && z * PI_SCAN_COLUMNS + cc < dv) ? src[tt * qkv_stride + v_col + cc] : 0.f;
    }
    float bt = 0.f, dc = 0.f;
    if constexpr (KIND != SCAN_DECAYED_OUTER) bt = lane < cn ? beta[(long)(qs + t0 + lane) * beta_stride + h] : 0.f;
    if constexpr (KIND == SCAN_HEAD_DELTA) dc = lane < cn ? decay[(long)(qs + t0 + lane) * decay_stride + h] : 0.f;
    qs_.store(sq[buf], lane);
    ks_.store(sk[buf], lane);
    if constexpr (KIND != SCAN_HEAD_DELTA) gs_.store(sg[buf], lane);
#pragma unroll
    for (int j = 0; j < XI; ++j) {
      const int i = lane + j * PI_WAVE;
      if (i < CH * PI_SCAN_COLUMNS) (&sv[buf][0][0])[i] = vs[j];
    }
    if (lane < CH) {
      sbeta[buf][lane] = bt;
      sdecay[buf][lane] = dc;
    }
  };

  float s[NR];
  const int cw = wave * 4 + lane / 16;                 // this lane's column within the block
  const int col = z * PI_SCAN_COLUMNS + cw;
  const bool live = col < dv;
  float* Sg = state + (long)slots[r] * state_stride + (((long)h * gridDim.z + z) * PI_SCAN_WAVES + (wave & 3)) * NR * PI_WAVE + lane;
  if (wave < PI_SCAN_WAVES) {
#pragma unroll
    for (int i = 0; i < NR; ++i) s[i] = Sg[i * PI_WAVE];
  } else {
    fill(0);
  }
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    if (wave == PI_SCAN_WAVES) {
      if (c + 1 < chunks) fill(c + 1);
    } else {
      const int buf = c & 1, cn = n - c * CH < CH ? n - c * CH : CH;
#pragma unroll 2
      for (int tt = 0; tt < cn; ++tt) {
        const float* qv = &sq[buf][tt * W + part * NR];
        const float* kv = &sk[buf][tt * W + part * NR];
        float u;
        if constexpr (KIND == SCAN_DECAYED_OUTER) {
          const float* gv = &sg[buf][tt * W + part * NR];
#pragma unroll
          for (int i = 0; i < NR; ++i) s[i] *= gv[i];
          u = sv[buf][tt][cw];
        } else {
          float d0 = 0.f, d1 = 0.f;
          if constexpr (KIND == SCAN_HEAD_DELTA) {
            const float g1 = sdecay[buf][tt];
#pragma unroll
            for (int i = 0; i < NR; ++i) {
              s[i] *= g1;
              if (i & 1) d1 = fmaf(s[i], kv[i], d1);
              else d0 = fmaf(s[i], kv[i], d0);
            }
          } else {
            const float* gv = &sg[buf][tt * W + part * NR];
#pragma unroll
            for (int i = 0; i < NR; ++i) {
              s[i] *= gv[i];
              if (i & 1) d1 = fmaf(s[i], kv[i], d1);
              else d0 = fmaf(s[i], kv[i], d0);
            }
          }
          u = sbeta[buf][tt] * (sv[buf][tt][cw] - row16_sum(d0 + d1));
        }
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          s[i] = fmaf(kv[i], u, s[i]);
          if (i & 1) a1 = fmaf(s[i], qv[i], a1);
          else a0 = fmaf(s[i], qv[i], a0);
        }
        const float acc = row16_sum(a0 + a1);
        if (live && part == 0) o[(long)(qs + c * CH + tt) * o_stride + (long)h * dv + col] = acc;
      }
    }
    __syncthreads();
  }
  if (wave < PI_SCAN_WAVES) {
#pragma unroll
    for (int i = 0; i < NR; ++i) Sg[i * PI_WAVE] = s[i];
  }
}

// qkv, a and b are changed in place (unit vectors or scaled queries, decays, beta); o gets the read-outs.
// kind: a ScanKind.  SCAN_HEAD_DELTA: a is [T, H] and dt_bias [H].  SCAN_DECAYED_OUTER: b is not read, A_log neither,
// unit_eps neither; tau is the root taken of the sigmoid.
extern "C" int pi_delta_scan(float* o, long o_stride, float* qkv, long qkv_stride, float* a, long a_stride,
                             const float* dt_bias, const float* A_log, float* b, long b_stride, const int* q_start,
                             const int* slots, int R, int T, int longest, float* state, long state_stride, int H, int G, int d, int dv,
                             float q_scale, float unit_eps, int kind, float tau, hipStream_t stream) {
  PI_REQUIRE(H > 0 && H <= 32767 && G > 0 && H % G == 0 && d > 0 && dv > 0, "state walk: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", H, G, d, dv);
  PI_REQUIRE(kind >= SCAN_CHANNEL_DELTA && kind <= SCAN_DECAYED_OUTER, "state walk: unknown kind %d", kind);
  PI_REQUIRE(kind != SCAN_DECAYED_OUTER || tau > 0.f, "state walk: the decay's root %g must be positive", (double)tau);
  PI_REQUIRE(kind == SCAN_DECAYED_OUTER || (b && A_log), "state walk: the delta rule needs beta and decay rates");
  const int nr = scan_rows_per_lane(d);
  PI_REQUIRE(nr > 0, "state walk: keys of %d channels are more than 256", d);
  PI_REQUIRE(R >= 0 && T >= 0 && state_stride >= pi_scan_state_floats(H, d, dv), "state walk: a state row of %ld floats cannot hold %d x %d x %d", state_stride, H, d, dv);
  if (R == 0 || T == 0) return 0;
  hipLaunchKernelGGL(delta_prepare_kernel, dim3(T, G + H), dim3(PI_WAVE), 0, stream, qkv, qkv_stride, a, a_stride, dt_bias, A_log, b,
                     b_stride, H, G, d, q_scale, unit_eps, kind, kind == SCAN_DECAYED_OUTER ? 1.0f / tau : 0.f);
  if (pi_check_launch("delta_prepare")) return -1;
  // bit 0: q and k may be fetched 16 bytes at a time; bit 1: the decays too
  const int vec = (d % 4 == 0 && qkv_stride % 4 == 0 && (uintptr_t)qkv % 16 == 0 ? 1 : 0) |
                  (d % 4 == 0 && a_stride % 4 == 0 && (uintptr_t)a % 16 == 0 ? 2 : 0);
  const dim3 grid(R, H, (dv + PI_SCAN_COLUMNS - 1) / PI_SCAN_COLUMNS), block((PI_SCAN_WAVES + 1) * PI_WAVE);
#define PI_LAUNCH_DELTA2(NR_, SHORT_, KIND_)                                                                                                   \
  hipLaunchKernelGGL((delta_scan_kernel<NR_, SHORT_, KIND_>), grid, block, 0, stream, o, o_stride, qkv, qkv_stride, a, a_stride, b, b_stride, \
                     q_start, slots, state, state_stride, H, G, d, dv, vec)
#define PI_LAUNCH_DELTA1(NR_, SHORT_)                                            \
  do {                                                                           \
    if (kind == SCAN_HEAD_DELTA) PI_LAUNCH_DELTA2(NR_, SHORT_, SCAN_HEAD_DELTA); \
    else if (kind == SCAN_DECAYED_OUTER) PI_LAUNCH_DELTA2(NR_, SHORT_, SCAN_DECAYED_OUTER); \
    else PI_LAUNCH_DELTA2(NR_, SHORT_, SCAN_CHANNEL_DELTA);                      \
  } while (0)
#define PI_LAUNCH_DELTA(NR_) do { if (longest <= 2) PI_LAUNCH_DELTA1(NR_, true); else PI_LAUNCH_DELTA1(NR_, false); } while (0)
  switch (nr) {
    case 1: PI_LAUNCH_DELTA(1); break;
    case 2: PI_LAUNCH_DELTA(2); break;
    case 4: PI_LAUNCH_DELTA(4); break;
    case 8: PI_LAUNCH_DELTA(8); break;
    default: PI_LAUNCH_DELTA(16); break;
  }
#undef PI_LAUNCH_DELTA
#undef PI_LAUNCH_DELTA1
#undef PI_LAUNCH_DELTA2
  return pi_check_launch("delta_scan");
}
