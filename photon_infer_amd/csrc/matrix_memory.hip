// A recurrent mixer with a matrix memory per head (the mLSTM cell of xLSTM), token by token.
//
// Per head, with state S [d, dv], n [d] and a running maximum m (all float32, zero at the
// start of a sequence), and per token the query q (already scaled), key k, value v and the two
// gate pre-activations zi, zf (biases added here):
//   i = cap * tanh(zi / cap)                     log input gate
//   f = logsigmoid(cap * tanh(zf / cap))         log forget gate
//   m' = max(f + m, i);  a = exp(f + m - m');  b = exp(i - m')
//   S' = a S + b k v^T;  n' = a n + b k
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// The scan is sequential in the tokens of a request and runs them in the order given, so its
// result for a token does not depend on how the tokens were cut into steps.
//
// One wave per (request, head, 16 value columns): lane = column + 16 * part; the four parts split
// the d rows of the state, which stays in registers over all tokens of the step (rows beyond d are
// zeros that never leave the registers).  n and m are kept
// once per group of 16 columns ([slices, d + 1] per head), so that no block reads what another writes.
//
// State row of one request (floats): [heads][d][dv] S, then [heads][slices][d + 1] (n, then m).
#include "common.h"

#define MM_COLS 16
#define MM_PARTS 4

__host__ __device__ inline long mm_state_floats(int heads, int d, int dv) {
  const int slices = (dv + MM_COLS - 1) / MM_COLS;
  return (long)heads * d * dv + (long)heads * slices * (d + 1);
}

extern "C" long pi_matrix_memory_state_floats(int heads, int d, int dv) { return mm_state_floats(heads, d, dv); }

// Tokens are staged through LDS a chunk at a time (one trip to memory per chunk instead of one
// per token).  Everything of a chunk that does not depend on the state is made before its walk:
// the gates (lane j, token j), the running maximum (a short sequential pass over the chunk's
// gates, the same in every lane) and from it each token's decay a, input weight b and floor
// exp(-m).  The walk itself is multiply-adds on registers and LDS reads.
//
// Long portions are cut into segments of MM_SEGMENT tokens that run side by side (with 64 tokens a
// 2,048-token prompt gives every SIMD of the chip four waves to switch between).  The state's
// recurrence is linear once a, b are known, and those depend on the gates alone:
//   1. a gates kernel (one wave per request and head) makes a, b, exp(-m) for every token;
//   2. every segment is walked from a zero state, leaving its summary (its own contribution L
//      and the product A of its decays);
//   3. a prefix kernel turns the summaries into the states at the segments' starts (S <- A S + L,
//      segment by segment, from the request's state) and stores the state after the step;
//   4. every segment is walked again for its outputs, from the state at its start.
// A step whose requests bring at most one segment each (decoding, short portions) is one kernel,
// which makes its own gates.
#define MM_SEGMENT 64

// floats of one segment summary for one (head, column group): L's part of S [d][16], of n [d], then A
__host__ __device__ inline long mm_summary_floats(int d) { return (long)d * MM_COLS + d + 1; }

enum { MM_SINGLE = 0, MM_SUMMARY = 1, MM_OUTPUT = 2 };

template <int DPP, int MODE>
__global__ __launch_bounds__(PI_WAVE) void matrix_memory_scan_kernel(
    float* __restrict__ out, long out_stride, const float* __restrict__ proj, long proj_stride, int q_off, int k_off, int v_off,
    int i_off, int f_off, const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ state, long state_stride, int max_slots,
    int heads, int d, int dv, int segs, const float* __restrict__ coef, float* __restrict__ summaries) {
  constexpr int DP = MM_PARTS * DPP;             // rows of the state as the lanes hold them (>= d)
  constexpr int CH = 2048 / DP < PI_WAVE ? 2048 / DP : PI_WAVE;   // tokens per chunk: 8 KB of queries, as much of keys
  __shared__ __attribute__((aligned(16))) float qs[CH][DP];
  __shared__ __attribute__((aligned(16))) float ks[CH][DP];
  __shared__ float vs[CH][MM_COLS];
  __shared__ float gi[CH], gf[CH], wa[CH], wb[CH], we[CH];
  const int r = blockIdx.x / segs, seg = blockIdx.x % segs, h = blockIdx.y, slice = blockIdx.z;
  const int lane = threadIdx.x, col = lane % MM_COLS, part = lane / MM_COLS;
  const int c = slice * MM_COLS + col;
  const bool col_ok = c < dv;
  const int slot = slots[r];
  if (slot < 0 || slot >= max_slots) return;
  const int slices = gridDim.z;
  const int t0 = MODE == MM_SINGLE ? q_start[r] : q_start[r] + seg * MM_SEGMENT;
  const int t1 = MODE == MM_SINGLE ? q_start[r + 1] : min(q_start[r + 1], t0 + MM_SEGMENT);
  if (t0 >= t1) return;                          // the request has fewer segments
  float* Sg = state + (long)slot * state_stride + (long)h * d * dv;
  float* nm = state + (long)slot * state_stride + (long)heads * d * dv + ((long)h * slices + slice) * (d + 1);
  const long sum_floats = mm_summary_floats(d);
  float* sums = MODE == MM_SINGLE ? nullptr : summaries + (((long)r * segs * heads + h) * slices + slice) * sum_floats;
  const long sum_stride = (long)heads * slices * sum_floats;      // from one segment's summary to the next
  const int r0 = part * DPP;                     // this lane's rows of the state: r0 .. r0 + DPP - 1 (those below d)
  float S[DPP], n[DPP];
#pragma unroll
  for (int i = 0; i < DPP; ++i) {
    const bool ok = r0 + i < d;
    S[i] = (MODE == MM_SINGLE && ok && col_ok) ? Sg[(long)(r0 + i) * dv + c] : 0.f;
    n[i] = (MODE == MM_SINGLE && ok) ? nm[r0 + i] : 0.f;
  }
  if (MODE == MM_OUTPUT) {                       // the state at the segment's start, left by the prefix kernel in the summary's place
    const float* L = sums + seg * sum_stride;
#pragma unroll
    for (int i = 0; i < DPP; ++i) {
      const bool ok = r0 + i < d;
      S[i] = ok ? L[(r0 + i) * MM_COLS + col] : 0.f;
      n[i] = ok ? L[d * MM_COLS + r0 + i] : 0.f;
    }
  }
  float m = MODE == MM_SINGLE ? nm[d] : 0.f;
  float decay = 1.0f;                            // MM_SUMMARY: the product of the segment's decays
  const float bi = i_bias[h], bf = f_bias[h];
  for (int tc = t0; tc < t1; tc += CH) {
    const int nt = min(CH, t1 - tc);
    // the chunk's queries (scaled), keys and this block's value columns; rows beyond d are zero
    // (all loads of a chunk are asked for before the first is stored: one wait for memory per chunk)
    {
      constexpr int PER = CH * DP / PI_WAVE;     // elements of q, and of k, per lane: 32 whatever the sizes
      float kreg[PER], qreg[PER];
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int idx = lane + u * PI_WAVE, j = idx / DP, i = idx % DP;
        const bool in = j < nt && i < d;
        const float* row = proj + (long)(tc + (in ? j : 0)) * proj_stride + h * d + (in ? i : 0);
        kreg[u] = row[k_off];
        if (MODE != MM_SUMMARY) qreg[u] = row[q_off];
      }
      constexpr int VPER = CH * MM_COLS / PI_WAVE;
      float vreg[VPER];
#pragma unroll
      for (int u = 0; u < VPER; ++u) {
        const int idx = lane + u * PI_WAVE, j = idx / MM_COLS, cc = slice * MM_COLS + idx % MM_COLS;
        const bool in = j < nt && cc < dv;
        vreg[u] = proj[(long)(tc + (in ? j : 0)) * proj_stride + v_off + h * dv + (in ? cc : 0)];
      }
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const int idx = lane + u * PI_WAVE, j = idx / DP, i = idx % DP;
        const bool in = j < nt && i < d;
        ks[j][i] = in ? kreg[u] : 0.f;
        if (MODE != MM_SUMMARY) qs[j][i] = in ? qreg[u] * q_scale : 0.f;
      }
#pragma unroll
      for (int u = 0; u < VPER; ++u) {
        const int idx = lane + u * PI_WAVE, j = idx / MM_COLS, cc = slice * MM_COLS + idx % MM_COLS;
        vs[j][idx % MM_COLS] = (j < nt && cc < dv) ? vreg[u] : 0.f;
      }
    }
    if (MODE == MM_SINGLE) {
      if (lane < nt) {
        const float* row = proj + (long)(tc + lane) * proj_stride;
        const float fz = cap * tanhf((row[f_off + h] + bf) / cap);
        gi[lane] = cap * tanhf((row[i_off + h] + bi) / cap);
        gf[lane] = fminf(fz, 0.f) - log1pf(expf(-fabsf(fz)));
      }
      __syncthreads();
      // the running maximum over the chunk (every lane the same); lane j keeps token j's
      float m_before = m, m_mine = m;
      for (int j = 0; j < nt; ++j) {
        const float m_new = fmaxf(gf[j] + m, gi[j]);
        if (j == lane) {
          m_before = m;
          m_mine = m_new;
        }
        m = m_new;
      }
      if (lane < nt) {
        wa[lane] = expf(gf[lane] + m_before - m_mine);
        wb[lane] = expf(gi[lane] - m_mine);
        we[lane] = expf(-m_mine);
      }
    } else if (lane < nt) {
      const float* cf = coef + ((long)(tc + lane) * heads + h) * 3;
      wa[lane] = cf[0];
      wb[lane] = cf[1];
      we[lane] = cf[2];
    }
    __syncthreads();
    for (int j = 0; j < nt; ++j) {
      const float a = wa[j], b = wb[j];
      const float bv = b * vs[j][col];
      float num[4] = {0.f, 0.f, 0.f, 0.f}, den[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < DPP; i += 4) {
        const float4 kk = *reinterpret_cast<const float4*>(&ks[j][r0 + i]);
        const float kv[4] = {kk.x, kk.y, kk.z, kk.w};
        if (MODE == MM_SUMMARY) {
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            S[i + u] = fmaf(a, S[i + u], kv[u] * bv);
            n[i + u] = fmaf(a, n[i + u], b * kv[u]);
          }
        } else {
          const float4 qq = *reinterpret_cast<const float4*>(&qs[j][r0 + i]);
          const float qv[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            S[i + u] = fmaf(a, S[i + u], kv[u] * bv);
            n[i + u] = fmaf(a, n[i + u], b * kv[u]);
            num[u] = fmaf(S[i + u], qv[u], num[u]);
            den[u] = fmaf(n[i + u], qv[u], den[u]);
          }
        }
      }
      if (MODE == MM_SUMMARY) {
        decay *= a;
      } else {
        float nu = (num[0] + num[1]) + (num[2] + num[3]), de = (den[0] + den[1]) + (den[2] + den[3]);
        nu += __shfl_xor(nu, 16, PI_WAVE);
        de += __shfl_xor(de, 16, PI_WAVE);
        nu += __shfl_xor(nu, 32, PI_WAVE);
        de += __shfl_xor(de, 32, PI_WAVE);
        if (part == 0 && col_ok) out[(long)(tc + j) * out_stride + h * dv + c] = nu / (fmaxf(fabsf(de), we[j]) + 1e-6f);
      }
    }
    __syncthreads();
  }
  if (MODE == MM_OUTPUT) return;                 // the state was stored by the prefix kernel
  if (MODE == MM_SUMMARY) {
    float* L = sums + seg * sum_stride;
#pragma unroll
    for (int i = 0; i < DPP; ++i) {
      if (r0 + i < d) {
        L[(r0 + i) * MM_COLS + col] = S[i];
        if (col == 0) L[d * MM_COLS + r0 + i] = n[i];
      }
    }
    if (lane == 0) L[sum_floats - 1] = decay;
    return;
  }
#pragma unroll
  for (int i = 0; i < DPP; ++i) {
    if (r0 + i < d) {
      if (col_ok) Sg[(long)(r0 + i) * dv + c] = S[i];
      if (col == 0) nm[r0 + i] = n[i];
    }
  }
  if (lane == 0) nm[d] = m;
}

// a, b and exp(-m) of every token of the step, [T, heads, 3], and the running maximum after each
// request's last token, [R, heads].  One block per (request, head): 256 tokens' gates at a time
// (thread j, token j) into LDS, then the maximum's chain over them (two operations per token, the
// same in every thread, its LDS reads independent of the chain), then each thread its token's three numbers.
#define MM_GATES_BLOCK 256
__global__ __launch_bounds__(MM_GATES_BLOCK) void matrix_memory_gates_kernel(
    float* __restrict__ coef, float* __restrict__ m_end, const float* __restrict__ proj, long proj_stride, int i_off, int f_off,
    const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, const int* __restrict__ q_start,
    const int* __restrict__ slots, const float* __restrict__ state, long state_stride, int max_slots, int heads, int d, int dv) {
  __shared__ float gis[MM_GATES_BLOCK], gfs[MM_GATES_BLOCK];
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int slot = slots[r];
  if (slot < 0 || slot >= max_slots) return;
  const int slices = (dv + MM_COLS - 1) / MM_COLS;
  float m = state[(long)slot * state_stride + (long)heads * d * dv + ((long)h * slices) * (d + 1) + d];
  const float bi = i_bias[h], bf = f_bias[h];
  const int t0 = q_start[r], t1 = q_start[r + 1];
  for (int tc = t0; tc < t1; tc += MM_GATES_BLOCK) {
    const int nt = min(MM_GATES_BLOCK, t1 - tc);
    float gi = 0.f, gf = 0.f;
    if (tid < nt) {
      const float* row = proj + (long)(tc + tid) * proj_stride;
      const float fz = cap * tanhf((row[f_off + h] + bf) / cap);
      gi = cap * tanhf((row[i_off + h] + bi) / cap);
      gf = fminf(fz, 0.f) - log1pf(expf(-fabsf(fz)));
    }
    __syncthreads();                 // the chain of the chunk before has been read
    gis[tid] = gi;
    gfs[tid] = gf;
    __syncthreads();
    float m_before = m, m_mine = m;
    for (int j = 0; j < nt; ++j) {
      const float m_new = fmaxf(gfs[j] + m, gis[j]);
      if (j == tid) {
        m_before = m;
        m_mine = m_new;
      }
      m = m_new;
    }
    if (tid < nt) {
      float* cf = coef + ((long)(tc + tid) * heads + h) * 3;
      cf[0] = expf(gf + m_before - m_mine);
      cf[1] = expf(gi - m_mine);
      cf[2] = expf(-m_mine);
    }
  }
  if (tid == 0) m_end[r * heads + h] = m;
}

// From the segments' summaries to the states at their starts: element by element, v = the request's
// state; for every segment in turn its summary is replaced by v and v <- A v + L.  What is left is
// the request's state after the step, which is stored (the walks for the outputs read the starts only).
__global__ __launch_bounds__(256) void matrix_memory_prefix_kernel(float* __restrict__ state, long state_stride, int max_slots,
                                                                   const int* __restrict__ q_start, const int* __restrict__ slots,
                                                                   float* __restrict__ summaries, const float* __restrict__ m_end,
                                                                   int heads, int d, int dv, int segs) {
  const int r = blockIdx.x, h = blockIdx.y, slice = blockIdx.z, slices = gridDim.z;
  const int slot = slots[r];
  if (slot < 0 || slot >= max_slots) return;
  const int n_seg = (q_start[r + 1] - q_start[r] + MM_SEGMENT - 1) / MM_SEGMENT;
  float* Sg = state + (long)slot * state_stride + (long)h * d * dv;
  float* nm = state + (long)slot * state_stride + (long)heads * d * dv + ((long)h * slices + slice) * (d + 1);
  const long sum_floats = mm_summary_floats(d);
  float* sums = summaries + (((long)r * segs * heads + h) * slices + slice) * sum_floats;
  const long sum_stride = (long)heads * slices * sum_floats;
  for (int idx = threadIdx.x; idx < d * MM_COLS + d; idx += blockDim.x) {
    const bool is_n = idx >= d * MM_COLS;
    const int row = is_n ? idx - d * MM_COLS : idx / MM_COLS, c = slice * MM_COLS + idx % MM_COLS;
    const bool there = is_n || c < dv;
    float* where = is_n ? nm + row : Sg + (long)row * dv + (there ? c : 0);
    float v = there ? *where : 0.f;
    for (int s = 0; s < n_seg; ++s) {
      const float A = sums[s * sum_stride + sum_floats - 1], L = sums[s * sum_stride + idx];
      sums[s * sum_stride + idx] = v;
      v = fmaf(A, v, L);
    }
    if (there) *where = v;
  }
  if (threadIdx.x == 0) nm[d] = m_end[r * heads + h];
}

extern "C" int pi_matrix_memory_segment() { return MM_SEGMENT; }

// out float32 [T, heads * dv]: the cell's raw output per head.  proj float32 rows hold q, k
// ([heads, d] each), v ([heads, dv]) and the gate pre-activations ([heads] each) at the given
// column offsets.  Requests r = 0 .. R-1 own tokens q_start[r] .. q_start[r+1]; their states are
// rows slots[r] of `state`.  max_q_len: the most tokens a request brings (an upper bound will do);
// above MM_SEGMENT the step runs in segments and needs `work`: float32, at least
// pi_matrix_memory_work_floats(T, R, max_q_len, heads, d, dv).
extern "C" long pi_matrix_memory_work_floats(int T, int R, int max_q_len, int heads, int d, int dv) {
  if (max_q_len <= MM_SEGMENT) return 0;
  const long segs = (max_q_len + MM_SEGMENT - 1) / MM_SEGMENT, slices = (dv + MM_COLS - 1) / MM_COLS;
  return (long)T * heads * 3 + (long)R * heads + (long)R * segs * heads * slices * mm_summary_floats(d);
}

extern "C" int pi_matrix_memory_scan(float* out, long out_stride, const float* proj, long proj_stride, int q_off, int k_off,
                                     int v_off, int i_off, int f_off, const float* i_bias, const float* f_bias, float cap,
                                     float q_scale, const int* q_start, const int* slots, int R, float* state,
                                     long state_stride, int max_slots, int heads, int d, int dv, int T, int max_q_len,
                                     float* work, long work_floats, hipStream_t stream) {
  PI_REQUIRE(R >= 0 && heads > 0 && d > 0 && dv > 0, "matrix memory: bad sizes");
  PI_REQUIRE(d <= 4 * 64, "matrix memory: key size %d is above %d", d, 4 * 64);
  PI_REQUIRE(state_stride >= mm_state_floats(heads, d, dv), "matrix memory: state rows of %ld floats are too short", state_stride);
  PI_REQUIRE(cap > 0.f, "matrix memory: the gates' cap must be positive");
  PI_REQUIRE(heads <= 65535, "matrix memory: too many heads");
  if (R == 0) return 0;
  const int slices = (dv + MM_COLS - 1) / MM_COLS;
  PI_REQUIRE(slices <= 65535, "matrix memory: value size %d is too large", dv);
  const int segs = max_q_len <= MM_SEGMENT ? 1 : (max_q_len + MM_SEGMENT - 1) / MM_SEGMENT;
  PI_REQUIRE((long)R * segs < 2147483647L, "matrix memory: too many segments");
  PI_REQUIRE(segs == 1 || (work && work_floats >= pi_matrix_memory_work_floats(T, R, max_q_len, heads, d, dv)),
             "matrix memory: a step in %d segments needs its workspace", segs);
  float* coef = work;
  float* m_end = segs > 1 ? coef + (long)T * heads * 3 : nullptr;
  float* summaries = segs > 1 ? m_end + (long)R * heads : nullptr;
  const dim3 grid(R * segs, heads, slices), block(PI_WAVE);
  const int dpp = (d + MM_PARTS - 1) / MM_PARTS;
#define MM_GO(DPP, MODE) hipLaunchKernelGGL((matrix_memory_scan_kernel<DPP, MODE>), grid, block, 0, stream, out, out_stride, proj, proj_stride, q_off, \
                                      k_off, v_off, i_off, f_off, i_bias, f_bias, cap, q_scale, q_start, slots, state, state_stride,    \
                                      max_slots, heads, d, dv, segs, coef, summaries)
#define MM_PICK(MODE)                \
  do {                               \
    if (dpp <= 8) MM_GO(8, MODE);    \
    else if (dpp <= 16) MM_GO(16, MODE); \
    else if (dpp <= 32) MM_GO(32, MODE); \
    else MM_GO(64, MODE);            \
  } while (0)
  if (segs == 1) {
    MM_PICK(MM_SINGLE);
    return pi_check_launch("matrix_memory_scan");
  }
  hipLaunchKernelGGL(matrix_memory_gates_kernel, dim3(R, heads), dim3(MM_GATES_BLOCK), 0, stream, coef, m_end, proj, proj_stride, i_off, f_off, i_bias,
                     f_bias, cap, q_start, slots, state, state_stride, max_slots, heads, d, dv);
  MM_PICK(MM_SUMMARY);
  hipLaunchKernelGGL(matrix_memory_prefix_kernel, dim3(R, heads, slices), dim3(256), 0, stream, state, state_stride, max_slots, q_start,
                     slots, summaries, m_end, heads, d, dv, segs);
  MM_PICK(MM_OUTPUT);
#undef MM_PICK
#undef MM_GO
  return pi_check_launch("matrix_memory_scan");
}

// y[t, h*dv + c] = o / sqrt(mean_c(o^2) + eps) * w[h*dv + c] * act(g[t, h*dv + c]); one wave per (token, head);
// act: the sigmoid, or (silu_gate) z * sigmoid(z)
template <typename T>
__global__ __launch_bounds__(PI_WAVE) void head_norm_gate_kernel(T* __restrict__ y, const float* __restrict__ o, long o_stride,
                                                                 const float* __restrict__ g, long g_stride,
                                                                 const float* __restrict__ w, float eps, int heads, int dv, float mult,
                                                                 int silu_gate) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + t * o_stride + (long)h * dv;
  float ss = 0.f;
  for (int c = lane; c < dv; c += PI_WAVE) ss = fmaf(orow[c], orow[c], ss);
  const float r = mult / sqrtf(wave_sum(ss) / dv + eps);
  for (int c = lane; c < dv; c += PI_WAVE) {
    const float z = g[t * g_stride + h * dv + c];
    const float sg = 1.0f / (1.0f + expf(-z));
    const float gate = silu_gate ? z * sg : sg;
    y[(t * heads + h) * dv + c] = from_float<T>(orow[c] * r * w[h * dv + c] * gate);
  }
}

extern "C" int pi_head_norm_gate(void* y, int dtype, const float* o, long o_stride, const float* g, long g_stride,
                                 const float* w, float eps, int T, int heads, int dv, float mult, int silu_gate, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && heads > 0 && heads <= 65535 && dv > 0, "head norm: bad sizes");
  if (T == 0) return 0;
  const dim3 grid(T, heads), block(PI_WAVE);
  if (dtype == PI_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, stream, (float*)y, o, o_stride, g, g_stride, w, eps, heads, dv, mult, silu_gate);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, o, o_stride, g, g_stride, w, eps, heads, dv, mult, silu_gate);
  else
    return pi_fail("head norm: unsupported dtype %d", dtype);
  return pi_check_launch("head_norm_gate");
}
