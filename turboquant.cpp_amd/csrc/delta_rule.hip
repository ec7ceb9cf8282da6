// The gated delta rule with one decay per head and key channel, over per-sequence state of fixed size.
//
// Per head, with a state S [D][V] (key channels by value channels) that starts at zero, token by token:
//   S <- diag(g) S ;  u = beta (v - S^T k) ;  S <- S + k u^T ;  o = S^T q
// with g = exp(-exp(A_log_h) * softplus(a + dt_bias)) in (0, 1) per key channel, beta = sigmoid(b) per head, and q, k
// unit vectors per head (q also times D^-1/2) made from projections that passed a short causal convolution over time
// and silu.  Each head's o is then divided by its root mean square, multiplied by a weight per value channel and by a
// sigmoid gate.  Everything here is float arithmetic on both libraries; the products around it are the library's.
//
// The kernels, for prompts and for decoding alike (a decoded token is a run of one):
//   delta_prep   per token: convolution (its first inputs from the sequence's state), silu, unit vectors, beta, and
//                the low-rank activations of the decay and the gate in the activation type, for the product behind
//   delta_decay  (steps of many tokens) the decays of all tokens, in parallel, in place of what they are made from
//   delta_scan   per (sequence, head, block of value channels): the recurrence over the run's tokens in order, the
//                state in registers (16 key channels of a value channel per lane), tokens staged through two LDS
//                buffers in chunks; a short step works out its decays as it stages them
//   delta_out    per token: norm and gate of every head; and per sequence: the convolution's new state
//   delta_decode (steps of one token per sequence) the second low-rank products, decays, recurrence, norm, gate and the
//                convolution's new state in one launch
//
// A second form (DeltaDims.mode 1) has one decay per head, g = exp(-exp(A_log_h) * softplus(a_h + dt_bias_h)) with a_h a
// projection of its own, and a gate that is a full projection with an activation of the caller's choice (gates.def); its
// projections are q | k | v | b (H) | a (H) | gate (H V), and it has no low-rank products.  The same kernels serve it.
//
// A sequence's row of state (float): S as [H][D][V], then for every convolution channel (q's, k's, v's) its last
// taps - 1 inputs, oldest first.  Projections P [T][NP] (float): q (G D) | k (G D) | v (H V) | b (H) | a1 (ra) | g1 (rg).
#include "common.h"

#define DR_ROWS 16        // key channels of a value channel that one lane keeps
#define DR_CHUNK 16       // tokens staged at a time

struct DeltaDims {
  int H, G, D, V;         // heads, q/k heads, key width, value width
  int taps;               // of the convolution
  int ra, rg;             // ranks of the decay's and the gate's first product
  int mode;               // 0: a decay per head and key channel, behind low-rank products; 1: a decay per head (ra = rg = 0)
};
__host__ __device__ __forceinline__ int dd_channels(const DeltaDims& d) { return 2 * d.G * d.D + d.H * d.V; }
__host__ __device__ __forceinline__ int dd_np(const DeltaDims& d) {
  return d.mode == 1 ? dd_channels(d) + 2 * d.H + d.H * d.V : dd_channels(d) + d.H + d.ra + d.rg;
}
__host__ __device__ __forceinline__ int64_t dd_state(const DeltaDims& d) {
  return (int64_t)d.H * d.D * d.V + (int64_t)dd_channels(d) * (d.taps - 1);
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// ------------------------------------------------------------------------------------------ per token
// grid (T, units / 4), block 256: a wave takes one "unit" of its token: one of the G query heads, the G key heads, the H
// value heads, or the unit of beta and the low-rank activations.  An input before the token's run comes from the
// state: the token is the c-th of its run if c of the taps - 1 tokens before it in the packed arrays have its slot
// (c < taps - 1), and then input i - d (d > c) is the state's (d - c)-th most recent.
__global__ __launch_bounds__(256) void delta_prep_kernel(const float* __restrict__ P, const int* __restrict__ slot_of_token,
                                                         const float* __restrict__ state, int64_t state_stride,
                                                         const float* __restrict__ conv_w, DeltaDims dm,
                                                         float* __restrict__ qn, float* __restrict__ kn,
                                                         float* __restrict__ vc, float* __restrict__ beta,
                                                         act_t* __restrict__ low, const float* __restrict__ a_log,
                                                         const float* __restrict__ dt_bias, float* __restrict__ dec) {
  const int t = blockIdx.x, wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int G = dm.G, D = dm.D, H = dm.H, V = dm.V, K = dm.taps;
  const int NP = dd_np(dm), C = dd_channels(dm);
  const int slot = slot_of_token[t];
  int before = 0;        // tokens of the same run right before this one, up to taps - 1
  while (before < K - 1 && t - before - 1 >= 0 && slot_of_token[t - before - 1] == slot) ++before;
  const float* hist = state + (size_t)slot * state_stride + (size_t)H * D * V;      // [C][K - 1]
  const float* row = P + (size_t)t * NP;
  const int units = 2 * G + H + 1;
  for (int u = blockIdx.y * 4 + wave; u < units; u += 4 * gridDim.y) {
    if (u == units - 1) {
      for (int h = lane; h < H; h += TQ_WAVE) beta[(size_t)t * H + h] = sigmoid_f(row[C + h]);
      if (dm.mode == 1) {       // the decay of every head
        for (int h = lane; h < H; h += TQ_WAVE)
          dec[(size_t)t * H + h] = expf(-expf(a_log[h]) * softplus_f(row[C + H + h] + dt_bias[h]));
        continue;
      }
      for (int i = lane; i < dm.ra + dm.rg; i += TQ_WAVE)
        low[(size_t)t * (dm.ra + dm.rg) + i] = from_f32<act_t>(row[C + H + i]);
      continue;
    }
    const bool is_v = u >= 2 * G;
    const int width = is_v ? V : D;
    const int c0 = is_v ? 2 * G * D + (u - 2 * G) * V : u * D;      // the unit's first channel
    float ss = 0.f;
    // (a unit wider than 64 goes in turns; its values wait in the output and are scaled afterwards)
    float* dst = is_v ? vc + (size_t)t * H * V + (size_t)(u - 2 * G) * V
                      : (u < G ? qn + (size_t)t * G * D + (size_t)u * D : kn + (size_t)t * G * D + (size_t)(u - G) * D);
    for (int i = lane; i < width; i += TQ_WAVE) {
      const int c = c0 + i;
      const float* w = conv_w + (size_t)c * K;
      float y = 0.f;
      for (int j = 0; j < K; ++j) {
        const int d = K - 1 - j;        // how many tokens back
        const float in = d <= before ? P[(size_t)(t - d) * NP + c] : hist[(size_t)c * (K - 1) + (K - 1) - (d - before)];
        y = fmaf(w[j], in, y);
      }
      y = silu_f(y);
      dst[i] = y;
      ss += y * y;
    }
    if (is_v) continue;
    ss = wave_sum(ss);
    const float f = (1.0f / sqrtf(ss + 1e-6f)) * (u < G ? 1.0f / sqrtf((float)D) : 1.0f);
    for (int i = lane; i < width; i += TQ_WAVE) dst[i] *= f;
  }
}

// ------------------------------------------------------------------------------------------ decays of a long step
// ag[t][h D + i] <- exp(-exp(a_log[h]) * softplus(ag[t][h D + i] + dt_bias[h D + i])), in place, for the first H D
// columns of every row: what the recurrence multiplies the state's rows by.  A step of many tokens works them out here,
// once and in parallel; the recurrence of a short step does it as it stages its tokens.
__global__ __launch_bounds__(256) void delta_decay_kernel(float* __restrict__ ag, const float* __restrict__ a_log,
                                                          const float* __restrict__ dt_bias, int HD, int D, int AGW,
                                                          int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % HD);
  float* at = ag + (i / HD) * AGW + c;
  *at = expf(-expf(a_log[c / D]) * softplus_f(*at + dt_bias[c]));
}

// ------------------------------------------------------------------------------------------ the recurrence
// Sums over the NSEG lanes that share a value channel (neighbours, aligned): within quads, then the two quads of
// eight lanes, then the two eights of a row of sixteen.  Every lane ends up with the total; the order is fixed.
template <int NSEG>
__device__ __forceinline__ float seg_sum(float v) {
#define TQ_DPP_ADD(ctrl) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xf, 0xf, false))
  if (NSEG >= 2) TQ_DPP_ADD(0xB1);        // quad_perm [1, 0, 3, 2]
  if (NSEG >= 4) TQ_DPP_ADD(0x4E);        // quad_perm [2, 3, 0, 1]
  if (NSEG >= 8) TQ_DPP_ADD(0x141);       // row_half_mirror
  if (NSEG >= 16) TQ_DPP_ADD(0x140);      // row_mirror
#undef TQ_DPP_ADD
  return v;
}

// grid (H * col_blocks, B), block NSEG * LC rounded up to whole waves: lane (lc, seg) keeps rows 16 seg .. 16 seg + 15 of the
// CPT value channels lc, lc + LC, ... of its block of cols = CPT * LC: several channels to a lane give it chains of
// multiply-adds that do not wait for each other, and one read of q, k and the decays from LDS serves them all.  The run's tokens pass through two LDS buffers in chunks of C = min(16, 8 block / DP) tokens:
// while a chunk is worked through, the next one's values are on their way from memory into registers (8 of q, k and
// decay per thread, 16 / NSEG of v), and go into the other buffer afterwards; one barrier a chunk.
// ag [T][H D + H V]: the decay's and the gate's second products; DECAYED: the first H D columns already hold the decays
// (delta_decay_kernel), else they hold what a_log [H] and dt_bias [H D] still have to be applied to (a kernel of its own
// for each, so that the one for long steps carries no exponentials).
#define DR_STAGE 8
// A lane's 16 rows of q, k and decays lie 20 floats from its neighbour's in LDS, not 16: the lanes of a wave that read
// different rows then hit different banks (blocks 80 bytes apart start at banks 0, 20, 8, 28, 16, 4, 24, 12).
#define DR_PAD 20
template <int NSEG, int CPT, bool DECAYED>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                                                         const float* __restrict__ vc, const float* __restrict__ beta,
                                                         const float* __restrict__ ag, const float* __restrict__ a_log,
                                                         const float* __restrict__ dt_bias,
                                                         const int* __restrict__ cu_seqlens, const int* __restrict__ slots,
                                                         float* __restrict__ state, int64_t state_stride, DeltaDims dm,
                                                         int cols, int col_blocks, int head_decay,
                                                         float* __restrict__ o_raw) {
  constexpr int DP = DR_ROWS * NSEG, RL = DR_PAD * NSEG;      // rows of a token, and the floats they take in LDS
  constexpr int EV = 16 * CPT / NSEG > 0 ? 16 * CPT / NSEG : 1;      // values of v per thread and chunk, at the most
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int C = min(DR_CHUNK, DR_STAGE * (int)blockDim.x / DP);
  // (a multiple of four floats, so that either buffer's rows of q, k and decays can be read 16 bytes at a time)
  const int buf_floats = 3 * C * RL + (C * cols + 3) / 4 * 4 + DR_CHUNK;
  const int H = dm.H, G = dm.G, D = dm.D, V = dm.V;
  const int h = blockIdx.x / col_blocks, cb = blockIdx.x % col_blocks, b = blockIdx.y;
  const int gq = h / (H / G);
  const int tid = threadIdx.x, seg = tid % NSEG, lc = tid / NSEG;
  const int LC = cols / CPT;                 // lanes' columns in the block; cols is a multiple of CPT
  int cloc[CPT];                             // this lane's channels within the block (0 where it has none)
  bool col_ok[CPT];
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0;
  float* S = state + (size_t)slots[b] * state_stride + (size_t)h * D * V;
  float s[CPT][DR_ROWS];
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    const int cl = lc + j * LC;
    col_ok[j] = lc < LC && cb * cols + cl < V;
    cloc[j] = col_ok[j] ? cl : 0;
#pragma unroll
    for (int i = 0; i < DR_ROWS; ++i) {
      const int r = seg * DR_ROWS + i;
      s[j][i] = col_ok[j] && r < D ? S[(size_t)r * V + cb * cols + cl] : 0.f;
    }
  }
  const float rate = expf(a_log[h]);
  const int AGW = H * D + H * V;

  float rq[DR_STAGE], rk[DR_STAGE], rg[DR_STAGE], rv[EV], rb = 0.f;
  // Asks memory for the chunk that starts at token c0 of the run.  Every load is unconditional, from an address that
  // is clamped into the chunk, and what lies outside is replaced when the values are staged: a load under a condition
  // is followed by a wait for it (its value is merged with the other branch's right away), and the loads of a chunk
  // then go out one by one, a memory latency each.
  auto fetch = [&](int c0) {
    const int nc = min(C, n - c0);
#pragma unroll
    for (int j = 0; j < DR_STAGE; ++j) {
      const int idx = tid + j * (int)blockDim.x, c = min(idx / DP, nc - 1), r = min(idx % DP, D - 1);
      const size_t t = (size_t)(t0 + c0 + c);
      rq[j] = qn[t * G * D + (size_t)gq * D + r];
      rk[j] = kn[t * G * D + (size_t)gq * D + r];
      rg[j] = head_decay ? ag[t * H + h] : ag[t * AGW + (size_t)h * D + r];      // (head_decay: ag is [T][H] decays)
    }
#pragma unroll
    for (int j = 0; j < EV; ++j) {
      const int idx = tid + j * (int)blockDim.x, c = min(idx / cols, nc - 1), jj = min(cb * cols + idx % cols, V - 1);
      rv[j] = vc[(size_t)(t0 + c0 + c) * H * V + (size_t)h * V + jj];
    }
    rb = beta[(size_t)(t0 + c0 + min(tid, nc - 1)) * H + h];
  };
  // puts what fetch brought into buffer `at`; a row beyond D keeps its zeros (q = k = 0, decay 1)
  auto stage = [&](float* at, int c0) {
    const int nc = min(C, n - c0);
    float* qs = at;
    float* ks = qs + C * RL;
    float* gs = ks + C * RL;
    float* vs = gs + C * RL;
    float* bs = vs + (C * cols + 3) / 4 * 4;
#pragma unroll
    for (int j = 0; j < DR_STAGE; ++j) {
      const int idx = tid + j * (int)blockDim.x, r = idx % DP;
      if (idx < nc * DP) {
        const bool row = r < D;
        const int to = idx / DP * RL + r / DR_ROWS * DR_PAD + r % DR_ROWS;
        qs[to] = row ? rq[j] : 0.f;
        ks[to] = row ? rk[j] : 0.f;
        float g = rg[j];
        if constexpr (!DECAYED) g = expf(-rate * softplus_f(g + dt_bias[h * D + min(r, D - 1)]));
        gs[to] = row ? g : 1.f;
      }
    }
#pragma unroll
    for (int j = 0; j < EV; ++j) {
      const int idx = tid + j * (int)blockDim.x;
      if (idx < nc * cols) vs[idx] = cb * cols + idx % cols < V ? rv[j] : 0.f;
    }
    if (tid < nc) bs[tid] = rb;
  };

  if (n > 0) {
    fetch(0);
    stage(lds, 0);
  }
  __syncthreads();
  int cur = 0;
  for (int c0 = 0; c0 < n; c0 += C, cur ^= 1) {
    const int nc = min(C, n - c0);
    const bool more = c0 + C < n;
    if (more) fetch(c0 + C);
    const float* qs = (const float*)__builtin_assume_aligned(lds + cur * buf_floats, 16);
    const float* ks = qs + C * RL;
    const float* gs = ks + C * RL;
    const float* vs = gs + C * RL;
    const float* bs = vs + (C * cols + 3) / 4 * 4;
    // One token: the rows' decays, the two sums over the state's rows, the write, the read-out.  The token's q, k and
    // decays (qq, kk, gg) were read from LDS while the token before was worked through (two sets of registers taking
    // turns, so that a read from LDS is never waited for right after it is asked).
    auto load_token = [&](int c, float (&qq)[DR_ROWS], float (&kk)[DR_ROWS], float (&gg)[DR_ROWS]) {
      const float* qr = (const float*)__builtin_assume_aligned(qs + c * RL + seg * DR_PAD, 16);
      const float* kr = (const float*)__builtin_assume_aligned(ks + c * RL + seg * DR_PAD, 16);
      const float* gr = (const float*)__builtin_assume_aligned(gs + c * RL + seg * DR_PAD, 16);
#pragma unroll
      for (int i = 0; i < DR_ROWS; ++i) {
        qq[i] = qr[i];
        kk[i] = kr[i];
        gg[i] = gr[i];
      }
    };
    auto one_token = [&](int c, const float (&qq)[DR_ROWS], const float (&kk)[DR_ROWS], const float (&gg)[DR_ROWS]) {
      float d1[CPT], d2[CPT], d3 = 0.f;
#pragma unroll
      for (int j = 0; j < CPT; ++j) d1[j] = d2[j] = 0.f;
#pragma unroll
      for (int i = 0; i < DR_ROWS; ++i) {
        d3 = fmaf(kk[i], qq[i], d3);
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
          s[j][i] *= gg[i];
          d1[j] = fmaf(s[j][i], kk[i], d1[j]);
          d2[j] = fmaf(s[j][i], qq[i], d2[j]);
        }
      }
      d3 = seg_sum<NSEG>(d3);
      const float bt = bs[c];
#pragma unroll
      for (int j = 0; j < CPT; ++j) {
        const float u = bt * (vs[c * cols + cloc[j]] - seg_sum<NSEG>(d1[j]));
#pragma unroll
        for (int i = 0; i < DR_ROWS; ++i) s[j][i] = fmaf(kk[i], u, s[j][i]);
        // the read-out of the state that holds this token's write: (g S)^T q + u (k . q)
        const float o = fmaf(u, d3, seg_sum<NSEG>(d2[j]));
        if (col_ok[j] && seg == 0) o_raw[(size_t)(t0 + c0 + c) * H * V + (size_t)h * V + cb * cols + cloc[j]] = o;
      }
    };
    float qa[DR_ROWS], ka[DR_ROWS], ga[DR_ROWS], qb[DR_ROWS], kb[DR_ROWS], gb[DR_ROWS];
    load_token(0, qa, ka, ga);
    for (int c = 0; c < nc; c += 2) {
      if (c + 1 < nc) load_token(c + 1, qb, kb, gb);
      one_token(c, qa, ka, ga);
      if (c + 1 < nc) {
        if (c + 2 < nc) load_token(c + 2, qa, ka, ga);
        one_token(c + 1, qb, kb, gb);
      }
    }
    if (more) stage(lds + (cur ^ 1) * buf_floats, c0 + C);
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < CPT; ++j) {
    if (!col_ok[j]) continue;
#pragma unroll
    for (int i = 0; i < DR_ROWS; ++i) {
      const int r = seg * DR_ROWS + i;
      if (r < D) S[(size_t)r * V + cb * cols + cloc[j]] = s[j][i];
    }
  }
}

// ------------------------------------------------------------------------------------------ norm, gate, new inputs
// grid (T + B, Y), block 256.  Blocks 0 .. T - 1 of x: a wave per head of its token: o / rms(o) * w * f(gate), the gate's row of token t at gates + t * gate_ld, f an activation of gates.def.
// Blocks T ..: the convolution's state of one sequence, its channels dealt over y: its last taps - 1 inputs, those of this run and, where the run
// is shorter, the most recent of the old state before them.
__global__ __launch_bounds__(256) void delta_out_kernel(const float* __restrict__ o_raw, const float* __restrict__ gates,
                                                        int64_t gate_ld, int gate_kind,
                                                        const float* __restrict__ norm_w, float eps,
                                                        const float* __restrict__ P, const int* __restrict__ cu_seqlens,
                                                        const int* __restrict__ slots, float* __restrict__ state,
                                                        int64_t state_stride, DeltaDims dm, int T,
                                                        act_t* __restrict__ out) {
  const int H = dm.H, D = dm.D, V = dm.V, K = dm.taps;
  if ((int)blockIdx.x < T) {
    const int t = blockIdx.x, wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
    for (int h = blockIdx.y * 4 + wave; h < H; h += 4 * gridDim.y) {
      const float* o = o_raw + (size_t)t * H * V + (size_t)h * V;
      float ss = 0.f;
      for (int j = lane; j < V; j += TQ_WAVE) ss += o[j] * o[j];
      ss = wave_sum(ss);
      const float rs = 1.0f / sqrtf(ss / (float)V + eps);
      const float* gate = gates + (size_t)t * gate_ld + (size_t)h * V;
      for (int j = lane; j < V; j += TQ_WAVE)
        out[(size_t)t * H * V + (size_t)h * V + j] = from_f32<act_t>(o[j] * rs * norm_w[j] * gate_fn(gate[j], gate_kind));
    }
    return;
  }
  const int b = blockIdx.x - T;
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0;
  const int C = dd_channels(dm), NP = dd_np(dm);
  float* hist = state + (size_t)slots[b] * state_stride + (size_t)H * D * V;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float* hc = hist + (size_t)c * (K - 1);
    // new[m], m = 0 .. K - 2 oldest first, is the input K - 1 - m tokens before the run's end
    for (int m = 0; m < K - 1; ++m) {
      const int back = K - 1 - m;           // 1 = the run's last token
      // ascending m reads old entries at m + n >= m: none that this loop has already overwritten
      hc[m] = back <= n ? P[(size_t)(t0 + n - back) * NP + c] : hc[m + n];
    }
  }
}

// ------------------------------------------------------------------------------------------ one token per sequence
// A decode step's form of what lies between delta_prep and the output product, in one launch: the second low-rank
// products of this head's decay and gate (four lanes to a row of the block-diagonal matrix), the decays, the recurrence for the one token, the read-out's norm and gate, and the convolution's new state.
// grid (H, B), block NSEG * V rounded up to whole waves (at most 1,024): lane (col, seg) keeps rows 16 seg .. 16 seg + 15
// of value channel col, all of a head's value channels in one workgroup, so that their norm needs no second kernel.
// The convolution's state of a head's own value channels is moved on by that head's workgroup, that of a q/k head by
// the workgroup of the first head that reads it; delta_prep, which read the old state, has finished by then.
template <int NSEG, class W>
__global__ __launch_bounds__(1024) void delta_decode_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                                                            const float* __restrict__ vc, const float* __restrict__ beta,
                                                            const act_t* __restrict__ low, const W* __restrict__ w_low,
                                                            const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                                            const float* __restrict__ norm_w, float eps,
                                                            const float* __restrict__ P, const int* __restrict__ cu_seqlens,
                                                            const int* __restrict__ slots, float* __restrict__ state,
                                                            int64_t state_stride, DeltaDims dm, int gate_kind,
                                                            act_t* __restrict__ out) {
  constexpr int DP = DR_ROWS * NSEG, RL = DR_PAD * NSEG;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;                 // [RL] each: a lane's 16 rows 20 floats from its neighbour's
  float* ks = qs + RL;
  float* gs = ks + RL;
  float* gate = gs + RL;           // [V]
  float* lowv = gate + (dm.V + 3) / 4 * 4;      // [ra + rg]
  float* red = lowv + (dm.ra + dm.rg + 3) / 4 * 4;      // one per wave
  const int H = dm.H, G = dm.G, D = dm.D, V = dm.V, K = dm.taps, R = dm.ra + dm.rg;
  const int h = blockIdx.x, b = blockIdx.y, gq = h / (H / G);
  const int tid = threadIdx.x, seg = tid % NSEG, col = tid / NSEG;
  const bool col_ok = col < V;
  const size_t t = (size_t)cu_seqlens[b];
  float* row = state + (size_t)slots[b] * state_stride;
  for (int i = tid; i < R; i += blockDim.x) lowv[i] = to_f32(low[t * R + i]);       // (mode 1: R is 0)
  __syncthreads();
  const float rate = expf(a_log[h]);
  // The head's D rows of the decay's product and V rows of the gate's, four neighbouring lanes to a row: lane p of the
  // four sums the elements p, p + 4, ... of the rank, and the four partial sums are added within the quad.
  const int part = tid & 3, rows_a_pass = (int)blockDim.x >> 2;
  if (dm.mode == 1) {
    // a decay per head and a gate that is a projection of its own: nothing to multiply here
    const int C1 = dd_channels(dm), NP1 = dd_np(dm);
    const float g = expf(-rate * softplus_f(P[t * NP1 + C1 + H + h] + dt_bias[h]));
    for (int r = tid; r < D + V; r += blockDim.x) {
      if (r < D) {
        const int to = r / DR_ROWS * DR_PAD + r % DR_ROWS;
        qs[to] = qn[t * G * D + (size_t)gq * D + r];
        ks[to] = kn[t * G * D + (size_t)gq * D + r];
        gs[to] = g;
      } else {
        gate[r - D] = P[t * NP1 + C1 + 2 * H + (size_t)h * V + (r - D)];
      }
    }
  }
  for (int r0 = 0; dm.mode == 0 && r0 < D + V; r0 += rows_a_pass) {
    const int r = r0 + (tid >> 2);
    const bool live = r < D + V, decay = r < D;
    float a = 0.f;
    if (live) {
      const W* wr = decay ? w_low + (size_t)(h * D + r) * R : w_low + (size_t)(H * D + h * V + (r - D)) * R + dm.ra;
      const float* lv = decay ? lowv : lowv + dm.ra;
      const int n = decay ? dm.ra : dm.rg;
#pragma unroll 4
      for (int j = part; j < n; j += 4) a = fmaf(to_f32(wr[j]), lv[j], a);
    }
    a = seg_sum<4>(a);
    if (live && part == 0) {
      if (decay) {
        const int to = r / DR_ROWS * DR_PAD + r % DR_ROWS;
        qs[to] = qn[t * G * D + (size_t)gq * D + r];
        ks[to] = kn[t * G * D + (size_t)gq * D + r];
        gs[to] = expf(-rate * softplus_f(a + dt_bias[h * D + r]));
      } else {
        gate[r - D] = a;
      }
    }
  }
  for (int r = D + tid; r < DP; r += blockDim.x) {      // rows beyond D keep their zeros
    const int to = r / DR_ROWS * DR_PAD + r % DR_ROWS;
    qs[to] = ks[to] = 0.f;
    gs[to] = 1.f;
  }
  __syncthreads();
  float* S = row + (size_t)h * D * V;
  float s[DR_ROWS];
  float d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
  for (int i = 0; i < DR_ROWS; ++i) {
    const int r = seg * DR_ROWS + i;
    s[i] = col_ok && r < D ? S[(size_t)r * V + col] : 0.f;
    const float q = qs[seg * DR_PAD + i], k = ks[seg * DR_PAD + i];
    s[i] *= gs[seg * DR_PAD + i];
    d1 = fmaf(s[i], k, d1);
    d2 = fmaf(s[i], q, d2);
    d3 = fmaf(k, q, d3);
  }
  d1 = seg_sum<NSEG>(d1);
  d2 = seg_sum<NSEG>(d2);
  d3 = seg_sum<NSEG>(d3);
  const float u = col_ok ? beta[t * H + h] * (vc[t * H * V + (size_t)h * V + col] - d1) : 0.f;
#pragma unroll
  for (int i = 0; i < DR_ROWS; ++i) {
    const int r = seg * DR_ROWS + i;
    if (col_ok && r < D) S[(size_t)r * V + col] = fmaf(ks[seg * DR_PAD + i], u, s[i]);
  }
  const float o = col_ok ? fmaf(u, d3, d2) : 0.f;
  const float ss = block_sum(seg == 0 ? o * o : 0.f, red);
  const float rs = 1.0f / sqrtf(ss / (float)V + eps);
  if (col_ok && seg == 0)
    out[t * H * V + (size_t)h * V + col] = from_f32<act_t>(o * rs * norm_w[col] * gate_fn(gate[col], gate_kind));
  // the convolution's inputs move on by this token: the head's own value channels, and its q/k head's if it is the first to read them
  const int C = dd_channels(dm), NP = dd_np(dm);
  float* hist = row + (size_t)H * D * V;
  const bool first = h % (H / G) == 0;
  const int mine = V + (first ? 2 * D : 0);
  for (int i = tid; i < mine; i += blockDim.x) {
    const int c = i < V ? 2 * G * D + h * V + i : (i - V < D ? gq * D + (i - V) : G * D + gq * D + (i - V - D));
    float* hc = hist + (size_t)c * (K - 1);
    for (int m = 0; m + 1 < K - 1; ++m) hc[m] = hc[m + 1];
    if (K > 1) hc[K - 2] = P[t * NP + c];
  }
  (void)C;
}

// ------------------------------------------------------------------------------------------ entry points
static int dims_ok(const DeltaDims& d) {
  return d.H > 0 && d.G > 0 && d.H % d.G == 0 && d.D > 0 && d.D <= 256 && d.V > 0 && d.taps >= 1 && d.taps <= 64 &&
         (d.mode == 1 ? d.ra == 0 && d.rg == 0 : d.mode == 0 && d.ra > 0 && d.rg > 0);
}

// Floats of one sequence's row of state.
TQ_API int64_t tq_delta_state_floats(int H, int G, int D, int V, int taps) {
  const DeltaDims d{H, G, D, V, taps, 1, 1, 0};
  return dd_state(d);
}

static int launch_prep(const float* P, const int* slot_of_token, const float* state, int64_t state_stride,
                       const float* conv_w, const DeltaDims& d, float* qn, float* kn, float* vc, float* beta, void* low,
                       const float* a_log, const float* dt_bias, float* dec, int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (!dims_ok(d) || state_stride < dd_state(d)) return TQ_ERR_BAD_ARG;
  const int units = 2 * d.G + d.H + 1;
  hipLaunchKernelGGL(delta_prep_kernel, dim3(T, (units + 3) / 4 < 65535 ? (units + 3) / 4 : 65535), dim3(256), 0, st, P,
                     slot_of_token, state, state_stride, conv_w, d, qn, kn, vc, beta, (act_t*)low, a_log, dt_bias, dec);
  TQ_LAUNCH_CHECK();
  return 0;
}

// P [T][NP] float (see the head of this file); slot_of_token [T]; state: rows of state_stride floats by slot;
// conv_w [channels][taps] float.  Writes qn, kn [T][G D], vc [T][H V], beta [T][H] (float) and low [T][ra + rg]
// (activation type).
TQ_API int tq_delta_prep(const float* P, const int* slot_of_token, const float* state, int64_t state_stride,
                         const float* conv_w, int H, int G, int D, int V, int taps, int ra, int rg, float* qn, float* kn,
                         float* vc, float* beta, void* low, int T, hipStream_t st) {
  return launch_prep(P, slot_of_token, state, state_stride, conv_w, DeltaDims{H, G, D, V, taps, ra, rg, 0}, qn, kn, vc, beta,
                     low, nullptr, nullptr, nullptr, T, st);
}

// The form with a decay per head: P [T][q | k | v | b (H) | a (H) | gate (H V)]; writes qn, kn, vc, beta as above and
// dec [T][H] = exp(-exp(a_log[h]) * softplus(a + dt_bias[h])).
TQ_API int tq_delta_prep_h(const float* P, const int* slot_of_token, const float* state, int64_t state_stride,
                           const float* conv_w, const float* a_log, const float* dt_bias, int H, int G, int D, int V,
                           int taps, float* qn, float* kn, float* vc, float* beta, float* dec, int T, hipStream_t st) {
  if (!a_log || !dt_bias || !dec) return TQ_ERR_BAD_ARG;
  return launch_prep(P, slot_of_token, state, state_stride, conv_w, DeltaDims{H, G, D, V, taps, 0, 0, 1}, qn, kn, vc, beta,
                     nullptr, a_log, dt_bias, dec, T, st);
}

// head_decay: ag is [T][H], the decay of every head, ready to use.
static int launch_scan(const float* qn, const float* kn, const float* vc, const float* beta, float* ag, const float* a_log,
                       const float* dt_bias, const int* cu_seqlens, const int* slots, float* state, int64_t state_stride,
                       const DeltaDims& d, int head_decay, int T, int B, float* o_raw, hipStream_t st) {
  if (B <= 0 || T <= 0) return 0;
  if (!dims_ok(d) || state_stride < dd_state(d)) return TQ_ERR_BAD_ARG;
  if (B > 65535) return TQ_ERR_UNSUPPORTED;
  const int H = d.H, D = d.D, V = d.V;
  int nseg = 1;
  while (nseg * DR_ROWS < D) nseg *= 2;
  // value channels per lane: as many of 4, 2, 1 as still leave the head's lanes a whole wave
  // (measured on 16 heads of 128 x 128, one sequence of 2,048 tokens: 0.51 us a token with one channel per lane, 0.65 with
  // two, 1.0 with four, since fewer lanes then share the head's work; several channels pay where the step's sequences
  // and heads alone give every compute unit its workgroups)
  const int lanes_one = nseg * V;                                  // lanes a head takes with one channel per lane
  const int64_t groups_one = (int64_t)B * H * ((lanes_one + 255) / 256);
  int cpt = groups_one >= 2048 ? 4 : groups_one >= 1024 ? 2 : 1;
  while (cpt > 1 && nseg * ((V + cpt - 1) / cpt) < TQ_WAVE) cpt /= 2;
  const int lane_cols = (V + cpt - 1) / cpt < 256 / nseg ? (V + cpt - 1) / cpt : 256 / nseg;     // LC
  const int cols = lane_cols * cpt;
  const int col_blocks = (V + cols - 1) / cols;
  // whole waves, so that the lanes of a value channel always lie in one
  const int threads = (nseg * lane_cols + TQ_WAVE - 1) / TQ_WAVE * TQ_WAVE;
  const int dp = DR_ROWS * nseg;
  const int chunk = DR_CHUNK < DR_STAGE * threads / dp ? DR_CHUNK : DR_STAGE * threads / dp;
  const size_t shmem = (size_t)2 * (3 * chunk * DR_PAD * nseg + (chunk * cols + 3) / 4 * 4 + DR_CHUNK) * sizeof(float);
  // the decays of a long step are worked out beforehand, once for all blocks of value channels
  const int decayed = head_decay || T > 16 * B || T >= 256;
  if (decayed && !head_decay) {
    const int64_t total = (int64_t)T * H * D;
    hipLaunchKernelGGL(delta_decay_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, ag, a_log, dt_bias,
                       H * D, D, H * D + H * V, total);
  }
#define TQ_SCAN_WITH(NS, CP, DEC)                                                                                     \
  do {                                                                                                                \
    if (shmem > 48 * 1024)                                                                                            \
      (void)hipFuncSetAttribute((const void*)delta_scan_kernel<NS, CP, DEC>,                                          \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);                              \
    hipLaunchKernelGGL((delta_scan_kernel<NS, CP, DEC>), dim3(H * col_blocks, B), dim3(threads), shmem, st, qn, kn,   \
                       vc, beta, ag, a_log, dt_bias, cu_seqlens, slots, state, state_stride, d, cols, col_blocks,     \
                       head_decay, o_raw);                                                                            \
  } while (0)
#define TQ_SCAN_AS(NS, CP)                   \
  do {                                       \
    if (decayed) TQ_SCAN_WITH(NS, CP, true); \
    else TQ_SCAN_WITH(NS, CP, false);        \
  } while (0)
#define TQ_SCAN(NS)                  \
  do {                               \
    if (cpt == 4) TQ_SCAN_AS(NS, 4); \
    else if (cpt == 2) TQ_SCAN_AS(NS, 2); \
    else TQ_SCAN_AS(NS, 1);          \
  } while (0)
  switch (nseg) {
    case 1: TQ_SCAN(1); break;
    case 2: TQ_SCAN(2); break;
    case 4: TQ_SCAN(4); break;
    case 8: TQ_SCAN(8); break;
    default: TQ_SCAN(16); break;
  }
#undef TQ_SCAN_AS
#undef TQ_SCAN_WITH
#undef TQ_SCAN
  TQ_LAUNCH_CHECK();
  return 0;
}

// The recurrence over runs of tokens, one run per sequence (cu_seqlens [B + 1], slots [B], T tokens in all); the state
// rows are read and written.  o_raw [T][H V] float.  In a step of many tokens the first H D columns of ag are replaced
// by the decays they stand for (nothing else reads them afterwards).
TQ_API int tq_delta_scan(const float* qn, const float* kn, const float* vc, const float* beta, float* ag,
                         const float* a_log, const float* dt_bias, const int* cu_seqlens, const int* slots, float* state,
                         int64_t state_stride, int H, int G, int D, int V, int taps, int T, int B, float* o_raw,
                         hipStream_t st) {
  return launch_scan(qn, kn, vc, beta, ag, a_log, dt_bias, cu_seqlens, slots, state, state_stride,
                     DeltaDims{H, G, D, V, taps, 1, 1, 0}, 0, T, B, o_raw, st);
}

// The same recurrence with one decay per head: dec [T][H] as tq_delta_prep_h wrote it.
TQ_API int tq_delta_scan_h(const float* qn, const float* kn, const float* vc, const float* beta, const float* dec,
                           const int* cu_seqlens, const int* slots, float* state, int64_t state_stride, int H, int G, int D,
                           int V, int taps, int T, int B, float* o_raw, hipStream_t st) {
  return launch_scan(qn, kn, vc, beta, const_cast<float*>(dec), nullptr, nullptr, cu_seqlens, slots, state, state_stride,
                     DeltaDims{H, G, D, V, taps, 0, 0, 1}, 1, T, B, o_raw, st);
}

static int launch_out(const float* o_raw, const float* gates, int64_t gate_ld, int gate_kind, const float* norm_w, float eps,
                      const float* P, const int* cu_seqlens, const int* slots, float* state, int64_t state_stride,
                      const DeltaDims& d, int T, int B, void* out, hipStream_t st) {
  if (T <= 0 || B <= 0) return 0;
  if (!dims_ok(d) || state_stride < dd_state(d) || gate_kind < 0 || gate_kind >= TQ_GATE_COUNT) return TQ_ERR_BAD_ARG;
  hipLaunchKernelGGL(delta_out_kernel, dim3(T + B, (d.H + 3) / 4 < 65535 ? (d.H + 3) / 4 : 65535), dim3(256), 0, st, o_raw,
                     gates, gate_ld, gate_kind, norm_w, eps, P, cu_seqlens, slots, state, state_stride, d, T, (act_t*)out);
  TQ_LAUNCH_CHECK();
  return 0;
}

// Norm and gate of every head's read-out into `out` [T][H V] (activation type), and every sequence's new convolution
// state from P.  norm_w [V] float.  The gate is the sigmoid of the last H V columns of ag.
TQ_API int tq_delta_out(const float* o_raw, const float* ag, const float* norm_w, float eps, const float* P,
                        const int* cu_seqlens, const int* slots, float* state, int64_t state_stride, int H, int G, int D,
                        int V, int taps, int ra, int rg, int T, int B, void* out, hipStream_t st) {
  return launch_out(o_raw, ag + (size_t)H * D, (int64_t)H * D + (int64_t)H * V, TQ_GATE_sigmoid, norm_w, eps, P, cu_seqlens,
                    slots, state, state_stride, DeltaDims{H, G, D, V, taps, ra, rg, 0}, T, B, out, st);
}

// The form with a decay per head: the gate is activation `gate_kind` (gates.def) of the last H V columns of P.
TQ_API int tq_delta_out_h(const float* o_raw, const float* norm_w, float eps, const float* P, int gate_kind,
                          const int* cu_seqlens, const int* slots, float* state, int64_t state_stride, int H, int G, int D,
                          int V, int taps, int T, int B, void* out, hipStream_t st) {
  const DeltaDims d{H, G, D, V, taps, 0, 0, 1};
  return launch_out(o_raw, P + dd_channels(d) + 2 * H, dd_np(d), gate_kind, norm_w, eps, P, cu_seqlens, slots, state,
                    state_stride, d, T, B, out, st);
}

template <class W>
static int launch_decode(const float* qn, const float* kn, const float* vc, const float* beta, const void* low,
                         const void* w_low, const float* a_log, const float* dt_bias, const float* norm_w, float eps,
                         const float* P, const int* cu_seqlens, const int* slots, float* state, int64_t state_stride,
                         const DeltaDims& d, int gate_kind, int B, void* out, hipStream_t st) {
  int nseg = 1;
  while (nseg * DR_ROWS < d.D) nseg *= 2;
  const int threads = (nseg * d.V + TQ_WAVE - 1) / TQ_WAVE * TQ_WAVE;
  if (threads > 1024 || B > 65535 || d.H > 65535) return TQ_ERR_UNSUPPORTED;
  const size_t shmem = (size_t)(3 * DR_PAD * nseg + (d.V + 3) / 4 * 4 + (d.ra + d.rg + 3) / 4 * 4 + 16) * sizeof(float);
  if (shmem > 60 * 1024) return TQ_ERR_UNSUPPORTED;
#define TQ_DECODE(NS)                                                                                                 \
  hipLaunchKernelGGL((delta_decode_kernel<NS, W>), dim3(d.H, B), dim3(threads), shmem, st, qn, kn, vc, beta,          \
                     (const act_t*)low, (const W*)w_low, a_log, dt_bias, norm_w, eps, P, cu_seqlens, slots, state,    \
                     state_stride, d, gate_kind, (act_t*)out)
  switch (nseg) {
    case 1: TQ_DECODE(1); break;
    case 2: TQ_DECODE(2); break;
    case 4: TQ_DECODE(4); break;
    case 8: TQ_DECODE(8); break;
    default: TQ_DECODE(16); break;
  }
#undef TQ_DECODE
  return 0;
}

// A decode step (one token per sequence, T == B) from delta_prep's outputs to the mixer's output `out` [T][H V]
// (activation type), in one launch: returns TQ_ERR_UNSUPPORTED where a head's lanes do not fit one workgroup (the caller
// then takes the kernels of longer steps).  low [T][ra + rg] (activation type); w_low [(H D + H V)][ra + rg] of wtype,
// the block-diagonal matrix of both second low-rank products.
TQ_API int tq_delta_decode(const float* qn, const float* kn, const float* vc, const float* beta, const void* low,
                           const void* w_low, int wtype, const float* a_log, const float* dt_bias, const float* norm_w,
                           float eps, const float* P, const int* cu_seqlens, const int* slots, float* state,
                           int64_t state_stride, int H, int G, int D, int V, int taps, int ra, int rg, int B, void* out,
                           hipStream_t st) {
  if (B <= 0) return 0;
  const DeltaDims d{H, G, D, V, taps, ra, rg, 0};
  if (!dims_ok(d) || state_stride < dd_state(d)) return TQ_ERR_BAD_ARG;
  TQ_DISPATCH_W(wtype, {
    const int rc = launch_decode<W>(qn, kn, vc, beta, low, w_low, a_log, dt_bias, norm_w, eps, P, cu_seqlens, slots, state,
                                    state_stride, d, TQ_GATE_sigmoid, B, out, st);
    if (rc) return rc;
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// The form with a decay per head and a gate of activation `gate_kind` that is a projection of its own (P as for
// tq_delta_prep_h): the decay, the recurrence for the one token, norm, gate and the convolution's new state.
TQ_API int tq_delta_decode_h(const float* qn, const float* kn, const float* vc, const float* beta, const float* a_log,
                             const float* dt_bias, const float* norm_w, float eps, const float* P, int gate_kind,
                             const int* cu_seqlens, const int* slots, float* state, int64_t state_stride, int H, int G,
                             int D, int V, int taps, int B, void* out, hipStream_t st) {
  if (B <= 0) return 0;
  const DeltaDims d{H, G, D, V, taps, 0, 0, 1};
  if (!dims_ok(d) || state_stride < dd_state(d) || gate_kind < 0 || gate_kind >= TQ_GATE_COUNT) return TQ_ERR_BAD_ARG;
  const int rc = launch_decode<float>(qn, kn, vc, beta, nullptr, nullptr, a_log, dt_bias, norm_w, eps, P, cu_seqlens, slots,
                                      state, state_stride, d, gate_kind, B, out, st);
  if (rc) return rc;
  TQ_LAUNCH_CHECK();
  return 0;
}
