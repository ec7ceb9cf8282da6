// A product per head: out[t][h N + n] = sum_k a[t][h K + k] * w[h][n][k], for the H heads of every token at once.
//
// It serves mixers whose heads have matrices of their own between the layer's projections and the attention: an
// attention over one compressed row per position folds each head's key matrix into its query before the scores
// (q_h W_uk,h: K = the head's query width, N = the compressed width) and expands each head's weighted sum of compressed
// rows afterwards (W_uv,h o_h: K = the compressed width, N = the head's value width).  `a` is float or of the
// activation type with a row stride of its own, so that it can be a run of columns of a wider product; `out` likewise.
// The epilogue can multiply by f(gate[t][h N + n]), f an activation of gates.def: an output gate costs no pass of its own.
//
// Three kernels.  bfloat16 library, bfloat16 matrices, K a multiple of 8: v_mfma_f32_16x16x32_bf16 with both operands
// straight from memory, 16 bytes per lane (the first operand is 16 rows n of the head's matrix, the second 16 tokens,
// so that a lane ends up with four neighbouring n of one token and stores them as one piece); a wave owns 32 tokens by
// 64 n, and a head's matrix is a few hundred KB at most, which the caches keep while the tokens pass.  Everything
// else: a tile of 64 tokens by 64 n per workgroup, staged through LDS in steps of 16 k, plain multiply-adds in float.
// (up to 16 tokens: a wave owns 16 tokens by 16 n and has eight steps of k in flight, head_gemm_few_kernel).
// All sum over k in ascending order whatever the number of tokens.
#include "common.h"

struct HeadGemmArgs {
  const void* a;
  int64_t lda;
  const void* w;           // [H][N][K]
  void* out;
  int64_t ldc;
  const float* gate;       // null: none
  int64_t ldg;
  int gate_kind;
  int T, H, N, K;
};

template <class A>
__device__ __forceinline__ float a_at(const A* p) { return to_f32(*p); }

template <bool OUT_ACT>
__device__ __forceinline__ void hg_store(const HeadGemmArgs& g, int t, int col, float v) {
  if (g.gate) v *= gate_fn(g.gate[(size_t)t * g.ldg + col], g.gate_kind);
  if (OUT_ACT)
    ((act_t*)g.out)[(size_t)t * g.ldc + col] = from_f32<act_t>(v);
  else
    ((float*)g.out)[(size_t)t * g.ldc + col] = v;
}

// ------------------------------------------------------------------------------------------ plain multiply-adds
// grid (ceil(T / 64), ceil(N / 64), H), block 256: thread (tx, ty) owns tokens 4 ty .. 4 ty + 3 and n 4 tx .. 4 tx + 3.
template <class A, class W, bool OUT_ACT>
__global__ __launch_bounds__(256) void head_gemm_plain_kernel(HeadGemmArgs g) {
  __shared__ float As[16][68], Ws[16][68];
  const int t0 = blockIdx.x * 64, n0 = blockIdx.y * 64, h = blockIdx.z;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const A* a = (const A*)g.a + (size_t)h * g.K;
  const W* w = (const W*)g.w + (size_t)h * g.N * g.K;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < g.K; k0 += 16) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int idx = tid + 256 * u, r = idx / 16, k = idx % 16;      // row of the tile, k within the step
      const bool k_ok = k0 + k < g.K;
      As[k][r] = k_ok && t0 + r < g.T ? a_at(a + (size_t)(t0 + r) * g.lda + k0 + k) : 0.f;
      Ws[k][r] = k_ok && n0 + r < g.N ? to_f32(w[(size_t)(n0 + r) * g.K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = As[k][4 * ty + i];
        wv[i] = Ws[k][4 * tx + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + 4 * ty + i;
    if (t >= g.T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + 4 * tx + j;
      if (n < g.N) hg_store<OUT_ACT>(g, t, h * g.N + n, acc[i][j]);
    }
  }
}

#if defined(TQ_ACT_BF16)
// ------------------------------------------------------------------------------------------ matrix cores
typedef __bf16 hg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float hg_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 hg_bf16x2 __attribute__((ext_vector_type(2)));

// eight consecutive elements of a row as one operand register set: bfloat16 as they are, float rounded to nearest even
__device__ __forceinline__ hg_bf16x8 hg_load8(const bf16_t* p) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(hg_bf16x8, v);
}
__device__ __forceinline__ hg_bf16x8 hg_load8(const float* p) {
  const float4 lo = *reinterpret_cast<const float4*>(p), hi = *reinterpret_cast<const float4*>(p + 4);
  const hg_bf16x8 v = {(__bf16)lo.x, (__bf16)lo.y, (__bf16)lo.z, (__bf16)lo.w, (__bf16)hi.x, (__bf16)hi.y, (__bf16)hi.z, (__bf16)hi.w};
  return v;
}
__device__ __forceinline__ hg_bf16x8 hg_zero8() {
  const uint4 v = make_uint4(0, 0, 0, 0);
  return __builtin_bit_cast(hg_bf16x8, v);
}

// grid (items / 4, 1, H), block 256: wave `id` of the grid's x takes token tile id / n_tiles (32 tokens) and n tile
// id % n_tiles (64 n) of head z.  Lane (r, c) = (lane % 16, lane / 16) reads k 8 c .. 8 c + 7 of every step of 32 k for
// row r of each operand tile; of a product tile it holds token r, n 4 c .. 4 c + 3.
template <class A, bool OUT_ACT>
__global__ __launch_bounds__(256) void head_gemm_mfma_kernel(HeadGemmArgs g, int n_tiles, int items) {
  const int id = blockIdx.x * 4 + threadIdx.x / 64;
  if (id >= items) return;
  const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
  const int t0 = id / n_tiles * 32, n0 = id % n_tiles * 64, h = blockIdx.z;
  const A* a = (const A*)g.a + (size_t)h * g.K;
  const bf16_t* w = (const bf16_t*)g.w + (size_t)h * g.N * g.K;
  const A* arow[2];
  const bf16_t* wrow[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) arow[i] = a + (size_t)min(t0 + 16 * i + r, g.T - 1) * g.lda;      // a row past the end is read again, never stored
#pragma unroll
  for (int j = 0; j < 4; ++j) wrow[j] = w + (size_t)min(n0 + 16 * j + r, g.N - 1) * g.K;
  hg_f32x4 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = hg_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < g.K; k0 += 32) {
    const int k = k0 + 8 * c;
    const bool k_ok = k < g.K;                 // K is a multiple of 8: a lane's eight are all inside or all outside
    hg_bf16x8 af[2], wf[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) af[i] = k_ok ? hg_load8(arow[i] + k) : hg_zero8();
#pragma unroll
    for (int j = 0; j < 4; ++j) wf[j] = k_ok ? hg_load8(wrow[j] + k) : hg_zero8();
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[i], acc[i][j], 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int t = t0 + 16 * i + r;
    if (t >= g.T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int n = n0 + 16 * j + 4 * c + v;
        if (n < g.N) hg_store<OUT_ACT>(g, t, h * g.N + n, acc[i][j][v]);
      }
  }
}

// A step of few tokens (a decode step): a wave takes 16 tokens by 16 n, so that a head's matrix is spread over eight times
// the waves of the kernel above, and fetches eight steps of k from clamped addresses before it multiplies any, so that
// the loads are in flight together (K = 512: two rounds of loads instead of sixteen).
template <class A, bool OUT_ACT>
__global__ __launch_bounds__(256) void head_gemm_few_kernel(HeadGemmArgs g, int n_tiles, int items) {
  const int id = blockIdx.x * 4 + threadIdx.x / 64;
  if (id >= items) return;
  const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
  const int t0 = id / n_tiles * 16, n0 = id % n_tiles * 16, h = blockIdx.z;
  const A* arow = (const A*)g.a + (size_t)h * g.K + (size_t)min(t0 + r, g.T - 1) * g.lda;
  const bf16_t* wrow = (const bf16_t*)g.w + ((size_t)h * g.N + min(n0 + r, g.N - 1)) * g.K;
  hg_f32x4 acc = hg_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < g.K; k0 += 256) {
    hg_bf16x8 af[8], wf[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int k = min(k0 + 32 * s + 8 * c, g.K - 8);
      af[s] = hg_load8(arow + k);
      wf[s] = hg_load8(wrow + k);
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      if (k0 + 32 * s + 8 * c >= g.K) af[s] = hg_zero8();        // a step past the end adds nothing
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s], af[s], acc, 0, 0, 0);
    }
  }
  const int t = t0 + r;
  if (t >= g.T) return;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int n = n0 + 4 * c + v;
    if (n < g.N) hg_store<OUT_ACT>(g, t, h * g.N + n, acc[v]);
  }
}
#endif

// a [T][>= H K] of a_type (TQ_F32, or TQ_BF16 on the bfloat16 library) with row stride lda; w [H][N][K] of wtype;
// out [T][>= H N] float, or the activation type if out_act, with row stride ldc; gate (or null) float [T][>= H N] with
// row stride ldg, passed through activation gate_kind of gates.def and multiplied into the result.
TQ_API int tq_head_gemm(const void* a, int a_type, int64_t lda, const void* w, int wtype, void* out, int out_act,
                        int64_t ldc, const float* gate, int64_t ldg, int gate_kind, int T, int H, int N, int K,
                        hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || N < 1 || K < 1 || lda < (int64_t)H * K || ldc < (int64_t)H * N || (gate && ldg < (int64_t)H * N))
    return TQ_ERR_BAD_ARG;
  if (gate && (gate_kind < 0 || gate_kind >= TQ_GATE_COUNT)) return TQ_ERR_BAD_ARG;
  if (a_type != TQ_F32 && a_type != TQ_ACT_TYPE) return TQ_ERR_BAD_ARG;
  if (H > 65535) return TQ_ERR_UNSUPPORTED;
  const HeadGemmArgs g{a, lda, w, out, ldc, gate, ldg, gate_kind, T, H, N, K};
#if defined(TQ_ACT_BF16)
  const bool a_f32 = a_type == TQ_F32;
  if (wtype == TQ_BF16 && K % 8 == 0 && lda % (a_f32 ? 4 : 8) == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0) {
    if (T <= 16) {
      const int n16 = (N + 15) / 16;
      const dim3 grid_few((unsigned)((n16 + 3) / 4), 1, H);
#define TQ_HG_FEW(AT)                                                                                               \
  do {                                                                                                              \
    if (out_act) hipLaunchKernelGGL((head_gemm_few_kernel<AT, true>), grid_few, dim3(256), 0, st, g, n16, n16);     \
    else hipLaunchKernelGGL((head_gemm_few_kernel<AT, false>), grid_few, dim3(256), 0, st, g, n16, n16);            \
  } while (0)
      if (a_f32) TQ_HG_FEW(float);
      else TQ_HG_FEW(bf16_t);
#undef TQ_HG_FEW
      TQ_LAUNCH_CHECK();
      return 0;
    }
    const int n_tiles = (N + 63) / 64;
    const int64_t items = (int64_t)((T + 31) / 32) * n_tiles;
    if (items > (int64_t)4 * 2147483647) return TQ_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((items + 3) / 4), 1, H);
#define TQ_HG_MFMA(AT)                                                                                              \
  do {                                                                                                              \
    if (out_act) hipLaunchKernelGGL((head_gemm_mfma_kernel<AT, true>), grid, dim3(256), 0, st, g, n_tiles, (int)items);  \
    else hipLaunchKernelGGL((head_gemm_mfma_kernel<AT, false>), grid, dim3(256), 0, st, g, n_tiles, (int)items);    \
  } while (0)
    if (a_f32) TQ_HG_MFMA(float);
    else TQ_HG_MFMA(bf16_t);
#undef TQ_HG_MFMA
    TQ_LAUNCH_CHECK();
    return 0;
  }
#endif
  if ((N + 63) / 64 > 65535) return TQ_ERR_UNSUPPORTED;
  const dim3 grid((T + 63) / 64, (N + 63) / 64, H);
#define TQ_HG_PLAIN(AT, WT)                                                                                  \
  do {                                                                                                       \
    if (out_act) hipLaunchKernelGGL((head_gemm_plain_kernel<AT, WT, true>), grid, dim3(256), 0, st, g);      \
    else hipLaunchKernelGGL((head_gemm_plain_kernel<AT, WT, false>), grid, dim3(256), 0, st, g);             \
  } while (0)
  TQ_DISPATCH_W(wtype, {
    if (a_type == TQ_F32) TQ_HG_PLAIN(float, W);
    else TQ_HG_PLAIN(act_t, W);
  });
#undef TQ_HG_PLAIN
  TQ_LAUNCH_CHECK();
  return 0;
}
