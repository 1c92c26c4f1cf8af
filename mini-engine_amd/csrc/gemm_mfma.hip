// Tiled bfloat16 product y = x . W^T on the matrix cores for prompt-sized batches (hundreds to
// thousands of rows), float32 accumulation, output in bfloat16 or float32, optionally with the SwiGLU
// of a gate/up projection as its epilogue.
//
// A block of WM x WN waves owns BM rows of x and BN rows of W (BN output columns). Both operands are
// k-contiguous in memory, which is what v_mfma_f32_16x16x32_bf16 wants from each lane (8 consecutive
// k of one row), so tiles go to LDS as they lie in memory, [row][64 k] = 128 bytes a row, with the eight
// 16-byte pieces of a row permuted by an XOR with (row / 2) % 8: the 16-byte fragment reads of a wave
// (16 rows, one piece each) are then free of bank conflicts without padding, and two blocks of 128 x 128 fit
// into the LDS of a compute unit.
//
// The loop over k is double-buffered in LDS, and tiles go there straight from memory (global_load_lds_dwordx4:
// a wave's instruction writes 64 consecutive 16-byte pieces of LDS, one per lane, and each lane fetches the piece
// that the swizzle puts at its place): no registers hold a tile, no LDS write instructions are issued. The
// request for tile s+1 stands at the head of step s; the barrier that ends the step waits for it. (With the next
// tile in registers and written to LDS in the middle of a step the gate/up product of a 2,048-token prompt took
// 33.6 us, now 32.4.) One barrier per step. Loads carry no bounds checks: rows past the matrix are clamped to
// its last row (their products are never stored), and k is a multiple of 64.
//
// Products are taken transposed, C^T[n, m] = sum_k W[n, k] x[m, k]: a lane then holds four
// consecutive columns n of one row m and stores them with one 8- or 16-byte store.
//
// Epilogue SWIGLU: W holds gate rows [0, N) and up rows [N, 2N). The BN rows of a block's W tile are
// BN/2 gate rows and the BN/2 up rows of the same columns, laid out so that every wave holds gate and
// up of a column in the same lane; the block writes silu(gate) * up, N columns in all.
//
// Blocks are numbered so that the blocks one XCD runs (every eighth block id) share W tiles.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

namespace {

constexpr int GK = 64;         // k per tile
constexpr int GROW = GK;       // LDS row length in elements

// (the reciprocal as one instruction: a division is a dozen, and a block of 256 x 192 ends with 48 of these per lane
// while its compute unit has nothing else to run)
__device__ __forceinline__ float silu_f(float g) { return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)); }

template <typename OutT>
__device__ __forceinline__ void store4(OutT* __restrict__ C, size_t ldc, int m, int n, int M, int N, const float (&v)[4]) {
  if (m >= M) return;
  OutT* p = C + (size_t)m * ldc + n;
  if (n + 3 < N && (((uintptr_t)p) & (sizeof(OutT) * 4 - 1)) == 0) {
    if constexpr (sizeof(OutT) == 2) {
      typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
      const bf16x4_t w = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};  // round to nearest even in hardware
      *reinterpret_cast<bf16x4_t*>(p) = w;
    } else {
      *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) p[i] = from_float<OutT>(v[i]);
  }
}

template <int BM, int BN, int WM, int WN, bool SWIGLU, typename OutT>
__global__ __launch_bounds__(WM * WN * 64) void gemm_tiled_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                   OutT* __restrict__ C, int M, int N, int K, int m_tiles,
                                                                   int n_tiles, int gate) {
  constexpr int THREADS = WM * WN * 64;
  constexpr int WMR = BM / WM, WNR = BN / WN;  // rows of x / rows of W per wave
  constexpr int FM = WMR / 16, FN = WNR / 16;  // 16 x 16 fragments per wave
  constexpr int NX = BM * 8 / THREADS, NW = BN * 8 / THREADS;  // 16-byte pieces of a tile per thread
  static_assert(WMR % 16 == 0 && WNR % 16 == 0, "wave tiles are multiples of 16");
  static_assert(BM * 8 % THREADS == 0 && BN * 8 % THREADS == 0, "tiles divide evenly among the threads");
  static_assert(!SWIGLU || FN % 2 == 0, "a wave needs gate and up fragments in pairs");
  constexpr int COLS = SWIGLU ? BN / 2 : BN;  // output columns of a block

  extern __shared__ __align__(16) unsigned char gemm_lds[];
  bf16_t* sx = reinterpret_cast<bf16_t*>(gemm_lds);  // [2][BM][GROW]
  bf16_t* sw = sx + 2 * BM * GROW;                   // [2][BN][GROW]

  // Block ids are dealt round-robin to the 8 XCDs: XCD x runs ids x, x+8, ... Give it a contiguous
  // range of tiles, ordered with m fastest, so that it walks through few tiles of W.
  const int total = m_tiles * n_tiles;
  int tile = blockIdx.x;
  if (total % 8 == 0) tile = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  const int tn = tile / m_tiles, tm = tile - tn * m_tiles;
  const int m0 = tm * BM, n0 = tn * COLS;

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave % WM, wn = wave / WM;
  const int r = lane & 15, g = lane >> 4;

  // This thread's pieces. A tile goes from memory straight into LDS: a wave's load instruction writes 64 consecutive
  // 16-byte pieces of LDS, one per lane, so piece p = tid + i THREADS of the tile (row p / 8, physical piece p % 8)
  // is fetched by the lane that writes it, from k offset ((p % 8) ^ swizzle(row)) * 8 of that row.
  const bf16_t* px[NX];
  const bf16_t* pw[NW];
#pragma unroll
  for (int i = 0; i < NX; ++i) {
    const int tr = (tid + i * THREADS) >> 3;
    px[i] = X + (size_t)min(m0 + tr, M - 1) * K + (((tid & 7) ^ ((tr >> 1) & 7)) * 8);
  }
  const int w_rows = SWIGLU ? 2 * N : N;
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int tr = (tid + i * THREADS) >> 3;
    int row = n0 + tr;
    if (SWIGLU) {  // wave w's WNR rows are WNR/2 gate rows, then the up rows of the same columns
      const int w = tr / WNR, q = tr % WNR;
      row = min(n0 + w * (WNR / 2) + q % (WNR / 2), N - 1) + (q >= WNR / 2 ? N : 0);
    }
    pw[i] = W + (size_t)min(row, w_rows - 1) * K + (((tid & 7) ^ ((tr >> 1) & 7)) * 8);
  }
  // requests tile `k` (in elements) into buffer `b`; the data is in LDS after the next __syncthreads(), which waits
  // for the wave's outstanding loads before the barrier
  auto request = [&](int k, int b) {
    char* dx = reinterpret_cast<char*>(sx + b * BM * GROW) + wave * 1024;
    char* dw = reinterpret_cast<char*>(sw + b * BN * GROW) + wave * 1024;
#pragma unroll
    for (int i = 0; i < NX; ++i)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(px[i] + k), (lds_ptr_t)(dx + i * THREADS * 16), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < NW; ++i)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pw[i] + k), (lds_ptr_t)(dw + i * THREADS * 16), 16, 0, 0);
  };

  float4_t acc[FN][FM];
#pragma unroll
  for (int a = 0; a < FN; ++a)
#pragma unroll
    for (int b = 0; b < FM; ++b) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

  const int steps = K / GK;
  request(0, 0);
  __syncthreads();

  // piece kk * 4 + g of row .. + r sits at piece (kk * 4 + g) ^ ((r / 2) % 8) (wave tiles start at multiples of 16 rows)
  const int frag_x = (wm * WMR + r) * GROW, frag_w = (wn * WNR + r) * GROW;
  const int piece[2] = {(g ^ ((r >> 1) & 7)) * 8, ((4 + g) ^ ((r >> 1) & 7)) * 8};
  for (int s = 0; s < steps; ++s) {
    const int cur = s & 1;
    const bf16_t* cx = sx + cur * BM * GROW + frag_x;
    const bf16_t* cw = sw + cur * BN * GROW + frag_w;
    // the next tile into the other buffer, which was last read before the barrier that ended step s - 1; past the
    // end the last tile is loaded again, unused
    request(min(s + 1, steps - 1) * GK, cur ^ 1);
#pragma unroll
    for (int kk = 0; kk < GK / 32; ++kk) {
      bf16x8_t fx[FM], fw[FN];
#pragma unroll
      for (int b = 0; b < FM; ++b) fx[b] = *reinterpret_cast<const bf16x8_t*>(cx + b * 16 * GROW + piece[kk]);
#pragma unroll
      for (int a = 0; a < FN; ++a) fw[a] = *reinterpret_cast<const bf16x8_t*>(cw + a * 16 * GROW + piece[kk]);
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[a], fx[b], acc[a][b], 0, 0, 0);
    }
    __syncthreads();
  }

  // lane holds C[m = .. + r][n = .. + 4 g + i]
  const size_t ldc = (size_t)N;
#pragma unroll
  for (int b = 0; b < FM; ++b) {
    const int m = m0 + wm * WMR + b * 16 + r;
    if constexpr (SWIGLU) {
#pragma unroll
      for (int a = 0; a < FN / 2; ++a) {
        const int n = n0 + wn * (WNR / 2) + a * 16 + 4 * g;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          v[i] = (gate == ME_GATE_GELU_TANH ? gate_act(acc[a][b][i], gate) : silu_f(acc[a][b][i])) * acc[a + FN / 2][b][i];
        store4<OutT>(C, ldc, m, n, M, N, v);
      }
    } else {
#pragma unroll
      for (int a = 0; a < FN; ++a) {
        const int n = n0 + wn * WNR + a * 16 + 4 * g;
        const float v[4] = {acc[a][b][0], acc[a][b][1], acc[a][b][2], acc[a][b][3]};
        store4<OutT>(C, ldc, m, n, M, N, v);
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, bool SWIGLU, typename OutT>
int launch_one(const void* X, const void* W, void* C, int M, int N, int K, int gate, hipStream_t stream) {
  constexpr int COLS = SWIGLU ? BN / 2 : BN;
  const int m_tiles = (M + BM - 1) / BM, n_tiles = (N + COLS - 1) / COLS;
  constexpr size_t LDS = (size_t)2 * (BM + BN) * GROW * sizeof(bf16_t);
  auto kernel = gemm_tiled_kernel<BM, BN, WM, WN, SWIGLU, OutT>;
  static bool raised = false;  // one flag per instantiation; the attribute belongs to the function
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS) !=
        hipSuccess)
      return me_fail("me_gemm_bf16_tiled: %zu bytes of LDS were refused", LDS);
    raised = true;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)(m_tiles * n_tiles)), dim3(WM * WN * 64), LDS, stream, (const bf16_t*)X,
                     (const bf16_t*)W, (OutT*)C, M, N, K, m_tiles, n_tiles, gate);
  return me_check_launch("me_gemm_bf16_tiled");
}

template <int BM, int BN, int WM, int WN>
int launch_tiled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype, hipStream_t stream) {
  if (swiglu) {
    if (out_dtype != ME_BF16) return me_fail("me_gemm_bf16_tiled: the gated form writes bfloat16");
    if constexpr ((BN / WN / 16) % 2 == 0)
      return launch_one<BM, BN, WM, WN, true, bf16_t>(X, W, C, M, N, K, swiglu, stream);
    else
      return me_fail("me_gemm_bf16_tiled: this tile shape has no gated form");
  }
  if (out_dtype == ME_BF16) return launch_one<BM, BN, WM, WN, false, bf16_t>(X, W, C, M, N, K, 0, stream);
  return launch_one<BM, BN, WM, WN, false, float>(X, W, C, M, N, K, 0, stream);
}

// The block tile for a product: all shapes here run at about the same rate per unit of tile area (the
// two largest a little ahead), so what decides is how evenly the tiles fill the compute units: the
// number of rounds of tiles times the tile's area. Measured on the gate/up projection (6,144 columns,
// k = 1,024): 2,048 rows, 256 x 192: 32 us against 34.6 with 128 x 192; 3,072 rows: 58.5 against 48.8;
// 4,096 rows: 60.7 against 66.0; 8,192 rows, 256 x 256: 121 against 127.
int choose_shape(int M, int N, int swiglu) {
  static int cus = 0;
  if (cus <= 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
  }
  struct Candidate {
    int shape, bm, bn;
    float weight;
  };
  const Candidate candidates[] = {{7, 128, 128, 1.f}, {9, 128, 192, 1.f}, {12, 256, 192, 0.94f}, {8, 256, 256, 0.93f}};
  int best = 7;
  float best_cost = 0.f;
  for (const Candidate& c : candidates) {
    const int cols = swiglu ? c.bn / 2 : c.bn;
    const long long tiles = (long long)((M + c.bm - 1) / c.bm) * ((N + cols - 1) / cols);
    const float cost = (float)((tiles + cus - 1) / cus) * c.bm * c.bn * c.weight;
    if (best_cost == 0.f || cost < best_cost) best = c.shape, best_cost = cost;
  }
  return best;
}

}  // namespace

// C[M, N] = X[M, K] . W[N, K]^T, or with `swiglu` (1 or 2, a MeGate code) C[M, N] = act(X . W[0:N]^T) * (X . W[N:2N]^T)
// with act silu or tanh-gelu.
// K is a multiple of 64. `shape` picks the block tile: 0 lets the entry point choose, others name one
// (for measurements).
extern "C" int me_gemm_bf16_tiled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                                  int shape, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % GK) return me_fail("me_gemm_bf16_tiled: K=%d must be a positive multiple of %d", K, GK);
  if (!X || !W || !C) return me_fail("me_gemm_bf16_tiled: null operand");
  if (((uintptr_t)X | (uintptr_t)W) & 15) return me_fail("me_gemm_bf16_tiled: operands must be 16-byte aligned");
  if (out_dtype != ME_BF16 && out_dtype != ME_F32) return me_fail("me_gemm_bf16_tiled: unknown output type %d", out_dtype);
  if (swiglu < ME_GATE_NONE || swiglu > ME_GATE_GELU_TANH) return me_fail("me_gemm_bf16_tiled: unknown gate activation %d", swiglu);
  if (shape == 0) shape = choose_shape(M, N, swiglu);
  switch (shape) {
    case 1: return launch_tiled<128, 128, 2, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 2: return launch_tiled<64, 128, 2, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 3: return launch_tiled<128, 64, 2, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 4: return launch_tiled<256, 128, 2, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 5: return launch_tiled<64, 64, 2, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 6: return launch_tiled<256, 128, 4, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 7: return launch_tiled<128, 128, 4, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 8: return launch_tiled<256, 256, 4, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 9: return launch_tiled<128, 192, 4, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 10: return launch_tiled<128, 256, 4, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 11: return launch_tiled<128, 128, 2, 4>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    case 12: return launch_tiled<256, 192, 4, 2>(X, W, C, M, N, K, swiglu, out_dtype, stream);
    default: return me_fail("me_gemm_bf16_tiled: unknown tile shape %d", shape);
  }
}
