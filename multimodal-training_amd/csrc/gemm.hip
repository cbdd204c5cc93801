// MFMA GEMM for gfx950 with fused epilogues:  C[M,N] = epi( sum_k A[m,k] * B[n,k] ).
//
// Block tile 256x128 (M x N), 4 waves in a 2x2 grid, each wave owning 128x64 as 4x2 MFMA 32x32 tiles.
//   bf16: v_mfma_f32_32x32x16_bf16, BK = 64.  Operands whose contraction index is contiguous in memory are
//         staged as [row][k] and read with 16-byte LDS loads; operands whose contraction index is the slow
//         dimension (dgrad's weight, both operands of wgrad) are staged as [k][row] exactly as they lie in
//         memory and read with ds_read_b64_tr_b16, which hands each lane 4 consecutive k for its row.
//   fp32: v_mfma_f32_32x32x2_f32, BK = 16 (parity mode; one LDS word per lane per MFMA operand).
// The next K tile is fetched into registers while the current one is consumed from LDS.
// Work-group ids are remapped so that the tiles a single XCD (one L2) works on are neighbours in N.
#include "mvit_common.h"

namespace {

constexpr int BM = 256, BN = 128;
constexpr int WAVE_M = 128, WAVE_N = 64;  // per-wave tile
constexpr int MT = WAVE_M / 32, NT = WAVE_N / 32;

struct GemmParams {
  int64_t M, N, K;
  const void* A;
  int64_t lda;
  const void* B;
  const void* B2;
  int64_t ldb;
  const void* bias;
  const void* bias2;
  void* C;
  int64_t ldc;
  const void* R;
  int64_t ldr;
  void* aux;
  int64_t ldaux;
  int64_t aux_off;
  int tiles_m, tiles_n;
  int split_k;        // K slices (1 = none)
  int64_t k_chunk;    // K extent of one slice (multiple of BK)
  float* workspace;   // [split_k][M][N] fp32 partial sums when split_k > 1
};

template <typename T>
struct Cfg;
template <>
struct Cfg<bf16_t> {
  static constexpr int BK = 64, VEC = 8;
  static constexpr int PITCH_K = BK + 8;  // [row][k] staging: 144-byte rows, conflict-free 16-byte reads
  static constexpr int PAD_T = 32;        // [k][row] staging: row pitch = rows + 32 elements
};
template <>
struct Cfg<float> {
  static constexpr int BK = 16, VEC = 4;
  static constexpr int PITCH_K = BK + 4;
  static constexpr int PAD_T = 4;
};

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752440f)); }
__device__ __forceinline__ float gelu_erf_grad(float z) {
  const float cdf = 0.5f * (1.f + erff(z * 0.70710678118654752440f));
  const float pdf = 0.39894228040143267794f * __expf(-0.5f * z * z);
  return cdf + z * pdf;
}
__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + __expf(-z)); }

// Stage one operand tile (ROWS rows of the output dimension x BK of the contraction) global -> registers.
// TR = false: memory is [row][k];  TR = true: memory is [k][row].
template <typename T, int ROWS, bool TR>
struct TileLoader {
  using C = Cfg<T>;
  static constexpr int V = C::VEC;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  static constexpr int CHUNKS = ROWS * C::BK / V;  // 16-byte chunks per tile
  static constexpr int PER_THREAD = CHUNKS / 256;
  static constexpr int LDS_ELEMS = TR ? C::BK * (ROWS + C::PAD_T) : ROWS * C::PITCH_K;
  vec_t regs[PER_THREAD];

  // row_map: SWIGLU packs two weight matrices into one B tile; otherwise identity.
  __device__ __forceinline__ void load(const T* __restrict__ base, const T* __restrict__ base2, int64_t ld,
                                       int64_t row0, int64_t row_limit, int64_t k0, int64_t K, bool dual) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = threadIdx.x + 256 * i;
      int r, kk;
      if (!TR) {
        r = c / (C::BK / V);
        kk = (c % (C::BK / V)) * V;
      } else {
        kk = c / (ROWS / V);
        r = (c % (ROWS / V)) * V;
      }
      const T* src = base;
      int64_t grow;
      if (dual) {
        // tile row r = wn*64 + half*32 + j  ->  matrix `half`, row row0 + wn*32 + j   (ROWS == 128, !TR)
        const int wn = r >> 6, half = (r >> 5) & 1, j = r & 31;
        grow = row0 + wn * 32 + j;
        if (half) src = base2;
      } else {
        grow = row0 + r;
      }
      const int64_t gk = k0 + kk;
      vec_t v;
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = from_f32<T>(0.f);
      if (!TR) {
        if (grow < row_limit && gk < K) v = *reinterpret_cast<const vec_t*>(src + grow * ld + gk);
      } else {
        if (grow < row_limit && gk < K) v = *reinterpret_cast<const vec_t*>(src + gk * ld + grow);
      }
      regs[i] = v;
    }
  }
  __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = threadIdx.x + 256 * i;
      int off;
      if (!TR) {
        const int r = c / (C::BK / V), kk = (c % (C::BK / V)) * V;
        off = r * C::PITCH_K + kk;
      } else {
        const int kk = c / (ROWS / V), r = (c % (ROWS / V)) * V;
        off = kk * (ROWS + C::PAD_T) + r;
      }
      *reinterpret_cast<vec_t*>(lds + off) = regs[i];
    }
  }
};

// MFMA operand fetch from LDS for the 32-row sub-tile starting at `row`, contraction offset `k`.
template <bool TR, int ROWS>
__device__ __forceinline__ bf16x8 frag_bf16(const bf16_t* lds, int row, int k) {
  using C = Cfg<bf16_t>;
  const int l = threadIdx.x & 63;
  if (!TR) {
    return *reinterpret_cast<const bf16x8*>(lds + (row + (l & 31)) * C::PITCH_K + k + 8 * (l >> 5));
  } else {
    // lane i of 16-lane group G fetches 4 elements of k-row (k + 8*(G/2) + i/4) at column 16*(G%2) + 4*(i%4);
    // the transposing read returns to lane j of the group the 4 consecutive k of column 16*(G%2) + j.
    constexpr int P = ROWS + C::PAD_T;
    const int G = l >> 4, i = l & 15;
    const bf16_t* p = lds + (k + 8 * (G >> 1) + (i >> 2)) * P + row + 16 * (G & 1) + 4 * (i & 3);
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p + 4 * P));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, both);
  }
}

template <bool TR, int ROWS>
__device__ __forceinline__ float frag_f32(const float* lds, int row, int k) {
  using C = Cfg<float>;
  const int l = threadIdx.x & 63;
  if (!TR)
    return lds[(row + (l & 31)) * C::PITCH_K + k + (l >> 5)];
  else
    return lds[(k + (l >> 5)) * (ROWS + C::PAD_T) + row + (l & 31)];
}

template <typename T, typename TO, bool TA, bool TB, int EPI>
__global__ __launch_bounds__(256) void gemm_kernel(const GemmParams p) {
  using C = Cfg<T>;
  constexpr int BK = C::BK;
  using LoaderA = TileLoader<T, BM, TA>;
  using LoaderB = TileLoader<T, BN, TB>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* lds_a = reinterpret_cast<T*>(smem_raw);
  T* lds_b = lds_a + LoaderA::LDS_ELEMS;

  // XCD-aware tile order: hardware deals consecutive work-group ids round-robin to the 8 XCDs; give each
  // XCD a contiguous range of tiles (N fastest) so that its L2 sees one A panel at a time.
  // With split-K the slices are the slowest index: all tiles of one K slice share the same rows of A and B.
  const int tiles = p.tiles_m * p.tiles_n;
  const int total = tiles * p.split_k;
  const int per_xcd = (total + 7) / 8;
  const int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (work >= total) return;
  const int slice = work / tiles, tile = work % tiles;
  const int tm = tile / p.tiles_n, tn = tile % p.tiles_n;
  const int64_t k_begin = (int64_t)slice * p.k_chunk;
  const int64_t k_end = p.split_k > 1 ? (k_begin + p.k_chunk < p.K ? k_begin + p.k_chunk : p.K) : p.K;
  constexpr bool DUAL = (EPI == MVIT_EPI_SWIGLU);
  constexpr int N_PER_BLOCK = DUAL ? BN / 2 : BN;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * N_PER_BLOCK;

  const int l = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int wm = wv >> 1, wn = wv & 1;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int a = 0; a < MT; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

  LoaderA la;
  LoaderB lb;
  const T* A = static_cast<const T*>(p.A);
  const T* B = static_cast<const T*>(p.B);
  const T* B2 = static_cast<const T*>(p.B2);
  la.load(A, nullptr, p.lda, m0, p.M, k_begin, k_end, false);
  lb.load(B, B2, p.ldb, n0, p.N, k_begin, k_end, DUAL);

  for (int64_t k0 = k_begin; k0 < k_end; k0 += BK) {
    __syncthreads();  // previous tile fully consumed
    la.store(lds_a);
    lb.store(lds_b);
    __syncthreads();
    if (k0 + BK < k_end) {
      la.load(A, nullptr, p.lda, m0, p.M, k0 + BK, k_end, false);
      lb.load(B, B2, p.ldb, n0, p.N, k0 + BK, k_end, DUAL);
    }
    if constexpr (sizeof(T) == 2) {
#pragma unroll
      for (int ks = 0; ks < BK; ks += 16) {
        bf16x8 fa[MT], fb[NT];
#pragma unroll
        for (int a = 0; a < MT; ++a) fa[a] = frag_bf16<TA, BM>(reinterpret_cast<const bf16_t*>(lds_a), wm * WAVE_M + a * 32, ks);
#pragma unroll
        for (int b = 0; b < NT; ++b) fb[b] = frag_bf16<TB, BN>(reinterpret_cast<const bf16_t*>(lds_b), wn * WAVE_N + b * 32, ks);
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
          for (int b = 0; b < NT; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[a], fb[b], acc[a][b], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < BK; ks += 2) {
        float fa[MT], fb[NT];
#pragma unroll
        for (int a = 0; a < MT; ++a) fa[a] = frag_f32<TA, BM>(reinterpret_cast<const float*>(lds_a), wm * WAVE_M + a * 32, ks);
#pragma unroll
        for (int b = 0; b < NT; ++b) fb[b] = frag_f32<TB, BN>(reinterpret_cast<const float*>(lds_b), wn * WAVE_N + b * 32, ks);
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
          for (int b = 0; b < NT; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a], fb[b], acc[a][b], 0, 0, 0);
      }
    }
  }

  // ---- epilogue.  acc[a][b][4*j+i] is C[m0 + wm*128 + a*32 + 8*j + 4*(l/32) + i][n-tile b, column l%32].
  TO* Cp = static_cast<TO*>(p.C);
  const T* Rp = static_cast<const T*>(p.R);
  T* auxp = static_cast<T*>(p.aux);
  const T* bias = static_cast<const T*>(p.bias);
  const T* bias2 = static_cast<const T*>(p.bias2);
  const int lc = l & 31, lr = 4 * (l >> 5);

  if constexpr (EPI == MVIT_EPI_NONE) {
    if (p.split_k > 1) {  // fp32 partial tile; summed over slices by splitk_reduce_kernel
      float* W = p.workspace + (int64_t)slice * p.M * p.N;
#pragma unroll
      for (int b = 0; b < NT; ++b) {
        const int64_t n = n0 + wn * WAVE_N + b * 32 + lc;
        if (n >= p.N) continue;
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int64_t m = m0 + wm * WAVE_M + a * 32 + 8 * j + lr + i;
              if (m < p.M) W[m * p.N + n] = acc[a][b][4 * j + i];
            }
      }
      return;
    }
  }
  if constexpr (DUAL) {
    const int64_t n = n0 + wn * 32 + lc;
    if (n < p.N) {
      const float bg = bias ? to_f32(bias[n]) : 0.f, bu = bias2 ? to_f32(bias2[n]) : 0.f;
#pragma unroll
      for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int64_t m = m0 + wm * WAVE_M + a * 32 + 8 * j + lr + i;
            if (m < p.M) {
              // round g and u to the storage type first: the backward recomputes from those stored values
              const T gs = from_f32<T>(acc[a][0][4 * j + i] + bg);
              const T us = from_f32<T>(acc[a][1][4 * j + i] + bu);
              auxp[m * p.ldaux + n] = gs;
              auxp[m * p.ldaux + p.aux_off + n] = us;
              const float g = to_f32(gs), u = to_f32(us);
              Cp[m * p.ldc + n] = from_f32<TO>(g * sigmoidf_(g) * u);
            }
          }
    }
  } else {
#pragma unroll
    for (int b = 0; b < NT; ++b) {
      const int64_t n = n0 + wn * WAVE_N + b * 32 + lc;
      if (n >= p.N) continue;
      float bv = 0.f;
      if constexpr (EPI == MVIT_EPI_BIAS || EPI == MVIT_EPI_BIAS_RES || EPI == MVIT_EPI_BIAS_GELU)
        bv = bias ? to_f32(bias[n]) : 0.f;
#pragma unroll
      for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int64_t m = m0 + wm * WAVE_M + a * 32 + 8 * j + lr + i;
            if (m >= p.M) continue;
            float v = acc[a][b][4 * j + i] + bv;
            if constexpr (EPI == MVIT_EPI_BIAS_RES) {
              v += to_f32(Rp[m * p.ldr + n]);
            } else if constexpr (EPI == MVIT_EPI_BIAS_GELU) {
              const T zs = from_f32<T>(v);
              auxp[m * p.ldaux + n] = zs;
              v = gelu_erf(to_f32(zs));
            } else if constexpr (EPI == MVIT_EPI_GELU_BWD) {
              v *= gelu_erf_grad(to_f32(Rp[m * p.ldr + n]));
            } else if constexpr (EPI == MVIT_EPI_ACCUM) {
              v += to_f32(Cp[m * p.ldc + n]);
            }
            if constexpr (EPI == MVIT_EPI_SWIGLU_BWD) {
              const float g = to_f32(Rp[m * p.ldr + n]), u = to_f32(Rp[m * p.ldr + p.aux_off + n]);
              const float sg = sigmoidf_(g);
              const float silu = g * sg;
              Cp[m * p.ldc + n] = from_f32<TO>(v * u * (sg + silu * (1.f - sg)));
              Cp[m * p.ldc + p.aux_off + n] = from_f32<TO>(v * silu);
            } else {
              Cp[m * p.ldc + n] = from_f32<TO>(v);
            }
          }
    }
  }
}

// C[m, n] = sum over slices of the fp32 partial tiles (fixed order, so the result is reproducible).
template <typename TO>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int split_k, int64_t M, int64_t N,
                                                            TO* __restrict__ C, int64_t ldc) {
  const int64_t total = M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    float s = 0.f;
    for (int k = 0; k < split_k; ++k) s += ws[(int64_t)k * total + i];
    C[(i / N) * ldc + (i % N)] = from_f32<TO>(s);
  }
}

template <typename T, typename TO, bool TA, bool TB, int EPI>
int launch(const GemmParams& p, hipStream_t stream) {
  using LA = TileLoader<T, BM, TA>;
  using LB = TileLoader<T, BN, TB>;
  const size_t lds = (size_t)(LA::LDS_ELEMS + LB::LDS_ELEMS) * sizeof(T);
  auto kern = gemm_kernel<T, TO, TA, TB, EPI>;
  static bool attr_set = false;  // dynamic LDS above 64 KiB needs opting in once per kernel
  if (!attr_set && lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return mvit_set_error(MVIT_ERR_LAUNCH, "gemm: hipFuncSetAttribute(%zu B LDS): %s", lds, hipGetErrorString(e));
    attr_set = true;
  }
  if (p.split_k > 1 && EPI != MVIT_EPI_NONE) return mvit_set_error(MVIT_ERR_UNSUPPORTED, "gemm: split_k needs EPI_NONE");
  const int total = p.tiles_m * p.tiles_n * p.split_k;
  const int grid = ((total + 7) / 8) * 8;
  hipLaunchKernelGGL(kern, grid, 256, lds, stream, p);
  MVIT_CHECK_LAUNCH("gemm");
  if (p.split_k > 1) {
    const int64_t elems = p.M * p.N;
    const int rgrid = (int)((elems + 255) / 256 < 8192 ? (elems + 255) / 256 : 8192);
    hipLaunchKernelGGL((splitk_reduce_kernel<TO>), rgrid, 256, 0, stream, p.workspace, p.split_k, p.M, p.N, static_cast<TO*>(p.C), p.ldc);
    MVIT_CHECK_LAUNCH("gemm split-k reduce");
  }
  return MVIT_OK;
}

template <typename T, typename TO, bool TA, bool TB>
int dispatch_epi(int epi, const GemmParams& p, hipStream_t s) {
  switch (epi) {
    case MVIT_EPI_NONE: return launch<T, TO, TA, TB, MVIT_EPI_NONE>(p, s);
    case MVIT_EPI_BIAS: return launch<T, TO, TA, TB, MVIT_EPI_BIAS>(p, s);
    case MVIT_EPI_ACCUM: return launch<T, TO, TA, TB, MVIT_EPI_ACCUM>(p, s);
    default: break;
  }
  if constexpr (!TA && !TB) {
    // forward-only epilogues (both operands contraction-contiguous)
    switch (epi) {
      case MVIT_EPI_BIAS_RES: return launch<T, TO, false, false, MVIT_EPI_BIAS_RES>(p, s);
      case MVIT_EPI_BIAS_GELU: return launch<T, TO, false, false, MVIT_EPI_BIAS_GELU>(p, s);
      case MVIT_EPI_SWIGLU: return launch<T, TO, false, false, MVIT_EPI_SWIGLU>(p, s);
      default: break;
    }
  }
  if constexpr (!TA && TB) {
    // data-gradient epilogues
    switch (epi) {
      case MVIT_EPI_SWIGLU_BWD: return launch<T, TO, false, true, MVIT_EPI_SWIGLU_BWD>(p, s);
      case MVIT_EPI_GELU_BWD: return launch<T, TO, false, true, MVIT_EPI_GELU_BWD>(p, s);
      default: break;
    }
  }
  return mvit_set_error(MVIT_ERR_UNSUPPORTED, "gemm: epilogue %d not built for trans_a=%d trans_b=%d", epi, (int)TA, (int)TB);
}

template <typename T, typename TO>
int dispatch_trans(int ta, int tb, int epi, const GemmParams& p, hipStream_t s) {
  if (!ta && !tb) return dispatch_epi<T, TO, false, false>(epi, p, s);
  if (!ta && tb) return dispatch_epi<T, TO, false, true>(epi, p, s);
  if (ta && tb) return dispatch_epi<T, TO, true, true>(epi, p, s);
  return mvit_set_error(MVIT_ERR_UNSUPPORTED, "gemm: trans_a=1, trans_b=0 is not built");
}

}  // namespace

extern "C" int mvit_gemm(const mvit_gemm_args* a, mvit_stream_t stream) {
  MVIT_REQUIRE(a, "gemm: null args");
  MVIT_REQUIRE(a->A && a->B && a->C, "gemm: null operand");
  MVIT_REQUIRE(a->M >= 0 && a->N > 0 && a->K > 0, "gemm: bad shape M=%lld N=%lld K=%lld", (long long)a->M, (long long)a->N, (long long)a->K);
  if (a->M == 0) return MVIT_OK;
  const int vec = a->dtype == MVIT_BF16 ? 8 : 4;
  MVIT_REQUIRE(a->dtype == MVIT_BF16 || a->dtype == MVIT_F32, "gemm: dtype %d", a->dtype);
  MVIT_REQUIRE(a->out_dtype == MVIT_BF16 || a->out_dtype == MVIT_F32, "gemm: out_dtype %d", a->out_dtype);
  MVIT_REQUIRE(mvit_aligned16(a->A) && mvit_aligned16(a->B) && (!a->B2 || mvit_aligned16(a->B2)), "gemm: operands must be 16-byte aligned");
  MVIT_REQUIRE(a->lda % vec == 0 && a->ldb % vec == 0, "gemm: lda=%lld ldb=%lld must be multiples of %d", (long long)a->lda, (long long)a->ldb, vec);
  // 16-byte vectors never straddle the edge of the contiguous dimension
  if (!a->trans_a) MVIT_REQUIRE(a->K % vec == 0 && a->lda >= a->K, "gemm: K=%lld must be a multiple of %d (lda=%lld)", (long long)a->K, vec, (long long)a->lda);
  else MVIT_REQUIRE(a->lda >= (a->M + vec - 1) / vec * vec, "gemm: transposed A needs lda=%lld >= M=%lld rounded up to %d", (long long)a->lda, (long long)a->M, vec);
  if (!a->trans_b) MVIT_REQUIRE(a->K % vec == 0 && a->ldb >= a->K, "gemm: K=%lld must be a multiple of %d (ldb=%lld)", (long long)a->K, vec, (long long)a->ldb);
  else MVIT_REQUIRE(a->ldb >= (a->N + vec - 1) / vec * vec, "gemm: transposed B needs ldb=%lld >= N=%lld rounded up to %d", (long long)a->ldb, (long long)a->N, vec);
  const int epi = a->epilogue;
  if (epi == MVIT_EPI_BIAS_RES || epi == MVIT_EPI_GELU_BWD || epi == MVIT_EPI_SWIGLU_BWD) MVIT_REQUIRE(a->R, "gemm: epilogue %d needs R", epi);
  if (epi == MVIT_EPI_BIAS_GELU || epi == MVIT_EPI_SWIGLU) MVIT_REQUIRE(a->aux, "gemm: epilogue %d needs aux", epi);
  if (epi == MVIT_EPI_SWIGLU) MVIT_REQUIRE(a->B2 && !a->trans_a && !a->trans_b, "gemm: SWIGLU needs B2 and untransposed operands");
  MVIT_REQUIRE(a->ldc >= a->N, "gemm: ldc=%lld < N=%lld", (long long)a->ldc, (long long)a->N);

  GemmParams p;
  p.M = a->M; p.N = a->N; p.K = a->K;
  p.A = a->A; p.lda = a->lda; p.B = a->B; p.B2 = a->B2; p.ldb = a->ldb;
  p.bias = a->bias; p.bias2 = a->bias2; p.C = a->C; p.ldc = a->ldc;
  p.R = a->R; p.ldr = a->ldr; p.aux = a->aux; p.ldaux = a->ldaux; p.aux_off = a->aux_off;
  const int n_per_block = (epi == MVIT_EPI_SWIGLU) ? BN / 2 : BN;
  const int64_t tm = (a->M + BM - 1) / BM, tn = (a->N + n_per_block - 1) / n_per_block;
  MVIT_REQUIRE(tm * tn < (1ll << 30), "gemm: too many tiles");
  p.tiles_m = (int)tm; p.tiles_n = (int)tn;
  p.split_k = 1; p.k_chunk = a->K; p.workspace = nullptr;
  if (a->split_k > 1) {
    const int bk = a->dtype == MVIT_BF16 ? 64 : 16;
    const int64_t chunk = ((a->K + a->split_k - 1) / a->split_k + bk - 1) / bk * bk;
    const int64_t slices = (a->K + chunk - 1) / chunk;  // never an empty slice
    MVIT_REQUIRE(epi == MVIT_EPI_NONE, "gemm: split_k is only available with EPI_NONE");
    MVIT_REQUIRE(a->workspace && a->workspace_bytes >= (int64_t)sizeof(float) * slices * a->M * a->N,
                 "gemm: split_k=%d needs a workspace of %lld bytes", a->split_k, (long long)(sizeof(float) * slices * a->M * a->N));
    MVIT_REQUIRE(tm * tn * slices < (1ll << 30), "gemm: too many tiles");
    if (slices > 1) { p.split_k = (int)slices; p.k_chunk = chunk; p.workspace = static_cast<float*>(a->workspace); }
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (a->dtype == MVIT_BF16) {
    if (a->out_dtype == MVIT_BF16) return dispatch_trans<bf16_t, bf16_t>(a->trans_a, a->trans_b, epi, p, s);
    return dispatch_trans<bf16_t, float>(a->trans_a, a->trans_b, epi, p, s);
  }
  MVIT_REQUIRE(a->out_dtype == MVIT_F32, "gemm: fp32 operands need fp32 output");
  return dispatch_trans<float, float>(a->trans_a, a->trans_b, epi, p, s);
}
