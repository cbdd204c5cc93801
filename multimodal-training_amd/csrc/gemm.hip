// MFMA GEMM for gfx950 with fused epilogues:  C[M,N] = epi( sum_k A[m,k] * B[n,k] ).
//
// Main loops:
//   bf16: 256x256 tile, 8 waves of 128x64 (4x2 MFMA 32x32x16 tiles each), BK = 32, four LDS stages filled by direct
//      global -> LDS loads (see gemm_dl_kernel).
//   fp32 (the parity path, v_mfma_f32_32x32x2_f32), and bf16 operands whose row pitch exceeds 2^22 elements (the
//      direct loads use 32-bit lane offsets): 256x256 tile, 8 waves, BK = 64 (fp32: 16), global -> registers -> LDS,
//      double-buffered LDS, one barrier per K step (gemm_kernel).
// Operands whose contraction index is contiguous in memory are staged as [row][k] and read with 16-byte LDS
// loads; operands whose contraction index is the slow dimension (dgrad's weight, both operands of wgrad) are
// staged as [k][row] exactly as they lie in memory and read with ds_read_b64_tr_b16, which hands each lane 4
// consecutive k for its row.
// The epilogue stages the accumulators through LDS (fp32) so that bias / residual / activation inputs are
// read and results written as 16-byte vectors along N.
// Work-group ids are remapped so that the tiles a single XCD (one L2) works on are neighbours in N.
#include "mvit_common.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <type_traits>

namespace {


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
  int reduce_epi;  // split_k > 1: the epilogue that the reduction over the K slices applies (none, bias, bias + residual)
  int tiles_m, tiles_n;
  int split_k;        // K slices (1 = none)
  int64_t k_chunk;    // K extent of one slice (multiple of BK)
  float* workspace;   // [split_k][M][N] fp32 partial sums when split_k > 1
  int vec_ok;         // every epilogue pointer / stride allows 16-byte accesses
  float* colsum;      // SWIGLU_BWD: per-tile-row column sums of the output, [tiles_m][ldc] (null: not wanted)
  int panel_w;        // tiles are walked in panels of this many tile columns (M fastest across a panel's rows)
  // A operand made from decoded frames (gemm_dl_kernel<..., PIX = true>): image table and the affine form of the
  // rescale / normalise step, value = byte * px_a[channel] + px_c[channel]
  const mvit_image* px_images;
  int px_n_images;
  float px_a[3], px_c[3];
};

// Tile order inside one K slice: panels of panel_w tile columns; within a panel row by row.  Work-groups that run
// at the same time on one XCD (consecutive tile indices) then cover a compact block of the output, e.g. 8 x 4
// tiles, so the A and B panels they stream through that XCD's L2 are shared as widely as possible.
__device__ __forceinline__ void tile_coords(const GemmParams& p, int tile, int& tm, int& tn) {
  const int pw = p.panel_w;
  const int full_panels = p.tiles_n / pw, per_panel = p.tiles_m * pw;
  if (tile < full_panels * per_panel) {
    const int r = tile % per_panel;
    tm = r / pw;
    tn = (tile / per_panel) * pw + r % pw;
  } else {
    const int r = tile - full_panels * per_panel, w = p.tiles_n - full_panels * pw;
    tm = r / w;
    tn = full_panels * pw + r % w;
  }
}

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

template <int VAR>
struct Waves;
template <>
struct Waves<1> {  // 256x256 tile, 8 waves of 128x64, double-buffered LDS, one work-group per CU
  static constexpr int BM = 256, BN = 256, WM = 128, WN = 64, NTHREADS = 512, MIN_WAVES = 2;
};

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752440f)); }
__device__ __forceinline__ float gelu_erf_grad(float z) {
  const float cdf = 0.5f * (1.f + erff(z * 0.70710678118654752440f));
  const float pdf = 0.39894228040143267794f * __expf(-0.5f * z * z);
  return cdf + z * pdf;
}
// 1 / (1 + e^-z) with the hardware reciprocal (1 ulp) instead of the IEEE division sequence
__device__ __forceinline__ float sigmoidf_(float z) { return __builtin_amdgcn_rcpf(1.f + __expf(-z)); }

// 8 consecutive elements <-> fp32 registers
__device__ __forceinline__ void load8(const bf16_t* p, float* v) {
  const bf16x8 x = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (float)x[e];
}
__device__ __forceinline__ void load8(const float* p, float* v) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[e] = a[e];
    v[4 + e] = b[e];
  }
}
template <typename T>
__device__ __forceinline__ void unpack8(const T __attribute__((ext_vector_type(8))) & x, float* v) {
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (float)x[e];
}
// Epilogue outputs and per-element epilogue inputs are touched once per launch: they are stored / loaded with the
// non-temporal hint, so that they do not push the operand panels of the tiles in flight out of the XCD's L2 (a round of
// 32 output tiles is as large as that L2; with plain stores the main loop after an epilogue ran 18 % slower).
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store8(bf16_t* p, const float* v) {
  bf16x8 x;
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (bf16_t)v[e];
  __builtin_nontemporal_store(__builtin_bit_cast(u32x4_t, x), reinterpret_cast<u32x4_t*>(p));
}
__device__ __forceinline__ void store8(float* p, const float* v) {
  __builtin_nontemporal_store(f32x4{v[0], v[1], v[2], v[3]}, reinterpret_cast<f32x4*>(p));
  __builtin_nontemporal_store(f32x4{v[4], v[5], v[6], v[7]}, reinterpret_cast<f32x4*>(p + 4));
}
// split-K partial tiles are read back by the reduction kernel right away: they stay cacheable
__device__ __forceinline__ void store8_cached(float* p, const float* v) {
  *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<f32x4*>(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
}
template <typename T>
__device__ __forceinline__ T __attribute__((ext_vector_type(8))) load8_stream(const void* p) {
  typedef T raw8 __attribute__((ext_vector_type(8)));
  if constexpr (sizeof(T) == 2) {
    return __builtin_bit_cast(raw8, __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p)));
  } else {
    raw8 r;
    const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
    const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p) + 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r[e] = a[e];
      r[4 + e] = b[e];
    }
    return r;
  }
}

// Stage one operand tile (ROWS rows of the output dimension x BK of the contraction) global -> registers -> LDS.
// TR = false: memory is [row][k];  TR = true: memory is [k][row].
// A thread's chunks are a fixed distance apart (NTHREADS/8 rows, or NTHREADS/(ROWS/V) k-rows when TR), so one
// pointer, one remaining-K counter and a row mask describe the whole K loop.  Loads are unconditional (masked
// chunks read the operand's first element) and zeroed, if need be, when written to LDS.
// DUAL (SWIGLU's B operand): rows alternate between two matrices, so every chunk keeps its own pointer.
template <typename T, int ROWS, bool TR, int NTHREADS, int WN, bool DUAL>
struct TileLoader {
  using C = Cfg<T>;
  static constexpr int V = C::VEC;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  static constexpr int CHUNKS = ROWS * C::BK / V;  // 16-byte chunks per tile
  static constexpr int PER_THREAD = CHUNKS / NTHREADS;
  static constexpr int LDS_ELEMS = TR ? C::BK * (ROWS + C::PAD_T) : ROWS * C::PITCH_K;
  static constexpr int ROW_STEP = TR ? 0 : NTHREADS / (C::BK / V);  // tile rows between consecutive chunks
  static constexpr int K_STEP = TR ? NTHREADS / (ROWS / V) : 0;     // k between consecutive chunks
  vec_t regs[PER_THREAD];
  const T* ptr[DUAL ? PER_THREAD : 1];
  const T* safe;      // always-valid address for masked chunks
  int64_t chunk_step; // elements between consecutive chunks of this thread
  int64_t step;       // pointer advance per K tile
  int k_left;         // K elements left from chunk 0's position (<= 0: exhausted)
  unsigned row_mask;  // bit i: chunk i lies on a valid row

  __device__ __forceinline__ void init(const T* __restrict__ base, const T* __restrict__ base2, int64_t ld,
                                       int64_t row0, int64_t row_limit, int64_t k_begin, int64_t k_end) {
    step = TR ? (int64_t)C::BK * ld : (int64_t)C::BK;
    chunk_step = TR ? (int64_t)K_STEP * ld : (int64_t)ROW_STEP * ld;
    safe = base;
    row_mask = 0;
    const int c0 = threadIdx.x;
    const int kk0 = TR ? c0 / (ROWS / V) : (c0 % (C::BK / V)) * V;
    const int64_t left = k_end - (k_begin + kk0);
    k_left = (int)(left > (1 << 30) ? (1 << 30) : left);
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = threadIdx.x + NTHREADS * i;
      const int r = TR ? (c % (ROWS / V)) * V : c / (C::BK / V);
      const int kk = TR ? c / (ROWS / V) : (c % (C::BK / V)) * V;
      const T* src = base;
      int64_t grow = row0 + r;
      if (DUAL) {  // tile row r = wn*WN + half*(WN/2) + j -> matrix `half`, row row0 + wn*(WN/2) + j
        const int wn = r / WN, w = r % WN, half = w / (WN / 2), j = w % (WN / 2);
        grow = row0 + wn * (WN / 2) + j;
        if (half) src = base2;
      }
      const bool row_ok = grow < row_limit;
      if (row_ok) row_mask |= 1u << i;
      const int64_t gk = k_begin + kk;
      const T* q = row_ok ? (TR ? src + gk * ld + grow : src + grow * ld + gk) : src;
      if (DUAL) ptr[i] = q;
      else if (i == 0) ptr[0] = TR ? src + gk * ld + grow : src + grow * ld + gk;  // may lie past the edge: never dereferenced then
    }
  }
  __device__ __forceinline__ bool live(int i, int kl) const { return ((row_mask >> i) & 1u) && (kl - i * K_STEP > 0); }
  __device__ __forceinline__ void load() {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const bool ok = live(i, k_left);
      const T* q = DUAL ? ptr[i] : ptr[0] + i * chunk_step;
      regs[i] = *reinterpret_cast<const vec_t*>(ok ? q : safe);
    }
    k_left -= C::BK;
    if (DUAL) {
#pragma unroll
      for (int i = 0; i < PER_THREAD; ++i) ptr[i] += step;
    } else {
      ptr[0] += step;
    }
  }
  __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      vec_t v = regs[i];
      if (!live(i, k_left + C::BK)) {  // this chunk was outside the matrix / K range when it was loaded
#pragma unroll
        for (int j = 0; j < V; ++j) v[j] = from_f32<T>(0.f);
      }
      const int c = threadIdx.x + NTHREADS * i;
      int off;
      if (!TR) {
        const int r = c / (C::BK / V), kk = (c % (C::BK / V)) * V;
        off = r * C::PITCH_K + kk;
      } else {
        const int kk = c / (ROWS / V), r = (c % (ROWS / V)) * V;
        off = kk * (ROWS + C::PAD_T) + r;
      }
      *reinterpret_cast<vec_t*>(lds + off) = v;
    }
  }
};

// The A operand of the patch embedding made on the fly from decoded uint8 frames (no [rows, 1176] matrix in memory).
// The contraction index is re-ordered so that it runs along memory: k' = line * 48 + b with line = frame-of-the-pair *
// 14 + y and b = x * 3 + channel for b < 42 (the 42 bytes of one pixel line of a patch are contiguous in the frame);
// b = 42..47 pads the line to six 8-byte pieces and meets zero weights (mvit_patch_embed_pack_weight).
// 1344 = 28 lines * 48 = 42 K tiles of 32.  A lane fetches one 8-byte piece per row and K tile with a single vector load
// and turns it into a 16-byte bf16 chunk with eight conversions byte -> float -> a * x + c -> bf16.  Pieces advance by a
// fixed count per K tile, so (line, piece) and the channel of the piece's first byte are stepped, not recomputed.
constexpr int PX_LINE = 48, PX_LINES = 28, PX_K = PX_LINE * PX_LINES, PX_PATCH = 14;
__device__ __forceinline__ int px_find_image(const mvit_image* t, int n, int64_t row) {
  int lo = 0, hi = n;  // invariant: t[lo].first_row <= row < t[hi].first_row
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (t[mid].first_row <= row) lo = mid;
    else hi = mid;
  }
  return lo;
}
// Where patch `row` of the batch lies: first byte of its 14 x 14 pixel square in the first frame of its temporal pair,
// bytes per image line, distance to the pair's second frame (0 when
// the last frame of an odd count, or a still image, fills both halves).
__device__ __forceinline__ void px_locate(const GemmParams& p, int64_t row, const uint8_t*& base, int& line_bytes, int& frame_off) {
  if (row >= p.M) row = p.M - 1;  // rows past the edge repeat the last row; their results are never stored
  const mvit_image im = p.px_images[px_find_image(p.px_images, p.px_n_images, row)];
  const int gh = im.height / PX_PATCH, gw = im.width / PX_PATCH, per_t = gh * gw;
  const int64_t local = row - im.first_row;
  const int t = (int)(local / per_t), rem = (int)(local % per_t);
  // rem = ((block row * (gw / 2) + block column) * 2 + row in block) * 2 + column in block
  const int blk = rem >> 2, hb = blk / (gw >> 1), wb = blk % (gw >> 1);
  const int y0 = (2 * hb + ((rem >> 1) & 1)) * PX_PATCH, x0 = (2 * wb + (rem & 1)) * PX_PATCH;
  const int f0 = 2 * t, f1 = f0 + 1 < im.frames ? f0 + 1 : im.frames - 1;
  const int lb = im.width * 3;
  const int64_t fb = (int64_t)lb * im.height;
  const int64_t first = f0 * fb + (int64_t)y0 * lb + x0 * 3;
  line_bytes = lb;
  frame_off = (int)((f1 - f0) * fb);
  base = im.pixels + first;
}
// The 8 bytes at p (2-byte aligned when the frame buffer is 4-byte aligned; global memory takes unaligned vector loads),
// as one load whose result is not touched until px_convert8, so that it can stay in flight.
struct PxRaw {
  u32x2 w;
};
__device__ __forceinline__ void px_fetch8(const uint8_t* p, PxRaw& r) {
  typedef __attribute__((address_space(1))) const uint8_t* global_bytes;  // frames are in device memory: no generic-address load
  __builtin_memcpy(&r.w, (global_bytes)(uintptr_t)p, 8);
}
// the normalisation constants as six scalars (kernel arguments indexed by a lane-varying channel would be fetched from
// memory for every use)
struct PxNorm {
  float a0, a1, a2, c0, c1, c2;
  __device__ __forceinline__ explicit PxNorm(const GemmParams& p) : a0(p.px_a[0]), a1(p.px_a[1]), a2(p.px_a[2]), c0(p.px_c[0]), c1(p.px_c[1]), c2(p.px_c[2]) {}
};
// 8 bytes -> bf16(byte * a + c), the first byte belonging to channel ch0.  tail: the load was moved 6 bytes back so that
// it ends with the line (piece 5 holds bytes 40, 41 of the line and six padding columns): its last two bytes are the
// piece's first two, the rest of the piece is padding.
__device__ __forceinline__ bf16x8 px_convert8(const PxRaw& r, int ch0, bool tail, const PxNorm nm) {
  const unsigned raw[2] = {tail ? r.w[1] >> 16 : r.w[0], tail ? 0u : r.w[1]};
  // a, c of bytes 0, 1, 2 (mod 3) of the piece: the constants rotated by ch0
  const bool r1 = ch0 == 1, r2 = ch0 == 2;
  const float ar0 = r2 ? nm.a2 : (r1 ? nm.a1 : nm.a0), ar1 = r2 ? nm.a0 : (r1 ? nm.a2 : nm.a1), ar2 = r2 ? nm.a1 : (r1 ? nm.a0 : nm.a2);
  const float cr0 = r2 ? nm.c2 : (r1 ? nm.c1 : nm.c0), cr1 = r2 ? nm.c0 : (r1 ? nm.c2 : nm.c1), cr2 = r2 ? nm.c1 : (r1 ? nm.c0 : nm.c2);
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float x = (float)((raw[e >> 2] >> (8 * (e & 3))) & 0xffu);
    v[e] = (bf16_t)__builtin_fmaf(x, e % 3 == 0 ? ar0 : (e % 3 == 1 ? ar1 : ar2), e % 3 == 0 ? cr0 : (e % 3 == 1 ? cr1 : cr2));
  }
  return v;
}
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

// Epilogue on 8 consecutive output columns n..n+7 of row m.  v: accumulators (gate half for SWIGLU), u: up half.
// FULL: all 8 columns exist and every pointer allows 16-byte accesses (compile-time trip counts, vector memory
// operations); otherwise a scalar path bounded by the matrix edge.
// PRE: the epilogue's per-element inputs (residual / saved activations) were fetched earlier into pre[0..1].
// hb / hb2: the 8 bias values of columns n .. n+7, already in registers (null: loaded here)
template <typename T, typename TO, int EPI, bool FULL, bool PRE = false>
__device__ __forceinline__ void emit8_impl(const GemmParams& p, int64_t m, int64_t n, float* v, const float* u,
                                           const T __attribute__((ext_vector_type(8))) * pre, float (&cs)[16], bool do_cs,
                                           const float* hb = nullptr, const float* hb2 = nullptr) {
  TO* Cp = static_cast<TO*>(p.C);
  const T* Rp = static_cast<const T*>(p.R);
  T* auxp = static_cast<T*>(p.aux);
  const T* bias = static_cast<const T*>(p.bias);
  const T* bias2 = static_cast<const T*>(p.bias2);
  const int cnt = FULL ? 8 : ((p.N - n) < 8 ? (int)(p.N - n) : 8);
  constexpr bool vec = FULL;

  if constexpr (EPI == MVIT_EPI_BIAS || EPI == MVIT_EPI_BIAS_RES || EPI == MVIT_EPI_BIAS_GELU || EPI == MVIT_EPI_SWIGLU) {
    if (hb) {
      for (int e = 0; e < 8; ++e) v[e] += hb[e];
    } else if (bias) {
      float b[8];
      if (vec) load8(bias + n, b);
      else
        for (int e = 0; e < cnt; ++e) b[e] = to_f32(bias[n + e]);
      for (int e = 0; e < cnt; ++e) v[e] += b[e];
    }
  }
  if constexpr (EPI == MVIT_EPI_SWIGLU) {
    float uu[8], h[8];
    for (int e = 0; e < 8; ++e) uu[e] = u[e];
    if (hb2) {
      for (int e = 0; e < 8; ++e) uu[e] += hb2[e];
    } else if (bias2) {
      float b[8];
      if (vec) load8(bias2 + n, b);
      else
        for (int e = 0; e < cnt; ++e) b[e] = to_f32(bias2[n + e]);
      for (int e = 0; e < cnt; ++e) uu[e] += b[e];
    }
    // round g and u to the storage type first: the backward recomputes from those stored values
    for (int e = 0; e < 8; ++e) {
      v[e] = to_f32(from_f32<T>(v[e]));
      uu[e] = to_f32(from_f32<T>(uu[e]));
      h[e] = v[e] * sigmoidf_(v[e]) * uu[e];
    }
    TO* h_out = Cp + m * p.ldc + n;
    if (auxp) {  // a caller that will not differentiate passes no aux and gets the product alone
      T* g_out = auxp + m * p.ldaux + n;
      T* u_out = g_out + p.aux_off;
      if (vec) {
        store8(g_out, v);
        store8(u_out, uu);
      } else {
        for (int e = 0; e < cnt; ++e) {
          g_out[e] = from_f32<T>(v[e]);
          u_out[e] = from_f32<T>(uu[e]);
        }
      }
    }
    if (vec) store8(h_out, h);
    else
      for (int e = 0; e < cnt; ++e) h_out[e] = from_f32<TO>(h[e]);
    return;
  }
  if constexpr (EPI == MVIT_EPI_SWIGLU_BWD) {
    const T* g_in = Rp + m * p.ldr + n;
    const T* u_in = g_in + p.aux_off;
    float g[8], uu[8], dg[8], du[8];
    if (PRE) {
      unpack8<T>(pre[0], g);
      unpack8<T>(pre[1], uu);
    } else if (vec) {
      load8(g_in, g);
      load8(u_in, uu);
    } else {
      for (int e = 0; e < 8; ++e) {
        g[e] = e < cnt ? to_f32(g_in[e]) : 0.f;
        uu[e] = e < cnt ? to_f32(u_in[e]) : 0.f;
      }
    }
    for (int e = 0; e < 8; ++e) {
      const float sg = sigmoidf_(g[e]);
      const float silu = g[e] * sg;
      dg[e] = v[e] * uu[e] * (sg + silu * (1.f - sg));
      du[e] = v[e] * silu;
    }
    if (do_cs) {  // running column sums of this thread's 8 columns (the gate / up bias gradient)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (e < cnt) {
          cs[e] += dg[e];
          cs[8 + e] += du[e];
        }
      }
    }
    TO* dg_out = Cp + m * p.ldc + n;
    TO* du_out = dg_out + p.aux_off;
    if (vec) {
      store8(dg_out, dg);
      store8(du_out, du);
    } else {
      for (int e = 0; e < cnt; ++e) {
        dg_out[e] = from_f32<TO>(dg[e]);
        du_out[e] = from_f32<TO>(du[e]);
      }
    }
    return;
  }
  if constexpr (EPI == MVIT_EPI_BIAS_RES || EPI == MVIT_EPI_GELU_BWD) {
    float r[8];
    if (PRE) unpack8<T>(pre[0], r);
    else if (vec) load8(Rp + m * p.ldr + n, r);
    else
      for (int e = 0; e < 8; ++e) r[e] = e < cnt ? to_f32(Rp[m * p.ldr + n + e]) : 0.f;
    for (int e = 0; e < 8; ++e) {
      if constexpr (EPI == MVIT_EPI_BIAS_RES) v[e] += r[e];
      else v[e] *= gelu_erf_grad(r[e]);
    }
  }
  if constexpr (EPI == MVIT_EPI_BIAS_GELU) {
    T* z_out = auxp + m * p.ldaux + n;
    for (int e = 0; e < 8; ++e) v[e] = to_f32(from_f32<T>(v[e]));  // gelu of the stored pre-activation
    if (vec) store8(z_out, v);
    else
      for (int e = 0; e < cnt; ++e) z_out[e] = from_f32<T>(v[e]);
    for (int e = 0; e < 8; ++e) v[e] = gelu_erf(v[e]);
  }
  TO* c_out = Cp + m * p.ldc + n;
  if constexpr (EPI == MVIT_EPI_ACCUM) {
    float c[8];
    if (vec) load8(c_out, c);
    else
      for (int e = 0; e < 8; ++e) c[e] = e < cnt ? to_f32(c_out[e]) : 0.f;
    for (int e = 0; e < 8; ++e) v[e] += c[e];
  }
  if (vec) store8(c_out, v);
  else
    for (int e = 0; e < cnt; ++e) c_out[e] = from_f32<TO>(v[e]);
}

template <typename T, typename TO, int EPI>
__device__ __forceinline__ void emit8(const GemmParams& p, int64_t m, int64_t n, float* v, const float* u, bool vec,
                                      float (&cs)[16], bool do_cs) {
  if (vec && n + 8 <= p.N) emit8_impl<T, TO, EPI, true>(p, m, n, v, u, nullptr, cs, do_cs);
  else emit8_impl<T, TO, EPI, false>(p, m, n, v, u, nullptr, cs, do_cs);
}

// Per-element epilogue inputs (residual / saved activations) of an interior tile, fetched ahead of their use.
// One pass of the epilogue covers (BM/WM)*32 rows; a thread owns ITEMS 8-column groups per pass.  Two passes are
// buffered (one when an element needs two inputs): the epilogue requests pass a+2 when pass a has been consumed.
template <typename T, int EPI, int BM, int BN, int WM, int NTHREADS>
struct EpiPre {
  static constexpr bool DUAL = (EPI == MVIT_EPI_SWIGLU);
  static constexpr int PASS_ROWS = (BM / WM) * 32, GROUPS = (DUAL ? BN / 2 : BN) / 8;
  static constexpr bool HAS_IN = (EPI == MVIT_EPI_BIAS_RES || EPI == MVIT_EPI_GELU_BWD || EPI == MVIT_EPI_SWIGLU_BWD) &&
                                 (PASS_ROWS * GROUPS) % NTHREADS == 0;
  static constexpr int ITEMS = HAS_IN ? PASS_ROWS * GROUPS / NTHREADS : 1, NLOAD = EPI == MVIT_EPI_SWIGLU_BWD ? 2 : 1;
  static constexpr int RPI = NTHREADS / GROUPS;  // rows between a thread's consecutive items
  static_assert(!HAS_IN || (NTHREADS % GROUPS == 0 && 32 % RPI == 0), "row mapping of the prefetched epilogue");
  typedef T raw8 __attribute__((ext_vector_type(8)));
  static constexpr int NBUF = NLOAD == 2 ? 1 : 2;  // passes buffered (two 16-byte inputs per element: one pass)
  raw8 pre[NBUF][ITEMS][NLOAD];
  const char* base;     // R + m0 * ldr + n0 (block-uniform)
  unsigned thread_off;  // this thread's byte offset inside a pass: row threadIdx / GROUPS, column group threadIdx % GROUPS
  bool active;          // block-uniform: this tile takes the prefetched path

  __device__ __forceinline__ void init(const GemmParams& p, int64_t m0, int64_t n0) {
    active = HAS_IN && p.vec_ok && m0 + BM <= p.M && n0 + GROUPS * 8 <= p.N && p.ldr * (int64_t)BM * sizeof(T) < (1ll << 31);
    base = reinterpret_cast<const char*>(static_cast<const T*>(p.R) + m0 * p.ldr + n0);
    thread_off = (unsigned)(((threadIdx.x / GROUPS) * p.ldr + (threadIdx.x % GROUPS) * 8) * sizeof(T));
  }
  // Item `it` of pass a is tile row (RPI*it/32)*WM + a*32 + (RPI*it)%32 + threadIdx/GROUPS: a uniform row offset
  // (scalar address arithmetic) plus the per-thread offset.
  __device__ __forceinline__ void load_item(const GemmParams& p, int a, int it, raw8 (&dst)[NLOAD]) const {
    const int rowoff = (RPI * it / 32) * WM + a * 32 + (RPI * it) % 32;
    const char* r = base + (int64_t)rowoff * p.ldr * (int64_t)sizeof(T);
    dst[0] = load8_stream<T>(r + thread_off);
    if (NLOAD == 2) dst[1] = load8_stream<T>(r + p.aux_off * (int64_t)sizeof(T) + thread_off);
  }
  template <int BUF>
  __device__ __forceinline__ void fetch(const GemmParams& p, int a) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) load_item(p, a, it, pre[BUF][it]);
  }
};

// Epilogue shared by every main loop.  acc[a][b][4*j+i] is C[m0 + wm*WM + a*32 + 8*j + 4*(l/32) + i][wave column
// b*32 + l%32].  Pass a: every wave parks its a-th 32-row sub-tile in LDS (fp32, [(BM/WM)*32 rows][BN + 8]), then
// the block walks the pass in 8-column groups.  The caller guarantees that no wave still reads operands from LDS.
template <typename T, typename TO, int EPI, int BM, int BN, int WM, int WN, int NTHREADS, bool MI16 = false>
__device__ __forceinline__ void run_epilogue(const GemmParams& p, f32x16 (&acc)[WM / 32][WN / 32], unsigned char* smem_raw,
                                             int64_t m0, int64_t n0, int wm, int wn, int slice,
                                             EpiPre<T, EPI, BM, BN, WM, NTHREADS>& ep) {
  constexpr int MT = WM / 32, NT = WN / 32;
  constexpr bool DUAL = (EPI == MVIT_EPI_SWIGLU);
  const int l = threadIdx.x & 63;
  // MI16: acc[a][b] holds the four 16x16 results of the 32x32 block, [(ra*2 + cb)*4 + i] = C[16*ra + 4*(l/16) + i][16*cb + l%16]
  // Staging rows are BN floats with no padding; 16-column chunks of a row are permuted by the row instead, so that the
  // rows one parking store touches (4 apart: four of them with the 16x16 results, two with the 32x32 ones) fall on
  // different banks.  Groups of 8 columns stay contiguous for the read-out.
  constexpr int SP = BN;
  auto swz = [](int row) { return MI16 ? ((row >> 2) & 3) << 4 : ((row >> 2) & 1) << 5; };
  constexpr int PASS_ROWS = (BM / WM) * 32;
  constexpr int NCOLS = DUAL ? BN / 2 : BN;
  constexpr int GROUPS = NCOLS / 8;
  float* stage = reinterpret_cast<float*>(smem_raw);
  const int lc = l & 31, lr = 4 * (l >> 5);
  const bool to_ws = (EPI == MVIT_EPI_NONE) && p.split_k > 1;
  float* ws = to_ws ? p.workspace + (int64_t)slice * p.M * p.N : nullptr;
  const bool ws_vec = (p.N % 4 == 0);
  // SWIGLU_BWD can hand back the column sums of dg | du (the bias gradient): a thread's items all lie in the same
  // 8 columns, so it keeps 2 x 8 running sums; after the last pass the rows-of-threads are added through LDS.
  constexpr bool CAN_CS = (EPI == MVIT_EPI_SWIGLU_BWD) && NTHREADS % GROUPS == 0 && NTHREADS == 2 * GROUPS * 8;
  float cs_acc[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) cs_acc[e] = 0.f;
  const bool do_cs = CAN_CS && p.colsum != nullptr;
  auto finish_colsum = [&]() {
    if constexpr (CAN_CS) {
      if (!do_cs) return;
      constexpr int TR_ = NTHREADS / GROUPS;  // thread rows sharing a column group
      __syncthreads();                        // the staging area is free
      float* red = stage;                     // [TR_][2][GROUPS * 8]
      const int trow = threadIdx.x / GROUPS, cgx = threadIdx.x % GROUPS;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        red[(trow * 2 + 0) * (GROUPS * 8) + cgx * 8 + e] = cs_acc[e];
        red[(trow * 2 + 1) * (GROUPS * 8) + cgx * 8 + e] = cs_acc[8 + e];
      }
      __syncthreads();
      const int half = threadIdx.x / (GROUPS * 8), col = threadIdx.x % (GROUPS * 8);  // NTHREADS == 2 * GROUPS * 8
      float t = 0.f;
#pragma unroll
      for (int k = 0; k < TR_; ++k) t += red[(k * 2 + half) * (GROUPS * 8) + col];
      if (n0 + col < p.N) p.colsum[(m0 / BM) * p.ldc + (half ? p.aux_off : 0) + n0 + col] = t;
    }
  };

  // Tiles inside the matrix: compile-time trip counts, no edge tests, 16-byte accesses only.  When the epilogue
  // reads one value per output element, those reads run up to two passes ahead, so their latency hides behind
  // the LDS staging and the previous passes' arithmetic and stores.
  using EP = EpiPre<T, EPI, BM, BN, WM, NTHREADS>;
  if constexpr ((PASS_ROWS * GROUPS) % NTHREADS == 0) {
    const bool interior = m0 + BM <= p.M && n0 + NCOLS <= p.N && (to_ws ? ws_vec : p.vec_ok != 0) && (!EP::HAS_IN || ep.active);
    if (interior) {
      constexpr int ITEMS = PASS_ROWS * GROUPS / NTHREADS;
      constexpr int NBUF = EP::NBUF;
      // a thread's items all lie in one 8-column group (NTHREADS is a multiple of GROUPS): its bias values are loaded
      // once per tile, before the accumulators are parked, instead of once per item behind the previous items' stores
      // (memory instructions of a wave complete in order, so a load issued after a store also waits for that store)
      constexpr bool HAS_BIAS = EPI == MVIT_EPI_BIAS || EPI == MVIT_EPI_BIAS_RES || EPI == MVIT_EPI_BIAS_GELU || EPI == MVIT_EPI_SWIGLU;
      static_assert(NTHREADS % GROUPS == 0, "a thread's items share their column group");
      float hb[8], hb2[8];
      if constexpr (HAS_BIAS) {
        const int64_t nb = n0 + (threadIdx.x % GROUPS) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) hb[e] = hb2[e] = 0.f;
        if (p.bias) load8(static_cast<const T*>(p.bias) + nb, hb);
        if (DUAL && p.bias2) load8(static_cast<const T*>(p.bias2) + nb, hb2);
      }
      if constexpr (EP::HAS_IN) {
        ep.template fetch<0>(p, 0);
        if (NBUF == 2 && MT > 1) ep.template fetch<(NBUF - 1)>(p, 1);
      }
#pragma unroll
      for (int a = 0; a < MT; ++a) {
        if (a > 0) __syncthreads();
#pragma unroll
        for (int b = 0; b < NT; ++b) {
          int col;
          if (DUAL) col = (b / (NT / 2)) * (BN / 2) + wn * (WN / 2) + (b % (NT / 2)) * 32 + lc;
          else col = wn * WN + b * 32 + lc;
          if constexpr (MI16) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
              for (int i = 0; i < 4; ++i)
                stage[(wm * 32 + 16 * (q >> 1) + 4 * (l >> 4) + i) * SP + (((col - lc) + 16 * (q & 1) + (l & 15)) ^ swz(4 * (l >> 4)))] = acc[a][b][4 * q + i];
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
              for (int i = 0; i < 4; ++i) stage[(wm * 32 + 8 * j + lr + i) * SP + (col ^ swz(lr))] = acc[a][b][4 * j + i];
          }
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
          const int c = threadIdx.x + NTHREADS * it, row = c / GROUPS, cg = c % GROUPS;
          const int64_t m = m0 + (row / 32) * WM + a * 32 + (row % 32), n = n0 + cg * 8;
          const float* sp = stage + row * SP + ((cg * 8) ^ swz(row));
          const f32x4 v0 = *reinterpret_cast<const f32x4*>(sp), v1 = *reinterpret_cast<const f32x4*>(sp + 4);
          float v[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
          float u[8];
          if (DUAL) {
            const f32x4 u0 = *reinterpret_cast<const f32x4*>(sp + BN / 2), u1 = *reinterpret_cast<const f32x4*>(sp + BN / 2 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              u[e] = u0[e];
              u[4 + e] = u1[e];
            }
          }
          if (to_ws) store8_cached(ws + m * p.N + n, v);
          else if constexpr (EP::HAS_IN) {
            // the same item of pass a + NBUF is requested before this item's stores are issued: a wave's memory
            // instructions complete in order, so the wait for a load also waits for every store issued before it
            typename EP::raw8 nx[EP::NLOAD];
            if (a + NBUF < MT) ep.load_item(p, a + NBUF, it, nx);
            emit8_impl<T, TO, EPI, true, true>(p, m, n, v, u, ep.pre[a % NBUF][it], cs_acc, do_cs, HAS_BIAS ? hb : nullptr, nullptr);
            if (a + NBUF < MT) {
#pragma unroll
              for (int k = 0; k < EP::NLOAD; ++k) ep.pre[a % NBUF][it][k] = nx[k];
            }
            if constexpr (EP::NLOAD == 2) __builtin_amdgcn_sched_barrier(0);  // keeps the items apart: registers
          } else emit8_impl<T, TO, EPI, true, false>(p, m, n, v, u, nullptr, cs_acc, false, HAS_BIAS ? hb : nullptr, (HAS_BIAS && DUAL) ? hb2 : nullptr);
        }
      }
      finish_colsum();
      return;
    }
  }
#pragma unroll
  for (int a = 0; a < MT; ++a) {
    if (a > 0) __syncthreads();
#pragma unroll
    for (int b = 0; b < NT; ++b) {
      int col;
      if (DUAL) col = (b / (NT / 2)) * (BN / 2) + wn * (WN / 2) + (b % (NT / 2)) * 32 + lc;
      else col = wn * WN + b * 32 + lc;
      if constexpr (MI16) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            stage[(wm * 32 + 16 * (q >> 1) + 4 * (l >> 4) + i) * SP + (((col - lc) + 16 * (q & 1) + (l & 15)) ^ swz(4 * (l >> 4)))] = acc[a][b][4 * q + i];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) stage[(wm * 32 + 8 * j + lr + i) * SP + (col ^ swz(lr))] = acc[a][b][4 * j + i];
      }
    }
    __syncthreads();
    for (int c = threadIdx.x; c < PASS_ROWS * GROUPS; c += NTHREADS) {
      const int row = c / GROUPS, cg = c % GROUPS;
      const int64_t m = m0 + (row / 32) * WM + a * 32 + (row % 32);
      const int64_t n = n0 + cg * 8;
      if (m >= p.M || n >= p.N) continue;
      float v[8], u[8];
      const float* sp = stage + row * SP + ((cg * 8) ^ swz(row));
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(sp), v1 = *reinterpret_cast<const f32x4*>(sp + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = v0[e];
        v[4 + e] = v1[e];
      }
      if (DUAL) {
        const f32x4 u0 = *reinterpret_cast<const f32x4*>(sp + BN / 2), u1 = *reinterpret_cast<const f32x4*>(sp + BN / 2 + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          u[e] = u0[e];
          u[4 + e] = u1[e];
        }
      }
      if (to_ws) {
        float* w = ws + m * p.N + n;
        if (ws_vec && n + 8 <= p.N) store8_cached(w, v);
        else
          for (int e = 0; e < 8 && n + e < p.N; ++e) w[e] = v[e];
      } else {
        emit8<T, TO, EPI>(p, m, n, v, u, p.vec_ok != 0, cs_acc, do_cs);
      }
    }
  }
  finish_colsum();
}

template <typename T, typename TO, bool TA, bool TB, int EPI, int VAR>
__global__ __launch_bounds__(Waves<VAR>::NTHREADS, Waves<VAR>::MIN_WAVES) void gemm_kernel(const GemmParams p) {
  using C = Cfg<T>;
  using W = Waves<VAR>;
  constexpr int BK = C::BK, BM = W::BM, BN = W::BN, WM = W::WM, WN = W::WN, NTHREADS = W::NTHREADS;
  constexpr int MT = WM / 32, NT = WN / 32, WGN = BN / WN;  // waves along N
  constexpr bool DUAL = (EPI == MVIT_EPI_SWIGLU);
  using LoaderA = TileLoader<T, BM, TA, NTHREADS, WN, false>;
  using LoaderB = TileLoader<T, BN, TB, NTHREADS, WN, DUAL>;
  constexpr int STAGE_ELEMS = LoaderA::LDS_ELEMS + LoaderB::LDS_ELEMS;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* lds = reinterpret_cast<T*>(smem_raw);

  // XCD-aware tile order: hardware deals consecutive work-group ids round-robin to the 8 XCDs; give each
  // XCD a contiguous range of tiles (N fastest) so that its L2 sees one A panel at a time.
  // With split-K the slices are the slowest index: all tiles of one K slice share the same rows of A and B.
  const int tiles = p.tiles_m * p.tiles_n;
  const int total = tiles * p.split_k;
  const int per_xcd = (total + 7) / 8;
  const int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (work >= total) return;
  const int slice = work / tiles, tile = work % tiles;
  int tm, tn;
  tile_coords(p, tile, tm, tn);
  const int64_t k_begin = (int64_t)slice * p.k_chunk;
  const int64_t k_end = p.split_k > 1 ? (k_begin + p.k_chunk < p.K ? k_begin + p.k_chunk : p.K) : p.K;
  constexpr int N_PER_BLOCK = DUAL ? BN / 2 : BN;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * N_PER_BLOCK;

  const int l = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int wm = wv / WGN, wn = wv % WGN;

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
  la.init(A, nullptr, p.lda, m0, p.M, k_begin, k_end);
  lb.init(B, B2, p.ldb, n0, p.N, k_begin, k_end);
  la.load();
  lb.load();
  la.store(lds);
  lb.store(lds + LoaderA::LDS_ELEMS);
  __syncthreads();

  int buf = 0;
  for (int64_t k0 = k_begin; k0 < k_end; k0 += BK) {
    const bool has_next = k0 + BK < k_end;
    if (has_next) {
      la.load();
      lb.load();
    }
    const T* lds_a = lds + buf * STAGE_ELEMS;
    const T* lds_b = lds_a + LoaderA::LDS_ELEMS;
    if constexpr (sizeof(T) == 2) {
      // operand fragments are fetched one 16-wide step ahead of the MFMAs that consume them
      const bf16_t* la_ = reinterpret_cast<const bf16_t*>(lds_a);
      const bf16_t* lb_ = reinterpret_cast<const bf16_t*>(lds_b);
      bf16x8 fa[2][MT], fb[2][NT];
#pragma unroll
      for (int a = 0; a < MT; ++a) fa[0][a] = frag_bf16<TA, BM>(la_, wm * WM + a * 32, 0);
#pragma unroll
      for (int b = 0; b < NT; ++b) fb[0][b] = frag_bf16<TB, BN>(lb_, wn * WN + b * 32, 0);
#pragma unroll
      for (int s4 = 0; s4 < BK / 16; ++s4) {
        const int cur = s4 & 1, nxt = cur ^ 1;
        if (s4 + 1 < BK / 16) {
#pragma unroll
          for (int a = 0; a < MT; ++a) fa[nxt][a] = frag_bf16<TA, BM>(la_, wm * WM + a * 32, (s4 + 1) * 16);
#pragma unroll
          for (int b = 0; b < NT; ++b) fb[nxt][b] = frag_bf16<TB, BN>(lb_, wn * WN + b * 32, (s4 + 1) * 16);
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the fetches of step s4+1 ahead of the MFMAs of step s4
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
          for (int b = 0; b < NT; ++b)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][a], fb[cur][b], acc[a][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < BK; ks += 2) {
        float fa[MT], fb[NT];
#pragma unroll
        for (int a = 0; a < MT; ++a) fa[a] = frag_f32<TA, BM>(reinterpret_cast<const float*>(lds_a), wm * WM + a * 32, ks);
#pragma unroll
        for (int b = 0; b < NT; ++b) fb[b] = frag_f32<TB, BN>(reinterpret_cast<const float*>(lds_b), wn * WN + b * 32, ks);
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
          for (int b = 0; b < NT; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a], fb[b], acc[a][b], 0, 0, 0);
      }
    }
    if (has_next) {
      T* nxt = lds + (buf ^ 1) * STAGE_ELEMS;
      la.store(nxt);
      lb.store(nxt + LoaderA::LDS_ELEMS);
    }
    __syncthreads();  // also: operands fully consumed before LDS is reused by the epilogue
    buf ^= 1;
  }

  EpiPre<T, EPI, BM, BN, WM, NTHREADS> ep;
  ep.init(p, m0, n0);
  run_epilogue<T, TO, EPI, BM, BN, WM, WN, NTHREADS>(p, acc, smem_raw, m0, n0, wm, wn, slice, ep);
}

// ---- bf16 main loop with direct global -> LDS loads (no staging registers) ----------------------------------
// 256x256 tile, 8 waves of 128x64, BK = 32, NSTAGE LDS stages of 16 KiB per operand.  global_load_lds_dwordx4 moves
// 16 bytes per lane straight into LDS at M0 + 16*lane, so one wave instruction fills 1 KiB of contiguous LDS and
// NSTAGE-1 K tiles are in flight while one is consumed; addresses are a per-lane 32-bit offset (constant over the
// K loop) plus a wave-uniform 64-bit base that a scalar add advances.  Because the LDS image of one instruction
// is contiguous, bank conflicts are avoided by permuting which global chunk a lane fetches:
//   [row][k] operands: 64-byte rows of 4 chunks, chunk c of row r lives in slot c ^ ((r >> 2) & 3);
//   [k][row] operands: 512-byte k-rows of 32 chunks, chunk c of k-row k lives in slot c ^ ((k & 3) << 2).
// Rows past the matrix edge are clamped to valid rows (they only feed outputs that are never stored).  A partial
// last K tile (K not a multiple of 32) is loaded through registers with zeros past the end of K.
// The compiler does not see these loads: s_waitcnt vmcnt is placed by hand (loads return in order).
// waves per work-group: 8 -> each owns 128x64 (two waves per SIMD), 4 -> 128x128 (one per SIMD).  BM_ = 128: an output
// tile of half the height for products whose 256-row tiles would leave most compute units idle: the eight waves own
// 64x64 each, the A stage holds 128 rows (in the first half of its 16 KiB slot), everything an output element sees
// (K order, MFMA form, epilogue arithmetic) is unchanged, so results are bit-identical to the 256-row tile's.
template <int NW, int BM_ = 256>
struct DL {
  static_assert(BM_ == 256 || (BM_ == 128 && NW == 8), "tile heights built: 256, and 128 with eight waves");
  static constexpr int BM = BM_, BN = 256, BK = 32, WM = BM_ / 2, WN = NW == 8 ? 64 : 128, NTHREADS = 64 * NW;
  static constexpr int TILE_BYTES = 256 * BK * 2;
  static constexpr int CPT = 16 / NW;          // 1 KiB load instructions per wave and K tile for a 256-row operand stage
  static constexpr int CPT_A = BM_ / 16 / NW;  // ... for the A stage of this tile height
};
constexpr int DL_BK = 32, DL_TILE_BYTES = 256 * DL_BK * 2;

__device__ __forceinline__ void dl_load(unsigned lds_addr, unsigned voff, const char* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <bool TR, bool DUAL, int NW, bool MI16 = false, int ROWS = 256>
struct DlOperand {
  static_assert(ROWS == 256 || !TR, "a [k][row] stage is always 256 rows wide");
  static constexpr int CPT = ROWS / 16 / NW, WN = DL<NW>::WN;
  unsigned voff[CPT];  // byte offset of this lane's 16-byte chunks from `base`
  const char* base;    // wave-uniform, advanced by `step` every K tile (DUAL: odd waves read the second matrix)
  int64_t step;

  __device__ __forceinline__ void init(const bf16_t* X, const bf16_t* X2, int64_t ld, int64_t row0, int64_t limit,
                                       int64_t k_begin, int wv) {
    const int l = threadIdx.x & 63;
    step = TR ? 2 * DL_BK * ld : 2 * DL_BK;
    // DUAL: tile row r = wn*WN + half*(WN/2) + j -> matrix `half`, row row0 + wn*(WN/2) + j; a wave's rows
    // [wv * 16 * CPT, +16 * CPT) all have half = wv & 1.
    const bf16_t* src = (DUAL && (wv & 1)) ? X2 : X;
    base = reinterpret_cast<const char*>(TR ? src + k_begin * ld + row0 : src + row0 * ld + k_begin);
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int q = wv * CPT + i;  // which 1 KiB of the stage this instruction fills
      if (!TR) {
        const int r = q * 16 + (l >> 2), c = (l & 3) ^ ((r >> 2) & 3);
        int64_t grow = row0 + r;
        if (DUAL) grow = row0 + (r / WN) * (WN / 2) + (r % (WN / 2));
        if (grow >= limit) grow = limit - 1;
        voff[i] = (unsigned)(((grow - row0) * ld + c * 8) * 2);
      } else {
        const int kr = 2 * q + (l >> 5);
        // MI16: the four 16-lane groups of a transposing read sit 8 k-rows apart; odd multiples of 8 are moved
        // by two chunks so that two neighbouring groups never share banks
        int ch = (l & 31) ^ ((kr & 3) << 2) ^ (MI16 ? ((kr >> 3) & 1) << 1 : 0);
        if (row0 + ch * 8 >= limit) ch = 0;
        voff[i] = (unsigned)((kr * ld + ch * 8) * 2);
      }
    }
  }
  // lds_addr: LDS byte address of this wave's CPT KiB slice of the operand's stage
  __device__ __forceinline__ void issue(unsigned lds_addr) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) dl_load(lds_addr + i * 1024, voff[i], base);
    base += step;
  }
  __device__ __forceinline__ void issue_tail(unsigned char* lds_slice, int k_rem, int wv) {
    const int l = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int q = wv * CPT + i;
      int k;  // first contraction index of the chunk
      if (!TR) {
        const int r = q * 16 + (l >> 2);
        k = ((l & 3) ^ ((r >> 2) & 3)) * 8;
      } else {
        k = 2 * q + (l >> 5);
      }
      bf16x8 v;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = from_f32<bf16_t>(0.f);
      if (k < k_rem) v = *reinterpret_cast<const bf16x8*>(base + voff[i]);
      *reinterpret_cast<bf16x8*>(lds_slice + i * 1024 + l * 16) = v;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // written before this wave's next barrier
  }
};

// The loader of that operand for the DL layout: this operand cannot travel global -> LDS directly, so a K tile takes two calls, a step of the main loop apart:
// request() loads this lane's 8 bytes of each of its CPT rows into registers, flush() converts them and writes the 16-byte
// chunk where the direct load of a [row][k] operand would have put it (slot l of the wave's 1 KiB slice holds chunk
// (l & 3) ^ ((row >> 2) & 3) of row 16 * slice + l / 4).  A K tile of 32 is 4 pieces, so pieces advance by 4 per tile.
template <int NW>
struct DlPixelOperand {
  static constexpr int CPT = DL<NW>::CPT;
  static_assert(PX_K % DL_BK == 0, "whole K tiles");
  const uint8_t* base[CPT];
  int line_bytes[CPT], frame_off[CPT];
  int line, piece;  // of the next request
  int ch0;          // channel of the first byte of the piece that the next flush converts
  PxRaw raw[CPT];

  __device__ __forceinline__ void init(const GemmParams& p, int64_t row0, int wv) {
    const int l = threadIdx.x & 63;
    line = 0;
    piece = (l & 3) ^ ((l >> 4) & 3);  // (row >> 2) & 3 = (l >> 4) & 3: slices start at multiples of 16 rows
    ch0 = (2 * piece) % 3;
#pragma unroll
    for (int i = 0; i < CPT; ++i) px_locate(p, row0 + (wv * CPT + i) * 16 + (l >> 2), base[i], line_bytes[i], frame_off[i]);
  }
  __device__ __forceinline__ void request() {
    const int second = line >= PX_PATCH ? 1 : 0, y = line - PX_PATCH * second;
    const int in_line = piece == 5 ? 8 * 5 - 6 : 8 * piece;  // the last piece is read as the last 8 bytes of the line
#pragma unroll
    for (int i = 0; i < CPT; ++i) px_fetch8(base[i] + ((second ? frame_off[i] : 0) + y * line_bytes[i] + in_line), raw[i]);
    piece += 4;
    if (piece >= 6) {
      piece -= 6;
      line += 1;
    }
  }
  // lds_slice: this wave's CPT KiB of the operand's stage.  The write is complete before the wave's next barrier
  // because the fragment reads that follow it in program order are (LDS operations of a wave complete in order).
  __device__ __forceinline__ void flush(unsigned char* lds_slice, const PxNorm nm) {
    const int l = threadIdx.x & 63;
    const bool tail = piece == 3;  // the piece in registers is 4 pieces (mod 6) before the next request's
#pragma unroll
    for (int i = 0; i < CPT; ++i) *reinterpret_cast<bf16x8*>(lds_slice + i * 1024 + l * 16) = px_convert8(raw[i], ch0, tail, nm);
    ch0 = ch0 == 0 ? 2 : ch0 - 1;  // 32 bytes further: + 2 mod 3 (a wrap to the next line moves by 48 = 0 mod 3)
  }
};

// MFMA operand fetch for the DL layout: sub-tile `a` (32 rows) of the wave, 16-wide contraction step ks, stage s.
template <bool TR, int NSUB, bool MI16 = false>
struct DlFrag {
  unsigned off[MI16 ? (TR ? 2 * NSUB : 1) : (TR ? NSUB : 2)];
  __device__ __forceinline__ void init(int rowbase, unsigned region) {
    const int l = threadIdx.x & 63;
    if constexpr (MI16) {
      // v_mfma_f32_16x16x32 operand: lane l holds row l%16 of a 16-row block, contraction 8*(l/16) .. +7 of the 32-wide stage
      if (!TR) {
        const int r = rowbase + (l & 15);  // blocks are 16 rows apart: (r >> 2) & 3 is the same for every block
        off[0] = region + r * 64 + (((l >> 4) ^ ((r >> 2) & 3)) << 4);
      } else {
        const int G = l >> 4, i = l & 15, k = 8 * G + (i >> 2);
#pragma unroll
        for (int a = 0; a < 2 * NSUB; ++a) {
          const int ch = (rowbase + a * 16) / 8 + ((i & 3) >> 1);
          off[a] = region + k * 512 + ((ch ^ ((k & 3) << 2) ^ (((k >> 3) & 1) << 1)) << 4) + (i & 1) * 8;
        }
      }
      return;
    }
    if (!TR) {
      const int x = ((l & 31) >> 2) & 3;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) off[ks] = region + (rowbase + (l & 31)) * 64 + (((ks * 2 + (l >> 5)) ^ x) << 4);
    } else {
      // lane i of 16-lane group G fetches 4 rows of k-row 8*(G/2) + i/4 at row 16*(G%2) + 4*(i%4); the transposing
      // read hands lane j of the group the 4 consecutive k of row 16*(G%2) + j.
      const int G = l >> 4, i = l & 15;
#pragma unroll
      for (int a = 0; a < NSUB; ++a) {
        const int ch = (rowbase + a * 32) / 8 + 2 * (G & 1) + ((i & 3) >> 1);
        off[a] = region + (8 * (G >> 1) + (i >> 2)) * 512 + ((ch ^ (((i >> 2) & 3) << 2)) << 4) + (i & 1) * 8;
      }
    }
  }
  // MI16: fragment of the 16-row block `blk` of the wave for the whole 32-wide stage s
  __device__ __forceinline__ bf16x8 read16(const unsigned char* smem, int blk, int s) const {
    if (!TR) {
      return *reinterpret_cast<const bf16x8*>(smem + off[0] + blk * 16 * 64 + s * DL_TILE_BYTES);
    } else {
      typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
      const unsigned char* p = smem + off[blk] + s * DL_TILE_BYTES;
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p + 4 * 512));
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      return __builtin_bit_cast(bf16x8, both);
    }
  }
  __device__ __forceinline__ bf16x8 read(const unsigned char* smem, int a, int ks, int s) const {
    if (!TR) {
      return *reinterpret_cast<const bf16x8*>(smem + off[ks] + a * 32 * 64 + s * DL_TILE_BYTES);
    } else {
      typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
      const unsigned char* p = smem + off[a] + s * DL_TILE_BYTES + ks * 16 * 512;
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p + 4 * 512));
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      return __builtin_bit_cast(bf16x8, both);
    }
  }
};

// Whether gemm_dl_kernel starts the next tile's loads before the epilogue of the current one: the weight-gradient
// GEMMs (A transposed) with a plain or bias epilogue.  Measured on the full tower: those kernels get 2-3 % faster and
// the step follows; the forward and input-gradient GEMMs also get 1-3 % faster alone, but the step with the
// weight gradients running beside them on a second stream gets slower, so they keep starting a tile after the
// epilogue.  The fused epilogues have no registers to spare for the next tile's addresses.
constexpr bool dl_prefetches(int epi, bool ta) { return (epi == MVIT_EPI_NONE || epi == MVIT_EPI_BIAS) && ta; }

// Wait until at most n K tiles' loads (PER per lane each) are still in flight.
template <int PER>
__device__ __forceinline__ void wait_tiles(int n) {
  if (n >= 3) wait_vm<3 * PER>();
  else if (n == 2) wait_vm<2 * PER>();
  else if (n == 1) wait_vm<PER>();
  else wait_vm<0>();
}

// PIX: the A operand is made from decoded frames (DlPixelOperand)
template <typename TO, bool TA, bool TB, int EPI, int NSTAGE, int NW, bool MI16 = false, bool PIX = false, int BM_ = 256>
__global__ __launch_bounds__(64 * NW, NW / 4) void gemm_dl_kernel(const GemmParams p) {
  static_assert(!PIX || (!TA && !MI16 && !dl_prefetches(EPI, TA)), "frames as the A operand: [row][k] layout, 32x32x16 fragments, no early loads");
  static_assert(BM_ == 256 || (!TA && !PIX && EPI != MVIT_EPI_SWIGLU_BWD), "half-height tiles: A in [row][k] layout, no per-256-row column sums");
  using T = bf16_t;
  using D = DL<NW, BM_>;
  constexpr int BM = D::BM, BN = D::BN, WM = D::WM, WN = D::WN, TILE = D::TILE_BYTES, SLICE = D::CPT * 1024, SLICE_A = D::CPT_A * 1024;
  constexpr int MT = WM / 32, NT = WN / 32, WGN = BN / WN;
  constexpr bool DUAL = (EPI == MVIT_EPI_SWIGLU);
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

  const int tiles = p.tiles_m * p.tiles_n;
  const int total = tiles * p.split_k;
  const int per_xcd = (total + 7) / 8;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wv / WGN, wn = wv % WGN;
  DlFrag<TA, MT, MI16> ra;
  DlFrag<TB, NT, MI16> rb;
  ra.init(wm * WM, 0);
  rb.init(wn * WN, NSTAGE * TILE);
  typedef __attribute__((address_space(3))) unsigned char lds_byte;
  const unsigned lds0 = (unsigned)(__UINTPTR_TYPE__)(lds_byte*)smem_raw + wv * SLICE;      // this wave's slice of a B stage
  const unsigned lds0a = (unsigned)(__UINTPTR_TYPE__)(lds_byte*)smem_raw + wv * SLICE_A;   // ... of an A stage

  // Persistent work-groups: the grid has at most one work-group per CU; work-group (xcd, slot) walks that XCD's
  // tile range with stride slots-per-XCD, the order a one-tile-per-work-group grid would be dispatched in.
  // Where dl_prefetches() says so, the first two K tiles of a work-group's next output tile are requested before the
  // epilogue of the current one, so they travel while the results are parked and stored: the epilogue then stages
  // through the later B stages and the LDS behind them, which those loads do not touch.
  constexpr bool PREFETCH = dl_prefetches(EPI, TA);
  constexpr int EARLY = PREFETCH ? (NSTAGE - 1 < 2 ? NSTAGE - 1 : 2) : NSTAGE - 1;  // K tiles requested by start_tile
  constexpr int STAGING_OFF = PREFETCH ? (NSTAGE + EARLY) * TILE : 0;
  typename std::conditional<PIX, DlPixelOperand<NW>, DlOperand<TA, false, NW, MI16, BM>>::type la;
  DlOperand<TB, DUAL, NW, MI16> lb;
  int T_ = 0, k_tail = 0;  // of the tile whose operands are being loaded
  [[maybe_unused]] int px_pending = -1;  // PIX: stage whose A bytes are in registers, requested by the previous issue()
  [[maybe_unused]] const PxNorm px_norm(p);
  const bool px_late = PIX && wv >= NW / 2;
  auto issue = [&](int t, int s) {  // K tile t into stage s (both wave-uniform)
    if constexpr (PIX) {
      // the A bytes requested one call ago are converted and written now (their K tile is read two barriers from here),
      // then K tile t is requested: B straight into LDS, A into registers
      if (px_pending >= 0) la.flush(smem_raw + px_pending * TILE + wv * SLICE_A, px_norm);
      px_pending = -1;
      if (t >= T_) return;
      lb.issue(lds0 + (NSTAGE + s) * TILE);
      la.request();
      px_pending = s;
    } else {
      if (t >= T_) return;
      if (k_tail != 0 && t == T_ - 1) {
        la.issue_tail(smem_raw + s * TILE + wv * SLICE_A, k_tail, wv);
        lb.issue_tail(smem_raw + (NSTAGE + s) * TILE + wv * SLICE, k_tail, wv);
      } else {
        la.issue(lds0a + s * TILE);
        lb.issue(lds0 + (NSTAGE + s) * TILE);
      }
    }
  };
  constexpr int N_PER_BLOCK = DUAL ? BN / 2 : BN;
  int next_slice = 0;
  int64_t next_m0 = 0, next_n0 = 0;
  // decodes work item `idx` of this work-group's XCD and starts its first loads; false past the end
  auto start_tile = [&](int idx) -> bool {
    if (idx >= per_xcd) return false;
    const int work = (blockIdx.x & 7) * per_xcd + idx;
    if (work >= total) return false;
    next_slice = work / tiles;
    int tm, tn;
    tile_coords(p, work % tiles, tm, tn);
    const int64_t k_begin = (int64_t)next_slice * p.k_chunk;
    const int64_t k_end = p.split_k > 1 ? (k_begin + p.k_chunk < p.K ? k_begin + p.k_chunk : p.K) : p.K;
    next_m0 = (int64_t)tm * BM;
    next_n0 = (int64_t)tn * N_PER_BLOCK;
    if constexpr (PIX) la.init(p, next_m0, wv);
    else la.init(static_cast<const T*>(p.A), nullptr, p.lda, next_m0, p.M, k_begin, wv);
    lb.init(static_cast<const T*>(p.B), static_cast<const T*>(p.B2), p.ldb, next_n0, p.N, k_begin, wv);
    const int klen = (int)(k_end - k_begin);
    T_ = (klen + DL_BK - 1) / DL_BK;
    k_tail = klen % DL_BK;
#pragma unroll
    for (int t = 0; t < EARLY; ++t) issue(t, t);
    return true;
  };
  int idx = blockIdx.x >> 3;
  [[maybe_unused]] bool have = PREFETCH ? start_tile(idx) : true;
  while (true) {
  if constexpr (PREFETCH) {
    if (!have) break;
  } else {
    if (!start_tile(idx)) break;
  }
  const int slice = next_slice;
  const int64_t m0 = next_m0, n0 = next_n0;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int a = 0; a < MT; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

  EpiPre<T, EPI, BM, BN, WM, D::NTHREADS> ep;
  ep.init(p, m0, n0);
#pragma unroll
  for (int t = EARLY; t < NSTAGE - 1; ++t) issue(t, t);  // the stages the previous tile's epilogue was using

  [[maybe_unused]] bf16x8 fa[2][MT], fb[2][NT];
  for (int t0 = 0; t0 < T_; t0 += NSTAGE) {
#pragma unroll
    for (int s = 0; s < NSTAGE; ++s) {
      const int t = t0 + s;
      if (t >= T_) break;
      // tile t has landed once only the tiles issued after it are pending
      const int rem = T_ - 1 - t;
      constexpr int AHEAD = NSTAGE - 2;
      wait_tiles<D::CPT_A + D::CPT>(rem < 0 ? 0 : (rem < AHEAD ? rem : AHEAD));
      __builtin_amdgcn_s_barrier();  // every wave's share of that tile is in LDS; stage (s-1) has been consumed
      // PIX: the conversion of the A bytes is vector work of about the length of a K tile's MFMAs.  The two waves of a
      // SIMD (w and w + NW/2) do it at opposite ends of the step, one before its MFMAs and one after, so that one
      // wave's conversions run under the other's MFMAs.
      if (!px_late) issue(t + NSTAGE - 1, (s + NSTAGE - 1) % NSTAGE);

      if constexpr (MI16) {
        // one 32-wide step per stage on v_mfma_f32_16x16x32_bf16: 2*MT x 2*NT blocks of 16x16
        bf16x8 ga[2 * MT], gb[2 * NT];
#pragma unroll
        for (int a = 0; a < 2 * MT; ++a) ga[a] = ra.read16(smem_raw, a, s);
#pragma unroll
        for (int b = 0; b < 2 * NT; ++b) gb[b] = rb.read16(smem_raw, b, s);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int a = 0; a < 2 * MT; ++a)
#pragma unroll
          for (int b = 0; b < 2 * NT; ++b) {
            f32x16& blk = acc[a >> 1][b >> 1];
            const int q = (a & 1) * 2 + (b & 1);
            f32x4 c = {blk[4 * q], blk[4 * q + 1], blk[4 * q + 2], blk[4 * q + 3]};
            c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga[a], gb[b], c, 0, 0, 0);
            blk[4 * q] = c[0];
            blk[4 * q + 1] = c[1];
            blk[4 * q + 2] = c[2];
            blk[4 * q + 3] = c[3];
          }
        __builtin_amdgcn_sched_barrier(0);
      } else {
#pragma unroll
      for (int a = 0; a < MT; ++a) fa[0][a] = ra.read(smem_raw, a, 0, s);
#pragma unroll
      for (int b = 0; b < NT; ++b) fb[0][b] = rb.read(smem_raw, b, 0, s);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int a = 0; a < MT; ++a) fa[1][a] = ra.read(smem_raw, a, 1, s);
#pragma unroll
      for (int b = 0; b < NT; ++b) fb[1][b] = rb.read(smem_raw, b, 1, s);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NT; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0][a], fb[0][b], acc[a][b], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NT; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][a], fb[1][b], acc[a][b], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (PIX) {
        if (px_late) {
          issue(t + NSTAGE - 1, (s + NSTAGE - 1) % NSTAGE);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // no LDS read follows the write before the barrier
        }
      }
    }
  }
  __syncthreads();  // operands fully consumed before the next tile's first loads (or the epilogue) overwrite them
  idx += gridDim.x >> 3;
  if constexpr (PREFETCH) have = start_tile(idx);
  run_epilogue<T, TO, EPI, BM, BN, WM, WN, D::NTHREADS, MI16>(p, acc, smem_raw + STAGING_OFF, m0, n0, wm, wn, slice, ep);
  __syncthreads();  // the staging area is free again before operands land in it
  }
}

// C[m, n] = epilogue(sum over slices of the fp32 partial tiles) (fixed order, so the result is reproducible); the
// epilogue is none, + bias[n] or + bias[n] + R[m, n], in the order of the one-pass kernels' epilogue.
// VEC: four consecutive columns per thread (N, the pitches and the pointers allow vector accesses).
template <typename T, typename TO, bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int split_k, int64_t M, int64_t N,
                                                            TO* __restrict__ C, int64_t ldc, int epi, const T* __restrict__ bias,
                                                            const T* __restrict__ R, int64_t ldr) {
  const int64_t total = M * N;
  if constexpr (VEC) {
    const int64_t quads = total / 4, nq = N / 4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < quads; i += (int64_t)gridDim.x * 256) {
      f32x4 s = {0.f, 0.f, 0.f, 0.f};  // the same sum, from the same zero, as the scalar form
      for (int k = 0; k < split_k; ++k) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(ws + (int64_t)k * total + 4 * i);
        s = f32x4{s[0] + v[0], s[1] + v[1], s[2] + v[2], s[3] + v[3]};
      }
      const int64_t m = i / nq, n = (i % nq) * 4;
      if (epi != MVIT_EPI_NONE) {
        const auto b = *reinterpret_cast<const T __attribute__((ext_vector_type(4)))*>(bias + n);
        s = f32x4{s[0] + to_f32(b[0]), s[1] + to_f32(b[1]), s[2] + to_f32(b[2]), s[3] + to_f32(b[3])};
      }
      if (epi == MVIT_EPI_BIAS_RES) {
        const auto r = *reinterpret_cast<const T __attribute__((ext_vector_type(4)))*>(R + m * ldr + n);
        s = f32x4{s[0] + to_f32(r[0]), s[1] + to_f32(r[1]), s[2] + to_f32(r[2]), s[3] + to_f32(r[3])};
      }
      TO* c = C + m * ldc + n;
      if constexpr (sizeof(TO) == 2) *reinterpret_cast<bf16x4*>(c) = bf16x4{(bf16_t)s[0], (bf16_t)s[1], (bf16_t)s[2], (bf16_t)s[3]};
      else *reinterpret_cast<f32x4*>(c) = s;
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
      float s = 0.f;
      for (int k = 0; k < split_k; ++k) s += ws[(int64_t)k * total + i];
      const int64_t m = i / N, n = i % N;
      if (epi != MVIT_EPI_NONE) s += to_f32(bias[n]);
      if (epi == MVIT_EPI_BIAS_RES) s += to_f32(R[m * ldr + n]);
      C[m * ldc + n] = from_f32<TO>(s);
    }
  }
}
template <typename T, typename TO>
void launch_splitk_reduce(const GemmParams& p, hipStream_t stream) {
  const int64_t elems = p.M * p.N;
  const int epi = p.reduce_epi;
  const T* bias = static_cast<const T*>(p.bias);
  const T* R = static_cast<const T*>(p.R);
  bool vec = p.N % 4 == 0 && p.ldc % 4 == 0 && mvit_aligned16(p.workspace) && (reinterpret_cast<uintptr_t>(p.C) % (4 * sizeof(TO))) == 0;
  if (epi != MVIT_EPI_NONE) vec = vec && reinterpret_cast<uintptr_t>(bias) % (4 * sizeof(T)) == 0;
  if (epi == MVIT_EPI_BIAS_RES) vec = vec && p.ldr % 4 == 0 && reinterpret_cast<uintptr_t>(R) % (4 * sizeof(T)) == 0;
  const int64_t items = vec ? elems / 4 : elems;
  const int rgrid = (int)((items + 255) / 256 < 8192 ? (items + 255) / 256 : 8192);
  if (vec) hipLaunchKernelGGL((splitk_reduce_kernel<T, TO, true>), rgrid, 256, 0, stream, p.workspace, p.split_k, p.M, p.N, static_cast<TO*>(p.C), p.ldc, epi, bias, R, p.ldr);
  else hipLaunchKernelGGL((splitk_reduce_kernel<T, TO, false>), rgrid, 256, 0, stream, p.workspace, p.split_k, p.M, p.N, static_cast<TO*>(p.C), p.ldc, epi, bias, R, p.ldr);
}

template <typename T, typename TO, bool TA, bool TB, int EPI, int VAR>
int launch(const GemmParams& p, hipStream_t stream) {
  using W = Waves<VAR>;
  constexpr int BM = W::BM, BN = W::BN;
  using LA = TileLoader<T, BM, TA, W::NTHREADS, W::WN, false>;
  using LB = TileLoader<T, BN, TB, W::NTHREADS, W::WN, false>;
  const size_t operands = 2 * (size_t)(LA::LDS_ELEMS + LB::LDS_ELEMS) * sizeof(T);
  const size_t staging = (size_t)(BM / W::WM) * 32 * (BN + 8) * sizeof(float);
  const size_t lds = operands > staging ? operands : staging;
  auto kern = gemm_kernel<T, TO, TA, TB, EPI, VAR>;
  static bool attr_set_on[MVIT_MAX_DEVICES] = {};  // dynamic LDS above 64 KiB needs opting in once per kernel and device
  const int dev = mvit_current_device("gemm");
  if (dev < 0) return MVIT_ERR_LAUNCH;
  bool& attr_set = attr_set_on[dev];
  if (!attr_set && lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return mvit_set_error(MVIT_ERR_LAUNCH, "gemm: hipFuncSetAttribute(%zu B LDS): %s", lds, hipGetErrorString(e));
    attr_set = true;
  }
  if (p.split_k > 1 && EPI != MVIT_EPI_NONE) return mvit_set_error(MVIT_ERR_UNSUPPORTED, "gemm: split_k needs EPI_NONE");
  const int total = p.tiles_m * p.tiles_n * p.split_k;
  const int grid = ((total + 7) / 8) * 8;
  hipLaunchKernelGGL(kern, grid, W::NTHREADS, lds, stream, p);
  MVIT_CHECK_LAUNCH("gemm");
  if (p.split_k > 1) {
    launch_splitk_reduce<T, TO>(p, stream);
    MVIT_CHECK_LAUNCH("gemm split-k reduce");
  }
  return MVIT_OK;
}

// Compute units of the device (rounded down to a multiple of the 8 XCDs): persistent GEMM work-groups run one per unit.
int device_cu_count(int dev) {
  static int n_cu_on[MVIT_MAX_DEVICES] = {};
  int& n_cu = n_cu_on[dev];
  if (n_cu == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    n_cu = v / 8 * 8 > 0 ? v / 8 * 8 : 8;
  }
  return n_cu;
}

template <typename TO, bool TA, bool TB, int EPI, int NSTAGE, int NW, bool MI16 = false, bool PIX = false, int BM_ = 256>
int launch_dl(const GemmParams& p, hipStream_t stream) {
  using D = DL<NW, BM_>;
  constexpr size_t operands = 2 * (size_t)NSTAGE * D::TILE_BYTES;
  constexpr size_t staging = (size_t)(D::BM / D::WM) * 32 * D::BN * sizeof(float);
  // with prefetching the staging area starts behind the B stages that the next tile's first two K tiles arrive in
  constexpr size_t staging_end = dl_prefetches(EPI, TA) ? (NSTAGE + (NSTAGE - 1 < 2 ? NSTAGE - 1 : 2)) * D::TILE_BYTES + staging : staging;
  constexpr size_t lds = staging_end > operands ? staging_end : operands;
  static_assert(lds <= 160 * 1024, "operand stages plus the epilogue staging area exceed the LDS of a CU");
  auto kern = gemm_dl_kernel<TO, TA, TB, EPI, NSTAGE, NW, MI16, PIX, BM_>;
  static bool attr_set_on[MVIT_MAX_DEVICES] = {};  // once per kernel and device
  const int dev = mvit_current_device("gemm");
  if (dev < 0) return MVIT_ERR_LAUNCH;
  bool& attr_set = attr_set_on[dev];
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return mvit_set_error(MVIT_ERR_LAUNCH, "gemm: hipFuncSetAttribute(%zu B LDS): %s", lds, hipGetErrorString(e));
    attr_set = true;
  }
  if (p.split_k > 1 && EPI != MVIT_EPI_NONE) return mvit_set_error(MVIT_ERR_UNSUPPORTED, "gemm: split_k needs EPI_NONE");
  const int total = p.tiles_m * p.tiles_n * p.split_k;
  const int n_cu = device_cu_count(dev);
  const int want = ((total + 7) / 8) * 8;
  const int grid = want < n_cu ? want : n_cu;
  hipLaunchKernelGGL(kern, grid, D::NTHREADS, lds, stream, p);
  MVIT_CHECK_LAUNCH("gemm");
  if (p.split_k > 1) {
    launch_splitk_reduce<bf16_t, TO>(p, stream);
    MVIT_CHECK_LAUNCH("gemm split-k reduce");
  }
  return MVIT_OK;
}

template <typename T, typename TO, bool TA, bool TB, int EPI>
int launch_var(int var, const GemmParams& p, hipStream_t s) {
  if constexpr (sizeof(T) == 2) {
    // direct-to-LDS main loop: v_mfma_f32_16x16x32_bf16 for the plain GEMMs with an operand behind the transposing
    // LDS read (weight gradients +6 %, input gradients +1 % on real data), v_mfma_f32_32x32x16_bf16 for the forward
    // GEMMs (both operands row-major: 3-5 % faster that way) and for the fused backward epilogues
    constexpr int NS = 4;
    if (var == 3) return (TB && EPI == MVIT_EPI_NONE) ? launch_dl<TO, TA, TB, EPI, NS, 8, true>(p, s) : launch_dl<TO, TA, TB, EPI, NS, 8>(p, s);
  }
  return launch<T, TO, TA, TB, EPI, 1>(p, s);  // register-staged main loop: fp32, and bf16 operands whose row pitch exceeds 32-bit lane offsets
}

template <typename T, typename TO, bool TA, bool TB>
int dispatch_epi(int epi, int var, const GemmParams& p, hipStream_t s) {
  switch (epi) {
    case MVIT_EPI_NONE: return launch_var<T, TO, TA, TB, MVIT_EPI_NONE>(var, p, s);
    case MVIT_EPI_BIAS: return launch_var<T, TO, TA, TB, MVIT_EPI_BIAS>(var, p, s);
    case MVIT_EPI_ACCUM: return launch_var<T, TO, TA, TB, MVIT_EPI_ACCUM>(var, p, s);
    default: break;
  }
  if constexpr (!TA && !TB) {
    // forward-only epilogues (both operands contraction-contiguous)
    switch (epi) {
      case MVIT_EPI_BIAS_RES: return launch_var<T, TO, false, false, MVIT_EPI_BIAS_RES>(var, p, s);
      case MVIT_EPI_BIAS_GELU: return launch_var<T, TO, false, false, MVIT_EPI_BIAS_GELU>(var, p, s);
      case MVIT_EPI_SWIGLU: return launch_var<T, TO, false, false, MVIT_EPI_SWIGLU>(var, p, s);
      default: break;
    }
  }
  if constexpr (!TA && TB) {
    // data-gradient epilogues
    switch (epi) {
      case MVIT_EPI_SWIGLU_BWD: return launch_var<T, TO, false, true, MVIT_EPI_SWIGLU_BWD>(var, p, s);
      case MVIT_EPI_GELU_BWD: return launch_var<T, TO, false, true, MVIT_EPI_GELU_BWD>(var, p, s);
      default: break;
    }
  }
  return mvit_set_error(MVIT_ERR_UNSUPPORTED, "gemm: epilogue %d not built for trans_a=%d trans_b=%d", epi, (int)TA, (int)TB);
}

template <typename T, typename TO>
int dispatch_trans(int ta, int tb, int epi, int var, const GemmParams& p, hipStream_t s) {
  if (!ta && !tb) return dispatch_epi<T, TO, false, false>(epi, var, p, s);
  if (!ta && tb) return dispatch_epi<T, TO, false, true>(epi, var, p, s);
  if (ta && tb) return dispatch_epi<T, TO, true, true>(epi, var, p, s);
  return mvit_set_error(MVIT_ERR_UNSUPPORTED, "gemm: trans_a=1, trans_b=0 is not built");
}

inline bool vec16(const void* ptr, int64_t ld, size_t esize) {
  return ptr == nullptr || (mvit_aligned16(ptr) && (ld * (int64_t)esize) % 16 == 0);
}

// packed[n][line * 48 + b] = w[n][channel * 392 + frame * 196 + y * 14 + x] for b = x * 3 + channel < 42, else 0
// (line = frame * 14 + y): the patch-embedding weight in the contraction order of DlPixelOperand
template <typename T>
__global__ __launch_bounds__(256) void pack_patch_weight_kernel(const T* __restrict__ w, int64_t ldw, int64_t n_out, bf16_t* __restrict__ packed) {
  const int64_t total = n_out * PX_K;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t n = i / PX_K;
    const int k = (int)(i % PX_K), ln = k / PX_LINE, b = k % PX_LINE;
    float v = 0.f;
    if (b < PX_PATCH * 3) {
      const int x = b / 3, ch = b % 3, fr = ln / PX_PATCH, y = ln % PX_PATCH;
      v = to_f32(w[n * ldw + ch * (2 * PX_PATCH * PX_PATCH) + fr * (PX_PATCH * PX_PATCH) + y * PX_PATCH + x]);
    }
    packed[i] = from_f32<bf16_t>(v);
  }
}

// float -> bf16 bits, round to nearest even (finite inputs)
inline uint16_t host_bf16_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

}  // namespace

extern "C" int mvit_patch_embed_pack_weight(const void* w, int dtype, int64_t ldw, int64_t n_out, void* packed, mvit_stream_t stream) {
  MVIT_REQUIRE(w && packed, "patch_embed_pack_weight: null pointer");
  MVIT_REQUIRE(dtype == MVIT_BF16 || dtype == MVIT_F32, "patch_embed_pack_weight: dtype %d", dtype);
  MVIT_REQUIRE(n_out > 0 && ldw >= MVIT_PIXEL_ROW, "patch_embed_pack_weight: n_out=%lld ldw=%lld", (long long)n_out, (long long)ldw);
  MVIT_REQUIRE(mvit_aligned16(packed), "patch_embed_pack_weight: packed must be 16-byte aligned");
  const int64_t total = n_out * PX_K;
  const int grid = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype == MVIT_BF16) hipLaunchKernelGGL((pack_patch_weight_kernel<bf16_t>), grid, 256, 0, s, static_cast<const bf16_t*>(w), ldw, n_out, static_cast<bf16_t*>(packed));
  else hipLaunchKernelGGL((pack_patch_weight_kernel<float>), grid, 256, 0, s, static_cast<const float*>(w), ldw, n_out, static_cast<bf16_t*>(packed));
  MVIT_CHECK_LAUNCH("patch_embed_pack_weight");
  return MVIT_OK;
}

extern "C" int mvit_patch_embed_frames(const mvit_image* images, int n_images, int64_t total_rows, const void* packed_w, int64_t n_out,
                                       void* out, int64_t ldo, int out_dtype, double rescale, float mean_r, float mean_g, float mean_b,
                                       float std_r, float std_g, float std_b, mvit_stream_t stream) {
  MVIT_REQUIRE(images && packed_w && out, "patch_embed_frames: null pointer");
  MVIT_REQUIRE(n_images > 0 && total_rows >= 0 && n_out > 0 && ldo >= n_out, "patch_embed_frames: n_images=%d total_rows=%lld n_out=%lld ldo=%lld",
               n_images, (long long)total_rows, (long long)n_out, (long long)ldo);
  MVIT_REQUIRE(out_dtype == MVIT_BF16 || out_dtype == MVIT_F32, "patch_embed_frames: out_dtype %d", out_dtype);
  MVIT_REQUIRE(mvit_aligned16(packed_w), "patch_embed_frames: packed_w must be 16-byte aligned");
  if (total_rows == 0) return MVIT_OK;
  GemmParams p;
  memset(&p, 0, sizeof(p));
  // the kernel computes byte * a + c in one fused multiply-add; that is only taken when, rounded to bf16, it gives
  // the table of mvit_patchify ((float)((double)byte * rescale) - mean) / std for all 256 bytes of every channel
  const float mean[3] = {mean_r, mean_g, mean_b}, stdv[3] = {std_r, std_g, std_b};
  for (int c = 0; c < 3; ++c) {
    MVIT_REQUIRE(stdv[c] != 0.f, "patch_embed_frames: std[%d] = 0", c);
    p.px_a[c] = (float)(rescale / (double)stdv[c]);
    p.px_c[c] = (float)(-(double)mean[c] / (double)stdv[c]);
    for (int b = 0; b < 256; ++b) {
      const float x = (float)((double)b * rescale);
      volatile float diff = x - mean[c];
      const float table = diff / stdv[c];
      const float affine = fmaf((float)b, p.px_a[c], p.px_c[c]);
      if (host_bf16_bits(table) != host_bf16_bits(affine))
        return mvit_set_error(MVIT_ERR_UNSUPPORTED, "patch_embed_frames: byte %d of channel %d: a * x + c does not round to the bf16 value of "
                              "(x * rescale - mean) / std for these constants; use mvit_patchify + mvit_gemm", b, c);
    }
  }
  p.M = total_rows; p.N = n_out; p.K = PX_K;
  p.B = packed_w; p.ldb = PX_K; p.C = out; p.ldc = ldo;
  p.px_images = images; p.px_n_images = n_images;
  p.vec_ok = vec16(out, ldo, out_dtype == MVIT_BF16 ? 2 : 4);
  const int64_t tm = (total_rows + 255) / 256, tn = (n_out + 255) / 256;
  MVIT_REQUIRE(tm * tn < (1ll << 30), "patch_embed_frames: too many tiles");
  p.tiles_m = (int)tm; p.tiles_n = (int)tn;
  p.panel_w = tn <= 6 ? (int)tn : 4;
  p.split_k = 1; p.k_chunk = PX_K; p.reduce_epi = MVIT_EPI_NONE;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == MVIT_BF16) return launch_dl<bf16_t, false, false, MVIT_EPI_NONE, 4, 8, false, true>(p, s);
  return launch_dl<float, false, false, MVIT_EPI_NONE, 4, 8, false, true>(p, s);
}

extern "C" int mvit_gemm(const mvit_gemm_args* a, mvit_stream_t stream) {
  MVIT_REQUIRE(a, "gemm: null args");
  MVIT_REQUIRE(a->M >= 0 && a->N > 0 && a->K > 0, "gemm: bad shape M=%lld N=%lld K=%lld", (long long)a->M, (long long)a->N, (long long)a->K);
  if (a->M == 0) return MVIT_OK;
  MVIT_REQUIRE(a->A && a->B && a->C, "gemm: null operand");
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
  int epi = a->epilogue;
  if (epi == MVIT_EPI_BIAS_RES || epi == MVIT_EPI_GELU_BWD || epi == MVIT_EPI_SWIGLU_BWD) MVIT_REQUIRE(a->R, "gemm: epilogue %d needs R", epi);
  if (epi == MVIT_EPI_BIAS_GELU) MVIT_REQUIRE(a->aux, "gemm: epilogue %d needs aux", epi);
  if (epi == MVIT_EPI_SWIGLU) MVIT_REQUIRE(a->B2 && !a->trans_a && !a->trans_b, "gemm: SWIGLU needs B2 and untransposed operands");
  MVIT_REQUIRE(a->ldc >= a->N, "gemm: ldc=%lld < N=%lld", (long long)a->ldc, (long long)a->N);

  GemmParams p;
  p.M = a->M; p.N = a->N; p.K = a->K;
  p.A = a->A; p.lda = a->lda; p.B = a->B; p.B2 = a->B2; p.ldb = a->ldb;
  p.bias = a->bias; p.bias2 = a->bias2; p.C = a->C; p.ldc = a->ldc;
  p.R = a->R; p.ldr = a->ldr; p.aux = a->aux; p.ldaux = a->ldaux; p.aux_off = a->aux_off;
  const size_t es = a->dtype == MVIT_BF16 ? 2 : 4, eo = a->out_dtype == MVIT_BF16 ? 2 : 4;
  p.vec_ok = vec16(a->C, a->ldc, eo) && vec16(a->R, a->ldr, es) && vec16(a->aux, a->ldaux, es) && vec16(a->bias, 0, es) &&
             vec16(a->bias2, 0, es) && (a->aux_off * (int64_t)(es < eo ? es : eo)) % 16 == 0;
  const int var = (a->lda > (1ll << 22) || a->ldb > (1ll << 22)) ? 1 : 3;  // 3: direct-to-LDS loads (32-bit lane offsets); 1: register-staged
  const int BM = 256, BN = 256;
  const int n_per_block = (epi == MVIT_EPI_SWIGLU) ? BN / 2 : BN;
  const int64_t tm = (a->M + BM - 1) / BM, tn = (a->N + n_per_block - 1) / n_per_block;
  MVIT_REQUIRE(tm * tn < (1ll << 30), "gemm: too many tiles");
  p.tiles_m = (int)tm; p.tiles_n = (int)tn;
  p.panel_w = tn <= 6 ? (int)tn : 4;
  p.split_k = 1; p.k_chunk = a->K; p.workspace = nullptr; p.reduce_epi = MVIT_EPI_NONE;
  p.colsum = nullptr;
  if (epi == MVIT_EPI_SWIGLU_BWD && a->workspace) {
    MVIT_REQUIRE(mvit_aligned16(a->workspace) && a->workspace_bytes >= (int64_t)sizeof(float) * tm * a->ldc,
                 "gemm: SWIGLU_BWD column sums need a workspace of %lld bytes", (long long)(sizeof(float) * tm * a->ldc));
    p.colsum = static_cast<float*>(a->workspace);
  }
  if (a->split_k > 1) {
    const int bk = a->dtype == MVIT_BF16 ? 64 : 16;
    const int64_t chunk = ((a->K + a->split_k - 1) / a->split_k + bk - 1) / bk * bk;
    const int64_t slices = (a->K + chunk - 1) / chunk;  // never an empty slice
    MVIT_REQUIRE(epi == MVIT_EPI_NONE || epi == MVIT_EPI_BIAS || epi == MVIT_EPI_BIAS_RES,
                 "gemm: split_k is available with the plain, bias and bias + residual epilogues (got %d)", epi);
    if (epi != MVIT_EPI_NONE) MVIT_REQUIRE(a->bias, "gemm: split_k with epilogue %d needs bias", epi);
    MVIT_REQUIRE(a->workspace && mvit_aligned16(a->workspace) && a->workspace_bytes >= (int64_t)sizeof(float) * slices * a->M * a->N,
                 "gemm: split_k=%d needs a 16-byte aligned workspace of %lld bytes", a->split_k, (long long)(sizeof(float) * slices * a->M * a->N));
    MVIT_REQUIRE(tm * tn * slices < (1ll << 30), "gemm: too many tiles");
    if (slices > 1) {
      // the main kernel leaves fp32 partial tiles; the reduction over the slices applies the epilogue
      p.split_k = (int)slices; p.k_chunk = chunk; p.workspace = static_cast<float*>(a->workspace);
      p.reduce_epi = epi;
      epi = MVIT_EPI_NONE;
    }
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // Half-height tiles (128 x 256) for the two products that have few tile columns (N = hidden size): when the 256-row
  // tiles would fill the last round of one-tile-per-unit work poorly and the 128-row tiles fill theirs better.  The
  // result does not depend on the choice (same arithmetic per output element), so it may follow M.
  if (a->dtype == MVIT_BF16 && a->out_dtype == MVIT_BF16 && var == 3 && !a->trans_a && p.split_k == 1 && getenv("MVIT_GEMM_NO_HALF_TILES") == nullptr &&
      ((!a->trans_b && epi == MVIT_EPI_BIAS_RES) || (a->trans_b && epi == MVIT_EPI_NONE))) {
    const int dev = mvit_current_device("gemm");
    if (dev < 0) return MVIT_ERR_LAUNCH;
    const double n_cu = device_cu_count(dev);
    const int64_t tm_half = (a->M + 127) / 128;
    const double r_full = (double)(tm * tn) / n_cu, r_half = (double)(tm_half * tn) / n_cu;
    const double fill_full = r_full / ceil(r_full), fill_half = r_half / ceil(r_half);
    if (fill_full < 0.75 && fill_half > fill_full + 0.1 && tm_half * tn < (1ll << 30)) {
      p.tiles_m = (int)tm_half;
      if (!a->trans_b) return launch_dl<bf16_t, false, false, MVIT_EPI_BIAS_RES, 4, 8, false, false, 128>(p, s);
      return launch_dl<bf16_t, false, true, MVIT_EPI_NONE, 4, 8, true, false, 128>(p, s);
    }
  }
  if (a->dtype == MVIT_BF16) {
    if (a->out_dtype == MVIT_BF16) return dispatch_trans<bf16_t, bf16_t>(a->trans_a, a->trans_b, epi, var, p, s);
    return dispatch_trans<bf16_t, float>(a->trans_a, a->trans_b, epi, var, p, s);
  }
  MVIT_REQUIRE(a->out_dtype == MVIT_F32, "gemm: fp32 operands need fp32 output");
  return dispatch_trans<float, float>(a->trans_a, a->trans_b, epi, var, p, s);
}
