// Variable-length (cu_seqlens) non-causal attention, forward and backward, for gfx950.
//
// bf16 path: flash-style kernels on v_mfma_f32_16x16x32_bf16; head_dim = 16*ND is contracted in 32-wide steps
// plus, for odd ND (head_dim 80 = 5 x 16), one half-filled 32-wide step.  All products are oriented so that the
// accumulator layout of one MFMA is directly the B-operand layout of the next:
//   forward : S^T = K Q^T   (lane: query l%16, keys 4*(l/16)+i)  ->  O^T += V^T P^T
//   dK/dV   : S = Q K^T, dP = dO V^T (lane: key l%16, queries 4*(l/16)+i)  ->  dV^T += dO^T P, dK^T += Q^T dS
//   dQ      : S^T, dP^T as in the forward  ->  dQ^T += K^T dS^T
// Operands that are needed "transposed" (V, dO, Q, K as the left factor of the second product) are read
// from their natural [row][head_dim] LDS tiles with ds_read_b64_tr_b16.  Softmax statistics live in
// registers; row reductions are two cross-lane exchanges (lanes l, l^16, l^32, l^48 share a query).
// The backward is split in two kernels (dK/dV, then dQ), which keeps it free of atomics and bit-reproducible.
//
// fp32 path (parity mode): one lane per query (or key) row, K/V (or Q/dO) tiles broadcast from LDS.
#include "mvit_common.h"

#include <algorithm>
#include <type_traits>

namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

struct AttnParams {
  const void *q, *k, *v, *o, *d_o;
  void *out, *dq, *dk, *dv;
  float* lse;
  float* delta;
  const int32_t* cu;
  int64_t total;
  int nheads;
  int64_t q_stride, k_stride, v_stride, o_stride, do_stride, dq_stride, dk_stride, dv_stride;
  float scale;
  const void* q_scaled;  // wide backward: bf16(Q * scale * log2(e)), row stride qs_stride
  int64_t qs_stride;
  const float *nlse2, *ndelta;  // wide backward: - lse * log2(e) and - delta, [nheads, total]
  const int32_t* order;  // optional: the segment scheduled at grid position i is order[i] (null: i)
  int seg_major;         // 0: grid (x, segment, head); 1: grid (x, head, segment), all heads of a segment together
};

// Which segment and head this work-group serves.  Work per work-group grows with its segment's length, so
// callers list long segments first: the short ones then fill the tail of the launch.
//
// seg_major = 2 (short segments, grid (1, n_seg, heads) with n_seg * heads a multiple of 8): a head's slice of a
// token row is 160 bytes at head_dim 80, so the heads of one segment share their 128-byte lines.  Work-group ids
// are dealt round-robin to the 8 XCDs; id i therefore takes work item (i % 8) * (total / 8) + i / 8 of the
// head-fastest list, which puts all heads of a segment on one XCD at about the same time and lets its L2 serve
// the shared lines (the natural order reads them from memory once per head).
__device__ __forceinline__ void seg_and_head(const AttnParams& p, int& seg, int& h) {
  int pos = p.seg_major == 1 ? blockIdx.z : blockIdx.y;
  h = p.seg_major == 1 ? blockIdx.y : blockIdx.z;
  const int n_seg = p.seg_major == 1 ? gridDim.z : gridDim.y;
  if (p.seg_major == 2) {
    const int nh = gridDim.z, lin = blockIdx.y + n_seg * blockIdx.z;
    const int w = (lin & 7) * ((n_seg * nh) >> 3) + (lin >> 3);
    pos = w / nh;
    h = w % nh;
  }
  seg = pos;
  if (p.order) {
    const int listed = p.order[pos];
    if ((unsigned)listed < (unsigned)n_seg) seg = listed;  // an entry outside the list never becomes an address
  }
}

typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
typedef short s16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ bf16x8 tr_pair(const bf16_t* p0, const bf16_t* p1) {
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p0);
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p1);
  s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, both);
}
__device__ __forceinline__ bf16x8 pack8(const f32x4& a, const f32x4& b) {
  bf16x8 r;
  r[0] = (bf16_t)a[0]; r[1] = (bf16_t)a[1]; r[2] = (bf16_t)a[2]; r[3] = (bf16_t)a[3];
  r[4] = (bf16_t)b[0]; r[5] = (bf16_t)b[1]; r[6] = (bf16_t)b[2]; r[7] = (bf16_t)b[3];
  return r;
}
__device__ __forceinline__ f32x4 mfma32(const bf16x8& a, const bf16x8& b, const f32x4& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

template <int ND>
struct Geo {
  static constexpr int HD = 16 * ND;
  static constexpr int NK32 = ND / 2;         // 32-wide contraction steps over head_dim
  static constexpr bool TAIL16 = (ND & 1);    // plus one 16-wide step
  static constexpr int PK = HD + 8;           // pitch of tiles read with 16-byte row loads
  static constexpr int PV = (HD % 32 == 0) ? HD + 16 : HD;  // pitch of tiles read only through transposing loads
  static constexpr int CH = 2 * ND;           // 16-byte chunks per row
};

// Bank-rotated LDS tile layout for tiles that are read both row-wise (16-byte fragments of 16 consecutive rows)
// and through the transposing load (8 consecutive rows x 32 bytes): chunk c (16 bytes) of row r lives at byte
// r * 512 + 16 * (c + rot(r)), rot(r) = 2 * (r & 7) + ((r >> 3) & 1).  Modulo the 256 bytes of one pass over the
// banks, sixteen consecutive rows put one chunk index into sixteen different 16-byte slots, and eight consecutive
// rows put one pair of chunks into eight disjoint 32-byte windows, so neither access pattern has bank conflicts
// (a plain pitch cannot satisfy both: the first needs pitch/16 odd, the second pitch/32 odd).  The rotation is
// additive, so every access is a per-lane base plus a compile-time offset; rows are 512 bytes so that it never
// wraps (10 chunks of data + rotation <= 25 slots; head_dim 128: 31).
constexpr int SWZ = 256;  // pitch in elements; used as the PITCH argument to select this layout
__device__ __forceinline__ int swz_off(int row, int chunk) {
  return row * SWZ + ((chunk + (((row & 7) << 1) | ((row >> 3) & 1))) << 3);
}
// Transposed operand of the 16 x 16 block (rows row0.., head-dim 16*d..) : two transposing loads 16 rows apart.
template <int PITCH>
__device__ __forceinline__ bf16x8 tr_block(const bf16_t* tile, int row0, int d, int g, int r) {
  const int row = row0 + 4 * g + (r >> 2);
  if (PITCH == SWZ) {
    const int chunk = 2 * d + ((r & 3) >> 1), sub = 4 * (r & 1);
    return tr_pair(tile + swz_off(row, chunk) + sub, tile + swz_off(row + 16, chunk) + sub);
  }
  const bf16_t* a = tile + row * PITCH + 16 * d + 4 * (r & 3);
  return tr_pair(a, a + 16 * PITCH);
}

// Operand fragments of 16 rows x head_dim for one lane, in the "row l%16, contraction 8*(l/16)+j" layout
// (serves as MFMA A for rows, or as MFMA B for columns).
template <int ND>
struct RowFrag {
  bf16x8 k32[Geo<ND>::NK32 > 0 ? Geo<ND>::NK32 : 1];
  bf16x4 k16;
};

template <int ND>
__device__ __forceinline__ void load_rowfrag_global(RowFrag<ND>& f, const bf16_t* row_ptr, bool valid, int g) {
  using G = Geo<ND>;
#pragma unroll
  for (int ks = 0; ks < G::NK32; ++ks) {
    bf16x8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (bf16_t)0.f;
    if (valid) v = *reinterpret_cast<const bf16x8*>(row_ptr + 32 * ks + 8 * g);
    f.k32[ks] = v;
  }
  if (G::TAIL16) {
    bf16x4 v = {(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
    if (valid) v = *reinterpret_cast<const bf16x4*>(row_ptr + 32 * G::NK32 + 4 * g);
    f.k16 = v;
  }
}
template <int ND, int PITCH>
__device__ __forceinline__ void load_rowfrag_lds(RowFrag<ND>& f, const bf16_t* tile, int row, int g) {
  using G = Geo<ND>;
  if (PITCH == SWZ) {
#pragma unroll
    for (int ks = 0; ks < G::NK32; ++ks) f.k32[ks] = *reinterpret_cast<const bf16x8*>(tile + swz_off(row, 4 * ks + g));
    if (G::TAIL16) f.k16 = *reinterpret_cast<const bf16x4*>(tile + swz_off(row, 4 * G::NK32 + (g >> 1)) + 4 * (g & 1));
    return;
  }
  const bf16_t* p = tile + row * PITCH;
#pragma unroll
  for (int ks = 0; ks < G::NK32; ++ks) f.k32[ks] = *reinterpret_cast<const bf16x8*>(p + 32 * ks + 8 * g);
  if (G::TAIL16) f.k16 = *reinterpret_cast<const bf16x4*>(p + 32 * G::NK32 + 4 * g);
}
// acc = rows(a) . rows(b)^T over head_dim  (16x16 tile).
// The 16-wide remainder of head_dim (odd ND) is issued as a 32-wide MFMA whose upper four contraction slots
// are zero: a v_mfma_f32_16x16x16_bf16 chained onto the accumulator of the 32-wide steps returned wrong sums
// on gfx950 (also with an all-zero remainder), so that instruction is not used here.
template <int ND>
__device__ __forceinline__ f32x4 dot_frag(const RowFrag<ND>& a, const RowFrag<ND>& b) {
  using G = Geo<ND>;
  f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < G::NK32; ++ks) c = mfma32(a.k32[ks], b.k32[ks], c);
  if (G::TAIL16) {
    const bf16_t z = (bf16_t)0.f;
    const bf16x8 ax = {a.k16[0], a.k16[1], a.k16[2], a.k16[3], z, z, z, z};
    const bf16x8 bx = {b.k16[0], b.k16[1], b.k16[2], b.k16[3], z, z, z, z};
    c = mfma32(ax, bx, c);
  }
  return c;
}

// Cooperative global -> LDS copy of `rows` x head_dim (zero-filled past `valid_rows`).
template <int ND, int PITCH, int NTHREADS>
__device__ __forceinline__ void stage_tile(bf16_t* tile, const bf16_t* src, int64_t stride, int rows, int valid_rows) {
  using G = Geo<ND>;
  const int nchunks = rows * G::CH;
  for (int c = threadIdx.x; c < nchunks; c += NTHREADS) {
    const int r = c / G::CH, dc = c % G::CH;
    bf16x8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (bf16_t)0.f;
    if (r < valid_rows) v = *reinterpret_cast<const bf16x8*>(src + (int64_t)r * stride + dc * 8);
    *reinterpret_cast<bf16x8*>(tile + r * PITCH + dc * 8) = v;
  }
}

// The same copy split in two halves (global -> registers, registers -> LDS) with the per-thread chunk
// coordinates computed once, so that the loads of the next tile can be in flight while the current one is used.
template <int ND, int ROWS, int PITCH, int NTHREADS>
struct TileStager {
  using G = Geo<ND>;
  static constexpr int CHUNKS = ROWS * G::CH;
  static constexpr int PER = (CHUNKS + NTHREADS - 1) / NTHREADS;
  int row[PER];      // tile row of chunk i (ROWS = "no chunk")
  int lds_off[PER];  // element offset in the LDS tile
  int64_t goff[PER]; // element offset from the tile's first row in global memory
  bf16x8 regs[PER];

  __device__ __forceinline__ void init(int64_t stride) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int c = threadIdx.x + NTHREADS * i;
      const int r = c / G::CH, dc = c % G::CH;
      row[i] = c < CHUNKS ? r : ROWS;
      lds_off[i] = PITCH == SWZ ? swz_off(r, dc) : r * PITCH + dc * 8;
      goff[i] = (int64_t)r * stride + dc * 8;
    }
  }
  __device__ __forceinline__ void load(const bf16_t* src, int valid_rows) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      bf16x8 v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (bf16_t)0.f;
      if (row[i] < valid_rows) v = *reinterpret_cast<const bf16x8*>(src + goff[i]);
      regs[i] = v;
    }
  }
  __device__ __forceinline__ void scale(float c) {  // the loaded chunks times c, rounded back to bf16
#pragma unroll
    for (int i = 0; i < PER; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) regs[i][j] = (bf16_t)((float)regs[i][j] * c);
  }
  __device__ __forceinline__ void store(bf16_t* tile) const {
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (row[i] < ROWS) *reinterpret_cast<bf16x8*>(tile + lds_off[i]) = regs[i];
  }
};

// Reductions over the four lanes l, l^16, l^32, l^48 (the lanes that share one query / key column) with the
// VALU lane-swap instructions of gfx950 instead of LDS permutes: v_permlane32_swap exchanges the upper half of its
// first operand with the lower half of its second, v_permlane16_swap does the same for the odd / even rows of 16.
__device__ __forceinline__ float quad_max(float x) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  x = fmaxf(a, b);
  a = x;
  b = x;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}

// dot_frag with one extra contraction slot (odd ND only: the 16-wide remainder leaves half of its 32-wide MFMA
// empty): adds a_x * b_x from lane group 0, which is how the forward folds "- running maximum" into the scores.
template <int ND>
__device__ __forceinline__ f32x4 dot_frag_plus(const RowFrag<ND>& a, const RowFrag<ND>& b, bf16_t a_x, bf16_t b_x) {
  using G = Geo<ND>;
  static_assert(G::TAIL16, "needs the spare slots of the padded remainder");
  f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < G::NK32; ++ks) c = mfma32(a.k32[ks], b.k32[ks], c);
  const bf16_t z = (bf16_t)0.f;
  const bf16x8 ax = {a.k16[0], a.k16[1], a.k16[2], a.k16[3], a_x, z, z, z};
  const bf16x8 bx = {b.k16[0], b.k16[1], b.k16[2], b.k16[3], b_x, z, z, z};
  return mfma32(ax, bx, c);
}

// A float as the sum of two bf16 numbers (16 bits of mantissa): for values that ride in spare contraction slots.
struct HiLo {
  bf16_t hi, lo;
};
__device__ __forceinline__ HiLo split_hilo(float x) {
  HiLo r;
  r.hi = (bf16_t)x;
  r.lo = (bf16_t)(x - (float)r.hi);
  return r;
}
// dot_frag with two extra contraction slots: adds a0*b0 + a1*b1 (operands given per lane; lane groups other than
// 0 must pass zeros on at least one side).  The backward uses it for "- lse" and "- delta", split as hi + lo.
template <int ND>
__device__ __forceinline__ f32x4 dot_frag_plus2(const RowFrag<ND>& a, const RowFrag<ND>& b, bf16_t a0, bf16_t a1, bf16_t b0, bf16_t b1) {
  using G = Geo<ND>;
  static_assert(G::TAIL16, "needs the spare slots of the padded remainder");
  f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < G::NK32; ++ks) c = mfma32(a.k32[ks], b.k32[ks], c);
  const bf16_t z = (bf16_t)0.f;
  const bf16x8 ax = {a.k16[0], a.k16[1], a.k16[2], a.k16[3], a0, a1, z, z};
  const bf16x8 bx = {b.k16[0], b.k16[1], b.k16[2], b.k16[3], b0, b1, z, z};
  return mfma32(ax, bx, c);
}
// Multiply a fragment by a scalar (rounded back to bf16): Q enters every score product as Q * scale * log2(e).
template <int ND>
__device__ __forceinline__ void scale_rowfrag(RowFrag<ND>& f, float c) {
  using G = Geo<ND>;
#pragma unroll
  for (int ks = 0; ks < G::NK32; ++ks)
#pragma unroll
    for (int j = 0; j < 8; ++j) f.k32[ks][j] = (bf16_t)((float)f.k32[ks][j] * c);
  if (G::TAIL16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) f.k16[j] = (bf16_t)((float)f.k16[j] * c);
  }
}

__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

// ================================================================================================
// Forward.  Block = NWAVES waves x 16*QB queries of one (segment, head); BNK keys per iteration.
// At least two work-groups share a CU, K/V tiles are double buffered in LDS and the next tile is
// fetched while the current one is used; key masking only runs on a segment's last, partial tile; the output
// accumulators are rescaled only in iterations where some row maximum of the wave actually grew.
template <int ND, int NWAVES, int BNK, bool PIPE, int QB = 4, int MINW = 2>
__global__ __launch_bounds__(64 * NWAVES, MINW) void attn_fwd_mfma(const AttnParams p) {
  using G = Geo<ND>;
  constexpr int HD = G::HD, NT = 64 * NWAVES, KT = BNK / 16, KK = BNK / 32, NBUF = PIPE ? 2 : 1;
  __shared__ __attribute__((aligned(16))) bf16_t lds_k[NBUF][BNK * G::PK];
  __shared__ __attribute__((aligned(16))) bf16_t lds_v[NBUF][BNK * G::PV];

  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int blk_q0 = blockIdx.x * (16 * QB * NWAVES);
  if (blk_q0 >= L) return;
  const int l = threadIdx.x & 63, wv = threadIdx.x >> 6, g = l >> 4, r = l & 15;
  const int q0 = blk_q0 + wv * (16 * QB);

  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD;
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;

  // Q is scaled by softmax_scale * log2(e) once (rounded to bf16), so the MFMA hands out scores in log2 units.
  // With an odd ND the spare contraction slot of the padded remainder also subtracts the row's running
  // stabiliser m_run (kept as a bf16-representable number): exp2 is then applied to the MFMA result directly.
  constexpr bool FOLD = G::TAIL16;
  constexpr float TAU = 2.f;  // the stabiliser only moves when a score exceeds it by more than TAU (log2 units)
  const float c = p.scale * LOG2E;
  RowFrag<ND> qf[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qi = q0 + qb * 16 + r;
    load_rowfrag_global<ND>(qf[qb], Q + (int64_t)qi * p.q_stride, qi < L, g);
    scale_rowfrag<ND>(qf[qb], c);
  }
  const bf16_t one_x = (bf16_t)(g == 0 ? 1.f : 0.f);  // key side of the extra slot
  bf16_t negm_x[QB];                                    // query side: -m_run in lane group 0

  f32x4 o[QB][ND], lacc[QB];  // lacc: row sums of P, accumulated by the MFMA against a tile of ones
  float m_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = 0.f;
    negm_x[qb] = (bf16_t)0.f;
    lacc[qb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) o[qb][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  bf16x8 ones;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones[j] = (bf16_t)1.f;

  TileStager<ND, BNK, G::PK, PIPE ? NT : BNK * G::CH> sk;  // (degenerate when not pipelined)
  TileStager<ND, BNK, G::PV, PIPE ? NT : BNK * G::CH> sv;
  if (PIPE) {
    sk.init(p.k_stride);
    sv.init(p.v_stride);
    sk.load(K, min(BNK, L));
    sv.load(V, min(BNK, L));
    sk.store(lds_k[0]);
    sv.store(lds_v[0]);
    __syncthreads();
  }

  int buf = 0;
  for (int k0 = 0; k0 < L; k0 += BNK) {
    const int valid = min(BNK, L - k0);
    const bool has_next = k0 + BNK < L;
    if (PIPE) {
      if (has_next) {
        const int nv = min(BNK, L - k0 - BNK);
        sk.load(K + (int64_t)(k0 + BNK) * p.k_stride, nv);
        sv.load(V + (int64_t)(k0 + BNK) * p.v_stride, nv);
      }
    } else {
      if (k0 > 0) __syncthreads();
      stage_tile<ND, G::PK, NT>(lds_k[0], K + (int64_t)k0 * p.k_stride, p.k_stride, BNK, valid);
      stage_tile<ND, G::PV, NT>(lds_v[0], V + (int64_t)k0 * p.v_stride, p.v_stride, BNK, valid);
      __syncthreads();
    }
    const bf16_t* tk = lds_k[PIPE ? buf : 0];
    const bf16_t* tv = lds_v[PIPE ? buf : 0];

    // raw scores: s[qb][kt][i] = S[query qb*16 + r][key kt*16 + 4g + i]
    f32x4 s[QB][KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      RowFrag<ND> kf;
      load_rowfrag_lds<ND, G::PK>(kf, tk, kt * 16 + r, g);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        if constexpr (FOLD) s[qb][kt] = dot_frag_plus<ND>(kf, qf[qb], one_x, negm_x[qb]);  // log2-scaled score - m_run
        else s[qb][kt] = dot_frag<ND>(kf, qf[qb]);
      }
    }
    if (valid < BNK) {  // last, partial tile of the segment
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (kt * 16 + 4 * g + i >= valid) s[qb][kt][i] = -INFINITY;
    }
    bf16x8 pb[QB][KK];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mx = fmaxf(s[qb][0][0], s[qb][0][1]);
      mx = max3(mx, s[qb][0][2], s[qb][0][3]);
#pragma unroll
      for (int kt = 1; kt < KT; ++kt) {
        mx = max3(mx, s[qb][kt][0], s[qb][kt][1]);
        mx = max3(mx, s[qb][kt][2], s[qb][kt][3]);
      }
      mx = quad_max(mx);
      if (!FOLD) mx -= m_run[qb];  // excess over the current stabiliser
      const bool grow = k0 == 0 || mx > TAU;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        float m_new = grow ? m_run[qb] + mx : m_run[qb];
        if (FOLD) m_new = (float)(bf16_t)m_new;
        const float delta = m_new - m_run[qb];
        const float alpha = k0 == 0 ? 1.f : __builtin_amdgcn_exp2f(-delta);
        m_run[qb] = m_new;
        lacc[qb] *= alpha;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) o[qb][dt] *= alpha;
        if (FOLD) {  // this tile's scores were taken against the old stabiliser
          negm_x[qb] = (bf16_t)(g == 0 ? -m_new : 0.f);
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s[qb][kt][i] -= delta;
        }
      }
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          s[qb][kt][i] = __builtin_amdgcn_exp2f(FOLD ? s[qb][kt][i] : s[qb][kt][i] - m_run[qb]);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) pb[qb][kk] = pack8(s[qb][2 * kk], s[qb][2 * kk + 1]);
    }
    // O^T[d][q] += sum_key V[key][d] P[q][key]; contraction slots (g, j): keys t0*16+4g+j | t1*16+4g+j-4
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int dt = 0; dt < ND; ++dt) {
        const bf16_t* a0 = tv + ((2 * kk) * 16 + 4 * g + (r >> 2)) * G::PV + 16 * dt + 4 * (r & 3);
        const bf16x8 vf = tr_pair(a0, a0 + 16 * G::PV);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) o[qb][dt] = mfma32(vf, pb[qb][kk], o[qb][dt]);
      }
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) lacc[qb] = mfma32(ones, pb[qb][kk], lacc[qb]);
    if (PIPE) {
      if (has_next) {
        sk.store(lds_k[buf ^ 1]);
        sv.store(lds_v[buf ^ 1]);
      }
      __syncthreads();
      buf ^= 1;
    }
  }

  bf16_t* O = static_cast<bf16_t*>(p.out) + (int64_t)s0 * p.o_stride + (int64_t)h * HD;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float lt = lacc[qb][0];  // every row of the ones tile holds the row sum
    const int qi = q0 + qb * 16 + r;
    if (qi < L) {
      const float inv = 1.f / lt;
#pragma unroll
      for (int dt = 0; dt < ND; ++dt) {
        bf16x4 ov;
#pragma unroll
        for (int i = 0; i < 4; ++i) ov[i] = (bf16_t)(o[qb][dt][i] * inv);
        *reinterpret_cast<bf16x4*>(O + (int64_t)qi * p.o_stride + 16 * dt + 4 * g) = ov;
      }
      if (g == 0) p.lse[(int64_t)h * p.total + s0 + qi] = (m_run[qb] + __builtin_amdgcn_logf(lt)) * LN2;
    }
  }
}

// ================================================================================================
// Long segments, "wide" kernels: a wave owns 64 rows (two 32-row blocks), four waves per work-group, one
// work-group per CU (up to 512 registers per lane).  Products whose contraction runs over head_dim use
// v_mfma_f32_32x32x16_bf16, so head_dim = 16 * ND is contracted exactly (80 = 5 x 16, no padding); products whose
// contraction runs over rows (keys or queries) use v_mfma_f32_16x16x32_bf16 with head_dim as the 16-wide M dimension.
// A 32x32 accumulator tile (lane: column l%32; register i: row 8*(i/4) + 4*(l/32) + i%4) becomes the B operand of the
// 16x16x32 product after packing to bf16 pairs and four v_permlane16_swap: lanes l and l^16 exchange halves, after
// which lane l holds, for columns l%16 (words 0-3) and 16 + l%16 (words 4-7), the rows
//     base(G) + {0..3}  and  base(G) + 8 + {0..3},   G = l / 16,  base = {0, 16, 4, 20}[G]
// in its eight contraction slots; the transposed left factor is read from LDS with the same row mapping.
// Row statistics ride in the accumulator input of the first MFMA of a chain (a tile of "- statistic" values), so
// exp2 is applied to the MFMA result directly.
// A wave that is alone on its SIMD issues about one instruction per seven cycles and hides no latency by itself:
// matrix and vector instructions are therefore interleaved by hand (__builtin_amdgcn_sched_barrier pins the order),
// LDS fragments are requested a phase before their use, and tiles reach LDS by direct loads three tiles ahead.
// d = a . b + c and d += a . b on v_mfma_f32_32x32x16_bf16 with the result in ordinary vector registers (the compiler's
// own MFMA selection would, in a kernel that uses accumulation registers, place results there and copy them back for
// the vector ALU).  The compiler does not see an MFMA here and inserts no wait states: ordinary instructions may read
// d only after mfma_drain() or after eleven or more other issue slots (every use below sits behind at least two
// further MFMAs).  The B operand `b` sits in accumulation registers (see to_acc_regs): an operand that never changes
// costs no ordinary register that way.
__device__ __forceinline__ void mfma32x32_init(f32x16& d, const bf16x8& a, const u32x4& b, const f32x16& c) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(__builtin_bit_cast(u32x4, a)), "a"(b), "v"(c));
}
__device__ __forceinline__ void mfma32x32_acc(f32x16& d, const bf16x8& a, const u32x4& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(__builtin_bit_cast(u32x4, a)), "a"(b));
}
// the same two with both operands in ordinary vector registers
__device__ __forceinline__ void mfma32x32_init_v(f32x16& d, const bf16x8& a, const bf16x8& b, const f32x16& c) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(__builtin_bit_cast(u32x4, a)), "v"(__builtin_bit_cast(u32x4, b)), "v"(c));
}
__device__ __forceinline__ void mfma32x32_acc_v(f32x16& d, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(__builtin_bit_cast(u32x4, a)), "v"(__builtin_bit_cast(u32x4, b)));
}
// Moves a fragment into accumulation registers through the lane's own 16-byte LDS slot (a DS load can target them).
__device__ __forceinline__ u32x4 to_acc_regs(const bf16x8& v, float* slot) {
  const unsigned addr = (unsigned)(uintptr_t)slot;
  *reinterpret_cast<volatile bf16x8*>(slot) = v;
  u32x4 r;
  asm volatile("s_waitcnt lgkmcnt(0)\n\tds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=a"(r) : "v"(addr) : "memory");
  return r;
}
__device__ __forceinline__ void mfma_drain() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}
__device__ __forceinline__ f32x16 splat16(float x) {
  f32x16 r;
#pragma unroll
  for (int i = 0; i < 16; ++i) r[i] = x;
  return r;
}
__device__ __forceinline__ unsigned pack2(float a, float b) {
  bf16x2 v = {(bf16_t)a, (bf16_t)b};
  return __builtin_bit_cast(unsigned, v);
}
// lanes l and l^16 trade: afterwards a = the pair's value for the lower lane's column, b = for the upper lane's
__device__ __forceinline__ void swap16(unsigned& a, unsigned& b) {
  const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);  // the compiler spaces it from the writes of a and b
  a = r[0];
  b = r[1];
}
struct BOps {
  bf16x8 lo, hi;  // B operands of the 16x16x32 product for columns l%16 and 16 + l%16 of the 32-column tile
};
__device__ __forceinline__ BOps to_b_operands(unsigned (&w)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) swap16(w[j], w[j + 4]);
  const u32x4 a = {w[0], w[1], w[2], w[3]}, b = {w[4], w[5], w[6], w[7]};
  BOps r;
  r.lo = __builtin_bit_cast(bf16x8, a);
  r.hi = __builtin_bit_cast(bf16x8, b);
  return r;
}
__device__ __forceinline__ bf16x8 scale_frag(bf16x8 v, float c) {
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (bf16_t)((float)v[j] * c);
  return v;
}
__device__ __forceinline__ bf16x8 load_frag_global(const bf16_t* p, bool valid) {
  bf16x8 v;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (bf16_t)0.f;
  if (valid) v = *reinterpret_cast<const bf16x8*>(p);
  return v;
}
// delta[h, s] = sum_d O[s,h,d] * dO[s,h,d].  One lane per (row, head), 16-byte loads; neighbouring lanes take
// neighbouring heads of the same row, so a wave sweeps contiguous memory.
template <typename T>
__global__ __launch_bounds__(256) void attn_delta_kernel(const T* __restrict__ o, const T* __restrict__ d_o,
                                                         float* __restrict__ delta, int64_t total, int nheads, int hd,
                                                         int64_t o_stride, int64_t do_stride) {
  constexpr int V = mvit_elem<T>::vec;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total * nheads) return;
  const int64_t s = i / nheads;
  const int h = (int)(i % nheads);
  const T* a = o + s * o_stride + (int64_t)h * hd;
  const T* b = d_o + s * do_stride + (int64_t)h * hd;
  float acc = 0.f;
  if (hd % V == 0 && (o_stride % V) == 0 && (do_stride % V) == 0) {
    for (int j = 0; j < hd; j += V) {
      const vec_t x = *reinterpret_cast<const vec_t*>(a + j);
      const vec_t y = *reinterpret_cast<const vec_t*>(b + j);
#pragma unroll
      for (int e = 0; e < V; ++e) acc += to_f32(x[e]) * to_f32(y[e]);
    }
  } else {
    for (int j = 0; j < hd; ++j) acc += to_f32(a[j]) * to_f32(b[j]);
  }
  delta[(int64_t)h * total + s] = acc;
}

// Same result with coalesced traffic: a block takes 16 consecutive rows; every thread multiplies 16-byte chunks
// (consecutive threads, consecutive chunks of a row), parks the chunk sums in LDS, and thread (h, r) then adds the
// chunks of its head in a fixed order and writes delta[h][s0 + r], 16 consecutive floats per head.
template <typename T>
__global__ __launch_bounds__(256) void attn_delta_rows_kernel(const T* __restrict__ o, const T* __restrict__ d_o,
                                                              float* __restrict__ delta, int64_t total, int nheads, int hd,
                                                              int64_t o_stride, int64_t do_stride) {
  constexpr int V = mvit_elem<T>::vec, R = 16;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  extern __shared__ float part[];  // [R][nheads * hd / V]
  const int cph = hd / V, cpr = nheads * cph;
  const int64_t s0 = (int64_t)blockIdx.x * R;
  const int rows = total - s0 < R ? (int)(total - s0) : R;
  for (int q = threadIdx.x; q < rows * cpr; q += 256) {
    const int r = q / cpr, c = q % cpr;
    const vec_t x = *reinterpret_cast<const vec_t*>(o + (s0 + r) * o_stride + (int64_t)c * V);
    const vec_t y = *reinterpret_cast<const vec_t*>(d_o + (s0 + r) * do_stride + (int64_t)c * V);
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < V; ++e) acc += to_f32(x[e]) * to_f32(y[e]);
    part[q] = acc;
  }
  __syncthreads();
  for (int t = threadIdx.x; t < nheads * R; t += 256) {
    const int h = t / R, r = t % R;
    if (r >= rows) continue;
    const float* src = part + r * cpr + h * cph;
    float acc = 0.f;
    for (int j = 0; j < cph; ++j) acc += src[j];
    delta[(int64_t)h * total + s0 + r] = acc;
  }
}

// ================================================================================================
// dK, dV.  Block = 64*NWAVES keys of one (segment, head); 32 queries per iteration, Q / dO tiles (and the
// rows' lse, delta) double buffered in LDS with the next tile's loads in flight during the MFMAs.
template <int ND, int NWAVES, int RB>
__global__ __launch_bounds__(64 * NWAVES) void attn_bwd_dkdv_mfma(const AttnParams p) {
  using G = Geo<ND>;
  constexpr int HD = G::HD, BQ = 32, NT = 64 * NWAVES, SPAN = 16 * RB * NWAVES;  // RB 16-row blocks per wave
  constexpr int P = SWZ;  // Q / dO tiles are read as row fragments and through the transposing load
  __shared__ __attribute__((aligned(16))) bf16_t lds_q[2][BQ * P];
  __shared__ __attribute__((aligned(16))) bf16_t lds_do[2][BQ * P];
  __shared__ __attribute__((aligned(16))) float lds_lse[2][BQ];
  __shared__ __attribute__((aligned(16))) float lds_delta[2][BQ];
  __shared__ __attribute__((aligned(8))) bf16_t lds_fold[2][BQ][4];  // -lse2 and -delta per row, each as hi + lo
  constexpr bool FOLD = G::TAIL16;

  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int blk_k0 = blockIdx.x * SPAN;
  if (blk_k0 >= L) return;
  const int l = threadIdx.x & 63, wv = threadIdx.x >> 6, g = l >> 4, r = l & 15;
  const int key0 = blk_k0 + wv * 16 * RB;

  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD;
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;
  const bf16_t* DO = static_cast<const bf16_t*>(p.d_o) + (int64_t)s0 * p.do_stride + (int64_t)h * HD;
  const float* LSE = p.lse + (int64_t)h * p.total + s0;
  const float* DELTA = p.delta + (int64_t)h * p.total + s0;

  RowFrag<ND> kf[RB], vf[RB];
#pragma unroll
  for (int kb = 0; kb < RB; ++kb) {
    const int ki = key0 + kb * 16 + r;
    load_rowfrag_global<ND>(kf[kb], K + (int64_t)ki * p.k_stride, ki < L, g);
    load_rowfrag_global<ND>(vf[kb], V + (int64_t)ki * p.v_stride, ki < L, g);
  }
  f32x4 dk[RB][ND], dv[RB][ND];
#pragma unroll
  for (int kb = 0; kb < RB; ++kb)
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
      dk[kb][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
      dv[kb][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  const float c = p.scale * LOG2E;
  const bf16_t one_x = (bf16_t)(g == 0 ? 1.f : 0.f);

  TileStager<ND, BQ, P, NT> sq, sdo;
  sq.init(p.q_stride);
  sdo.init(p.do_stride);
  float r_lse = 0.f, r_delta = 0.f;  // threads 0..31 carry one row's statistics
  auto load_stats = [&](int qs, int valid) {
    if (threadIdx.x < BQ) {
      const bool ok = (int)threadIdx.x < valid;
      r_lse = ok ? LSE[qs + threadIdx.x] * LOG2E : 1e30f;  // huge => p = 0 for padded queries
      r_delta = ok ? DELTA[qs + threadIdx.x] : 0.f;
    }
  };
  auto store_stats = [&](int b) {
    if (threadIdx.x < BQ) {
      lds_lse[b][threadIdx.x] = r_lse;
      lds_delta[b][threadIdx.x] = r_delta;
      const HiLo nl = split_hilo(-r_lse), nd = split_hilo(-r_delta);
      lds_fold[b][threadIdx.x][0] = nl.hi;
      lds_fold[b][threadIdx.x][1] = nl.lo;
      lds_fold[b][threadIdx.x][2] = nd.hi;
      lds_fold[b][threadIdx.x][3] = nd.lo;
    }
  };
  sq.load(Q, min(BQ, L));
  sdo.load(DO, min(BQ, L));
  load_stats(0, min(BQ, L));
  sq.scale(c);  // the Q tile holds Q * scale * log2(e): scores leave the MFMA in log2 units
  sq.store(lds_q[0]);
  sdo.store(lds_do[0]);
  store_stats(0);
  __syncthreads();

  int buf = 0;
  for (int qs = 0; qs < L; qs += BQ) {
    const bool has_next = qs + BQ < L;
    if (has_next) {
      const int nv = min(BQ, L - qs - BQ);
      sq.load(Q + (int64_t)(qs + BQ) * p.q_stride, nv);
      sdo.load(DO + (int64_t)(qs + BQ) * p.do_stride, nv);
      load_stats(qs + BQ, nv);
    }
    const bf16_t* tq = lds_q[buf];
    const bf16_t* tdo = lds_do[buf];

    RowFrag<ND> qa[2], da[2];  // natural-layout A operands: row = query t*16 + r
    bf16x8 qt[ND], dt_[ND];    // transposed A operands: row = head-dim 16*dt + r, slots = queries
    f32x4 lse2[2], dl[2];
    bf16x4 fold[2];  // FOLD: (-lse2 hi, lo, -delta hi, lo) of query t*16 + r, riding in the padded MFMA's spare slots
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      load_rowfrag_lds<ND, P>(qa[t], tq, t * 16 + r, g);
      load_rowfrag_lds<ND, P>(da[t], tdo, t * 16 + r, g);
      if (FOLD) {
        fold[t] = *reinterpret_cast<const bf16x4*>(lds_fold[buf][t * 16 + r]);
        if (g != 0) fold[t] = bf16x4{(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
      } else {
        lse2[t] = *reinterpret_cast<const f32x4*>(lds_lse[buf] + t * 16 + 4 * g);
        dl[t] = *reinterpret_cast<const f32x4*>(lds_delta[buf] + t * 16 + 4 * g);
      }
    }
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      qt[d] = tr_block<P>(tq, 0, d, g, r);
      dt_[d] = tr_block<P>(tdo, 0, d, g, r);
    }
#pragma unroll
    for (int kb = 0; kb < RB; ++kb) {
      f32x4 pv[2], ds[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        // S[q = t*16+4g+i][key = kb*16+r] in log2 units, and dP in the same layout
        if constexpr (FOLD) {
          const f32x4 s = dot_frag_plus2<ND>(qa[t], kf[kb], fold[t][0], fold[t][1], one_x, one_x);   // - lse2
          const f32x4 dp = dot_frag_plus2<ND>(da[t], vf[kb], fold[t][2], fold[t][3], one_x, one_x);  // - delta
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float e = __builtin_amdgcn_exp2f(s[i]);
            pv[t][i] = e;
            ds[t][i] = e * dp[i];
          }
        } else {
          const f32x4 s = dot_frag<ND>(qa[t], kf[kb]);
          const f32x4 dp = dot_frag<ND>(da[t], vf[kb]);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float e = __builtin_amdgcn_exp2f(s[i] - lse2[t][i]);
            pv[t][i] = e;
            ds[t][i] = e * (dp[i] - dl[t][i]);
          }
        }
      }
      const bf16x8 pb = pack8(pv[0], pv[1]);
      const bf16x8 dsb = pack8(ds[0], ds[1]);
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        dv[kb][d] = mfma32(dt_[d], pb, dv[kb][d]);
        dk[kb][d] = mfma32(qt[d], dsb, dk[kb][d]);
      }
    }
    if (has_next) {
      sq.scale(c);
      sq.store(lds_q[buf ^ 1]);
      sdo.store(lds_do[buf ^ 1]);
      store_stats(buf ^ 1);
    }
    __syncthreads();
    buf ^= 1;
  }

  bf16_t* DK = static_cast<bf16_t*>(p.dk) + (int64_t)s0 * p.dk_stride + (int64_t)h * HD;
  bf16_t* DV = static_cast<bf16_t*>(p.dv) + (int64_t)s0 * p.dv_stride + (int64_t)h * HD;
#pragma unroll
  for (int kb = 0; kb < RB; ++kb) {
    const int ki = key0 + kb * 16 + r;
    if (ki < L) {
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        bf16x4 a, b;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[i] = (bf16_t)(dk[kb][d][i] * LN2);  // dS^T (Q scale log2e) / log2e
          b[i] = (bf16_t)dv[kb][d][i];
        }
        *reinterpret_cast<bf16x4*>(DK + (int64_t)ki * p.dk_stride + 16 * d + 4 * g) = a;
        *reinterpret_cast<bf16x4*>(DV + (int64_t)ki * p.dv_stride + 16 * d + 4 * g) = b;
      }
    }
  }
}

// ================================================================================================
// LDS tile layout of the wide backward kernels: 32 rows of 256 bytes (16 slots of 16 bytes, 10 of them used at head_dim
// 80); chunk c of row r lives in slot c ^ xs(r), xs(r) = 2*(r & 3) + ((r >> 2) & 1).  Eight consecutive rows put one
// chunk index into eight different slots (16-byte row-fragment reads), four consecutive rows put one pair of chunks
// into four different 32-byte windows (transposing reads): neither pattern has bank conflicts.  The tile is filled by
// global_load_lds_dwordx4 (16 bytes per lane straight into LDS at M0 + 16 * lane, no staging registers): lane i of
// instruction j fills slot 64*j + i, i.e. it fetches chunk (i & 15) ^ xs(row) of row 4*j + i/16.
constexpr int XS_PITCH = 128;                 // elements per LDS row
constexpr int XS_TILE = 32 * XS_PITCH;        // elements per 32-row tile (8 KiB)
__device__ __forceinline__ int xs(int row) { return ((row & 3) << 1) | ((row >> 2) & 1); }
__device__ __forceinline__ bf16x8 xs_row_frag(const bf16_t* tile, int row, int s, int h) {
  return *reinterpret_cast<const bf16x8*>(tile + row * XS_PITCH + (((2 * s + h) ^ xs(row)) << 3));
}
// transposed A operand (see tr_block_wide) of head-dim block d from rows base(G) + (r >> 2) and + 8
__device__ __forceinline__ bf16x8 xs_tr_block(const bf16_t* tile, int d, int G, int r) {
  const int row = 16 * (G & 1) + 4 * (G >> 1) + (r >> 2);
  const bf16_t* a = tile + row * XS_PITCH + (((2 * d + ((r & 3) >> 1)) ^ xs(row)) << 3) + 4 * (r & 1);
  return tr_pair(a, a + 8 * XS_PITCH);  // xs(row + 8) == xs(row)
}
// wave-uniform values as scalars (the compiler cannot prove uniformity of values derived from the wave index)
__device__ __forceinline__ unsigned uniform_u32(unsigned x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ const void* uniform_ptr(const void* q) {
  const uint64_t v = (uint64_t)(uintptr_t)q;
  const uint64_t u = (uint64_t)uniform_u32((unsigned)v) | ((uint64_t)uniform_u32((unsigned)(v >> 32)) << 32);
  return (const void*)(uintptr_t)u;
}
// lds_addr and base must be wave-uniform (scalar registers)
__device__ __forceinline__ void lds_direct_16(unsigned lds_addr, unsigned voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
__device__ __forceinline__ void lds_direct_4(unsigned lds_addr, unsigned voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// q_scaled[s, h, :] = bf16(q[s, h, :] * c) for the wide backward kernels (the forward rounds Q * scale * log2(e) to
// bf16 the same way, so the recomputed probabilities match the forward's), and the row statistics in the form the
// MFMA accumulators are initialised with: nlse2 = - lse * log2(e), ndelta = - delta.
__global__ __launch_bounds__(256) void attn_bwd_prepare_kernel(const bf16_t* __restrict__ q, int64_t q_stride, bf16_t* __restrict__ qs,
                                                               int64_t qs_stride, int64_t total, int cols, float c,
                                                               const float* __restrict__ lse, const float* __restrict__ delta,
                                                               float* __restrict__ nlse2, float* __restrict__ ndelta, int64_t nstat) {
  const int cpr = cols / 8;
  const int64_t nchunk = total * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nchunk; i += (int64_t)gridDim.x * 256) {
    const int64_t row = i / cpr;
    const int ch = (int)(i % cpr);
    bf16x8 v = *reinterpret_cast<const bf16x8*>(q + row * q_stride + ch * 8);
    *reinterpret_cast<bf16x8*>(qs + row * qs_stride + ch * 8) = scale_frag(v, c);
  }
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nstat; i += (int64_t)gridDim.x * 256) {
    nlse2[i] = -lse[i] * LOG2E;
    ndelta[i] = -delta[i];
  }
}

// ================================================================================================
// dK, dV for long segments, "wide" form: a wave owns 64 keys (two groups of 32), four waves = 256 keys per work-group,
// one work-group per CU.  K / V fragments of the wave's keys and the 2 x 80 accumulators live in accumulation
// registers; pre-scaled Q / dO tiles of 32 queries and their statistics stream through an LDS ring of four tiles,
// written by direct global -> LDS loads three tiles ahead.  Per tile and key group:
//   S = Q K^T - lse2, dP = dO V^T - delta   (v_mfma_f32_32x32x16_bf16, head_dim contracted exactly; the first MFMA of
//                                            a chain takes the tile of "- statistic" values as its accumulator input)
//   P = exp2(S), dS = P * dP                 (vector ALU), packed to bf16 and turned into B operands by lane swaps
//   dV^T += dO^T P, dK^T += Q^T dS           (v_mfma_f32_16x16x32_bf16, transposed left factors read from LDS)
// A wave is alone on its SIMD, so matrix and vector instructions are interleaved by hand: the second key group's
// score MFMAs run under the first group's exp / pack, the first group's dV / dK MFMAs under the second group's.
template <int ND>
__global__ __launch_bounds__(256, 1) void attn_bwd_dkdv_wide(const AttnParams p) {
  static_assert(ND == 5, "the hand-placed instruction order below is laid out for head_dim 80");
  using G = Geo<ND>;
  constexpr int HD = G::HD, BQ = 32, NT = 256, RING = 4;
  __shared__ __attribute__((aligned(1024))) bf16_t lds_q[RING][XS_TILE];
  __shared__ __attribute__((aligned(1024))) bf16_t lds_do[RING][XS_TILE];
  __shared__ __attribute__((aligned(256))) float lds_nlse[RING][64];  // - lse * log2(e) per query of the tile (32 used)
  __shared__ __attribute__((aligned(256))) float lds_ndel[RING][64];  // - delta
  __shared__ __attribute__((aligned(16))) float lds_fix[NT * 4];

  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int blk_k0 = blockIdx.x * 256;
  if (blk_k0 >= L) return;
  const int l = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), hh = l >> 5, c32 = l & 31, G4 = l >> 4, r = l & 15;
  const int key0 = blk_k0 + wv * 64;

  const bf16_t* QS = static_cast<const bf16_t*>(p.q_scaled) + (int64_t)s0 * p.qs_stride + (int64_t)h * HD;
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;
  const bf16_t* DO = static_cast<const bf16_t*>(p.d_o) + (int64_t)s0 * p.do_stride + (int64_t)h * HD;
  const float* NLSE = p.nlse2 + (int64_t)h * p.total + s0;
  const float* NDEL = p.ndelta + (int64_t)h * p.total + s0;

  // B operands of the score products (column = key 32*kg + l%32, contraction = head-dim 16*s + 8*(l/32) ..)
  u32x4 kf[2][ND], vf[2][ND];
#pragma unroll
  for (int kg = 0; kg < 2; ++kg) {
    const int ki = key0 + 32 * kg + c32;
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      kf[kg][s] = to_acc_regs(load_frag_global(K + (int64_t)ki * p.k_stride + 16 * s + 8 * hh, ki < L), lds_fix + threadIdx.x * 4);
      vf[kg][s] = to_acc_regs(load_frag_global(V + (int64_t)ki * p.v_stride + 16 * s + 8 * hh, ki < L), lds_fix + threadIdx.x * 4);
    }
  }
  f32x4 dk[4][ND], dv[4][ND];  // [16-key block][16-wide head-dim block]: lane = key l%16, registers = head-dim 4*(l/16) + i
#pragma unroll
  for (int kb = 0; kb < 4; ++kb)
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      dk[kb][d] = f32x4{0.f, 0.f, 0.f, 0.f};
      dv[kb][d] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  // Direct global -> LDS loads: per tile and tensor eight 1 KiB instructions, two of them this wave's; wave 0 and 1 also
  // fetch one array of statistics each.  Rows past the segment end are read from the segment's last row (they stay
  // finite and meet a probability of exactly zero: their statistics are overwritten before use).
  int trow[2], tchunk[2];
  unsigned voff_q[2], voff_do[2];  // byte offsets of this lane's chunks from the tile's first row (tiles without a tail)
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int slot = 64 * (2 * wv + j) + l;
    trow[j] = slot >> 4;
    tchunk[j] = min(((slot & 15) ^ xs(trow[j])), 2 * ND - 1);  // padding slots re-fetch the last chunk
    voff_q[j] = (unsigned)(trow[j] * (int)p.qs_stride * 2 + tchunk[j] * 16);
    voff_do[j] = (unsigned)(trow[j] * (int)p.do_stride * 2 + tchunk[j] * 16);
  }
  const unsigned lds_q0 = (unsigned)(uintptr_t)&lds_q[0][0], lds_do0 = (unsigned)(uintptr_t)&lds_do[0][0];
  const unsigned lds_nl0 = (unsigned)(uintptr_t)&lds_nlse[0][0], lds_nd0 = (unsigned)(uintptr_t)&lds_ndel[0][0];
  auto request_tile = [&](int qs, int slot) {  // 5 (waves 0, 1) or 4 load instructions
    if (qs >= L) return;
    const int last = L - 1 - qs;  // last valid row of the tile (>= 0)
    const bool tail = last < BQ - 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      unsigned vq = voff_q[j], vd = voff_do[j];
      if (tail) {
        const int row = min(trow[j], last);
        vq = (unsigned)(row * (int)p.qs_stride * 2 + tchunk[j] * 16);
        vd = (unsigned)(row * (int)p.do_stride * 2 + tchunk[j] * 16);
      }
      lds_direct_16(lds_q0 + slot * (XS_TILE * 2) + (2 * wv + j) * 1024, vq, QS + (int64_t)qs * p.qs_stride);
      lds_direct_16(lds_do0 + slot * (XS_TILE * 2) + (2 * wv + j) * 1024, vd, DO + (int64_t)qs * p.do_stride);
    }
    if (wv < 2) lds_direct_4((wv == 0 ? lds_nl0 : lds_nd0) + slot * 256, (unsigned)(min(l, last) * 4), (wv == 0 ? NLSE : NDEL) + qs);
  };
  auto request_inner_tile = [&](int qs, int slot) {  // the same for a tile of 32 rows inside the segment
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      lds_direct_16(lds_q0 + slot * (XS_TILE * 2) + (2 * wv + j) * 1024, voff_q[j], QS + (int64_t)qs * p.qs_stride);
      lds_direct_16(lds_do0 + slot * (XS_TILE * 2) + (2 * wv + j) * 1024, voff_do[j], DO + (int64_t)qs * p.do_stride);
    }
    // every wave fetches one array of statistics (waves 2 and 3 the same bytes as 0 and 1): five loads per wave and
    // tile, so the wait at the end of the step is the same instruction for all of them
    lds_direct_4(((wv & 1) == 0 ? lds_nl0 : lds_nd0) + slot * 256, (unsigned)(l < BQ ? l * 4 : (BQ - 1) * 4), ((wv & 1) == 0 ? NLSE : NDEL) + qs);
  };
  // statistics of rows past the segment end: probability zero, no contribution
  auto fix_tail = [&](int qs, int slot) {
    if (qs < L && qs + BQ > L && threadIdx.x < BQ && qs + (int)threadIdx.x >= L) {
      lds_nlse[slot][threadIdx.x] = -1e30f;
      lds_ndel[slot][threadIdx.x] = 0.f;
    }
  };
  request_tile(0, 0);
  request_tile(BQ, 1);
  request_tile(2 * BQ, 2);
  wait_vmcnt<0>();
  fix_tail(0, 0);
  fix_tail(BQ, 1);
  fix_tail(2 * BQ, 2);
  __syncthreads();

  bf16x8 qa[ND], da[ND];  // A operands of the score products: row = query l%32 of the tile
  f32x16 nl, nd;          // - lse2 and - delta of the tile's queries in accumulator layout (register i: query 8*(i/4) + 4*(l/32) + i%4)
  f32x16 sc[2], dp[2];    // per key group: S - lse2 and dP - delta, lane = key l%32
  auto fetch_rows = [&](int slot) {
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      qa[s] = xs_row_frag(lds_q[slot], c32, s, hh);
      da[s] = xs_row_frag(lds_do[slot], c32, s, hh);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(&lds_nlse[slot][8 * j + 4 * hh]);
      const f32x4 b = *reinterpret_cast<const f32x4*>(&lds_ndel[slot][8 * j + 4 * hh]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        nl[4 * j + i] = a[i];
        nd[4 * j + i] = b[i];
      }
    }
  };
  fetch_rows(0);
  // the same reads in five parts (one per head-dim step), to sit between MFMAs
  auto fetch_rows_part = [&](int slot, int s) {
    qa[s] = xs_row_frag(lds_q[slot], c32, s, hh);
    da[s] = xs_row_frag(lds_do[slot], c32, s, hh);
    if (s < 4) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(&lds_nlse[slot][8 * s + 4 * hh]);
      const f32x4 b = *reinterpret_cast<const f32x4*>(&lds_ndel[slot][8 * s + 4 * hh]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        nl[4 * s + i] = a[i];
        nd[4 * s + i] = b[i];
      }
    }
  };

  // One step of the loop over tiles.  INNER: tile it+3 lies wholly inside the segment, so its request needs no bounds,
  // the wait at the end always leaves one tile in flight and no statistics need fixing: the steady state of a long
  // segment runs without the scalar bookkeeping of the general step, which only the last tiles take.
  int it = 0, qs = 0;
  auto step = [&](auto inner_tag) {
    constexpr bool INNER = decltype(inner_tag)::value;
    const int b0 = it & 3, b1 = (it + 1) & 3, b3 = (it + 3) & 3;
    // tile it+3 is requested into the slot that tile it-1 left (every wave is past the barrier that ended iteration it-1)
    if constexpr (INNER) request_inner_tile(qs + 3 * BQ, b3);
    else request_tile(qs + 3 * BQ, b3);
    // ---- phase 1: score products of key group 0; the transposed left factors that phase 3 needs are read from LDS
    // between the MFMAs
    bf16x8 qt[ND], dt_[ND];
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      if (s == 0) {
        mfma32x32_init(sc[0], qa[0], kf[0][0], nl);
        mfma32x32_init(dp[0], da[0], vf[0][0], nd);
      } else {
        mfma32x32_acc(sc[0], qa[s], kf[0][s]);
        mfma32x32_acc(dp[0], da[s], vf[0][s]);
      }
      qt[s] = xs_tr_block(lds_q[b0], s, G4, r);
      dt_[s] = xs_tr_block(lds_do[b0], s, G4, r);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- phase 2: score products of key group 1 under the vector work of group 0
    unsigned pw[8], dw[8];
    auto words = [&](int j) {
      const float e0 = __builtin_amdgcn_exp2f(sc[0][2 * j]), e1 = __builtin_amdgcn_exp2f(sc[0][2 * j + 1]);
      pw[j] = pack2(e0, e1);
      dw[j] = pack2(e0 * dp[0][2 * j], e1 * dp[0][2 * j + 1]);
    };
    BOps pb, db;
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      // from the second step on the vector work is split between the two MFMAs: a wave issues in order, so whatever
      // stands behind a second MFMA waits with it for the pipe, and only work placed between the two fills the first
      // one's shadow.  (Step 0 keeps both MFMAs first: they separate group 0's last score MFMAs from the first read of
      // their results, which the compiler does not guard.)
      if (s == 0) {
        mfma32x32_init(sc[1], qa[0], kf[1][0], nl);
        mfma32x32_init(dp[1], da[0], vf[1][0], nd);
        words(0);
        words(1);
      } else if (s < 4) {
        mfma32x32_acc(sc[1], qa[s], kf[1][s]);
        __builtin_amdgcn_sched_barrier(0);
        words(2 * s);
        __builtin_amdgcn_sched_barrier(0);
        mfma32x32_acc(dp[1], da[s], vf[1][s]);
        __builtin_amdgcn_sched_barrier(0);
        words(2 * s + 1);
      } else {  // the lane swaps of group 0 under the last two score MFMAs
        mfma32x32_acc(sc[1], qa[s], kf[1][s]);
        __builtin_amdgcn_sched_barrier(0);
        pb = to_b_operands(pw);
        __builtin_amdgcn_sched_barrier(0);
        mfma32x32_acc(dp[1], da[s], vf[1][s]);
        __builtin_amdgcn_sched_barrier(0);
        db = to_b_operands(dw);
        asm volatile("s_nop 1");
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- phase 3: dV / dK of key group 0 under the vector work of group 1
    unsigned pw1[8], dw1[8];
    auto words1 = [&](int j) {
      const float e0 = __builtin_amdgcn_exp2f(sc[1][2 * j]), e1 = __builtin_amdgcn_exp2f(sc[1][2 * j + 1]);
      pw1[j] = pack2(e0, e1);
      dw1[j] = pack2(e0 * dp[1][2 * j], e1 * dp[1][2 * j + 1]);
    };
    BOps pb1, db1;
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      dv[0][d] = mfma32(dt_[d], pb.lo, dv[0][d]);
      dk[0][d] = mfma32(qt[d], db.lo, dk[0][d]);
      dv[1][d] = mfma32(dt_[d], pb.hi, dv[1][d]);
      dk[1][d] = mfma32(qt[d], db.hi, dk[1][d]);
      if (d < 4) {
        words1(2 * d);
        words1(2 * d + 1);
      } else {
        pb1 = to_b_operands(pw1);
        db1 = to_b_operands(dw1);
        asm volatile("s_nop 1");
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- phase 4: dV / dK of key group 1 under the fragment reads of the next tile; the barrier is waited for while
    // these MFMAs drain
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      dv[2][d] = mfma32(dt_[d], pb1.lo, dv[2][d]);
      dk[2][d] = mfma32(qt[d], db1.lo, dk[2][d]);
      dv[3][d] = mfma32(dt_[d], pb1.hi, dv[3][d]);
      dk[3][d] = mfma32(qt[d], db1.hi, dk[3][d]);
      fetch_rows_part(b1, d);
      __builtin_amdgcn_sched_barrier(0);
    }
    // tile it+2 (requested in iteration it-1) must have landed before any wave reads it in the next iteration; the
    // loads requested in this iteration (five by waves 0 and 1, four by the others) may stay in flight
    if constexpr (INNER) {
      wait_vmcnt<5>();
    } else if (qs + 3 * BQ < L) {
      if (wv < 2) wait_vmcnt<5>();
      else wait_vmcnt<4>();
    } else {
      wait_vmcnt<0>();
    }
    if constexpr (!INNER) fix_tail(qs + 2 * BQ, (it + 2) & 3);
    __syncthreads();
  };
  for (; qs + 4 * BQ <= L; qs += BQ, ++it) step(std::true_type{});
  for (; qs < L; qs += BQ, ++it) step(std::false_type{});

  bf16_t* DK = static_cast<bf16_t*>(p.dk) + (int64_t)s0 * p.dk_stride + (int64_t)h * HD;
  bf16_t* DV = static_cast<bf16_t*>(p.dv) + (int64_t)s0 * p.dv_stride + (int64_t)h * HD;
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    const int ki = key0 + kb * 16 + r;
    if (ki < L) {
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        bf16x4 a, b;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[i] = (bf16_t)(dk[kb][d][i] * LN2);  // dS^T (Q scale log2e) / log2e
          b[i] = (bf16_t)dv[kb][d][i];
        }
        *reinterpret_cast<bf16x4*>(DK + (int64_t)ki * p.dk_stride + 16 * d + 4 * G4) = a;
        *reinterpret_cast<bf16x4*>(DV + (int64_t)ki * p.dv_stride + 16 * d + 4 * G4) = b;
      }
    }
  }
}

// ================================================================================================
// Forward for long segments on v_mfma_f32_32x32x16_bf16 only.  A wave owns two blocks of 32 queries (the N dimension of
// every product), eight waves = 512 queries per work-group, one work-group per CU (two waves per SIMD, ~250 registers).
// Per tile of 32 keys and query block:
//   S^T = K Q'^T          5 MFMAs, head_dim contracted exactly; A = a row fragment of the K tile, B = Q' in registers
//                         the accumulator input is a tile of -m (the running stabiliser), so scores arrive stabilised
//   P^T = exp2(S^T)       the accumulator layout (lane: query l%32; register i: key 8*(i/4) + 4*(l/32) + i%4) is, after
//                         packing pairs, already the B operand of the next product: registers 0-7 are contraction
//                         step 0 (keys 0-15), registers 8-15 step 1, with contraction slot j of lane half hh standing
//                         for key 16*ks + 4*hh + (j < 4 ? j : j + 4); no lane exchange is needed
//   O^T += V^T P^T        6 MFMAs: head_dim padded to 96 rows (three 32-row blocks).  Columns 80-95 of the V tile in LDS
//                         hold ones, so rows 80-95 of O^T accumulate the row sums of P for free.
// The transposed left factor V^T is read from the natural [key][head_dim] tile with the transposing LDS load using the
// same slot -> key map.  K / V tiles reach a four-slot LDS ring by direct global -> LDS loads three tiles ahead; lanes
// that would fill the padding chunks are switched off, so the ones written once at the start stay in place.
// 16-byte chunk c of row r of a tile sits in slot c ^ xs16(r): sixteen consecutive rows put one chunk index into sixteen
// different slots (row fragments), four consecutive rows put a pair of chunks into four different 32-byte windows
// (transposing reads).
__device__ __forceinline__ int xs16(int row) { return ((row & 3) << 1) | ((row >> 2) & 1) | (((row >> 3) & 1) << 3); }
__device__ __forceinline__ f32x16 mfma32x32(const bf16x8& a, const bf16x8& b, const f32x16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
// v_max3_f32 / v_max_f32 as they are: the compiler's fmaxf first quiets a possible signalling NaN in every operand
// (one more instruction each); scores are finite or -inf
__device__ __forceinline__ float raw_max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float raw_max(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
// the full maximum of a value held by lanes l and l ^ 32 (the two halves hold different keys of the same query)
__device__ __forceinline__ float max_across_halves(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));  // a = low half's value, b = high half's, in every lane
  return raw_max(a, b);
}

template <int ND>
__global__ __launch_bounds__(512, 1) void attn_fwd_x32(const AttnParams p) {
  static_assert(ND == 5, "the padded third block of head_dim and its ones columns are laid out for head_dim 80");
  using G = Geo<ND>;
  constexpr int HD = G::HD, BK = 32, RING = 4, QB = 2, WQ = 32 * QB;  // QB blocks of 32 queries per wave
  constexpr float TAU = 2.f;  // the stabiliser only moves when a score exceeds it by more than TAU (log2 units)
  __shared__ __attribute__((aligned(1024))) bf16_t lds_k[RING][XS_TILE];
  __shared__ __attribute__((aligned(1024))) bf16_t lds_v[RING][XS_TILE];

  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int blk_q0 = blockIdx.x * (8 * WQ);
  if (blk_q0 >= L) return;
  const int l = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), hh = l >> 5, c32 = l & 31, G4 = l >> 4, r = l & 15;
  const int q_first = blk_q0 + wv * WQ + c32;  // block qb: query q_first + 32 * qb

  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD;
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;

  // ones in chunks 10 and 11 (head_dim 80 .. 95) of every row of every V slot
  for (int i = threadIdx.x; i < RING * 32 * 2; i += 512) {
    const int slot = i >> 6, row = (i >> 1) & 31, ch = 10 + (i & 1);  // i < RING * 64
    bf16x8 ones;
#pragma unroll
    for (int j = 0; j < 8; ++j) ones[j] = (bf16_t)1.f;
    *reinterpret_cast<bf16x8*>(&lds_v[slot][row * XS_PITCH + ((ch ^ xs16(row)) << 3)]) = ones;
  }

  // B operand of the score product: Q * scale * log2(e), rounded to bf16 (scores then come out in log2 units)
  bf16x8 qf[QB][ND];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      const int qi = q_first + 32 * qb;
      qf[qb][s] = scale_frag(load_frag_global(Q + (int64_t)qi * p.q_stride + 16 * s + 8 * hh, qi < L), p.scale * LOG2E);
    }

  // direct global -> LDS loads: one 1 KiB instruction per wave, tensor and tile (rows 4*wv .. 4*wv + 3)
  const int trow = 4 * wv + (l >> 4);
  const int tchunk = (l & 15) ^ xs16(trow);
  const bool tactive = tchunk < 2 * ND;
  const unsigned lds_k0 = (unsigned)(uintptr_t)&lds_k[0][0], lds_v0 = (unsigned)(uintptr_t)&lds_v[0][0];
  auto request_tile = [&](int ks, int slot) {
    if (ks >= L) return;
    const int row = min(trow, L - 1 - ks);  // rows past the segment end repeat its last row; their scores are masked
    const unsigned vk = (unsigned)(row * (int)p.k_stride * 2 + tchunk * 16), vv = (unsigned)(row * (int)p.v_stride * 2 + tchunk * 16);
    if (tactive) {
      lds_direct_16(lds_k0 + slot * (XS_TILE * 2) + wv * 1024, vk, K + (int64_t)ks * p.k_stride);
      lds_direct_16(lds_v0 + slot * (XS_TILE * 2) + wv * 1024, vv, V + (int64_t)ks * p.v_stride);
    }
  };
  f32x16 o[QB][3];  // O^T: block mt, register i = head_dim 32*mt + 8*(i/4) + 4*hh + i%4 of query l%32; rows 80-95 = row sum of P
  float m_run[QB];
  f32x16 negm[QB];  // - m_run in every register: the accumulator input of the score product, so that scores arrive stabilised

  // V^T fragment (block mt of head_dim, contraction step ks): lane i of 16-lane group g4 supplies four consecutive
  // head-dim values of one key row; the transposing load hands lane j of the group head_dim 32*mt + 16*(g4 & 1) + j
  // for the four keys 16*ks + 4*(g4 >> 1) + {0..3}, a second load the keys 8 further on
  auto vt_frag = [&](const bf16_t* tile, int mt, int ks) {
    const int row = 16 * ks + 4 * (G4 >> 1) + (r >> 2);
    const int ch = 4 * mt + 2 * (G4 & 1) + ((r & 3) >> 1);
    const bf16_t* a0 = tile + row * XS_PITCH + ((ch ^ xs16(row)) << 3) + 4 * (r & 1);
    const bf16_t* a1 = tile + (row + 8) * XS_PITCH + ((ch ^ xs16(row + 8)) << 3) + 4 * (r & 1);
    return tr_pair(a0, a1);
  };

  // K row fragments (A operand of the score product) are fetched one tile ahead: tile it+1 is complete in LDS from the
  // start of iteration it on (see the wait before the barrier), so its fragments are requested under the last MFMAs of
  // tile it and no LDS latency opens the next iteration
  bf16x8 kf[ND];
  auto fetch_k = [&](int slot) {
#pragma unroll
    for (int s = 0; s < ND; ++s) kf[s] = *reinterpret_cast<const bf16x8*>(lds_k[slot] + c32 * XS_PITCH + (((2 * s + hh) ^ xs16(c32)) << 3));
  };
  // One tile of 32 keys.  CHECK: the tile's row maxima are taken and the stabiliser follows them.  The first sweep over
  // the keys does that for the first tile only and then leaves the stabiliser where it is: exp2 of a bf16 / fp32 value has
  // 250 binary orders of range, so a later score may exceed the first tile's maximum by more than a hundred (base-2
  // units) before anything overflows, and scores far below it vanish exactly as they would against the true maximum.
  // A row whose sums did overflow is seen at the end (an infinity or NaN in its accumulators) and the work-group sweeps
  // again with the maxima taken on every tile.
  int it = 0;
  auto tile_step = [&](int k0, auto check_tag) {
    constexpr bool CHECK = decltype(check_tag)::value;
    const int b0 = it & (RING - 1), b1 = (it + 1) & (RING - 1), b3 = (it + 3) & (RING - 1);
    request_tile(k0 + 3 * BK, b3);
    const bf16_t* tv = lds_v[b0];
    f32x16 sc[QB];
    unsigned pw[QB][8];
    auto mask_tail = [&](int qb) {
      if (k0 + BK > L) {  // last, partial tile
        asm volatile("" ::: "memory");
        const int valid = L - k0;
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (4 * hh >= valid - (8 * (i >> 2) + (i & 3))) sc[qb][i] = -INFINITY;  // key 8*(i/4) + 4*hh + i%4 >= valid
      }
    };
    auto row_max = [&](int qb) {
      float mx = raw_max3(sc[qb][0], sc[qb][1], sc[qb][2]);
#pragma unroll
      for (int i = 3; i < 15; i += 2) mx = raw_max3(mx, sc[qb][i], sc[qb][i + 1]);
      mx = raw_max(mx, sc[qb][15]);
      return max_across_halves(mx);
    };
    // mx = the largest score of the tile minus the current stabiliser; the stabiliser moves when that excess is above
    // TAU for some query of the wave (rare after the first tiles): accumulators and this tile's scores are rebased
    auto rescale = [&](int qb, float mx) {
      const bool grow = k0 == 0 || mx > TAU;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        asm volatile("" ::: "memory");
        const float delta = grow ? mx : 0.f;
        const float alpha = k0 == 0 ? 1.f : __builtin_amdgcn_exp2f(-delta);
        m_run[qb] += delta;
        negm[qb] = splat16(-m_run[qb]);
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[qb][i] -= delta;
#pragma unroll
        for (int mt = 0; mt < 3; ++mt) o[qb][mt] *= alpha;
      }
    };
    auto p_operand = [&](int qb, int ks) {
      const u32x4 w4 = {pw[qb][4 * ks], pw[qb][4 * ks + 1], pw[qb][4 * ks + 2], pw[qb][4 * ks + 3]};
      return __builtin_bit_cast(bf16x8, w4);
    };
    {
      // Two query blocks per wave, software-pipelined by hand: the second block's score MFMAs run under the first
      // block's softmax arithmetic, the first block's P.V MFMAs under the second block's; scheduling barriers pin the
      // order.  Only the first score MFMA of each block is inline assembly (its accumulator input is the stabiliser
      // tile, which the compiler's own MFMA selection would first copy into the result registers).  The compiler sees
      // no MFMA there and inserts no wait states for its result: the two are issued together, so that a whole MFMA
      // separates each from the accumulating MFMA that reads its result; all later dependencies are the compiler's.
      auto words = [&](int qb, int w0, int w1) {
#pragma unroll
        for (int w = w0; w < w1; ++w) pw[qb][w] = pack2(__builtin_amdgcn_exp2f(sc[qb][2 * w]), __builtin_amdgcn_exp2f(sc[qb][2 * w + 1]));
      };
      mfma32x32_init_v(sc[0], kf[0], qf[0][0], negm[0]);
      mfma32x32_init_v(sc[1], kf[0], qf[1][0], negm[1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 1; s < ND; ++s) sc[0] = mfma32x32(kf[s], qf[0][s], sc[0]);
      sc[1] = mfma32x32(kf[1], qf[1][1], sc[1]);
      __builtin_amdgcn_sched_barrier(0);
      mask_tail(0);
      if constexpr (CHECK) rescale(0, row_max(0));
      __builtin_amdgcn_sched_barrier(0);
      sc[1] = mfma32x32(kf[2], qf[1][2], sc[1]);
      __builtin_amdgcn_sched_barrier(0);
      words(0, 0, 3);
      __builtin_amdgcn_sched_barrier(0);
      sc[1] = mfma32x32(kf[3], qf[1][3], sc[1]);
      __builtin_amdgcn_sched_barrier(0);
      words(0, 3, 6);
      __builtin_amdgcn_sched_barrier(0);
      sc[1] = mfma32x32(kf[4], qf[1][4], sc[1]);
      __builtin_amdgcn_sched_barrier(0);
      words(0, 6, 8);
      // the V fragments (kept for both blocks) and the first two P.V MFMAs of block 0 separate the last score MFMA of
      // block 1 from the first read of its result
      bf16x8 vf[6];
#pragma unroll
      for (int n = 0; n < 6; ++n) vf[n] = vt_frag(tv, n % 3, n / 3);
      o[0][0] = mfma32x32(vf[0], p_operand(0, 0), o[0][0]);
      o[0][1] = mfma32x32(vf[1], p_operand(0, 0), o[0][1]);
      __builtin_amdgcn_sched_barrier(0);
      mask_tail(1);
      if constexpr (CHECK) rescale(1, row_max(1));
      __builtin_amdgcn_sched_barrier(0);
      o[0][2] = mfma32x32(vf[2], p_operand(0, 0), o[0][2]);
      __builtin_amdgcn_sched_barrier(0);
      words(1, 0, 2);
      __builtin_amdgcn_sched_barrier(0);
      o[0][0] = mfma32x32(vf[3], p_operand(0, 1), o[0][0]);
      __builtin_amdgcn_sched_barrier(0);
      words(1, 2, 4);
      __builtin_amdgcn_sched_barrier(0);
      o[0][1] = mfma32x32(vf[4], p_operand(0, 1), o[0][1]);
      __builtin_amdgcn_sched_barrier(0);
      words(1, 4, 6);
      __builtin_amdgcn_sched_barrier(0);
      o[0][2] = mfma32x32(vf[5], p_operand(0, 1), o[0][2]);
      __builtin_amdgcn_sched_barrier(0);
      words(1, 6, 8);
      __builtin_amdgcn_sched_barrier(0);
      fetch_k(b1);  // next tile's K fragments (garbage past the last tile, never used)
#pragma unroll
      for (int n = 0; n < 6; ++n) o[1][n % 3] = mfma32x32(vf[n], p_operand(1, n / 3), o[1][n % 3]);
    }
    // tile it+2 (requested one iteration ago) must have landed before any wave reads it; this iteration's own two
    // requests may stay in flight
    if (k0 + 3 * BK < L) wait_vmcnt<2>();
    else wait_vmcnt<0>();
    __syncthreads();
  };
  auto sweep = [&](auto every_tile_tag) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      m_run[qb] = 0.f;
      negm[qb] = splat16(0.f);
#pragma unroll
      for (int mt = 0; mt < 3; ++mt) o[qb][mt] = splat16(0.f);
    }
    request_tile(0, 0);
    request_tile(BK, 1);
    request_tile(2 * BK, 2);
    wait_vmcnt<0>();
    __syncthreads();
    fetch_k(0);
    it = 0;
    tile_step(0, std::true_type{});
    ++it;
    for (int k0 = BK; k0 < L; k0 += BK, ++it) tile_step(k0, every_tile_tag);
  };
  sweep(std::false_type{});
  {
    // x * 0 is NaN for an infinity or a NaN and 0 otherwise: one chain of multiply-adds over a block's accumulators
    float chk = 0.f;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int mt = 0; mt < 3; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) chk = __builtin_fmaf(o[qb][mt][i], 0.f, chk);
    if (__syncthreads_or(chk != chk)) sweep(std::true_type{});  // the ring is idle: every wave is past its last tile
  }

#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qi = q_first + 32 * qb;
    if (qi < L) {
      const float lsum = o[qb][2][8];  // head_dim row 80 (or 84): the row sum of P
      const float inv = 1.f / lsum;
      bf16_t* O = static_cast<bf16_t*>(p.out) + (int64_t)(s0 + qi) * p.o_stride + (int64_t)h * HD;
#pragma unroll
      for (int mt = 0; mt < 3; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (32 * mt + 8 * j >= HD) continue;
          bf16x4 ov;
#pragma unroll
          for (int i = 0; i < 4; ++i) ov[i] = (bf16_t)(o[qb][mt][4 * j + i] * inv);
          *reinterpret_cast<bf16x4*>(O + 32 * mt + 8 * j + 4 * hh) = ov;
        }
      if (hh == 0) p.lse[(int64_t)h * p.total + s0 + qi] = (m_run[qb] + __builtin_amdgcn_logf(lsum)) * LN2;
    }
  }
}

// ================================================================================================
// dQ for long segments, "wide" form: a wave owns 64 queries (two blocks of 32), four waves = 256 queries per
// work-group, one work-group per CU.  Pre-scaled Q and dO fragments of the wave's queries, and the 80 accumulators,
// live in accumulation registers; K / V tiles of 32 keys stream through an LDS ring of four tiles (direct
// global -> LDS loads, three tiles ahead).  Per tile and query block:
//   S^T = K Q^T - lse2, dP^T = V dO^T - delta   (v_mfma_f32_32x32x16_bf16; lane = query, so the statistics are per-lane
//                                                constants kept as ready-made accumulator input tiles)
//   dS^T = exp2(S^T) * dP^T                      (vector ALU), packed to bf16, lane swaps
//   dQ^T += K^T dS^T                             (v_mfma_f32_16x16x32_bf16, K^T read from LDS with the transposing load)
template <int ND>
__global__ __launch_bounds__(256, 1) void attn_bwd_dq_wide(const AttnParams p) {
  static_assert(ND == 5, "the hand-placed instruction order below is laid out for head_dim 80");
  using G = Geo<ND>;
  constexpr int HD = G::HD, BK = 32, NT = 256, RING = 4;
  // one array for both streamed tensors: a fragment's address in the V tile is its address in the K tile plus a
  // constant that fits the instruction's offset field, so one address computation serves both
  __shared__ __attribute__((aligned(1024))) bf16_t lds_kv[2 * RING][XS_TILE];
  bf16_t (*const lds_k)[XS_TILE] = lds_kv;
  bf16_t (*const lds_v)[XS_TILE] = lds_kv + RING;
  __shared__ __attribute__((aligned(16))) float lds_fix[NT * 4];

  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int blk_q0 = blockIdx.x * 256;
  if (blk_q0 >= L) return;
  const int l = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), hh = l >> 5, c32 = l & 31, G4 = l >> 4, r = l & 15;
  const int q0 = blk_q0 + wv * 64;

  const bf16_t* QS = static_cast<const bf16_t*>(p.q_scaled) + (int64_t)s0 * p.qs_stride + (int64_t)h * HD;
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;
  const bf16_t* DO = static_cast<const bf16_t*>(p.d_o) + (int64_t)s0 * p.do_stride + (int64_t)h * HD;
  const float* NLSE = p.nlse2 + (int64_t)h * p.total + s0;
  const float* NDEL = p.ndelta + (int64_t)h * p.total + s0;

  // B operands of the score products (column = query 32*qb + l%32, contraction = head-dim 16*s + 8*(l/32) ..) and the
  // accumulator input tiles holding the query's - lse2 / - delta in all sixteen registers
  u32x4 qf[2][ND], dof[2][ND];
  f32x16 nl[2], nd[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = q0 + 32 * qb + c32;
    const bool ok = qi < L;
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      qf[qb][s] = to_acc_regs(load_frag_global(QS + (int64_t)qi * p.qs_stride + 16 * s + 8 * hh, ok), lds_fix + threadIdx.x * 4);
      dof[qb][s] = to_acc_regs(load_frag_global(DO + (int64_t)qi * p.do_stride + 16 * s + 8 * hh, ok), lds_fix + threadIdx.x * 4);
    }
    nl[qb] = splat16(ok ? NLSE[qi] : -1e30f);  // hugely negative => p = 0 for queries past the end
    nd[qb] = splat16(ok ? NDEL[qi] : 0.f);
  }
  f32x4 dq[2][2][ND];  // [query block][half][head-dim block]: lane = query l%16 of the half, registers = head-dim 4*(l/16) + i
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int d = 0; d < ND; ++d) dq[qb][hf][d] = f32x4{0.f, 0.f, 0.f, 0.f};

  // direct global -> LDS loads of the K / V tiles (see attn_bwd_dkdv_wide); rows past the segment end repeat its last row
  int trow[2], tchunk[2];
  unsigned voff_k[2], voff_v[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int slot = 64 * (2 * wv + j) + l;
    trow[j] = slot >> 4;
    tchunk[j] = min(((slot & 15) ^ xs(trow[j])), 2 * ND - 1);
    voff_k[j] = (unsigned)(trow[j] * (int)p.k_stride * 2 + tchunk[j] * 16);
    voff_v[j] = (unsigned)(trow[j] * (int)p.v_stride * 2 + tchunk[j] * 16);
  }
  const unsigned lds_k0 = (unsigned)(uintptr_t)&lds_k[0][0], lds_v0 = (unsigned)(uintptr_t)&lds_v[0][0];
  auto request_tile = [&](int k0, int slot) {  // 4 load instructions
    if (k0 >= L) return;
    const int last = L - 1 - k0;
    const bool tail = last < BK - 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      unsigned vk = voff_k[j], vv = voff_v[j];
      if (tail) {
        const int row = min(trow[j], last);
        vk = (unsigned)(row * (int)p.k_stride * 2 + tchunk[j] * 16);
        vv = (unsigned)(row * (int)p.v_stride * 2 + tchunk[j] * 16);
      }
      lds_direct_16(lds_k0 + slot * (XS_TILE * 2) + (2 * wv + j) * 1024, vk, K + (int64_t)k0 * p.k_stride);
      lds_direct_16(lds_v0 + slot * (XS_TILE * 2) + (2 * wv + j) * 1024, vv, V + (int64_t)k0 * p.v_stride);
    }
  };
  request_tile(0, 0);
  request_tile(BK, 1);
  request_tile(2 * BK, 2);
  wait_vmcnt<0>();
  __syncthreads();

  bf16x8 ka[ND], va[ND];  // A operands of the score products: row = key l%32 of the tile
  auto fetch_rows = [&](int slot) {
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      ka[s] = xs_row_frag(lds_k[slot], c32, s, hh);
      va[s] = xs_row_frag(lds_v[slot], c32, s, hh);
    }
  };
  fetch_rows(0);

  f32x16 sc[2], dp[2];  // per query block: S^T - lse2 and dP^T - delta, lane = query l%32, register i = key 8*(i/4) + 4*(l/32) + i%4
  int it = 0;
  for (int k0 = 0; k0 < L; k0 += BK, ++it) {
    const int b0 = it & 3, b1 = (it + 1) & 3, b3 = (it + 3) & 3;
    request_tile(k0 + 3 * BK, b3);
    const int valid = L - k0;  // keys of this tile inside the segment (>= 1)
    // ---- phase 1: score products of query block 0; K^T fragments for the dQ products are read between the MFMAs
    bf16x8 kt[ND];
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      if (s == 0) {
        mfma32x32_init(sc[0], ka[0], qf[0][0], nl[0]);
        mfma32x32_init(dp[0], va[0], dof[0][0], nd[0]);
      } else {
        mfma32x32_acc(sc[0], ka[s], qf[0][s]);
        mfma32x32_acc(dp[0], va[s], dof[0][s]);
      }
      kt[s] = xs_tr_block(lds_k[b0], s, G4, r);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- phase 2: score products of query block 1 under the vector work of block 0
    unsigned dw[2][8];
    auto word = [&](int qb, int j) {
      const float x0 = __builtin_amdgcn_exp2f(sc[qb][2 * j]) * dp[qb][2 * j], x1 = __builtin_amdgcn_exp2f(sc[qb][2 * j + 1]) * dp[qb][2 * j + 1];
      dw[qb][j] = pack2(x0, x1);
    };
    // keys past the segment end (last tile only) contribute nothing: their dP is zeroed before it is used
    auto mask_tail = [&](int qb) {
      if (valid < BK) {
        asm volatile("" ::: "memory");  // keeps this rare block a branch
        mfma_drain();
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (8 * (i >> 2) + 4 * hh + (i & 3) >= valid) dp[qb][i] = 0.f;
      }
    };
    mask_tail(0);
    BOps d0;
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      // vector work between the two MFMAs from the second step on (see attn_bwd_dkdv_wide)
      if (s == 0) {
        mfma32x32_init(sc[1], ka[0], qf[1][0], nl[1]);
        mfma32x32_init(dp[1], va[0], dof[1][0], nd[1]);
        word(0, 0);
        word(0, 1);
      } else if (s < 4) {
        mfma32x32_acc(sc[1], ka[s], qf[1][s]);
        __builtin_amdgcn_sched_barrier(0);
        word(0, 2 * s);
        __builtin_amdgcn_sched_barrier(0);
        mfma32x32_acc(dp[1], va[s], dof[1][s]);
        __builtin_amdgcn_sched_barrier(0);
        word(0, 2 * s + 1);
      } else {  // the lane swaps of block 0 under the last two score MFMAs
        mfma32x32_acc(sc[1], ka[s], qf[1][s]);
        mfma32x32_acc(dp[1], va[s], dof[1][s]);
        d0 = to_b_operands(dw[0]);
        asm volatile("s_nop 1");
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- phase 3: dQ of query block 0 under the vector work of block 1
    mask_tail(1);
    BOps d1;
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      dq[0][0][d] = mfma32(kt[d], d0.lo, dq[0][0][d]);
      dq[0][1][d] = mfma32(kt[d], d0.hi, dq[0][1][d]);
      if (d < 4) {
        word(1, 2 * d);
        word(1, 2 * d + 1);
      } else {
        d1 = to_b_operands(dw[1]);
        asm volatile("s_nop 1");
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- phase 4: dQ of query block 1 under the fragment reads of the next tile
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      dq[1][0][d] = mfma32(kt[d], d1.lo, dq[1][0][d]);
      dq[1][1][d] = mfma32(kt[d], d1.hi, dq[1][1][d]);
      ka[d] = xs_row_frag(lds_k[b1], c32, d, hh);
      va[d] = xs_row_frag(lds_v[b1], c32, d, hh);
      __builtin_amdgcn_sched_barrier(0);
    }
    // tile it+2 (requested in iteration it-1) must have landed before any wave reads it in the next iteration
    if (k0 + 3 * BK < L) wait_vmcnt<4>();
    else wait_vmcnt<0>();
    __syncthreads();
  }

  bf16_t* DQ = static_cast<bf16_t*>(p.dq) + (int64_t)s0 * p.dq_stride + (int64_t)h * HD;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int qi = q0 + 32 * qb + 16 * hf + r;
      if (qi < L) {
#pragma unroll
        for (int d = 0; d < ND; ++d) {
          bf16x4 a;
#pragma unroll
          for (int i = 0; i < 4; ++i) a[i] = (bf16_t)(dq[qb][hf][d][i] * p.scale);
          *reinterpret_cast<bf16x4*>(DQ + (int64_t)qi * p.dq_stride + 16 * d + 4 * G4) = a;
        }
      }
    }
}

// ================================================================================================
// dQ.  Block = 64*NWAVES queries of one (segment, head); 32 keys per iteration, K / V tiles double buffered.
template <int ND, int NWAVES, int RB>
__global__ __launch_bounds__(64 * NWAVES) void attn_bwd_dq_mfma(const AttnParams p) {
  using G = Geo<ND>;
  constexpr int HD = G::HD, BK = 32, NT = 64 * NWAVES, SPAN = 16 * RB * NWAVES;  // RB 16-row blocks per wave
  constexpr int P = SWZ;  // the K tile is read as row fragments and through the transposing load
  __shared__ __attribute__((aligned(16))) bf16_t lds_k[2][BK * P];
  __shared__ __attribute__((aligned(16))) bf16_t lds_v[2][BK * P];

  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int blk_q0 = blockIdx.x * SPAN;
  if (blk_q0 >= L) return;
  const int l = threadIdx.x & 63, wv = threadIdx.x >> 6, g = l >> 4, r = l & 15;
  const int q0 = blk_q0 + wv * 16 * RB;

  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD;
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;
  const bf16_t* DO = static_cast<const bf16_t*>(p.d_o) + (int64_t)s0 * p.do_stride + (int64_t)h * HD;
  const float* LSE = p.lse + (int64_t)h * p.total + s0;
  const float* DELTA = p.delta + (int64_t)h * p.total + s0;

  constexpr bool FOLD = G::TAIL16;
  const float c = p.scale * LOG2E;
  const bf16_t one_x = (bf16_t)(g == 0 ? 1.f : 0.f);
  RowFrag<ND> qf[RB], dof[RB];
  float neg_lse2[RB], dl[RB];
  HiLo f_lse[RB], f_dl[RB];  // FOLD: -lse2 and -delta of the lane's query as hi + lo (lane group 0 only)
#pragma unroll
  for (int qb = 0; qb < RB; ++qb) {
    const int qi = q0 + qb * 16 + r;
    const bool ok = qi < L;
    load_rowfrag_global<ND>(qf[qb], Q + (int64_t)qi * p.q_stride, ok, g);
    scale_rowfrag<ND>(qf[qb], c);  // scores leave the MFMA in log2 units
    load_rowfrag_global<ND>(dof[qb], DO + (int64_t)qi * p.do_stride, ok, g);
    neg_lse2[qb] = ok ? -LSE[qi] * LOG2E : -1e30f;  // hugely negative => p = 0 for padded queries
    dl[qb] = ok ? DELTA[qi] : 0.f;
    f_lse[qb] = split_hilo(g == 0 ? neg_lse2[qb] : 0.f);
    f_dl[qb] = split_hilo(g == 0 ? -dl[qb] : 0.f);
  }
  f32x4 dq[RB][ND];
#pragma unroll
  for (int qb = 0; qb < RB; ++qb)
#pragma unroll
    for (int d = 0; d < ND; ++d) dq[qb][d] = f32x4{0.f, 0.f, 0.f, 0.f};

  TileStager<ND, BK, P, NT> sk, sv;
  sk.init(p.k_stride);
  sv.init(p.v_stride);
  sk.load(K, min(BK, L));
  sv.load(V, min(BK, L));
  sk.store(lds_k[0]);
  sv.store(lds_v[0]);
  __syncthreads();

  int buf = 0;
  for (int k0 = 0; k0 < L; k0 += BK) {
    const int valid = min(BK, L - k0);
    const bool has_next = k0 + BK < L;
    if (has_next) {
      const int nv = min(BK, L - k0 - BK);
      sk.load(K + (int64_t)(k0 + BK) * p.k_stride, nv);
      sv.load(V + (int64_t)(k0 + BK) * p.v_stride, nv);
    }
    const bf16_t* tk = lds_k[buf];
    const bf16_t* tv = lds_v[buf];

    RowFrag<ND> ka[2], va[2];
    bf16x8 kt[ND];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      load_rowfrag_lds<ND, P>(ka[t], tk, t * 16 + r, g);
      load_rowfrag_lds<ND, P>(va[t], tv, t * 16 + r, g);
    }
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      kt[d] = tr_block<P>(tk, 0, d, g, r);
    }
#pragma unroll
    for (int qb = 0; qb < RB; ++qb) {
      f32x4 ds[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        // S[q = qb*16+r][key = t*16+4g+i] in log2 units, and dP in the same layout
        if constexpr (FOLD) {
          const f32x4 s = dot_frag_plus2<ND>(ka[t], qf[qb], one_x, one_x, f_lse[qb].hi, f_lse[qb].lo);   // - lse2
          const f32x4 dp = dot_frag_plus2<ND>(va[t], dof[qb], one_x, one_x, f_dl[qb].hi, f_dl[qb].lo);  // - delta
#pragma unroll
          for (int i = 0; i < 4; ++i) ds[t][i] = __builtin_amdgcn_exp2f(s[i]) * dp[i];
        } else {
          const f32x4 s = dot_frag<ND>(ka[t], qf[qb]);
          const f32x4 dp = dot_frag<ND>(va[t], dof[qb]);
#pragma unroll
          for (int i = 0; i < 4; ++i) ds[t][i] = __builtin_amdgcn_exp2f(s[i] + neg_lse2[qb]) * (dp[i] - dl[qb]);
        }
      }
      if (valid < BK) {  // keys past the segment end contribute nothing
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (t * 16 + 4 * g + i >= valid) ds[t][i] = 0.f;
      }
      const bf16x8 dsb = pack8(ds[0], ds[1]);
#pragma unroll
      for (int d = 0; d < ND; ++d) dq[qb][d] = mfma32(kt[d], dsb, dq[qb][d]);
    }
    if (has_next) {
      sk.store(lds_k[buf ^ 1]);
      sv.store(lds_v[buf ^ 1]);
    }
    __syncthreads();
    buf ^= 1;
  }

  bf16_t* DQ = static_cast<bf16_t*>(p.dq) + (int64_t)s0 * p.dq_stride + (int64_t)h * HD;
#pragma unroll
  for (int qb = 0; qb < RB; ++qb) {
    const int qi = q0 + qb * 16 + r;
    if (qi < L) {
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        bf16x4 a;
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = (bf16_t)(dq[qb][d][i] * p.scale);
        *reinterpret_cast<bf16x4*>(DQ + (int64_t)qi * p.dq_stride + 16 * d + 4 * g) = a;
      }
    }
  }
}

// ================================================================================================
// Whole backward of a short segment (<= 64 rows, the windowed layers) in one work-group: Q, K, V and dO of one
// (segment, head) are staged in LDS once.  Pass A works in the dQ orientation (a lane owns a query), where
// delta_q = sum_k P[q,k] * dP[q,k] (equal to dO_q . O_q, so O is never read) is a lane-local sum, and writes dQ;
// pass B repeats the dK/dV kernel's tile loop on the staged tiles.  HBM traffic: four tiles in, three out.
template <int ND, int NW, int MINW = 1>  // NW waves share the staged tiles; wave w owns query / key blocks [w*4/NW, (w+1)*4/NW)
__global__ __launch_bounds__(64 * NW, MINW) void attn_bwd_window_mfma(const AttnParams p) {
  using G = Geo<ND>;
  constexpr int HD = G::HD, R = 64, PK = G::PK, NB = 4 / NW;  // NB 16-row blocks per wave
  __shared__ __attribute__((aligned(16))) bf16_t lds_q[R * PK];
  __shared__ __attribute__((aligned(16))) bf16_t lds_k[R * PK];
  __shared__ __attribute__((aligned(16))) bf16_t lds_v[R * PK];
  __shared__ __attribute__((aligned(16))) bf16_t lds_do[R * PK];
  __shared__ __attribute__((aligned(16))) float lds_lse[R];
  __shared__ __attribute__((aligned(16))) float lds_delta[R];

  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg];
  const int L = min(p.cu[seg + 1] - s0, R);
  if (L <= 0) return;
  const int l = threadIdx.x & 63, wv = threadIdx.x >> 6, g = l >> 4, r = l & 15;
  const float c = p.scale * LOG2E;
  {
    TileStager<ND, R, PK, 64 * NW> sq, sk, sv, sdo;
    sq.init(p.q_stride);
    sk.init(p.k_stride);
    sv.init(p.v_stride);
    sdo.init(p.do_stride);
    sq.load(static_cast<const bf16_t*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD, L);
    sk.load(static_cast<const bf16_t*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD, L);
    sv.load(static_cast<const bf16_t*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD, L);
    sdo.load(static_cast<const bf16_t*>(p.d_o) + (int64_t)s0 * p.do_stride + (int64_t)h * HD, L);
    if (wv == 0) lds_lse[l] = l < L ? p.lse[(int64_t)h * p.total + s0 + l] * LOG2E : INFINITY;  // +inf => p = 0 for padded queries
    sq.scale(c);  // the Q tile holds Q * scale * log2(e): scores leave the MFMA in log2 units
    sq.store(lds_q);
    sk.store(lds_k);
    sv.store(lds_v);
    sdo.store(lds_do);
  }
  __syncthreads();

  // ---- pass A: dQ^T += K^T dS^T per 16-query block, keys in two chunks of 32
  {
    RowFrag<ND> ka[2][2], va[2][2];
    bf16x8 kt[2][ND];
#pragma unroll
    for (int kc = 0; kc < 2; ++kc) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        load_rowfrag_lds<ND, PK>(ka[kc][t], lds_k, kc * 32 + t * 16 + r, g);
        load_rowfrag_lds<ND, PK>(va[kc][t], lds_v, kc * 32 + t * 16 + r, g);
      }
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        const int off = (kc * 32 + 4 * g + (r >> 2)) * PK + 16 * d + 4 * (r & 3);
        kt[kc][d] = tr_pair(lds_k + off, lds_k + off + 16 * PK);
      }
    }
    bf16_t* DQ = static_cast<bf16_t*>(p.dq) + (int64_t)s0 * p.dq_stride + (int64_t)h * HD;
    float* DELTA = p.delta + (int64_t)h * p.total + s0;
#pragma unroll 1
    for (int qb = wv * NB; qb < (wv + 1) * NB; ++qb) {
      if (qb * 16 >= L) break;
      const int qi = qb * 16 + r;
      RowFrag<ND> qf, dof;
      load_rowfrag_lds<ND, PK>(qf, lds_q, qi, g);
      load_rowfrag_lds<ND, PK>(dof, lds_do, qi, g);
      const float neg_lse2 = -lds_lse[qi];
      f32x4 e[2][2], dp[2][2];
      float part = 0.f;
#pragma unroll
      for (int kc = 0; kc < 2; ++kc)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const f32x4 sc = dot_frag<ND>(ka[kc][t], qf);  // S[q = qb*16+r][key = kc*32+t*16+4g+i]
          dp[kc][t] = dot_frag<ND>(va[kc][t], dof);      // dP, same layout
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float x = __builtin_amdgcn_exp2f(sc[i] + neg_lse2);
            if (kc * 32 + t * 16 + 4 * g + i >= L) x = 0.f;  // keys past the segment end
            e[kc][t][i] = x;
            part = __builtin_fmaf(x, dp[kc][t][i], part);
          }
        }
      part += __shfl_xor(part, 16);
      part += __shfl_xor(part, 32);  // lanes r, r+16, r+32, r+48 share query qb*16+r
      if (g == 0) {
        lds_delta[qi] = part;
        if (qi < L) DELTA[qi] = part;
      }
      f32x4 dq[ND];
#pragma unroll
      for (int d = 0; d < ND; ++d) dq[d] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < 2; ++kc) {
        f32x4 ds[2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) ds[t][i] = e[kc][t][i] * (dp[kc][t][i] - part);
        const bf16x8 dsb = pack8(ds[0], ds[1]);
#pragma unroll
        for (int d = 0; d < ND; ++d) dq[d] = mfma32(kt[kc][d], dsb, dq[d]);
      }
      if (qi < L) {
#pragma unroll
        for (int d = 0; d < ND; ++d) {
          bf16x4 a;
#pragma unroll
          for (int i = 0; i < 4; ++i) a[i] = (bf16_t)(dq[d][i] * p.scale);
          *reinterpret_cast<bf16x4*>(DQ + (int64_t)qi * p.dq_stride + 16 * d + 4 * g) = a;
        }
      }
    }
    for (int q = 16 * ((L + 15) / 16) + (int)threadIdx.x; q < R; q += 64 * NW) lds_delta[q] = 0.f;  // query blocks that were skipped
  }
  __syncthreads();

  // ---- pass B: dV^T += dO^T P, dK^T += Q^T dS per 16-key block, queries in two tiles of 32
  {
    RowFrag<ND> kf[NB], vf[NB];
    f32x4 dk[NB][ND], dv[NB][ND];
    const int key0 = wv * NB * 16;  // this wave's first key
#pragma unroll
    for (int kb = 0; kb < NB; ++kb) {
      load_rowfrag_lds<ND, PK>(kf[kb], lds_k, key0 + kb * 16 + r, g);
      load_rowfrag_lds<ND, PK>(vf[kb], lds_v, key0 + kb * 16 + r, g);
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        dk[kb][d] = f32x4{0.f, 0.f, 0.f, 0.f};
        dv[kb][d] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
    }
#pragma unroll 1
    for (int qs = 0; qs < L; qs += 32) {
      const bf16_t* tq = lds_q + qs * PK;
      const bf16_t* tdo = lds_do + qs * PK;
      RowFrag<ND> qa[2], da[2];
      bf16x8 qt[ND], dt_[ND];
      f32x4 lse2[2], dl[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        load_rowfrag_lds<ND, PK>(qa[t], tq, t * 16 + r, g);
        load_rowfrag_lds<ND, PK>(da[t], tdo, t * 16 + r, g);
        lse2[t] = *reinterpret_cast<const f32x4*>(lds_lse + qs + t * 16 + 4 * g);
        dl[t] = *reinterpret_cast<const f32x4*>(lds_delta + qs + t * 16 + 4 * g);
      }
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        const int off = (4 * g + (r >> 2)) * PK + 16 * d + 4 * (r & 3);
        qt[d] = tr_pair(tq + off, tq + off + 16 * PK);
        dt_[d] = tr_pair(tdo + off, tdo + off + 16 * PK);
      }
#pragma unroll
      for (int kb = 0; kb < NB; ++kb) {
        f32x4 pv[2], ds[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const f32x4 sc = dot_frag<ND>(qa[t], kf[kb]);   // S[q = qs+t*16+4g+i][key = kb*16+r]
          const f32x4 dpp = dot_frag<ND>(da[t], vf[kb]);  // dP, same layout
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float x = __builtin_amdgcn_exp2f(sc[i] - lse2[t][i]);
            pv[t][i] = x;
            ds[t][i] = x * (dpp[i] - dl[t][i]);
          }
        }
        const bf16x8 pb = pack8(pv[0], pv[1]);
        const bf16x8 dsb = pack8(ds[0], ds[1]);
#pragma unroll
        for (int d = 0; d < ND; ++d) {
          dv[kb][d] = mfma32(dt_[d], pb, dv[kb][d]);
          dk[kb][d] = mfma32(qt[d], dsb, dk[kb][d]);
        }
      }
    }
    bf16_t* DK = static_cast<bf16_t*>(p.dk) + (int64_t)s0 * p.dk_stride + (int64_t)h * HD;
    bf16_t* DV = static_cast<bf16_t*>(p.dv) + (int64_t)s0 * p.dv_stride + (int64_t)h * HD;
#pragma unroll
    for (int kb = 0; kb < NB; ++kb) {
      const int ki = key0 + kb * 16 + r;
      if (ki < L) {
#pragma unroll
        for (int d = 0; d < ND; ++d) {
          bf16x4 a, b;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            a[i] = (bf16_t)(dk[kb][d][i] * LN2);  // dS^T (Q scale log2e) / log2e
            b[i] = (bf16_t)dv[kb][d][i];
          }
          *reinterpret_cast<bf16x4*>(DK + (int64_t)ki * p.dk_stride + 16 * d + 4 * g) = a;
          *reinterpret_cast<bf16x4*>(DV + (int64_t)ki * p.dv_stride + 16 * d + 4 * g) = b;
        }
      }
    }
  }
}

// ================================================================================================
// fp32 parity kernels: one lane per row, 32-row tiles of the other side broadcast from LDS.
template <int HD>
__global__ __launch_bounds__(64) void attn_fwd_f32(const AttnParams p) {
  constexpr int TB = 32;
  __shared__ float sk[TB * HD];
  __shared__ float sv[TB * HD];
  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int q0 = blockIdx.x * 64;
  if (q0 >= L) return;
  const int qi = q0 + threadIdx.x;
  const bool valid = qi < L;
  const float* Q = static_cast<const float*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD;
  const float* K = static_cast<const float*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const float* V = static_cast<const float*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;
  float qr[HD], acc[HD];
#pragma unroll
  for (int j = 0; j < HD; ++j) {
    qr[j] = valid ? Q[(int64_t)qi * p.q_stride + j] : 0.f;
    acc[j] = 0.f;
  }
  float m = -INFINITY, lsum = 0.f;
  for (int k0 = 0; k0 < L; k0 += TB) {
    const int nk = min(TB, L - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < TB * HD; i += 64) {
      const int rr = i / HD, j = i % HD;
      sk[i] = rr < nk ? K[(int64_t)(k0 + rr) * p.k_stride + j] : 0.f;
      sv[i] = rr < nk ? V[(int64_t)(k0 + rr) * p.v_stride + j] : 0.f;
    }
    __syncthreads();
    float s[TB];
    float mx = m;
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      float d = 0.f;
#pragma unroll
      for (int j = 0; j < HD; ++j) d += qr[j] * sk[t * HD + j];
      s[t] = t < nk ? d * p.scale : -INFINITY;
      mx = fmaxf(mx, s[t]);
    }
    const float alpha = expf(m - mx);
    m = mx;
    lsum *= alpha;
#pragma unroll
    for (int j = 0; j < HD; ++j) acc[j] *= alpha;
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      const float e = expf(s[t] - mx);
      lsum += e;
#pragma unroll
      for (int j = 0; j < HD; ++j) acc[j] += e * sv[t * HD + j];
    }
  }
  if (valid) {
    float* O = static_cast<float*>(p.out) + (int64_t)(s0 + qi) * p.o_stride + (int64_t)h * HD;
    const float inv = 1.f / lsum;
#pragma unroll
    for (int j = 0; j < HD; ++j) O[j] = acc[j] * inv;
    p.lse[(int64_t)h * p.total + s0 + qi] = m + logf(lsum);
  }
}

template <int HD>
__global__ __launch_bounds__(64) void attn_bwd_dq_f32(const AttnParams p) {
  constexpr int TB = 32;
  __shared__ float sk[TB * HD];
  __shared__ float sv[TB * HD];
  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int q0 = blockIdx.x * 64;
  if (q0 >= L) return;
  const int qi = q0 + threadIdx.x;
  const bool valid = qi < L;
  const float* Q = static_cast<const float*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD;
  const float* K = static_cast<const float*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const float* V = static_cast<const float*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;
  const float* DO = static_cast<const float*>(p.d_o) + (int64_t)s0 * p.do_stride + (int64_t)h * HD;
  float qr[HD], dor[HD], acc[HD];
#pragma unroll
  for (int j = 0; j < HD; ++j) {
    qr[j] = valid ? Q[(int64_t)qi * p.q_stride + j] : 0.f;
    dor[j] = valid ? DO[(int64_t)qi * p.do_stride + j] : 0.f;
    acc[j] = 0.f;
  }
  const float lse = valid ? p.lse[(int64_t)h * p.total + s0 + qi] : INFINITY;
  const float dl = valid ? p.delta[(int64_t)h * p.total + s0 + qi] : 0.f;
  for (int k0 = 0; k0 < L; k0 += TB) {
    const int nk = min(TB, L - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < TB * HD; i += 64) {
      const int rr = i / HD, j = i % HD;
      sk[i] = rr < nk ? K[(int64_t)(k0 + rr) * p.k_stride + j] : 0.f;
      sv[i] = rr < nk ? V[(int64_t)(k0 + rr) * p.v_stride + j] : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < nk; ++t) {
      float d = 0.f, dp = 0.f;
#pragma unroll
      for (int j = 0; j < HD; ++j) {
        d += qr[j] * sk[t * HD + j];
        dp += dor[j] * sv[t * HD + j];
      }
      const float ds = expf(d * p.scale - lse) * (dp - dl);
#pragma unroll
      for (int j = 0; j < HD; ++j) acc[j] += ds * sk[t * HD + j];
    }
  }
  if (valid) {
    float* DQ = static_cast<float*>(p.dq) + (int64_t)(s0 + qi) * p.dq_stride + (int64_t)h * HD;
#pragma unroll
    for (int j = 0; j < HD; ++j) DQ[j] = acc[j] * p.scale;
  }
}

template <int HD>
__global__ __launch_bounds__(64) void attn_bwd_dkdv_f32(const AttnParams p) {
  constexpr int TB = 32;
  __shared__ float sq[TB * HD];
  __shared__ float sdo[TB * HD];
  __shared__ float slse[TB];
  __shared__ float sdl[TB];
  int seg, h;
  seg_and_head(p, seg, h);
  const int s0 = p.cu[seg], L = p.cu[seg + 1] - s0;
  const int kb0 = blockIdx.x * 64;
  if (kb0 >= L) return;
  const int ki = kb0 + threadIdx.x;
  const bool valid = ki < L;
  const float* Q = static_cast<const float*>(p.q) + (int64_t)s0 * p.q_stride + (int64_t)h * HD;
  const float* K = static_cast<const float*>(p.k) + (int64_t)s0 * p.k_stride + (int64_t)h * HD;
  const float* V = static_cast<const float*>(p.v) + (int64_t)s0 * p.v_stride + (int64_t)h * HD;
  const float* DO = static_cast<const float*>(p.d_o) + (int64_t)s0 * p.do_stride + (int64_t)h * HD;
  float kr[HD], vr[HD], dk[HD], dv[HD];
#pragma unroll
  for (int j = 0; j < HD; ++j) {
    kr[j] = valid ? K[(int64_t)ki * p.k_stride + j] : 0.f;
    vr[j] = valid ? V[(int64_t)ki * p.v_stride + j] : 0.f;
    dk[j] = 0.f;
    dv[j] = 0.f;
  }
  for (int qs = 0; qs < L; qs += TB) {
    const int nq = min(TB, L - qs);
    __syncthreads();
    for (int i = threadIdx.x; i < TB * HD; i += 64) {
      const int rr = i / HD, j = i % HD;
      sq[i] = rr < nq ? Q[(int64_t)(qs + rr) * p.q_stride + j] : 0.f;
      sdo[i] = rr < nq ? DO[(int64_t)(qs + rr) * p.do_stride + j] : 0.f;
    }
    if (threadIdx.x < TB) {
      const bool ok = (int)threadIdx.x < nq;
      slse[threadIdx.x] = ok ? p.lse[(int64_t)h * p.total + s0 + qs + threadIdx.x] : INFINITY;
      sdl[threadIdx.x] = ok ? p.delta[(int64_t)h * p.total + s0 + qs + threadIdx.x] : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < nq; ++t) {
      float d = 0.f, dp = 0.f;
#pragma unroll
      for (int j = 0; j < HD; ++j) {
        d += sq[t * HD + j] * kr[j];
        dp += sdo[t * HD + j] * vr[j];
      }
      const float e = expf(d * p.scale - slse[t]);
      const float ds = e * (dp - sdl[t]);
#pragma unroll
      for (int j = 0; j < HD; ++j) {
        dv[j] += e * sdo[t * HD + j];
        dk[j] += ds * sq[t * HD + j];
      }
    }
  }
  if (valid) {
    float* DK = static_cast<float*>(p.dk) + (int64_t)(s0 + ki) * p.dk_stride + (int64_t)h * HD;
    float* DV = static_cast<float*>(p.dv) + (int64_t)(s0 + ki) * p.dv_stride + (int64_t)h * HD;
#pragma unroll
    for (int j = 0; j < HD; ++j) {
      DK[j] = dk[j] * p.scale;
      DV[j] = dv[j];
    }
  }
}

// ------------------------------------------------------------------------------------------------
constexpr int WIDE_MIN_SEQLEN = 512;  // from here on the 64-rows-per-wave kernels fill their work-groups well enough
inline int pick_waves(int max_seqlen) { return max_seqlen <= 64 ? 1 : (max_seqlen <= 128 ? 2 : 4); }

template <int ND>
int launch_fwd_mfma(const AttnParams& p, int n_seg, int max_seqlen, hipStream_t s) {
  const int nw = pick_waves(max_seqlen);
  dim3 grid((unsigned)((max_seqlen + 64 * nw - 1) / (64 * nw)), (unsigned)n_seg, (unsigned)p.nheads);
  if (nw == 1 && ND <= 5) {
    // windows: two waves x 32 queries share the staged K / V tiles (more waves per CU hide the load latency)
    AttnParams pw = p;
    if (grid.x == 1 && ((int64_t)n_seg * p.nheads) % 8 == 0) pw.seg_major = 2;  // heads of a segment together on one XCD
    if constexpr (ND <= 5) hipLaunchKernelGGL((attn_fwd_mfma<ND, 2, 64, false, 2, 4>), grid, 128, 0, s, pw);
  } else if (nw == 1) hipLaunchKernelGGL((attn_fwd_mfma<ND, 1, 64, false>), grid, 64, 0, s, p);
  else if (nw == 2) hipLaunchKernelGGL((attn_fwd_mfma<ND, 2, 64, false>), grid, 128, 0, s, p);
  else if constexpr (ND <= 5) {
    // long segments: 8 waves x 32 queries, <= 128 registers, so that four waves share a SIMD and cover each
    // other's MFMA -> softmax -> MFMA dependency stalls
    // all heads of a segment are neighbours in the launch order: with the caller's longest-first segment order
    // the work-groups then start in order of decreasing run time
    AttnParams pl = p;
    pl.seg_major = 1;  // n_seg fits gridDim.z: checked at the entry point
    dim3 gl = pl.seg_major ? dim3(grid.x, grid.z, grid.y) : grid;
    if constexpr (ND == 5) {
      if (max_seqlen >= WIDE_MIN_SEQLEN) {  // 64 queries per wave, 512 per work-group
        hipLaunchKernelGGL((attn_fwd_x32<ND>), dim3((unsigned)((max_seqlen + 511) / 512), gl.y, gl.z), 512, 0, s, pl);
        MVIT_CHECK_LAUNCH("attn_fwd");
        return MVIT_OK;
      }
    }
    hipLaunchKernelGGL((attn_fwd_mfma<ND, 8, 32, true, 2, 4>), gl, 512, 0, s, pl);
  }
  else hipLaunchKernelGGL((attn_fwd_mfma<ND, 4, 32, true>), grid, 256, 0, s, p);  // head_dim 128: register budget
  MVIT_CHECK_LAUNCH("attn_fwd");
  return MVIT_OK;
}
using G5 = Geo<5>;
template <int ND>
int launch_bwd_mfma(const AttnParams& p, int n_seg, int max_seqlen, hipStream_t s) {
  // short segments (windows): one work-group does the whole backward of a (segment, head); long ones: 8 waves x 32 rows
  if (max_seqlen <= 64) {
    dim3 grid(1, (unsigned)n_seg, (unsigned)p.nheads);
    if constexpr (ND <= 5) {
      // four waves x 16 rows: ~160 registers, three work-groups (12 waves) per CU to cover the load -> MFMA -> store latency
      AttnParams pw = p;
      if (((int64_t)n_seg * p.nheads) % 8 == 0) pw.seg_major = 2;  // heads of a segment together on one XCD
      hipLaunchKernelGGL((attn_bwd_window_mfma<ND, 4, 2>), grid, 256, 0, s, pw);  // computes delta itself
    } else {
      hipLaunchKernelGGL((attn_bwd_dkdv_mfma<ND, 1, 4>), grid, 64, 0, s, p);
      hipLaunchKernelGGL((attn_bwd_dq_mfma<ND, 1, 4>), grid, 64, 0, s, p);
    }
  } else if (max_seqlen <= 128) {
    dim3 grid(1, (unsigned)n_seg, (unsigned)p.nheads);
    hipLaunchKernelGGL((attn_bwd_dkdv_mfma<ND, 2, 4>), grid, 128, 0, s, p);
    hipLaunchKernelGGL((attn_bwd_dq_mfma<ND, 2, 4>), grid, 128, 0, s, p);
  } else {
    dim3 grid((unsigned)((max_seqlen + 255) / 256), (unsigned)n_seg, (unsigned)p.nheads);
    AttnParams pl = p;
    pl.seg_major = 1;  // as in the forward: segment-major launch order
    dim3 gl = pl.seg_major ? dim3(grid.x, grid.z, grid.y) : grid;
    if (ND == 5 && max_seqlen >= WIDE_MIN_SEQLEN) {
      if constexpr (ND == 5) {
        // the dq buffer holds the pre-scaled queries until the dQ kernel overwrites it with the result
        const int64_t nstat = (int64_t)p.nheads * p.total;
        pl.q_scaled = p.dq;
        pl.qs_stride = p.dq_stride;
        pl.nlse2 = p.delta + nstat;
        pl.ndelta = p.delta + 2 * nstat;
        const int cols = p.nheads * G5::HD;
        const int64_t nchunk = p.total * (cols / 8);
        const unsigned pgrid = (unsigned)std::min<int64_t>(8192, (std::max(nchunk, nstat) + 255) / 256);
        hipLaunchKernelGGL(attn_bwd_prepare_kernel, dim3(pgrid), 256, 0, s, static_cast<const bf16_t*>(p.q), p.q_stride,
                           static_cast<bf16_t*>(p.dq), p.dq_stride, p.total, cols, p.scale * LOG2E, (const float*)p.lse,
                           (const float*)p.delta, p.delta + nstat, p.delta + 2 * nstat, nstat);
        hipLaunchKernelGGL((attn_bwd_dkdv_wide<ND>), gl, 256, 0, s, pl);
        hipLaunchKernelGGL((attn_bwd_dq_wide<ND>), gl, 256, 0, s, pl);
      }
    } else {
      hipLaunchKernelGGL((attn_bwd_dkdv_mfma<ND, 8, 2>), gl, 512, 0, s, pl);
      hipLaunchKernelGGL((attn_bwd_dq_mfma<ND, 8, 2>), gl, 512, 0, s, pl);
    }
  }
  MVIT_CHECK_LAUNCH("attn_bwd");
  return MVIT_OK;
}
template <int HD>
int launch_f32(const AttnParams& p, int n_seg, int max_seqlen, bool bwd, hipStream_t s) {
  dim3 grid((unsigned)((max_seqlen + 63) / 64), (unsigned)n_seg, (unsigned)p.nheads);
  if (!bwd) {
    hipLaunchKernelGGL((attn_fwd_f32<HD>), grid, 64, 0, s, p);
  } else {
    hipLaunchKernelGGL((attn_bwd_dkdv_f32<HD>), grid, 64, 0, s, p);
    hipLaunchKernelGGL((attn_bwd_dq_f32<HD>), grid, 64, 0, s, p);
  }
  MVIT_CHECK_LAUNCH("attn_f32");
  return MVIT_OK;
}

int check_common(const char* who, const int32_t* cu, int n_seg, int max_seqlen, int64_t total, int nheads, int head_dim,
                 int dtype, std::initializer_list<int64_t> strides, std::initializer_list<const void*> ptrs) {
  MVIT_REQUIRE(cu && n_seg >= 0 && max_seqlen >= 0 && total >= 0 && nheads > 0 && nheads <= 65535 && n_seg <= 65535,
               "%s: bad sizes (n_seg=%d max_seqlen=%d total=%lld nheads=%d)", who, n_seg, max_seqlen, (long long)total, nheads);
  MVIT_REQUIRE(dtype == MVIT_BF16 || dtype == MVIT_F32, "%s: dtype %d", who, dtype);
  MVIT_REQUIRE(head_dim == 32 || head_dim == 64 || head_dim == 80 || head_dim == 128, "%s: head_dim %d not built (32, 64, 80, 128)", who, head_dim);
  const int vec = dtype == MVIT_BF16 ? 8 : 1;
  for (int64_t st : strides)
    MVIT_REQUIRE(st >= (int64_t)nheads * head_dim && st % vec == 0, "%s: row stride %lld must cover %d heads and be a multiple of %d", who, (long long)st, nheads, vec);
  if (n_seg == 0 || max_seqlen == 0 || total == 0) return MVIT_OK;  // nothing to do: empty tensors have no address to check
  for (const void* q : ptrs) MVIT_REQUIRE(q && mvit_aligned16(q), "%s: null or unaligned pointer", who);
  return MVIT_OK;
}

// Do two sets of `rows` rows of `width` bytes, starting at a and b with row pitches pa and pb (bytes), share a byte?
// Exact when the pitches are equal (tensors interleaved in one buffer, like q | k | v, are told apart); otherwise the
// two address ranges are compared as wholes.
bool strided_rows_overlap(const void* a, int64_t pa, const void* b, int64_t pb, int64_t rows, int64_t width) {
  const int64_t x = (int64_t)reinterpret_cast<uintptr_t>(a), y = (int64_t)reinterpret_cast<uintptr_t>(b);
  const int64_t ea = x + (rows - 1) * pa + width, eb = y + (rows - 1) * pb + width;
  if (ea <= y || eb <= x) return false;
  if (pa != pb || pa < width) return true;
  // equal pitch: row i of a starts at x + i*pa; relative to b's rows the column offset is constant
  int64_t off = (x - y) % pa;
  if (off < 0) off += pa;
  // a's row covers [off, off + width) modulo the pitch; b's rows cover [0, width)
  return off < width || off + width > pa;
}

}  // namespace

extern "C" {

int64_t mvit_attn_bwd_delta_elems(int max_seqlen, int64_t total, int nheads, int head_dim, int dtype) {
  const bool wide = dtype == MVIT_BF16 && head_dim == 80 && max_seqlen >= WIDE_MIN_SEQLEN;
  return (wide ? 3 : 1) * (int64_t)nheads * total;
}

int mvit_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens,
                  const int32_t* seg_order, int n_seg, int max_seqlen, int64_t total, int nheads, int head_dim, int64_t q_stride, int64_t k_stride,
                  int64_t v_stride, int64_t o_stride, float scale, int dtype, mvit_stream_t stream) {
  if (int rc = check_common("attn_fwd", cu_seqlens, n_seg, max_seqlen, total, nheads, head_dim, dtype,
                            {q_stride, k_stride, v_stride, o_stride}, {q, k, v, o, (const void*)lse}))
    return rc;
  if (n_seg == 0 || max_seqlen == 0 || total == 0) return MVIT_OK;
  AttnParams p = {};
  p.q = q; p.k = k; p.v = v; p.out = o; p.lse = lse; p.cu = cu_seqlens; p.order = seg_order; p.total = total; p.nheads = nheads;
  p.q_stride = q_stride; p.k_stride = k_stride; p.v_stride = v_stride; p.o_stride = o_stride; p.scale = scale;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype == MVIT_BF16) {
    switch (head_dim) {
      case 32: return launch_fwd_mfma<2>(p, n_seg, max_seqlen, s);
      case 64: return launch_fwd_mfma<4>(p, n_seg, max_seqlen, s);
      case 80: return launch_fwd_mfma<5>(p, n_seg, max_seqlen, s);
      default: return launch_fwd_mfma<8>(p, n_seg, max_seqlen, s);
    }
  }
  switch (head_dim) {
    case 32: return launch_f32<32>(p, n_seg, max_seqlen, false, s);
    case 64: return launch_f32<64>(p, n_seg, max_seqlen, false, s);
    case 80: return launch_f32<80>(p, n_seg, max_seqlen, false, s);
    default: return launch_f32<128>(p, n_seg, max_seqlen, false, s);
  }
}

int mvit_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse, void* dq,
                  void* dk, void* dv, float* delta, int64_t delta_elems, const int32_t* cu_seqlens, const int32_t* seg_order, int n_seg, int max_seqlen,
                  int64_t total, int nheads, int head_dim, int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                  int64_t do_stride, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride, float scale, int dtype,
                  mvit_stream_t stream) {
  if (int rc = check_common("attn_bwd", cu_seqlens, n_seg, max_seqlen, total, nheads, head_dim, dtype,
                            {q_stride, k_stride, v_stride, o_stride, do_stride, dq_stride, dk_stride, dv_stride},
                            {q, k, v, o, d_o, (const void*)lse, dq, dk, dv, (const void*)delta}))
    return rc;
  if (total == 0) return MVIT_OK;
  // the long-segment kernels keep three arrays of row statistics in the workspace and park the pre-scaled queries in dq
  const bool wide = dtype == MVIT_BF16 && head_dim == 80 && max_seqlen >= WIDE_MIN_SEQLEN;
  const int64_t need = (wide ? 3 : 1) * (int64_t)nheads * total;
  MVIT_REQUIRE(delta_elems >= need, "attn_bwd: the delta workspace holds %lld floats, this call needs %lld (%d x nheads x total)",
               (long long)delta_elems, (long long)need, wide ? 3 : 1);
  {
    const int64_t e = dtype == MVIT_BF16 ? 2 : 4, width = (int64_t)nheads * head_dim * e;
    const struct { const void* ptr; int64_t stride; const char* name; } ins[] = {{q, q_stride, "q"}, {k, k_stride, "k"}, {v, v_stride, "v"}, {o, o_stride, "o"}, {d_o, do_stride, "d_o"}};
    const struct { const void* ptr; int64_t stride; const char* name; } outs[] = {{dq, dq_stride, "dq"}, {dk, dk_stride, "dk"}, {dv, dv_stride, "dv"}};
    for (const auto& w : outs)
      for (const auto& r : ins)
        MVIT_REQUIRE(!strided_rows_overlap(w.ptr, w.stride * e, r.ptr, r.stride * e, total, width),
                     "attn_bwd: %s overlaps %s (outputs are written, and dq is used as scratch, before all inputs have been read)", w.name, r.name);
  }
  if (n_seg == 0 || max_seqlen == 0 || total == 0) return MVIT_OK;
  AttnParams p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.d_o = d_o; p.lse = const_cast<float*>(lse); p.delta = delta;
  p.dq = dq; p.dk = dk; p.dv = dv; p.cu = cu_seqlens; p.order = seg_order; p.total = total; p.nheads = nheads;
  p.q_stride = q_stride; p.k_stride = k_stride; p.v_stride = v_stride; p.o_stride = o_stride; p.do_stride = do_stride;
  p.dq_stride = dq_stride; p.dk_stride = dk_stride; p.dv_stride = dv_stride; p.scale = scale;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int vecw = dtype == MVIT_BF16 ? 8 : 4;
  const size_t part_bytes = (size_t)16 * nheads * (head_dim / vecw) * sizeof(float);
  if (dtype == MVIT_BF16 && max_seqlen <= 64 && head_dim <= 80) {
    // the window kernel derives delta from P and dP itself
  } else if (head_dim % vecw == 0 && o_stride % vecw == 0 && do_stride % vecw == 0 && part_bytes <= 48 * 1024 && mvit_aligned16(o) && mvit_aligned16(d_o)) {
    const int dgrid = (int)((total + 15) / 16);
    if (dtype == MVIT_BF16)
      hipLaunchKernelGGL((attn_delta_rows_kernel<bf16_t>), dgrid, 256, part_bytes, s, (const bf16_t*)o, (const bf16_t*)d_o, delta, total, nheads, head_dim, o_stride, do_stride);
    else
      hipLaunchKernelGGL((attn_delta_rows_kernel<float>), dgrid, 256, part_bytes, s, (const float*)o, (const float*)d_o, delta, total, nheads, head_dim, o_stride, do_stride);
  } else {
    const int64_t npairs = total * nheads;
    const int dgrid = (int)((npairs + 255) / 256);
    if (dtype == MVIT_BF16)
      hipLaunchKernelGGL((attn_delta_kernel<bf16_t>), dgrid, 256, 0, s, (const bf16_t*)o, (const bf16_t*)d_o, delta, total, nheads, head_dim, o_stride, do_stride);
    else
      hipLaunchKernelGGL((attn_delta_kernel<float>), dgrid, 256, 0, s, (const float*)o, (const float*)d_o, delta, total, nheads, head_dim, o_stride, do_stride);
  }
  MVIT_CHECK_LAUNCH("attn_delta");
  if (dtype == MVIT_BF16) {
    switch (head_dim) {
      case 32: return launch_bwd_mfma<2>(p, n_seg, max_seqlen, s);
      case 64: return launch_bwd_mfma<4>(p, n_seg, max_seqlen, s);
      case 80: return launch_bwd_mfma<5>(p, n_seg, max_seqlen, s);
      default: return launch_bwd_mfma<8>(p, n_seg, max_seqlen, s);
    }
  }
  switch (head_dim) {
    case 32: return launch_f32<32>(p, n_seg, max_seqlen, true, s);
    case 64: return launch_f32<64>(p, n_seg, max_seqlen, true, s);
    case 80: return launch_f32<80>(p, n_seg, max_seqlen, true, s);
    default: return launch_f32<128>(p, n_seg, max_seqlen, true, s);
  }
}

}  // extern "C"
