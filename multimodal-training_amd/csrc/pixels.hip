// Decoded RGB frames (uint8) -> rows of pixel_values for gfx950: rescale, normalise and cut into 14x14x2 patches in
// the row order the vision tower expects, for a whole batch of images and videos in one launch.  HBM-bound: every
// output row is 1176 values (4704 bytes in fp32) made from 2 x 588 input bytes (588 for a still image, whose one
// frame fills both halves).  A work-group makes the four rows of a 2x2 merge block, one wave per row: it stages
// the block's 28x28 pixel square (28 lines of 84 bytes = 21 aligned dwords) in LDS with dword loads, reads single
// bytes from there, and the output leaves as 16-byte (fp32) or 8-byte (bf16) stores.
//
// The arithmetic is that of the image processor the reference calls (transformers 4.57.0,
// Qwen2VLImageProcessor._preprocess: rescale in float64 rounded to float32, then (x - mean) / std in float32
// with an IEEE division), so fp32 results can be compared bit for bit with a numpy restatement.
#include "mvit_common.h"

namespace {

constexpr int PATCH = 14, TPS = 2, ROW = MVIT_PIXEL_ROW;
constexpr int PLANE = PATCH * PATCH;   // 196 values of one (channel, frame) plane of a row
constexpr int QUADS = PLANE / 4;       // 49 groups of four consecutive values per plane

struct Norm {
  double rescale;
  float mean[3], std[3];
};

__device__ __forceinline__ int find_image(const mvit_image* t, int n, int64_t row) {
  int lo = 0, hi = n;  // invariant: t[lo].first_row <= row < t[hi].first_row
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (t[mid].first_row <= row) lo = mid;
    else hi = mid;
  }
  return lo;
}

__device__ __forceinline__ void store4(float* dst, const float (&v)[4]) {
  *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void store4(bf16_t* dst, const float (&v)[4]) {
  *reinterpret_cast<bf16x4*>(dst) = bf16x4{from_f32<bf16_t>(v[0]), from_f32<bf16_t>(v[1]), from_f32<bf16_t>(v[2]), from_f32<bf16_t>(v[3])};
}

constexpr int SQ = 2 * PATCH;          // a merge block is a square of 28 x 28 pixels
constexpr int SQ_LINE = SQ * 3;        // 84 bytes (21 dwords) per line of the square
constexpr int SQ_DWORDS = SQ * SQ_LINE / 4;  // 588

template <typename TO>
__global__ __launch_bounds__(256) void patchify_kernel(const mvit_image* __restrict__ images, int n_images, TO* __restrict__ out,
                                                       int64_t total_rows, Norm nm) {
#pragma clang fp contract(off)
  // a byte has 256 values: the work-group computes the result for each of them and each channel once (exact
  // arithmetic, three divisions per thread) and every element of its rows is then a byte read and a table lookup
  __shared__ float lut[3][256];
  __shared__ __attribute__((aligned(16))) uint32_t square[TPS][SQ_DWORDS];  // the block's pixels, one copy per frame of the pair
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    const float x = (float)((double)(int)threadIdx.x * nm.rescale);
    lut[c][threadIdx.x] = (x - nm.mean[c]) / nm.std[c];
  }
  // everything up to the barrier is the same for the whole work-group: its four rows are one merge block
  const int64_t row0 = (int64_t)blockIdx.x * 4;
  const mvit_image im = images[find_image(images, n_images, row0)];
  const int gh = im.height / PATCH, gw = im.width / PATCH;
  const int per_t = gh * gw;
  const int64_t local = (row0 - im.first_row) & ~(int64_t)3;
  bool ok = row0 < total_rows && im.frames > 0 && gh > 0 && gw > 0 && !((gh | gw) & 1);  // malformed entry: nothing is read
  const int t = ok ? (int)(local / per_t) : 0, rem = ok ? (int)(local % per_t) : 0;
  ok = ok && t * TPS < im.frames;  // first_row entries that promise more rows than the frames give
  // rem = ((block row * (gw / 2) + block column) * 2 + row in block) * 2 + column in block
  const int blk = rem >> 2, hb = ok ? blk / (gw >> 1) : 0, wb = ok ? blk % (gw >> 1) : 0;
  const int64_t line = (int64_t)im.width * 3, frame_bytes = line * im.height;
  const int f0 = t * TPS, f1 = f0 + 1 < im.frames ? f0 + 1 : im.frames - 1;  // the last frame fills an odd count up
  if (ok) {
    const int nf = f1 != f0 ? 2 : 1;
    const uint8_t* corner = im.pixels + (int64_t)hb * SQ * line + wb * SQ_LINE;  // of the square in frame 0
    // width is a multiple of 28, so lines are a multiple of 84 bytes: with a 4-byte aligned frame buffer every
    // line of the square is 21 aligned dwords
    if ((reinterpret_cast<uintptr_t>(im.pixels) & 3u) == 0) {
      for (int i = threadIdx.x; i < nf * SQ_DWORDS; i += 256) {
        const int fi = i / SQ_DWORDS, j = i % SQ_DWORDS, y = j / (SQ_LINE / 4), xw = j % (SQ_LINE / 4);
        square[fi][j] = *reinterpret_cast<const uint32_t*>(corner + (fi ? f1 : f0) * frame_bytes + y * line + xw * 4);
      }
    } else {
      uint8_t* sq8 = reinterpret_cast<uint8_t*>(&square[0][0]);
      for (int i = threadIdx.x; i < nf * SQ_DWORDS * 4; i += 256) {
        const int fi = i / (SQ_DWORDS * 4), j = i % (SQ_DWORDS * 4), y = j / SQ_LINE, xb = j % SQ_LINE;
        sq8[i] = corner[(fi ? f1 : f0) * frame_bytes + y * line + xb];
      }
    }
  }
  __syncthreads();
  if (!ok) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint8_t* p0 = reinterpret_cast<const uint8_t*>(&square[0][0]) + (wave >> 1) * PATCH * SQ_LINE + (wave & 1) * PATCH * 3;
  const uint8_t* p1 = f1 != f0 ? p0 + SQ_DWORDS * 4 : p0;
  TO* dst = out + (row0 + wave) * ROW;
  for (int g = lane; g < 3 * QUADS; g += 64) {
    const int c = g / QUADS, q = g % QUADS;
    float v0[4], v1[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int p = 4 * q + e, off = (p / PATCH) * SQ_LINE + (p % PATCH) * 3 + c;
      v0[e] = lut[c][p0[off]];
      v1[e] = lut[c][p1[off]];
    }
    store4(dst + (c * TPS + 0) * PLANE + 4 * q, v0);
    store4(dst + (c * TPS + 1) * PLANE + 4 * q, v1);
  }
}

}  // namespace
// A window as the kernels use it: first tap and tap count forced into the table's row (ksize entries) and into the
// input axis, so that a table that breaks the entry point's contract cannot make a kernel read outside its arrays.
struct TapWindow {
  int xmin, n;
};
__device__ __forceinline__ TapWindow tap_window(const int32_t* __restrict__ bounds, int64_t x, int ksize, int64_t in_len) {
  int xmin = bounds[2 * x], n = bounds[2 * x + 1];
  xmin = max(0, min(xmin, (int)in_len - 1));
  n = max(0, min(n, min(ksize, (int)in_len - xmin)));
  return {xmin, n};
}


// ------------------------------------------------------------------------------------------------
// One resampling pass along the middle axis of a uint8 array [outer][in_len][inner] -> [outer][out_len][inner], with
// Pillow's 8-bit arithmetic (libImaging/Resample.c, ImagingResampleHorizontal_8bpc / Vertical_8bpc): per output
// coordinate a window of `bounds[2*x + 1]` input coordinates starting at `bounds[2*x]`, 22-bit fixed-point weights
// kk[x * ksize + i], an accumulator that starts at one half, an arithmetic shift and a clamp to 0..255.
// A thread makes four consecutive output bytes of one output coordinate (inner is the contiguous dimension: pixels
// times channels for the vertical pass, 3 channels for the horizontal one) or, when inner is not a multiple of four,
// four consecutive bytes of the flattened [out_len * inner] row, each with its own window.
constexpr int RESAMPLE_PRECISION_BITS = 22;
__device__ __forceinline__ unsigned clip8(int v) {
  v >>= RESAMPLE_PRECISION_BITS;
  return (unsigned)(v < 0 ? 0 : (v > 255 ? 255 : v));
}
template <bool WIDE>  // WIDE: inner % 4 == 0 and 4-byte aligned rows, the four bytes share one window
__global__ __launch_bounds__(256) void resample_pass_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t outer,
                                                            int64_t in_len, int64_t out_len, int64_t inner,
                                                            const int32_t* __restrict__ bounds, const int32_t* __restrict__ kk, int ksize) {
  const int64_t row_out = out_len * inner, row_in = in_len * inner;
  const int64_t quads = (row_out + 3) / 4;
  const int64_t total = outer * quads;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t o = i / quads, q = i % quads;
    const uint8_t* s = src + o * row_in;
    uint8_t* d = dst + o * row_out + 4 * q;
    if (WIDE) {
      const int64_t x = (4 * q) / inner, c = (4 * q) % inner;
      const TapWindow tw = tap_window(bounds, x, ksize, in_len);
      const int xmin = tw.xmin, n = tw.n;
      const int32_t* k = kk + x * ksize;
      int a0 = 1 << (RESAMPLE_PRECISION_BITS - 1), a1 = a0, a2 = a0, a3 = a0;
      for (int t = 0; t < n; ++t) {
        const unsigned w = *reinterpret_cast<const unsigned*>(s + (int64_t)(xmin + t) * inner + c);
        const int kt = k[t];
        a0 += (int)(w & 0xff) * kt;
        a1 += (int)((w >> 8) & 0xff) * kt;
        a2 += (int)((w >> 16) & 0xff) * kt;
        a3 += (int)(w >> 24) * kt;
      }
      *reinterpret_cast<unsigned*>(d) = clip8(a0) | (clip8(a1) << 8) | (clip8(a2) << 16) | (clip8(a3) << 24);
    } else {
      for (int b = 0; b < 4; ++b) {
        const int64_t e = 4 * q + b;
        if (e >= row_out) break;
        const int64_t x = e / inner, c = e % inner;
        const TapWindow tw = tap_window(bounds, x, ksize, in_len);
      const int xmin = tw.xmin, n = tw.n;
        const int32_t* k = kk + x * ksize;
        int a = 1 << (RESAMPLE_PRECISION_BITS - 1);
        for (int t = 0; t < n; ++t) a += (int)s[(int64_t)(xmin + t) * inner + c] * k[t];
        d[b] = (uint8_t)clip8(a);
      }
    }
  }
}

// The same pass for a short contiguous dimension (the horizontal pass: inner = channels): neighbouring output bytes have
// different windows and every tap is a single byte, so a work-group first copies its input row into LDS with aligned
// 4-byte loads and then reads the taps from there.  One work-group per row of the outer dimension; a thread makes whole
// pixels (up to four channels).
constexpr int RESAMPLE_LDS_BYTES = 60 * 1024, RESAMPLE_MAX_CHANNELS = 4;
__global__ __launch_bounds__(256) void resample_rows_lds_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t outer,
                                                                int64_t in_len, int64_t out_len, int inner,
                                                                const int32_t* __restrict__ bounds, const int32_t* __restrict__ kk, int ksize) {
  __shared__ __attribute__((aligned(16))) uint8_t row[RESAMPLE_LDS_BYTES + 8];
  const int64_t row_in = in_len * inner, row_out = out_len * inner;
  const uint8_t* src_end = src + outer * row_in;
  for (int64_t o = blockIdx.x; o < outer; o += gridDim.x) {
    const uint8_t* b = src + o * row_in;
    const int lead = (int)((uintptr_t)b & 3);  // the row starts `lead` bytes into an aligned word
    const uint8_t* a = b - lead;
    const int words = (int)((lead + row_in + 3) / 4);
    __syncthreads();  // the previous row has been consumed
    for (int j = threadIdx.x; j < words; j += 256) {
      const uint8_t* g = a + 4 * j;
      unsigned w;
      if (g >= src && g + 4 <= src_end) {
        w = *reinterpret_cast<const unsigned*>(g);
      } else {  // first / last word of the array: only the bytes that belong to it
        w = 0;
        for (int e = 0; e < 4; ++e)
          if (g + e >= src && g + e < src_end) w |= (unsigned)g[e] << (8 * e);
      }
      *reinterpret_cast<unsigned*>(row + 4 * j) = w;
    }
    __syncthreads();
    const uint8_t* r = row + lead;
    uint8_t* d = dst + o * row_out;
    // a thread makes whole pixels: the channels of a pixel share its window and its weights
    for (int x = threadIdx.x; x < (int)out_len; x += 256) {
      const TapWindow tw = tap_window(bounds, x, ksize, in_len);
      const int xmin = tw.xmin, n = tw.n;
      const int32_t* k = kk + (int64_t)x * ksize;
      int acc[RESAMPLE_MAX_CHANNELS];
#pragma unroll
      for (int c = 0; c < RESAMPLE_MAX_CHANNELS; ++c) acc[c] = 1 << (RESAMPLE_PRECISION_BITS - 1);
      const uint8_t* px = r + xmin * inner;
      for (int t = 0; t < n; ++t) {
        const int kt = k[t];
#pragma unroll
        for (int c = 0; c < RESAMPLE_MAX_CHANNELS; ++c)
          if (c < inner) acc[c] += (int)px[c] * kt;
        px += inner;
      }
#pragma unroll
      for (int c = 0; c < RESAMPLE_MAX_CHANNELS; ++c)
        if (c < inner) d[x * inner + c] = (uint8_t)clip8(acc[c]);
    }
  }
}

// The horizontal pass again, for windows of at most RESAMPLE_KMAX taps: a work-group owns 256 consecutive output
// coordinates and a strip of rows.  A thread keeps its coordinate's window and weights in registers for the whole strip
// (they are the same for every row, and fetching them per row was most of the row kernel's time); per row the
// work-group stages just the input bytes its 256 windows cover (two LDS buffers, one barrier per row) and every thread
// makes one pixel.  A work-group whose windows cover more than the LDS buffer (windows are the caller's) reads its taps
// from global memory instead.
constexpr int RESAMPLE_KMAX = 16, RESAMPLE_SPAN_BYTES = 8 * 1024;
__global__ __launch_bounds__(256) void resample_cols_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t outer,
                                                            int64_t in_len, int64_t out_len, int inner, const int32_t* __restrict__ bounds,
                                                            const int32_t* __restrict__ kk, int ksize, int rows_per_group) {
  __shared__ __attribute__((aligned(16))) uint8_t buf[2][RESAMPLE_SPAN_BYTES + 8];
  const int64_t row_in = in_len * inner, row_out = out_len * inner;
  const uint8_t* src_end = src + outer * row_in;
  const int x_first = blockIdx.x * 256, x_last = min(x_first + 255, (int)out_len - 1);
  const bool mine = x_first + (int)threadIdx.x <= x_last;
  const int x = mine ? x_first + (int)threadIdx.x : x_last;
  const TapWindow tw = tap_window(bounds, x, ksize, in_len);
      const int xmin = tw.xmin, n = tw.n;
  int k[RESAMPLE_KMAX];
#pragma unroll
  for (int t = 0; t < RESAMPLE_KMAX; ++t) k[t] = t < n ? kk[(int64_t)x * ksize + t] : 0;
  // bytes of a row that the work-group's windows cover (window starts and ends do not decrease with the coordinate
  // for a resampling; anything else shows up as a span that does not fit and takes the global path)
  int lo = bounds[2 * x_first] * inner, hi = (bounds[2 * x_last] + bounds[2 * x_last + 1]) * inner;
  bool fits = hi - lo + 4 <= RESAMPLE_SPAN_BYTES && xmin * inner >= lo && (xmin + n) * inner <= hi;
  fits = __syncthreads_and(fits);
  const int64_t o_begin = (int64_t)blockIdx.y * rows_per_group, o_end = min(o_begin + rows_per_group, outer);
  for (int64_t o = o_begin; o < o_end; ++o) {
    int acc[RESAMPLE_MAX_CHANNELS];
#pragma unroll
    for (int c = 0; c < RESAMPLE_MAX_CHANNELS; ++c) acc[c] = 1 << (RESAMPLE_PRECISION_BITS - 1);
    if (fits) {
      const uint8_t* b = src + o * row_in + lo;
      const int lead = (int)((uintptr_t)b & 3);
      const uint8_t* a = b - lead;
      const int words = (lead + (hi - lo) + 3) / 4;
      uint8_t* stage = buf[o & 1];
      for (int j = threadIdx.x; j < words; j += 256) {
        const uint8_t* g = a + 4 * j;
        unsigned w;
        if (g >= src && g + 4 <= src_end) {
          w = *reinterpret_cast<const unsigned*>(g);
        } else {  // first / last word of the array: only the bytes that belong to it
          w = 0;
          for (int e = 0; e < 4; ++e)
            if (g + e >= src && g + e < src_end) w |= (unsigned)g[e] << (8 * e);
        }
        *reinterpret_cast<unsigned*>(stage + 4 * j) = w;
      }
      __syncthreads();  // also: every thread is done with the buffer of two rows ago
      const uint8_t* px = stage + lead + (xmin * inner - lo);
#pragma unroll
      for (int t = 0; t < RESAMPLE_KMAX; ++t) {
        if (t >= ksize) break;
        const uint8_t* q = px + max(min(t, n - 1), 0) * inner;  // taps past the window have weight 0 and re-read its last one
#pragma unroll
        for (int c = 0; c < RESAMPLE_MAX_CHANNELS; ++c)
          if (c < inner) acc[c] += (int)q[c] * k[t];
      }
    } else {
      const uint8_t* px = src + o * row_in + (int64_t)xmin * inner;
#pragma unroll
      for (int t = 0; t < RESAMPLE_KMAX; ++t) {
        if (t >= n) break;
#pragma unroll
        for (int c = 0; c < RESAMPLE_MAX_CHANNELS; ++c)
          if (c < inner) acc[c] += (int)px[t * inner + c] * k[t];
      }
    }
    if (mine) {
      uint8_t* d = dst + o * row_out + (int64_t)x * inner;
#pragma unroll
      for (int c = 0; c < RESAMPLE_MAX_CHANNELS; ++c)
        if (c < inner) d[c] = (uint8_t)clip8(acc[c]);
    }
  }
}

extern "C" {

int mvit_patchify(const mvit_image* images, int n_images, int64_t total_rows, void* out, double rescale, float mean_r,
                  float mean_g, float mean_b, float std_r, float std_g, float std_b, int dtype, mvit_stream_t stream) {
  MVIT_REQUIRE(images != nullptr && n_images > 0, "patchify: empty image table");
  MVIT_REQUIRE(total_rows >= 0 && total_rows % 4 == 0 && total_rows / 4 <= 0x7fffffffLL,
               "patchify: total_rows %lld must be a multiple of 4 (2x2 merge blocks) below 2^33", (long long)total_rows);
  MVIT_REQUIRE(dtype == MVIT_BF16 || dtype == MVIT_F32, "patchify: dtype %d", dtype);
  MVIT_REQUIRE(std_r != 0.f && std_g != 0.f && std_b != 0.f, "patchify: zero std");
  if (total_rows == 0) return MVIT_OK;
  MVIT_REQUIRE(out != nullptr && mvit_aligned16(out), "patchify: output must be a 16-byte aligned device pointer");
  Norm nm{rescale, {mean_r, mean_g, mean_b}, {std_r, std_g, std_b}};
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const unsigned grid = (unsigned)(total_rows / 4);
  if (dtype == MVIT_BF16)
    hipLaunchKernelGGL((patchify_kernel<bf16_t>), dim3(grid), 256, 0, s, images, n_images, static_cast<bf16_t*>(out), total_rows, nm);
  else
    hipLaunchKernelGGL((patchify_kernel<float>), dim3(grid), 256, 0, s, images, n_images, static_cast<float*>(out), total_rows, nm);
  MVIT_CHECK_LAUNCH("patchify");
  return MVIT_OK;
}

int mvit_resample_u8(const uint8_t* src, uint8_t* dst, int64_t outer, int64_t in_len, int64_t out_len, int64_t inner,
                     const int32_t* bounds, const int32_t* kk, int ksize, mvit_stream_t stream) {
  MVIT_REQUIRE(src && dst && bounds && kk, "resample_u8: null pointer");
  MVIT_REQUIRE(outer >= 0 && in_len > 0 && out_len > 0 && inner > 0 && ksize > 0, "resample_u8: bad sizes (outer=%lld in=%lld out=%lld inner=%lld ksize=%d)",
               (long long)outer, (long long)in_len, (long long)out_len, (long long)inner, ksize);
  MVIT_REQUIRE(in_len < (1 << 24) && out_len < (1 << 24) && in_len * inner < (1ll << 40) && out_len * inner < (1ll << 40), "resample_u8: axis too long");
  if (outer == 0) return MVIT_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t quads = (out_len * inner + 3) / 4, total = outer * quads;
  const unsigned grid = (unsigned)((total + 255) / 256 < 65535 * 16 ? (total + 255) / 256 : 65535 * 16);
  const bool wide = inner % 4 == 0 && ((uintptr_t)src % 4 == 0) && ((uintptr_t)dst % 4 == 0);
  if (!wide && inner <= RESAMPLE_MAX_CHANNELS && ksize <= RESAMPLE_KMAX) {
    const int rows_per_group = 32;
    const dim3 g((unsigned)((out_len + 255) / 256), (unsigned)((outer + rows_per_group - 1) / rows_per_group));
    MVIT_REQUIRE(g.y <= 65535, "resample_u8: outer=%lld too large for a short inner dimension", (long long)outer);
    hipLaunchKernelGGL(resample_cols_kernel, g, 256, 0, s, src, dst, outer, in_len, out_len, (int)inner, bounds, kk, ksize, rows_per_group);
  } else if (!wide && inner <= RESAMPLE_MAX_CHANNELS && in_len * inner + 4 <= RESAMPLE_LDS_BYTES) {
    const unsigned rows = (unsigned)(outer < 65535 * 16 ? outer : 65535 * 16);
    hipLaunchKernelGGL(resample_rows_lds_kernel, dim3(rows), 256, 0, s, src, dst, outer, in_len, out_len, (int)inner, bounds, kk, ksize);
  } else if (wide) hipLaunchKernelGGL((resample_pass_kernel<true>), dim3(grid), 256, 0, s, src, dst, outer, in_len, out_len, inner, bounds, kk, ksize);
  else hipLaunchKernelGGL((resample_pass_kernel<false>), dim3(grid), 256, 0, s, src, dst, outer, in_len, out_len, inner, bounds, kk, ksize);
  MVIT_CHECK_LAUNCH("resample_u8");
  return MVIT_OK;
}

}  // extern "C"
