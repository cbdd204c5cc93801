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

}  // extern "C"
