// HBM-bound kernels of the vision tower: RMSNorm fwd/bwd, rotary embedding, row gather, segment copy,
// pad, cast, column sums.  One wave (64 lanes) owns a row where a row reduction is needed; all global
// accesses are 16-byte vectors along the contiguous dimension whenever shapes allow it.
#include "mvit_common.h"

// ------------------------------------------------------------------------------------------------
// RMSNorm forward.  One wave per row, 4 rows per 256-thread block; grid-stride over rows.
// Algorithmic bytes per row: read cols*e, write cols*e (+ the weight once, + 4 B rstd).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          T* __restrict__ y, float* __restrict__ rstd,
                                                          int64_t rows, int cols, float eps) {
  constexpr int V = mvit_elem<T>::vec;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * 4;
  for (int64_t r = wave; r < rows; r += nwaves) {
    const T* xr = x + r * cols;
    T* yr = y + r * cols;
    float ss = 0.f;
    if (VEC) {
      for (int c = lane * V; c < cols; c += 64 * V) {
        vec_t v = *reinterpret_cast<const vec_t*>(xr + c);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          float f = to_f32(v[j]);
          ss += f * f;
        }
      }
    } else {
      for (int c = lane; c < cols; c += 64) {
        float f = to_f32(xr[c]);
        ss += f * f;
      }
    }
    ss = wave_sum(ss);
    const float rs = rsqrtf(ss / (float)cols + eps);
    if (lane == 0) rstd[r] = rs;
    if (VEC) {
      for (int c = lane * V; c < cols; c += 64 * V) {
        vec_t v = *reinterpret_cast<const vec_t*>(xr + c);
        vec_t g = *reinterpret_cast<const vec_t*>(w + c);
        vec_t o;
#pragma unroll
        for (int j = 0; j < V; ++j) {
          // normalise in fp32, round to the storage type, then scale (two roundings, like the reference)
          T n = from_f32<T>(to_f32(v[j]) * rs);
          o[j] = from_f32<T>(to_f32(g[j]) * to_f32(n));
        }
        *reinterpret_cast<vec_t*>(yr + c) = o;
      }
    } else {
      for (int c = lane; c < cols; c += 64) {
        T n = from_f32<T>(to_f32(xr[c]) * rs);
        yr[c] = from_f32<T>(to_f32(w[c]) * to_f32(n));
      }
    }
  }
}

// RMSNorm backward.  Same row ownership; each block keeps its weight-gradient partial in LDS (fp32 [cols])
// and writes it to dw_partial[blockIdx.x, :] at the end, so the result does not depend on atomics order.
// Algorithmic bytes per row: read dy, x (2*cols*e) [+ dx_add], write dx (cols*e).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                          const T* __restrict__ w, const float* __restrict__ rstd,
                                                          const T* dx_add, T* dx, float* __restrict__ dw_partial,
                                                          int64_t rows, int cols) {
  constexpr int V = mvit_elem<T>::vec;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  extern __shared__ float dw_lds[];  // [4][cols]
  const int lane = threadIdx.x & 63;
  const int wv = threadIdx.x >> 6;
  float* my_dw = dw_lds + (size_t)wv * cols;
  for (int c = lane; c < cols; c += 64) my_dw[c] = 0.f;
  const int64_t wave = (int64_t)blockIdx.x * 4 + wv;
  const int64_t nwaves = (int64_t)gridDim.x * 4;
  const float inv_cols = 1.f / (float)cols;
  for (int64_t r = wave; r < rows; r += nwaves) {
    const T* xr = x + r * cols;
    const T* gr = dy + r * cols;
    const float rs = rstd[r];
    float dot = 0.f;
    if (VEC) {
      for (int c = lane * V; c < cols; c += 64 * V) {
        vec_t xv = *reinterpret_cast<const vec_t*>(xr + c);
        vec_t gv = *reinterpret_cast<const vec_t*>(gr + c);
        vec_t wv_ = *reinterpret_cast<const vec_t*>(w + c);
#pragma unroll
        for (int j = 0; j < V; ++j) dot += to_f32(gv[j]) * to_f32(wv_[j]) * to_f32(xv[j]);
      }
    } else {
      for (int c = lane; c < cols; c += 64) dot += to_f32(gr[c]) * to_f32(w[c]) * to_f32(xr[c]);
    }
    dot = wave_sum(dot) * rs * inv_cols;  // mean(dy*w*xhat)
    if (VEC) {
      for (int c = lane * V; c < cols; c += 64 * V) {
        vec_t xv = *reinterpret_cast<const vec_t*>(xr + c);
        vec_t gv = *reinterpret_cast<const vec_t*>(gr + c);
        vec_t wv_ = *reinterpret_cast<const vec_t*>(w + c);
        vec_t av;
        if (dx_add) av = *reinterpret_cast<const vec_t*>(dx_add + r * cols + c);
        vec_t o;
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float xhat = to_f32(xv[j]) * rs;
          const float g = to_f32(gv[j]);
          float d = rs * (g * to_f32(wv_[j]) - xhat * dot);
          if (dx_add) d += to_f32(av[j]);
          o[j] = from_f32<T>(d);
          my_dw[c + j] += g * xhat;
        }
        *reinterpret_cast<vec_t*>(dx + r * cols + c) = o;
      }
    } else {
      for (int c = lane; c < cols; c += 64) {
        const float xhat = to_f32(xr[c]) * rs;
        const float g = to_f32(gr[c]);
        float d = rs * (g * to_f32(w[c]) - xhat * dot);
        if (dx_add) d += to_f32(dx_add[r * cols + c]);
        dx[r * cols + c] = from_f32<T>(d);
        my_dw[c] += g * xhat;
      }
    }
  }
  __syncthreads();
  float* out = dw_partial + (size_t)blockIdx.x * cols;
  for (int c = threadIdx.x; c < cols; c += 256)
    out[c] = dw_lds[c] + dw_lds[cols + c] + dw_lds[2 * (size_t)cols + c] + dw_lds[3 * (size_t)cols + c];
}

// out[c] = sum_b partial[b, c].  A block owns 32 columns; its 8 row groups each add every 8th partial row
// (fixed order, so the sum is reproducible), then combine through LDS.
template <typename T>
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ partial, int n_partial,
                                                              int64_t cols, T* __restrict__ out) {
  __shared__ float red[8][33];
  const int cx = threadIdx.x & 31, ry = threadIdx.x >> 5;
  const int64_t c = (int64_t)blockIdx.x * 32 + cx;
  float s = 0.f;
  if (c < cols)
    for (int b = ry; b < n_partial; b += 8) s += partial[(size_t)b * cols + c];
  red[ry][cx] = s;
  __syncthreads();
  if (ry == 0 && c < cols) {
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) t += red[k][cx];
    out[c] = from_f32<T>(t);
  }
}

// The same sum for cols % 4 == 0: a block owns 16 columns (4 lanes x float4) and 64 row groups, so that a tall
// partial array (1024 rows from the RMSNorm backward) is walked by many short, independent load chains.
template <typename T>
__global__ __launch_bounds__(256) void reduce_partials_vec_kernel(const float* __restrict__ partial, int n_partial,
                                                                  int64_t cols, T* __restrict__ out) {
  __shared__ float red[64][17];
  const int cx = threadIdx.x & 3, ry = threadIdx.x >> 2;
  const int64_t c = (int64_t)blockIdx.x * 16 + cx * 4;
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  if (c < cols) {
#pragma unroll 4
    for (int b = ry; b < n_partial; b += 64) s += *reinterpret_cast<const f32x4*>(partial + (size_t)b * cols + c);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) red[ry][cx * 4 + e] = s[e];
  __syncthreads();
  if (threadIdx.x < 16 && (int64_t)blockIdx.x * 16 + threadIdx.x < cols) {
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 64; ++k) t += red[k][threadIdx.x];
    out[(int64_t)blockIdx.x * 16 + threadIdx.x] = from_f32<T>(t);
  }
}

// Column sums with 16-byte loads: a block owns 128 columns (16 lanes x 8/4 elements) and 16 row phases.
template <typename T>
__global__ __launch_bounds__(256) void colsum_vec_kernel(const T* __restrict__ x, int64_t ld, int64_t rows, int64_t cols,
                                                         float* __restrict__ partial) {
  constexpr int V = mvit_elem<T>::vec;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  __shared__ float red[16][16 * V + 1];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int64_t c0 = ((int64_t)blockIdx.x * 16 + tx) * V;
  float acc[V];
#pragma unroll
  for (int j = 0; j < V; ++j) acc[j] = 0.f;
  if (c0 < cols) {
    for (int64_t r = (int64_t)blockIdx.y * 16 + ty; r < rows; r += (int64_t)gridDim.y * 16) {
      const vec_t v = *reinterpret_cast<const vec_t*>(x + r * ld + c0);
#pragma unroll
      for (int j = 0; j < V; ++j) acc[j] += to_f32(v[j]);
    }
  }
#pragma unroll
  for (int j = 0; j < V; ++j) red[ty][tx * V + j] = acc[j];
  __syncthreads();
  if (threadIdx.x < 16 * V) {
    const int64_t c = (int64_t)blockIdx.x * 16 * V + threadIdx.x;
    if (c < cols) {
      float t = 0.f;
#pragma unroll
      for (int k = 0; k < 16; ++k) t += red[k][threadIdx.x];
      partial[(size_t)blockIdx.y * cols + c] = t;
    }
  }
}

// Column sums: block b accumulates rows b, b+grid, ... ; thread owns columns.  Partials [grid, cols].
template <typename T>
__global__ __launch_bounds__(256) void colsum_kernel(const T* __restrict__ x, int64_t ld, int64_t rows, int64_t cols,
                                                     float* __restrict__ partial) {
  // blockIdx.x: column chunk of 256*2 columns; blockIdx.y: row slice
  const int64_t c0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (c0 >= cols) return;
  const bool two = (c0 + 1 < cols);
  float s0 = 0.f, s1 = 0.f;
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
    const T* p = x + r * ld + c0;
    s0 += to_f32(p[0]);
    if (two) s1 += to_f32(p[1]);
  }
  partial[(size_t)blockIdx.y * cols + c0] = s0;
  if (two) partial[(size_t)blockIdx.y * cols + c0 + 1] = s1;
}

// ------------------------------------------------------------------------------------------------
// Rotary embedding in place.  A thread owns V consecutive elements of the first half of one head and
// the matching V of the second half.  Algorithmic bytes per (row, head): 2*head_dim*e + table share.
// The first `lead_heads` heads are multiplied by `lead_scale` before the one rounding to the storage type (the
// queries of an attention layer take the softmax scale here, so that no later pass rounds them a second time).
template <typename T, int V>
__global__ __launch_bounds__(256) void rope_kernel(T* __restrict__ x, const float* __restrict__ cosb,
                                                   const float* __restrict__ sinb, int64_t rows, int nheads,
                                                   int head_dim, int64_t row_stride, int backward, int lead_heads,
                                                   float lead_scale) {
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int half = head_dim / 2;
  const int chunks = half / V;  // per head
  const int64_t total = rows * nheads * chunks;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int ch = (int)(i % chunks);
    const int64_t rh = i / chunks;
    const int h = (int)(rh % nheads);
    const int64_t r = rh / nheads;
    T* p = x + r * row_stride + (int64_t)h * head_dim + ch * V;
    const float gain = h < lead_heads ? lead_scale : 1.f;
    const float* c = cosb + r * head_dim + ch * V;
    const float* s = sinb + r * head_dim + ch * V;
    vec_t lo, hi, olo, ohi;
    if (V > 1) {
      lo = *reinterpret_cast<const vec_t*>(p);
      hi = *reinterpret_cast<const vec_t*>(p + half);
    } else {
      lo[0] = p[0];
      hi[0] = p[half];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float a = to_f32(lo[j]), b = to_f32(hi[j]);
      const float c0 = c[j], c1 = c[j + half], s0 = s[j], s1 = s[j + half];
      float oa, ob;
      if (!backward) {
        oa = a * c0 - b * s0;
        ob = b * c1 + a * s1;
      } else {
        oa = a * c0 + b * s1;
        ob = b * c1 - a * s0;
      }
      olo[j] = from_f32<T>(oa * gain);
      ohi[j] = from_f32<T>(ob * gain);
    }
    if (V > 1) {
      *reinterpret_cast<vec_t*>(p) = olo;
      *reinterpret_cast<vec_t*>(p + half) = ohi;
    } else {
      p[0] = olo[0];
      p[half] = ohi[0];
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Row gather / segment copy: pure byte movement in 16-byte (or 4-byte) words.
template <typename W>
__global__ __launch_bounds__(256) void gather_rows_kernel(const W* __restrict__ src, const int64_t* __restrict__ index,
                                                          W* __restrict__ dst, int64_t n_rows, int64_t row_words) {
  // blockIdx.y strides over rows; threads over words
  for (int64_t r = blockIdx.y; r < n_rows; r += gridDim.y) {
    const W* s = src + index[r] * row_words;
    W* d = dst + r * row_words;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < row_words; c += (int64_t)gridDim.x * 256) d[c] = s[c];
  }
}

template <typename W>
__global__ __launch_bounds__(256) void segment_copy_kernel(const W* __restrict__ src, W* __restrict__ dst,
                                                           const int64_t* __restrict__ desc, int64_t row_words) {
  // blockIdx.z: segment; blockIdx.y strides over the segment's rows
  const int64_t* d3 = desc + 3 * (int64_t)blockIdx.z;
  const int64_t s0 = d3[0], d0 = d3[1], n = d3[2];
  for (int64_t r = blockIdx.y; r < n; r += gridDim.y) {
    const W* s = src + (s0 + r) * row_words;
    W* d = dst + (d0 + r) * row_words;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < row_words; c += (int64_t)gridDim.x * 256) d[c] = s[c];
  }
}

template <typename E>
__global__ __launch_bounds__(256) void pad_pack_kernel(const E* __restrict__ pack, E* __restrict__ padded,
                                                       uint8_t* __restrict__ mask, const int64_t* __restrict__ lens,
                                                       const int64_t* __restrict__ offsets, int64_t pad_len,
                                                       int64_t row_elems, E pad_value) {
  const int64_t b = blockIdx.z;
  const int64_t len = lens[b], off = offsets[b];
  for (int64_t r = blockIdx.y; r < pad_len; r += gridDim.y) {
    E* d = padded + (b * pad_len + r) * row_elems;
    const bool real = r < len;
    const E* s = pack + (off + (real ? r : 0)) * row_elems;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < row_elems; c += (int64_t)gridDim.x * 256)
      d[c] = real ? s[c] : pad_value;
    if (blockIdx.x == 0 && threadIdx.x == 0) mask[b * pad_len + r] = real ? 1 : 0;
  }
}

template <typename S, typename D>
__global__ __launch_bounds__(256) void cast2d_kernel(const S* __restrict__ src, int64_t src_ld, D* __restrict__ dst,
                                                     int64_t dst_ld, int64_t rows, int64_t cols) {
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y)
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < cols; c += (int64_t)gridDim.x * 256)
      dst[r * dst_ld + c] = from_f32<D>(to_f32(src[r * src_ld + c]));
}

// ------------------------------------------------------------------------------------------------
static inline hipStream_t S_(mvit_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
// ------------------------------------------------------------------------------------------------
// Vision -> text hand-off: where the token ids equal the image placeholder, the rows of the text embedding are
// replaced by the vision rows, the k-th placeholder taking vision row k (masked_scatter with a row mask).
// One work-group ranks the placeholders (each thread counts a contiguous slice, the counts are scanned in LDS, the
// slice is walked again to write ranks and positions); the row merge is then a pure byte copy.
__global__ __launch_bounds__(1024) void image_token_ranks_kernel(const int64_t* __restrict__ ids, const int64_t* __restrict__ labels,
                                                                 int64_t n, int64_t image_id, int64_t ignore_label,
                                                                 int32_t* __restrict__ rank, int64_t* __restrict__ positions,
                                                                 int64_t* __restrict__ counts) {
  __shared__ int scan[1024];
  __shared__ int bad[1024];
  const int t = threadIdx.x;
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = per * t < n ? per * t : n;
  const int64_t hi = lo + per < n ? lo + per : n;
  int cnt = 0, wrong = 0;
  for (int64_t i = lo; i < hi; ++i) {
    const bool img = ids[i] == image_id;
    cnt += img;
    if (img && labels != nullptr && labels[i] != ignore_label) ++wrong;
  }
  scan[t] = cnt;
  bad[t] = wrong;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {  // inclusive scan (Hillis-Steele), and a plain sum for the label check
    const int v = t >= off ? scan[t - off] : 0;
    const int w = t >= off ? bad[t - off] : 0;
    __syncthreads();
    scan[t] += v;
    bad[t] += w;
    __syncthreads();
  }
  int k = scan[t] - cnt;  // exclusive prefix of this slice
  for (int64_t i = lo; i < hi; ++i) {
    if (ids[i] == image_id) {
      rank[i] = k;
      positions[k] = i;
      ++k;
    } else {
      rank[i] = -1;
    }
  }
  if (t == 1023) {
    counts[0] = scan[1023];
    counts[1] = bad[1023];
  }
}

template <typename W>
__global__ __launch_bounds__(256) void merge_rows_kernel(const W* __restrict__ embeds, const W* __restrict__ vision,
                                                         const int32_t* __restrict__ rank, W* __restrict__ merged, int64_t n_rows,
                                                         int64_t n_vision, int64_t row_words) {
  for (int64_t r = blockIdx.y; r < n_rows; r += gridDim.y) {
    const int k = rank[r];
    const bool img = k >= 0 && k < n_vision;  // a rank beyond the vision rows keeps the text row (the caller has refused that case)
    const W* s = img ? (vision ? vision + (int64_t)k * row_words : nullptr) : embeds + r * row_words;
    W* d = merged + r * row_words;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < row_words; c += (int64_t)gridDim.x * 256) d[c] = s ? s[c] : W{};
  }
}

static inline int clamp_grid(int64_t v, int64_t hi) { return (int)(v < 1 ? 1 : (v > hi ? hi : v)); }

extern "C" {

int mvit_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t rows, int64_t cols, float eps,
                     int dtype, mvit_stream_t stream) {
  MVIT_REQUIRE(rows >= 0 && cols > 0 && cols < (1 << 24), "rmsnorm_fwd: bad shape %lld x %lld", (long long)rows, (long long)cols);
  if (rows == 0) return MVIT_OK;
  MVIT_REQUIRE(x && w && y && rstd, "rmsnorm_fwd: null pointer");
  const int grid = clamp_grid((rows + 3) / 4, 8192);
  if (dtype == MVIT_BF16) {
    const bool vec = cols % 8 == 0 && mvit_aligned16(x) && mvit_aligned16(y) && mvit_aligned16(w);
    if (vec)
      hipLaunchKernelGGL((rmsnorm_fwd_kernel<bf16_t, true>), grid, 256, 0, S_(stream), (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, rstd, rows, (int)cols, eps);
    else
      hipLaunchKernelGGL((rmsnorm_fwd_kernel<bf16_t, false>), grid, 256, 0, S_(stream), (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, rstd, rows, (int)cols, eps);
  } else if (dtype == MVIT_F32) {
    const bool vec = cols % 4 == 0 && mvit_aligned16(x) && mvit_aligned16(y) && mvit_aligned16(w);
    if (vec)
      hipLaunchKernelGGL((rmsnorm_fwd_kernel<float, true>), grid, 256, 0, S_(stream), (const float*)x, (const float*)w, (float*)y, rstd, rows, (int)cols, eps);
    else
      hipLaunchKernelGGL((rmsnorm_fwd_kernel<float, false>), grid, 256, 0, S_(stream), (const float*)x, (const float*)w, (float*)y, rstd, rows, (int)cols, eps);
  } else {
    return mvit_set_error(MVIT_ERR_UNSUPPORTED, "rmsnorm_fwd: dtype %d", dtype);
  }
  MVIT_CHECK_LAUNCH("rmsnorm_fwd");
  return MVIT_OK;
}

int mvit_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, const void* dx_add, void* dx,
                     float* dw_partial, int n_partial, int64_t rows, int64_t cols, int dtype, mvit_stream_t stream) {
  MVIT_REQUIRE(dw_partial && w && (rows == 0 || (dy && x && rstd && dx)), "rmsnorm_bwd: null pointer");  // no rows: only the partial sums are written (zeros)
  MVIT_REQUIRE(rows >= 0 && cols > 0 && n_partial > 0, "rmsnorm_bwd: bad shape");
  const size_t lds = 4 * (size_t)cols * sizeof(float);
  MVIT_REQUIRE(lds <= 160 * 1024, "rmsnorm_bwd: cols %lld needs %zu B of LDS (> 160 KiB)", (long long)cols, lds);
  const int grid = n_partial;  // every block writes its partial row, rows or not
  bool al = mvit_aligned16(dy) && mvit_aligned16(x) && mvit_aligned16(w) && mvit_aligned16(dx) && (!dx_add || mvit_aligned16(dx_add));
  if (dtype == MVIT_BF16) {
    if (cols % 8 == 0 && al)
      hipLaunchKernelGGL((rmsnorm_bwd_kernel<bf16_t, true>), grid, 256, lds, S_(stream), (const bf16_t*)dy, (const bf16_t*)x, (const bf16_t*)w, rstd, (const bf16_t*)dx_add, (bf16_t*)dx, dw_partial, rows, (int)cols);
    else
      hipLaunchKernelGGL((rmsnorm_bwd_kernel<bf16_t, false>), grid, 256, lds, S_(stream), (const bf16_t*)dy, (const bf16_t*)x, (const bf16_t*)w, rstd, (const bf16_t*)dx_add, (bf16_t*)dx, dw_partial, rows, (int)cols);
  } else if (dtype == MVIT_F32) {
    if (cols % 4 == 0 && al)
      hipLaunchKernelGGL((rmsnorm_bwd_kernel<float, true>), grid, 256, lds, S_(stream), (const float*)dy, (const float*)x, (const float*)w, rstd, (const float*)dx_add, (float*)dx, dw_partial, rows, (int)cols);
    else
      hipLaunchKernelGGL((rmsnorm_bwd_kernel<float, false>), grid, 256, lds, S_(stream), (const float*)dy, (const float*)x, (const float*)w, rstd, (const float*)dx_add, (float*)dx, dw_partial, rows, (int)cols);
  } else {
    return mvit_set_error(MVIT_ERR_UNSUPPORTED, "rmsnorm_bwd: dtype %d", dtype);
  }
  MVIT_CHECK_LAUNCH("rmsnorm_bwd");
  return MVIT_OK;
}

int mvit_reduce_partials(const float* partial, int n_partial, int64_t cols, void* out, int out_dtype, mvit_stream_t stream) {
  MVIT_REQUIRE(partial && out && n_partial > 0 && cols > 0, "reduce_partials: bad arguments");
  if (cols % 4 == 0 && mvit_aligned16(partial) && (out_dtype == MVIT_BF16 || out_dtype == MVIT_F32)) {
    const int vgrid = (int)((cols + 15) / 16);
    if (out_dtype == MVIT_BF16)
      hipLaunchKernelGGL((reduce_partials_vec_kernel<bf16_t>), vgrid, 256, 0, S_(stream), partial, n_partial, cols, (bf16_t*)out);
    else
      hipLaunchKernelGGL((reduce_partials_vec_kernel<float>), vgrid, 256, 0, S_(stream), partial, n_partial, cols, (float*)out);
    MVIT_CHECK_LAUNCH("reduce_partials");
    return MVIT_OK;
  }
  const int grid = (int)((cols + 31) / 32);
  if (out_dtype == MVIT_BF16)
    hipLaunchKernelGGL((reduce_partials_kernel<bf16_t>), grid, 256, 0, S_(stream), partial, n_partial, cols, (bf16_t*)out);
  else if (out_dtype == MVIT_F32)
    hipLaunchKernelGGL((reduce_partials_kernel<float>), grid, 256, 0, S_(stream), partial, n_partial, cols, (float*)out);
  else
    return mvit_set_error(MVIT_ERR_UNSUPPORTED, "reduce_partials: dtype %d", out_dtype);
  MVIT_CHECK_LAUNCH("reduce_partials");
  return MVIT_OK;
}

int mvit_colsum(const void* x, int64_t ld, int64_t rows, int64_t cols, float* partial, int n_partial, int dtype, mvit_stream_t stream) {
  MVIT_REQUIRE((x || rows == 0) && partial && n_partial > 0 && n_partial <= 65535 && cols > 0 && rows >= 0 && ld >= cols, "colsum: bad arguments");
  MVIT_REQUIRE(dtype == MVIT_BF16 || dtype == MVIT_F32, "colsum: dtype %d", dtype);
  const int vec = dtype == MVIT_BF16 ? 8 : 4;
  if (cols % vec == 0 && ld % vec == 0 && mvit_aligned16(x)) {
    dim3 grid((unsigned)((cols + 16 * vec - 1) / (16 * vec)), (unsigned)n_partial);
    if (dtype == MVIT_BF16)
      hipLaunchKernelGGL((colsum_vec_kernel<bf16_t>), grid, 256, 0, S_(stream), (const bf16_t*)x, ld, rows, cols, partial);
    else
      hipLaunchKernelGGL((colsum_vec_kernel<float>), grid, 256, 0, S_(stream), (const float*)x, ld, rows, cols, partial);
  } else {
    dim3 grid((unsigned)((cols + 511) / 512), (unsigned)n_partial);
    if (dtype == MVIT_BF16)
      hipLaunchKernelGGL((colsum_kernel<bf16_t>), grid, 256, 0, S_(stream), (const bf16_t*)x, ld, rows, cols, partial);
    else
      hipLaunchKernelGGL((colsum_kernel<float>), grid, 256, 0, S_(stream), (const float*)x, ld, rows, cols, partial);
  }
  MVIT_CHECK_LAUNCH("colsum");
  return MVIT_OK;
}

int mvit_rope(void* x, const float* cosb, const float* sinb, int64_t rows, int nheads, int head_dim, int64_t row_stride,
              int backward, int dtype, mvit_stream_t stream) {
  return mvit_rope_scaled(x, cosb, sinb, rows, nheads, head_dim, row_stride, backward, 0, 1.f, dtype, stream);
}

int mvit_rope_scaled(void* x, const float* cosb, const float* sinb, int64_t rows, int nheads, int head_dim, int64_t row_stride,
                     int backward, int lead_heads, float lead_scale, int dtype, mvit_stream_t stream) {
  MVIT_REQUIRE(lead_heads >= 0 && lead_heads <= nheads, "rope: lead_heads=%d of %d heads", lead_heads, nheads);
  MVIT_REQUIRE(rows >= 0 && nheads > 0 && head_dim > 0 && head_dim % 2 == 0 && row_stride >= (int64_t)nheads * head_dim,
               "rope: bad shape rows=%lld heads=%d head_dim=%d stride=%lld", (long long)rows, nheads, head_dim, (long long)row_stride);
  if (rows == 0) return MVIT_OK;
  MVIT_REQUIRE(x && cosb && sinb, "rope: null pointer");
  const int half = head_dim / 2;
  const int64_t work_scalar = rows * nheads * half;
  if (dtype == MVIT_BF16) {
    if (half % 8 == 0 && row_stride % 8 == 0 && mvit_aligned16(x)) {
      const int grid = clamp_grid((work_scalar / 8 + 255) / 256, 65535 * 16);
      hipLaunchKernelGGL((rope_kernel<bf16_t, 8>), grid, 256, 0, S_(stream), (bf16_t*)x, cosb, sinb, rows, nheads, head_dim, row_stride, backward, lead_heads, lead_scale);
    } else {
      const int grid = clamp_grid((work_scalar + 255) / 256, 65535 * 16);
      hipLaunchKernelGGL((rope_kernel<bf16_t, 1>), grid, 256, 0, S_(stream), (bf16_t*)x, cosb, sinb, rows, nheads, head_dim, row_stride, backward, lead_heads, lead_scale);
    }
  } else if (dtype == MVIT_F32) {
    if (half % 4 == 0 && row_stride % 4 == 0 && mvit_aligned16(x)) {
      const int grid = clamp_grid((work_scalar / 4 + 255) / 256, 65535 * 16);
      hipLaunchKernelGGL((rope_kernel<float, 4>), grid, 256, 0, S_(stream), (float*)x, cosb, sinb, rows, nheads, head_dim, row_stride, backward, lead_heads, lead_scale);
    } else {
      const int grid = clamp_grid((work_scalar + 255) / 256, 65535 * 16);
      hipLaunchKernelGGL((rope_kernel<float, 1>), grid, 256, 0, S_(stream), (float*)x, cosb, sinb, rows, nheads, head_dim, row_stride, backward, lead_heads, lead_scale);
    }
  } else {
    return mvit_set_error(MVIT_ERR_UNSUPPORTED, "rope: dtype %d", dtype);
  }
  MVIT_CHECK_LAUNCH("rope");
  return MVIT_OK;
}

int mvit_gather_rows(const void* src, const int64_t* index, void* dst, int64_t n_rows, int64_t row_bytes, mvit_stream_t stream) {
  MVIT_REQUIRE(n_rows >= 0 && row_bytes > 0 && row_bytes % 2 == 0, "gather_rows: row_bytes %lld must be a positive multiple of 2", (long long)row_bytes);
  if (n_rows == 0) return MVIT_OK;
  MVIT_REQUIRE(src && index && dst, "gather_rows: null pointer");
  const unsigned gy = (unsigned)clamp_grid(n_rows, 65535);
  if (row_bytes % 16 == 0 && mvit_aligned16(src) && mvit_aligned16(dst)) {
    const int64_t words = row_bytes / 16;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy);
    hipLaunchKernelGGL((gather_rows_kernel<u32x4>), grid, 256, 0, S_(stream), (const u32x4*)src, index, (u32x4*)dst, n_rows, words);
  } else if (row_bytes % 4 == 0) {
    const int64_t words = row_bytes / 4;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy);
    hipLaunchKernelGGL((gather_rows_kernel<uint32_t>), grid, 256, 0, S_(stream), (const uint32_t*)src, index, (uint32_t*)dst, n_rows, words);
  } else {
    const int64_t words = row_bytes / 2;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy);
    hipLaunchKernelGGL((gather_rows_kernel<uint16_t>), grid, 256, 0, S_(stream), (const uint16_t*)src, index, (uint16_t*)dst, n_rows, words);
  }
  MVIT_CHECK_LAUNCH("gather_rows");
  return MVIT_OK;
}

int mvit_segment_copy(const void* src, void* dst, const int64_t* desc, int64_t nseg, int64_t max_seg_rows, int64_t row_bytes, mvit_stream_t stream) {
  MVIT_REQUIRE(nseg >= 0 && nseg <= 65535 && row_bytes > 0 && row_bytes % 2 == 0, "segment_copy: bad nseg/row_bytes");
  if (nseg == 0 || max_seg_rows <= 0) return MVIT_OK;
  MVIT_REQUIRE(src && dst && desc, "segment_copy: null pointer");
  const unsigned gy = (unsigned)clamp_grid(max_seg_rows, 4096);
  if (row_bytes % 16 == 0 && mvit_aligned16(src) && mvit_aligned16(dst)) {
    const int64_t words = row_bytes / 16;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy, (unsigned)nseg);
    hipLaunchKernelGGL((segment_copy_kernel<u32x4>), grid, 256, 0, S_(stream), (const u32x4*)src, (u32x4*)dst, desc, words);
  } else if (row_bytes % 4 == 0) {
    const int64_t words = row_bytes / 4;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy, (unsigned)nseg);
    hipLaunchKernelGGL((segment_copy_kernel<uint32_t>), grid, 256, 0, S_(stream), (const uint32_t*)src, (uint32_t*)dst, desc, words);
  } else {
    const int64_t words = row_bytes / 2;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy, (unsigned)nseg);
    hipLaunchKernelGGL((segment_copy_kernel<uint16_t>), grid, 256, 0, S_(stream), (const uint16_t*)src, (uint16_t*)dst, desc, words);
  }
  MVIT_CHECK_LAUNCH("segment_copy");
  return MVIT_OK;
}

int mvit_pad_pack(const void* pack, void* padded, uint8_t* mask, const int64_t* lens, const int64_t* offsets, int64_t batch,
                  int64_t pad_len, int64_t row_elems, int elem_size, uint32_t pad_bits, mvit_stream_t stream) {
  MVIT_REQUIRE(batch >= 0 && batch <= 65535 && pad_len >= 0 && row_elems > 0, "pad_pack: bad shape");
  MVIT_REQUIRE(elem_size == 2 || elem_size == 4, "pad_pack: elem_size %d", elem_size);
  if (batch == 0 || pad_len == 0) return MVIT_OK;
  MVIT_REQUIRE(padded && mask && lens && offsets, "pad_pack: null pointer");
  dim3 grid((unsigned)clamp_grid((row_elems + 255) / 256, 64), (unsigned)clamp_grid(pad_len, 4096), (unsigned)batch);
  if (elem_size == 2)
    hipLaunchKernelGGL((pad_pack_kernel<uint16_t>), grid, 256, 0, S_(stream), (const uint16_t*)pack, (uint16_t*)padded, mask, lens, offsets, pad_len, row_elems, (uint16_t)pad_bits);
  else
    hipLaunchKernelGGL((pad_pack_kernel<uint32_t>), grid, 256, 0, S_(stream), (const uint32_t*)pack, (uint32_t*)padded, mask, lens, offsets, pad_len, row_elems, pad_bits);
  MVIT_CHECK_LAUNCH("pad_pack");
  return MVIT_OK;
}

int mvit_cast2d(const void* src, int64_t src_ld, int src_dtype, void* dst, int64_t dst_ld, int dst_dtype, int64_t rows,
                int64_t cols, mvit_stream_t stream) {
  MVIT_REQUIRE(rows >= 0 && cols >= 0 && src_ld >= cols && dst_ld >= cols, "cast2d: bad arguments");
  if (rows == 0 || cols == 0) return MVIT_OK;
  MVIT_REQUIRE(src && dst, "cast2d: null pointer");
  dim3 grid((unsigned)clamp_grid((cols + 255) / 256, 256), (unsigned)clamp_grid(rows, 16384));
  hipStream_t s = S_(stream);
  if (src_dtype == MVIT_F32 && dst_dtype == MVIT_BF16)
    hipLaunchKernelGGL((cast2d_kernel<float, bf16_t>), grid, 256, 0, s, (const float*)src, src_ld, (bf16_t*)dst, dst_ld, rows, cols);
  else if (src_dtype == MVIT_BF16 && dst_dtype == MVIT_F32)
    hipLaunchKernelGGL((cast2d_kernel<bf16_t, float>), grid, 256, 0, s, (const bf16_t*)src, src_ld, (float*)dst, dst_ld, rows, cols);
  else if (src_dtype == MVIT_F32 && dst_dtype == MVIT_F32)
    hipLaunchKernelGGL((cast2d_kernel<float, float>), grid, 256, 0, s, (const float*)src, src_ld, (float*)dst, dst_ld, rows, cols);
  else if (src_dtype == MVIT_BF16 && dst_dtype == MVIT_BF16)
    hipLaunchKernelGGL((cast2d_kernel<bf16_t, bf16_t>), grid, 256, 0, s, (const bf16_t*)src, src_ld, (bf16_t*)dst, dst_ld, rows, cols);
  else
    return mvit_set_error(MVIT_ERR_UNSUPPORTED, "cast2d: dtypes %d -> %d", src_dtype, dst_dtype);
  MVIT_CHECK_LAUNCH("cast2d");
  return MVIT_OK;
}

int mvit_image_token_ranks(const int64_t* input_ids, const int64_t* labels, int64_t n_tokens, int64_t image_token_id,
                           int64_t ignore_label, int32_t* rank, int64_t* positions, int64_t* counts, mvit_stream_t stream) {
  MVIT_REQUIRE(counts && (n_tokens == 0 || (input_ids && rank && positions)), "image_token_ranks: null pointer");  // no tokens: only the counts are written (zeros)
  MVIT_REQUIRE(n_tokens >= 0 && n_tokens <= 0x7fffffffLL, "image_token_ranks: n_tokens %lld out of range", (long long)n_tokens);
  hipLaunchKernelGGL(image_token_ranks_kernel, dim3(1), 1024, 0, S_(stream), input_ids, labels, n_tokens, image_token_id, ignore_label,
                     rank, positions, counts);
  MVIT_CHECK_LAUNCH("image_token_ranks");
  return MVIT_OK;
}

int mvit_merge_rows(const void* embeds, const void* vision, const int32_t* rank, void* merged, int64_t n_tokens, int64_t n_vision,
                    int64_t row_bytes, mvit_stream_t stream) {
  MVIT_REQUIRE(n_tokens >= 0 && n_vision >= 0 && row_bytes > 0 && row_bytes % 2 == 0, "merge_rows: bad sizes (row_bytes %lld)", (long long)row_bytes);
  if (n_tokens == 0) return MVIT_OK;
  MVIT_REQUIRE(embeds && rank && merged, "merge_rows: null pointer");
  const unsigned gy = (unsigned)clamp_grid(n_tokens, 65535);
  const bool al = mvit_aligned16(embeds) && mvit_aligned16(merged) && (vision == nullptr || mvit_aligned16(vision));
  if (row_bytes % 16 == 0 && al) {
    const int64_t words = row_bytes / 16;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy);
    hipLaunchKernelGGL((merge_rows_kernel<u32x4>), grid, 256, 0, S_(stream), (const u32x4*)embeds, (const u32x4*)vision, rank, (u32x4*)merged, n_tokens, n_vision, words);
  } else if (row_bytes % 4 == 0) {
    const int64_t words = row_bytes / 4;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy);
    hipLaunchKernelGGL((merge_rows_kernel<uint32_t>), grid, 256, 0, S_(stream), (const uint32_t*)embeds, (const uint32_t*)vision, rank, (uint32_t*)merged, n_tokens, n_vision, words);
  } else {
    const int64_t words = row_bytes / 2;
    dim3 grid((unsigned)clamp_grid((words + 255) / 256, 64), gy);
    hipLaunchKernelGGL((merge_rows_kernel<uint16_t>), grid, 256, 0, S_(stream), (const uint16_t*)embeds, (const uint16_t*)vision, rank, (uint16_t*)merged, n_tokens, n_vision, words);
  }
  MVIT_CHECK_LAUNCH("merge_rows");
  return MVIT_OK;
}

}  // extern "C"
