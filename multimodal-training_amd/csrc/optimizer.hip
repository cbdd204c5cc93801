// Multi-tensor Adam step and gradient sum of squares for gfx950: one launch over every parameter tensor
// instead of several launches (and one host read-back) per tensor.  Both kernels are HBM-bound streams.
//
// Work is cut into chunks of CHUNK elements that never straddle two tensors; chunk c belongs to the tensor t
// with tensors[t].first_chunk <= c < tensors[t + 1].first_chunk (binary search by the block, the table has one
// extra sentinel entry).  The arithmetic follows torch.optim.Adam's single-tensor path operation by operation
// (torch/optim/adam.py, _single_tensor_adam; called from the reference's trainer.py:479-577 with the default
// betas / eps, amsgrad and maximize off), including one rounding to the storage type after every operation
// when parameters, gradients and moments are bf16.  Association and fused multiply-adds are those of torch's
// own element-wise kernels on the host (a + alpha * b, lerp and the last product of addcmul fused;
// addcdiv as a + (value * b) / c), with no other contraction, so fp32 results can be compared bit for bit.
#include "mvit_common.h"

#include <mutex>

// Scratch of the entry point that allocates nothing (mvit_grad_sumsq_static): per-chunk partial sums.  Every GPU the
// library runs on holds its own copy of this array until the process ends.  In host code the name is only a handle
// for hipGetSymbolAddress; kernels and every other use take the device address looked up once per device.
static __device__ __align__(256) float scratch[MVIT_SUMSQ_STATIC_MAX_CHUNKS];

namespace {

constexpr int CHUNK = MVIT_ADAM_CHUNK;
constexpr int NT = 256;

struct AdamConsts {
  float beta2, one_minus_beta1, one_minus_beta2, eps, grad_scale;
  int write_grad;
};

__device__ __forceinline__ int find_tensor(const mvit_adam_tensor* t, int n_tensors, int64_t chunk) {
  int lo = 0, hi = n_tensors;  // invariant: t[lo].first_chunk <= chunk < t[hi].first_chunk
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (t[mid].first_chunk <= chunk) lo = mid;
    else hi = mid;
  }
  return lo;
}

// Rounds to the storage type and back: a no-op for fp32 tensors.
template <typename T>
__device__ __forceinline__ float rs(float x) { return to_f32(from_f32<T>(x)); }

// Second copy of an updated parameter ("shadow"): the operand buffer the GEMMs read, in its own dtype and with its
// own row pitch.  Element e of the parameter, seen as rows of `cols` elements, lands at shadow[row * ld + col].
template <typename TS>
__device__ __forceinline__ void shadow_store(void* shadow, int64_t e0, int n, int64_t cols, int64_t ld, const float* vals) {
  TS* S = static_cast<TS*>(shadow);
  int64_t idx = e0;
  int64_t run = n;
  if (cols != ld) {
    const int64_t row = e0 / cols, col = e0 - row * cols;
    idx = row * ld + col;
    run = cols - col;
  }
  constexpr int V = mvit_elem<TS>::vec;
  if (run >= n && n == V) {  // one contiguous piece: 16-byte store, or two 8-byte halves, by the address's alignment
    typedef __attribute__((ext_vector_type(V))) TS vec_t;
    typedef __attribute__((ext_vector_type(V / 2))) TS half_t;
    vec_t out;
#pragma unroll
    for (int j = 0; j < V; ++j) out[j] = from_f32<TS>(vals[j]);
    const uintptr_t a = reinterpret_cast<uintptr_t>(S + idx);
    if ((a & 15u) == 0) {
      *reinterpret_cast<vec_t*>(S + idx) = out;
      return;
    }
    if ((a & 7u) == 0) {
      half_t lo, hi;
#pragma unroll
      for (int j = 0; j < V / 2; ++j) {
        lo[j] = out[j];
        hi[j] = out[j + V / 2];
      }
      *reinterpret_cast<half_t*>(S + idx) = lo;
      *reinterpret_cast<half_t*>(S + idx + V / 2) = hi;
      return;
    }
  }
  for (int j = 0; j < n; ++j) {  // pieces that wrap to the next row, odd tails, unaligned targets
    const int64_t e = e0 + j;
    const int64_t d = cols != ld ? (e / cols) * ld + (e % cols) : e;
    S[d] = from_f32<TS>(vals[j]);
  }
}

template <typename T>
__device__ __forceinline__ void adam_elem(float& p, float& g, float& m, float& v, const AdamConsts& c, float wd,
                                          float neg_step_size, float bc2_sqrt) {
#pragma clang fp contract(off)
  if (c.grad_scale != 1.0f) g = rs<T>(g * c.grad_scale);     // p.grad.mul_(clip_coeff)
  float gg = g;
  if (wd != 0.0f) gg = rs<T>(__builtin_fmaf(wd, p, g));                          // grad.add(param, alpha=weight_decay)
  m = rs<T>(__builtin_fmaf(c.one_minus_beta1, gg - m, m));                       // exp_avg.lerp_(grad, 1 - beta1), weight < 0.5
  v = rs<T>(v * c.beta2);                                                        // exp_avg_sq.mul_(beta2)
  v = rs<T>(__builtin_fmaf(c.one_minus_beta2 * gg, gg, v));                      //   .addcmul_(grad, grad, value=1 - beta2)
  float d = rs<T>(sqrtf(v));                                                     // exp_avg_sq.sqrt() (correctly rounded)
  d = rs<T>(d / bc2_sqrt);                                                       //   / bias_correction2_sqrt
  d = rs<T>(d + c.eps);                                                          //   .add_(eps)
  p = rs<T>(p + (neg_step_size * m) / d);                                        // param.addcdiv_(exp_avg, denom, value=-step_size)
}

template <typename T>
__global__ __launch_bounds__(NT) void adam_multi_kernel(const mvit_adam_tensor* __restrict__ tensors, int n_tensors,
                                                        AdamConsts c) {
  constexpr int V = mvit_elem<T>::vec;
  typedef __attribute__((ext_vector_type(V))) T vec_t;
  const int64_t chunk = blockIdx.x;
  const int ti = find_tensor(tensors, n_tensors, chunk);
  const mvit_adam_tensor t = tensors[ti];
  const int64_t base = (chunk - t.first_chunk) * CHUNK;
  const int64_t left = t.numel - base;
  const int n = left < CHUNK ? (int)left : CHUNK;
  T* P = static_cast<T*>(t.param) + base;
  T* G = static_cast<T*>(t.grad) + base;
  T* M = static_cast<T*>(t.exp_avg) + base;
  T* Vv = static_cast<T*>(t.exp_avg_sq) + base;
  const float wd = t.weight_decay, nss = -t.step_size, bc2 = t.bias_correction2_sqrt;
  const bool wg = c.write_grad && c.grad_scale != 1.0f;
  const int64_t sh_cols = t.shadow_cols > 0 ? t.shadow_cols : t.numel, sh_ld = t.shadow_cols > 0 ? t.shadow_ld : t.numel;
  const bool sh_bf16 = t.shadow_dtype == MVIT_BF16;
  const uintptr_t mis = (reinterpret_cast<uintptr_t>(P) | reinterpret_cast<uintptr_t>(G) | reinterpret_cast<uintptr_t>(M) |
                         reinterpret_cast<uintptr_t>(Vv)) & 15u;
  int done = 0;
  if (mis == 0) {  // 16-byte vectors over the aligned body
    const int nvec = n / V;
    for (int i = threadIdx.x; i < nvec; i += NT) {
      vec_t p = reinterpret_cast<vec_t*>(P)[i], g = reinterpret_cast<const vec_t*>(G)[i];
      vec_t m = reinterpret_cast<vec_t*>(M)[i], v = reinterpret_cast<vec_t*>(Vv)[i];
      float pnew[V];
#pragma unroll
      for (int j = 0; j < V; ++j) {
        float pf = to_f32(p[j]), gf = to_f32(g[j]), mf = to_f32(m[j]), vf = to_f32(v[j]);
        adam_elem<T>(pf, gf, mf, vf, c, wd, nss, bc2);
        pnew[j] = pf;
        p[j] = from_f32<T>(pf);
        g[j] = from_f32<T>(gf);
        m[j] = from_f32<T>(mf);
        v[j] = from_f32<T>(vf);
      }
      reinterpret_cast<vec_t*>(P)[i] = p;
      reinterpret_cast<vec_t*>(M)[i] = m;
      reinterpret_cast<vec_t*>(Vv)[i] = v;
      if (wg) reinterpret_cast<vec_t*>(G)[i] = g;
      if (t.shadow) {
        if (sh_bf16) shadow_store<bf16_t>(t.shadow, base + (int64_t)i * V, V, sh_cols, sh_ld, pnew);  // fp32 parameters: element-wise
        else shadow_store<float>(t.shadow, base + (int64_t)i * V, V, sh_cols, sh_ld, pnew);
      }
    }
    done = nvec * V;
  }
  for (int i = done + threadIdx.x; i < n; i += NT) {
    float pf = to_f32(P[i]), gf = to_f32(G[i]), mf = to_f32(M[i]), vf = to_f32(Vv[i]);
    adam_elem<T>(pf, gf, mf, vf, c, wd, nss, bc2);
    P[i] = from_f32<T>(pf);
    M[i] = from_f32<T>(mf);
    Vv[i] = from_f32<T>(vf);
    if (wg) G[i] = from_f32<T>(gf);
    if (t.shadow) {
      if (sh_bf16) shadow_store<bf16_t>(t.shadow, base + i, 1, sh_cols, sh_ld, &pf);
      else shadow_store<float>(t.shadow, base + i, 1, sh_cols, sh_ld, &pf);
    }
  }
}

// partial[chunk] = sum of g^2 over the chunk (fp32 per thread and per block; the chunks are added in fp64 below)
template <typename T>
__global__ __launch_bounds__(NT) void sumsq_multi_kernel(const mvit_adam_tensor* __restrict__ tensors, int n_tensors,
                                                         float* __restrict__ partial) {
  constexpr int V = mvit_elem<T>::vec;
  typedef __attribute__((ext_vector_type(V))) T vec_t;
  __shared__ float red[NT / MVIT_WAVE];
  const int64_t chunk = blockIdx.x;
  const int ti = find_tensor(tensors, n_tensors, chunk);
  const mvit_adam_tensor t = tensors[ti];
  const int64_t base = (chunk - t.first_chunk) * CHUNK;
  const int64_t left = t.numel - base;
  const int n = left < CHUNK ? (int)left : CHUNK;
  const T* G = static_cast<const T*>(t.grad) + base;
  float acc = 0.f;
  int done = 0;
  if ((reinterpret_cast<uintptr_t>(G) & 15u) == 0) {
    const int nvec = n / V;
    for (int i = threadIdx.x; i < nvec; i += NT) {
      const vec_t g = reinterpret_cast<const vec_t*>(G)[i];
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float x = to_f32(g[j]);
        acc += x * x;
      }
    }
    done = nvec * V;
  }
  for (int i = done + threadIdx.x; i < n; i += NT) {
    const float x = to_f32(G[i]);
    acc += x * x;
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NT / MVIT_WAVE; ++w) s += red[w];
    partial[chunk] = s;
  }
}

// out[0] = sum of the partials, in fp64 and in a fixed order (one block)
__global__ __launch_bounds__(1024) void sumsq_final_kernel(const float* __restrict__ partial, int64_t n, double* __restrict__ out) {
  __shared__ double red[1024];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += 1024) acc += (double)partial[i];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int s = 512; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = red[0];
}

int check_table(const char* what, const mvit_adam_tensor* tensors, int n_tensors, int64_t n_chunks, int dtype) {
  MVIT_REQUIRE(tensors != nullptr && n_tensors > 0, "%s: empty tensor table", what);
  MVIT_REQUIRE(n_chunks > 0 && n_chunks <= 0x7fffffffLL, "%s: n_chunks %lld out of range", what, (long long)n_chunks);
  MVIT_REQUIRE(dtype == MVIT_BF16 || dtype == MVIT_F32, "%s: dtype %d", what, dtype);
  static_assert(sizeof(mvit_adam_tensor) == 96, "table rows are 96 bytes");
  return MVIT_OK;
}

std::mutex g_scratch_mutex;
float* g_scratch_ptr[MVIT_MAX_DEVICES] = {};  // device address of `scratch` on each device, looked up on first use

// Address of `scratch` on the device that owns `stream` (set-up on the first call per device; no allocation).  The
// launch goes to the current device, so a stream of another device is refused instead of being handed this one's array.
int static_scratch(float** out, hipStream_t stream) {
  const int dev = mvit_current_device("grad_sumsq_static");
  if (dev < 0) return MVIT_ERR_LAUNCH;
  hipError_t e = hipSuccess;
  if (stream != nullptr) {
    hipDevice_t sdev = -1;
    e = hipStreamGetDevice(stream, &sdev);
    if (e != hipSuccess || (int)sdev != dev)
      return mvit_set_error(MVIT_ERR_ARG, "grad_sumsq_static: the stream belongs to device %d, the current device is %d (%s)", (int)sdev, dev,
                            hipGetErrorString(e));
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return mvit_set_error(MVIT_ERR_LAUNCH, "grad_sumsq_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<float*>(p);
  }
  *out = g_scratch_ptr[dev];
  return MVIT_OK;
}

}  // namespace

extern "C" {

int mvit_adam_step(const mvit_adam_tensor* tensors, int n_tensors, int64_t n_chunks, double beta1, double beta2, double eps,
                   double grad_scale, int write_grad, int dtype, mvit_stream_t stream) {
  if (int rc = check_table("adam_step", tensors, n_tensors, n_chunks, dtype)) return rc;
  MVIT_REQUIRE(beta1 > 0.5 && beta1 < 1.0 && beta2 >= 0.0 && beta2 < 1.0 && eps >= 0.0,
               "adam_step: betas (%g, %g) / eps %g outside the supported range (beta1 in (0.5, 1))", beta1, beta2, eps);
  AdamConsts c;
  // the scalars reach torch's kernels as doubles rounded once to fp32: 1 - beta is formed in double first
  c.beta2 = (float)beta2;
  c.one_minus_beta1 = (float)(1.0 - beta1);
  c.one_minus_beta2 = (float)(1.0 - beta2);
  c.eps = (float)eps;
  c.grad_scale = (float)grad_scale;
  c.write_grad = write_grad;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype == MVIT_BF16)
    hipLaunchKernelGGL((adam_multi_kernel<bf16_t>), dim3((unsigned)n_chunks), NT, 0, s, tensors, n_tensors, c);
  else
    hipLaunchKernelGGL((adam_multi_kernel<float>), dim3((unsigned)n_chunks), NT, 0, s, tensors, n_tensors, c);
  MVIT_CHECK_LAUNCH("adam_step");
  return MVIT_OK;
}

int mvit_grad_sumsq(const mvit_adam_tensor* tensors, int n_tensors, int64_t n_chunks, float* partial, double* out, int dtype,
                    mvit_stream_t stream) {
  if (int rc = check_table("grad_sumsq", tensors, n_tensors, n_chunks, dtype)) return rc;
  MVIT_REQUIRE(partial != nullptr && out != nullptr, "grad_sumsq: null output");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype == MVIT_BF16)
    hipLaunchKernelGGL((sumsq_multi_kernel<bf16_t>), dim3((unsigned)n_chunks), NT, 0, s, tensors, n_tensors, partial);
  else
    hipLaunchKernelGGL((sumsq_multi_kernel<float>), dim3((unsigned)n_chunks), NT, 0, s, tensors, n_tensors, partial);
  MVIT_CHECK_LAUNCH("grad_sumsq");
  hipLaunchKernelGGL(sumsq_final_kernel, dim3(1), 1024, 0, s, (const float*)partial, n_chunks, out);
  MVIT_CHECK_LAUNCH("grad_sumsq (final)");
  return MVIT_OK;
}

int mvit_grad_sumsq_static(const mvit_adam_tensor* tensors, int n_tensors, int64_t n_chunks, double* out, int dtype,
                           mvit_stream_t stream) {
  if (int rc = check_table("grad_sumsq_static", tensors, n_tensors, n_chunks, dtype)) return rc;
  MVIT_REQUIRE(out != nullptr, "grad_sumsq_static: null output");
  MVIT_REQUIRE(n_chunks <= (int64_t)MVIT_SUMSQ_STATIC_MAX_CHUNKS,
               "grad_sumsq_static: %lld chunks exceed the built-in scratch of %d chunks (%lld elements); use mvit_grad_sumsq with a workspace",
               (long long)n_chunks, MVIT_SUMSQ_STATIC_MAX_CHUNKS, (long long)MVIT_SUMSQ_STATIC_MAX_CHUNKS * MVIT_ADAM_CHUNK);
  float* partial = nullptr;
  if (int rc = static_scratch(&partial, reinterpret_cast<hipStream_t>(stream))) return rc;
  // every partial in [0, n_chunks) is overwritten by the first kernel, so nothing has to be cleared between calls
  return mvit_grad_sumsq(tensors, n_tensors, n_chunks, partial, out, dtype, stream);
}

}  // extern "C"
