// RMSNorm fused with the residual add that precedes it.
//   resid (float, in place) += delta;  out = resid * rsqrt(mean(resid^2) + eps) * w
// delta is a tensor in the activation dtype, or the float partial sums of a
// product whose K was split over workgroups (parts [nparts][T][H], optionally a
// bias [H]): the partial sums are then added here instead of by a kernel of
// their own.
// Formula and float32 math: servelab/attention/triton/paged_attention.py:76-91,
// tests/test_triton_kernels.py:57-59; the adds it absorbs are
// servelab/parallel/tp_model.py:131,133.  One block per row.
#include "common.h"

// rows == nullptr: row r of the stream, which is updated in place.
// rows != nullptr: row rows[r] of the stream (and of delta) is read, nothing
// but out[r] is written.
struct SplitDelta {
  const float* parts;            // [nparts][stride], or nullptr
  int nparts;
  size_t stride;                 // T * H
  const float* bias;             // [H] or nullptr
};

__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const act_t* __restrict__ delta,
                                   const SplitDelta sd, const int* __restrict__ rows,
                                   const float* __restrict__ w, act_t* __restrict__ out, int H,
                                   float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* d = delta != nullptr ? delta + src * H : nullptr;
  const float* p = sd.parts != nullptr ? sd.parts + src * H : nullptr;
  const bool adds = d != nullptr || p != nullptr;
  auto delta_at = [&](int i) {
    float v = d != nullptr ? to_f(d[i]) : 0.f;
    if (p != nullptr) {
      for (int j = 0; j < sd.nparts; ++j) v += p[j * sd.stride + i];
      if (sd.bias != nullptr) v += sd.bias[i];
    }
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (adds) {
      v += delta_at(i);
      if (rows == nullptr) x[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)H + eps);
  act_t* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (adds && rows != nullptr) v += delta_at(i);
    o[i] = from_f<act_t>(v * inv * w[i]);
  }
}

// The same for rows of up to 4 * 8 * blockDim values that are a multiple of 4
// wide: every value is read once with 16-byte loads and kept in registers
// between the sum of squares and the scaling.
struct __attribute__((aligned(16))) f4 { float v[4]; };
#if defined(SL_F32)
struct __attribute__((aligned(16))) a4 { act_t v[4]; };
#else
struct __attribute__((aligned(8))) a4 { act_t v[4]; };
#endif

template <int ITERS>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ resid, const act_t* __restrict__ delta,
                                       const SplitDelta sd, const int* __restrict__ rows,
                                       const float* __restrict__ w, act_t* __restrict__ out, int H,
                                       float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* d = delta != nullptr ? delta + src * H : nullptr;
  const float* p = sd.parts != nullptr ? sd.parts + src * H : nullptr;
  const int H4 = H / 4;
  f4 v[ITERS];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = threadIdx.x + it * blockDim.x;
    if (i < H4) {
      v[it] = ((const f4*)x)[i];
      if (d != nullptr) {
        const a4 dv = ((const a4*)d)[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[it].v[j] += to_f(dv.v[j]);
      }
      if (p != nullptr) {
#pragma unroll 4
        for (int q = 0; q < sd.nparts; ++q) {
          const f4 pv = ((const f4*)(p + q * sd.stride))[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[it].v[j] += pv.v[j];
        }
        if (sd.bias != nullptr) {
          const f4 bv = ((const f4*)sd.bias)[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[it].v[j] += bv.v[j];
        }
      }
      if ((d != nullptr || p != nullptr) && rows == nullptr) ((f4*)x)[i] = v[it];
#pragma unroll
      for (int j = 0; j < 4; ++j) ss += v[it].v[j] * v[it].v[j];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)H + eps);
  act_t* o = out + (size_t)r * H;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = threadIdx.x + it * blockDim.x;
    if (i < H4) {
      const f4 wv = ((const f4*)w)[i];
      a4 ov;
#pragma unroll
      for (int j = 0; j < 4; ++j) ov.v[j] = from_f<act_t>(v[it].v[j] * inv * wv.v[j]);
      ((a4*)o)[i] = ov;
    }
  }
}

// parts != nullptr: nparts float partial sums [nparts][T][H] (T rows in each)
// and an optional bias [H] are the delta (or are added to it).
extern "C" const char* sl_add_rmsnorm(float* resid, const void* delta, const float* parts,
                                      int nparts, int T, const float* bias, const int* rows,
                                      const float* w, void* out, int R, int H, float eps,
                                      hipStream_t stream) {
  SL_CHECK(R >= 0 && H > 0, "add_rmsnorm: sizes must be positive");
  SL_CHECK(parts == nullptr || (nparts >= 1 && T >= 1), "add_rmsnorm: partial sums need their counts");
  SL_CHECK(parts != nullptr || bias == nullptr, "add_rmsnorm: a bias comes with partial sums only");
  if (R == 0) return nullptr;
  const SplitDelta sd{parts, nparts, (size_t)T * H, bias};
  const bool aligned = ((uintptr_t)resid % 16) == 0 && ((uintptr_t)out % sizeof(a4)) == 0 &&
                       ((uintptr_t)delta % sizeof(a4)) == 0 && ((uintptr_t)parts % 16) == 0 &&
                       ((uintptr_t)bias % 16) == 0 && ((uintptr_t)w % 16) == 0;
  if (H % 4 == 0 && H <= 4 * 8 * 512 && aligned) {
    const int H4 = H / 4;
    const int threads = H4 <= 64 ? 64 : (H4 <= 128 ? 128 : (H4 <= 256 ? 256 : 512));
    const int iters = (H4 + threads - 1) / threads;
    const act_t* dl = (const act_t*)delta;
    act_t* o = (act_t*)out;
    if (iters == 1) add_rmsnorm_vec_kernel<1><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    else if (iters == 2) add_rmsnorm_vec_kernel<2><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    else if (iters <= 4) add_rmsnorm_vec_kernel<4><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    else add_rmsnorm_vec_kernel<8><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    return sl_launch_status();
  }
  const int threads = H >= 2048 ? 512 : 256;
  add_rmsnorm_kernel<<<R, threads, 0, stream>>>(resid, (const act_t*)delta, sd, rows, w,
                                                (act_t*)out, H, eps);
  return sl_launch_status();
}

// Layer norm with a gain and no bias, fused with the residual add that precedes it:
//   resid (float, in place) += d1 + d2;  out = (resid - mean) / sqrt(var + eps) * w
// where var is the mean of the squared deviations.  Either delta may be absent.
// rows as above: with rows the stream is only read.  One block per row; the
// row is read three times (sum, squared deviations, output), from cache after
// the first.
__global__ void add_layernorm_kernel(float* __restrict__ resid, const act_t* __restrict__ d1,
                                     const act_t* __restrict__ d2, const int* __restrict__ rows,
                                     const float* __restrict__ w, act_t* __restrict__ out, int H,
                                     float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* a = d1 != nullptr ? d1 + src * H : nullptr;
  const act_t* b = d2 != nullptr ? d2 + src * H : nullptr;
  const bool adds = a != nullptr || b != nullptr;
  const bool again = adds && rows != nullptr;        // the sum is not stored: form it on every pass
  auto value = [&](int i) {
    float d = 0.f;
    if (a != nullptr) d = to_f(a[i]);
    if (b != nullptr) d += to_f(b[i]);
    return x[i] + d;
  };
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (adds) {
      v = value(i);
      if (rows == nullptr) x[i] = v;
    }
    sum += v;
  }
  const float mean = block_sum(sum, scratch) / (float)H;
  float sq = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float dv = (again ? value(i) : x[i]) - mean;
    sq += dv * dv;
  }
  const float inv = 1.f / sqrtf(block_sum(sq, scratch) / (float)H + eps);
  act_t* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    o[i] = from_f<act_t>(((again ? value(i) : x[i]) - mean) * inv * w[i]);
}

// The same for rows of up to 4 * 8 * blockDim values that are a multiple of 4 wide: every value
// is read once with 16-byte loads and stays in registers for the mean, the squared deviations
// and the output.
template <int ITERS>
__global__ void add_layernorm_vec_kernel(float* __restrict__ resid, const act_t* __restrict__ d1,
                                         const act_t* __restrict__ d2, const int* __restrict__ rows,
                                         const float* __restrict__ w, act_t* __restrict__ out, int H,
                                         float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* a = d1 != nullptr ? d1 + src * H : nullptr;
  const act_t* b = d2 != nullptr ? d2 + src * H : nullptr;
  const int H4 = H / 4;
  f4 v[ITERS];
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = threadIdx.x + it * blockDim.x;
    if (i < H4) {
      v[it] = ((const f4*)x)[i];
      if (a != nullptr || b != nullptr) {
        float d[4] = {0.f, 0.f, 0.f, 0.f};
        if (a != nullptr) {
          const a4 av = ((const a4*)a)[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) d[j] = to_f(av.v[j]);
        }
        if (b != nullptr) {
          const a4 bv = ((const a4*)b)[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) d[j] += to_f(bv.v[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) v[it].v[j] += d[j];
        if (rows == nullptr) ((f4*)x)[i] = v[it];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) sum += v[it].v[j];
    }
  }
  const float mean = block_sum(sum, scratch) / (float)H;
  float sq = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = threadIdx.x + it * blockDim.x;
    if (i < H4) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[it].v[j] -= mean;
        sq += v[it].v[j] * v[it].v[j];
      }
    }
  }
  const float inv = 1.f / sqrtf(block_sum(sq, scratch) / (float)H + eps);
  act_t* o = out + (size_t)r * H;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = threadIdx.x + it * blockDim.x;
    if (i < H4) {
      const f4 wv = ((const f4*)w)[i];
      a4 ov;
#pragma unroll
      for (int j = 0; j < 4; ++j) ov.v[j] = from_f<act_t>(v[it].v[j] * inv * wv.v[j]);
      ((a4*)o)[i] = ov;
    }
  }
}

extern "C" const char* sl_add_layernorm(float* resid, const void* d1, const void* d2, const int* rows,
                                        const float* w, void* out, int R, int H, float eps,
                                        hipStream_t stream) {
  SL_CHECK(R >= 0 && H > 0, "add_layernorm: sizes must be positive");
  if (R == 0) return nullptr;
  const bool aligned = ((uintptr_t)resid % 16) == 0 && ((uintptr_t)out % sizeof(a4)) == 0 &&
                       ((uintptr_t)d1 % sizeof(a4)) == 0 && ((uintptr_t)d2 % sizeof(a4)) == 0 &&
                       ((uintptr_t)w % 16) == 0;
  if (H % 4 == 0 && H <= 4 * 8 * 512 && aligned) {
    const int H4 = H / 4;
    const int nthreads = H4 <= 64 ? 64 : (H4 <= 128 ? 128 : (H4 <= 256 ? 256 : 512));
    const int iters = (H4 + nthreads - 1) / nthreads;
    const act_t* a = (const act_t*)d1;
    const act_t* b = (const act_t*)d2;
    act_t* o = (act_t*)out;
    if (iters == 1) add_layernorm_vec_kernel<1><<<R, nthreads, 0, stream>>>(resid, a, b, rows, w, o, H, eps);
    else if (iters == 2) add_layernorm_vec_kernel<2><<<R, nthreads, 0, stream>>>(resid, a, b, rows, w, o, H, eps);
    else if (iters <= 4) add_layernorm_vec_kernel<4><<<R, nthreads, 0, stream>>>(resid, a, b, rows, w, o, H, eps);
    else add_layernorm_vec_kernel<8><<<R, nthreads, 0, stream>>>(resid, a, b, rows, w, o, H, eps);
    return sl_launch_status();
  }
  const int threads = H >= 2048 ? 512 : 256;
  add_layernorm_kernel<<<R, threads, 0, stream>>>(resid, (const act_t*)d1, (const act_t*)d2, rows, w,
                                                  (act_t*)out, H, eps);
  return sl_launch_status();
}

// resid (float, in place) += delta: for a delta that a norm cannot take with its own add.
__global__ void add_into_kernel(float* __restrict__ resid, const act_t* __restrict__ delta, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) resid[i] += to_f(delta[i]);
}

extern "C" const char* sl_add_into(float* resid, const void* delta, long long n, hipStream_t stream) {
  SL_CHECK(n >= 0, "add_into: the count must not be negative");
  if (n == 0) return nullptr;
  add_into_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(resid, (const act_t*)delta, (size_t)n);
  return sl_launch_status();
}

// RMS norm on a sublayer's output: resid (float, in place) += mult * y * rsqrt(mean(y^2) + eps) * w,
// and the stream's new rows in the activation type for the sublayer that reads them next.  y == nullptr:
// only those rows.  One block per row; sums and the stream in float.
__global__ void add_postnorm_kernel(float* __restrict__ resid, const act_t* __restrict__ y,
                                    const float* __restrict__ w, act_t* __restrict__ out, int H, float eps,
                                    float mult) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  float* x = resid + r * H;
  act_t* o = out + r * H;
  if (y == nullptr) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = from_f<act_t>(x[i]);
    return;
  }
  const act_t* yr = y + r * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = to_f(yr[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = x[i] + mult * (to_f(yr[i]) * inv * w[i]);
    x[i] = v;
    o[i] = from_f<act_t>(v);
  }
}

extern "C" const char* sl_add_postnorm(float* resid, const void* y, const float* w, void* out, int T, int H,
                                       float eps, float mult, hipStream_t stream) {
  SL_CHECK(T >= 0 && H > 0, "add_postnorm: sizes must be positive");
  if (T == 0) return nullptr;
  add_postnorm_kernel<<<T, H >= 2048 ? 512 : 256, 0, stream>>>(resid, (const act_t*)y, w, (act_t*)out, H, eps, mult);
  return sl_launch_status();
}

// A sublayer's output joins the stream through a norm of its own, and the next sublayer's input norm
// follows at once: v = resid + y * rsqrt(mean(y^2) + eps_y) * wy, out = v * rsqrt(mean(v^2) + eps) * w.
// rows == nullptr: every row, and v goes back to the stream; else only the listed rows are computed
// and the stream stays as it is (the head reads few rows of the last layer's result).  One block per
// row, up to NORMED_KEEP values a thread kept in registers between the passes; all sums in float.
constexpr int NORMED_KEEP = 8;
__global__ void add_normed_rmsnorm_kernel(float* __restrict__ resid, const act_t* __restrict__ y,
                                          const float* __restrict__ wy, float eps_y,
                                          const int* __restrict__ rows, const float* __restrict__ w, float eps,
                                          act_t* __restrict__ out, int H) {
  __shared__ float scratch[16];
  const size_t r = rows != nullptr ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  float* x = resid + r * H;
  const act_t* yr = y + r * H;
  act_t* o = out + (size_t)blockIdx.x * H;
  float keep[NORMED_KEEP];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < NORMED_KEEP; ++u) {
    const int i = threadIdx.x + u * blockDim.x;
    keep[u] = i < H ? to_f(yr[i]) : 0.f;
    ss += keep[u] * keep[u];
  }
  for (int i = threadIdx.x + NORMED_KEEP * blockDim.x; i < H; i += blockDim.x) {
    const float v = to_f(yr[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv_y = 1.f / sqrtf(ss / (float)H + eps_y);
  float s2 = 0.f;
#pragma unroll
  for (int u = 0; u < NORMED_KEEP; ++u) {
    const int i = threadIdx.x + u * blockDim.x;
    if (i < H) {
      keep[u] = x[i] + keep[u] * inv_y * wy[i];
      if (rows == nullptr) x[i] = keep[u];
      s2 += keep[u] * keep[u];
    }
  }
  for (int i = threadIdx.x + NORMED_KEEP * blockDim.x; i < H; i += blockDim.x) {
    const float v = x[i] + to_f(yr[i]) * inv_y * wy[i];
    if (rows == nullptr) x[i] = v;
    s2 += v * v;
  }
  s2 = block_sum(s2, scratch);
  const float inv = 1.f / sqrtf(s2 / (float)H + eps);
#pragma unroll
  for (int u = 0; u < NORMED_KEEP; ++u) {
    const int i = threadIdx.x + u * blockDim.x;
    if (i < H) o[i] = from_f<act_t>(keep[u] * inv * w[i]);
  }
  for (int i = threadIdx.x + NORMED_KEEP * blockDim.x; i < H; i += blockDim.x) {
    const float v = rows == nullptr ? x[i] : x[i] + to_f(yr[i]) * inv_y * wy[i];
    o[i] = from_f<act_t>(v * inv * w[i]);
  }
}

extern "C" const char* sl_add_normed_rmsnorm(float* resid, const void* y, const float* wy, float eps_y,
                                             const int* rows, const float* w, float eps, void* out, int R,
                                             int H, hipStream_t stream) {
  SL_CHECK(R >= 0 && H > 0, "add_normed_rmsnorm: sizes must be positive");
  SL_CHECK(y != nullptr && wy != nullptr && w != nullptr, "add_normed_rmsnorm: the output and both gains are required");
  if (R == 0) return nullptr;
  add_normed_rmsnorm_kernel<<<R, H >= 2048 ? 512 : 256, 0, stream>>>(resid, (const act_t*)y, wy, eps_y, rows, w,
                                                                    eps, (act_t*)out, H);
  return sl_launch_status();
}

// out = sa * a + sb * b, float sums: the outputs of two mixers that ran side by side.
__global__ void scaled_sum_kernel(const act_t* __restrict__ a, float sa, const act_t* __restrict__ b, float sb,
                                  act_t* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f<act_t>(sa * to_f(a[i]) + sb * to_f(b[i]));
}

extern "C" const char* sl_scaled_sum(const void* a, float sa, const void* b, float sb, void* out, long long n,
                                     hipStream_t stream) {
  SL_CHECK(n >= 0, "scaled_sum: the count must not be negative");
  if (n == 0) return nullptr;
  scaled_sum_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((const act_t*)a, sa, (const act_t*)b, sb,
                                                                    (act_t*)out, (size_t)n);
  return sl_launch_status();
}

// x = cap * tanh(x / cap) in place on float values (logits).
__global__ void softcap_kernel(float* __restrict__ x, float cap, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" const char* sl_softcap(float* x, float cap, long long n, hipStream_t stream) {
  SL_CHECK(n >= 0 && cap > 0.f, "softcap: the count must not be negative, the cap positive");
  if (n == 0) return nullptr;
  softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, cap, (size_t)n);
  return sl_launch_status();
}

// x *= factor in place on float values (logits).
__global__ void scale_kernel(float* __restrict__ x, float factor, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] *= factor;
}

extern "C" const char* sl_scale(float* x, float factor, long long n, hipStream_t stream) {
  SL_CHECK(n >= 0, "scale: the count must not be negative");
  if (n == 0) return nullptr;
  scale_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, factor, (size_t)n);
  return sl_launch_status();
}
