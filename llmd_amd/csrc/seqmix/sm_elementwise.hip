// Row kernels of per-layer stacks: embedding with scale, zero-centred RMS norms on the fp32
// residual, post-norm + layer scale + residual add (+ the next pre-norm in the same pass),
// the depth average (+ the norm that follows it), xIELU and the logit soft cap; the embedding with
// a hashed bigram table and the plain post-norm residual add of stacks that norm only outputs; the
// embedding with the first plain norm, the plain norm of a projection's rows and the squared ReLU.
// One workgroup of 256 threads per token row; the fp32 residual is read and written once.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void embed_scale_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                        float scale, float* __restrict__ o0, float* __restrict__ o1,
                                                        int d, int64_t V) {
  const int64_t row = blockIdx.x;
  const int64_t id = min(max(ids[row], (int64_t)0), V - 1);  // a bad id must not read outside the table
  const T* src = table + id * (int64_t)d;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = ld(src + c) * scale;
    o0[row * d + c] = v;
    o1[row * d + c] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void zc_norm_kernel(const float* __restrict__ x, const T* __restrict__ w, float eps,
                                                    T* __restrict__ out, int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  const float* xr = x + row * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) ss += xr[c] * xr[c];
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, xr[c] * inv * (1.f + ld(w + c)));
}

// x += ls * (y / rms(y) * (1 + wp));  optionally out = x / rms(x) * (1 + wn)
template <typename T>
__global__ __launch_bounds__(NT) void add_post_norm_kernel(const T* __restrict__ y, int64_t y_stride,
                                                          const T* __restrict__ wp, const T* __restrict__ ls,
                                                          float* __restrict__ x, float eps, const T* __restrict__ wn,
                                                          T* __restrict__ out, int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float* xr = x + row * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = ld(yr + c);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = xr[c] + ld(ls + c) * (ld(yr + c) * inv * (1.f + ld(wp + c)));
    xr[c] = v;
    s2 += v * v;
  }
  if (wn == nullptr) return;
  s2 = block_sum<NT>(s2, red);
  const float inv2 = 1.f / sqrtf(s2 / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, xr[c] * inv2 * (1.f + ld(wn + c)));
}

// hist[dst] = sum_{j<n} coef[j] hist[j];  out = zero-centred norm of it
template <typename T>
__global__ __launch_bounds__(NT) void depth_avg_norm_kernel(float* __restrict__ hist, int64_t plane, int n,
                                                           const float* __restrict__ coef, int dst,
                                                           const T* __restrict__ w, float eps, T* __restrict__ out,
                                                           int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  float* dr = hist + dst * plane + row * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    float s = 0.f;
    for (int j = 0; j < n; ++j) s += coef[j] * hist[j * plane + row * d + c];
    dr[c] = s;
    ss += s * s;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, dr[c] * inv * (1.f + ld(w + c)));
}

template <typename T>
__global__ __launch_bounds__(NT) void xielu_kernel(const T* __restrict__ z, float ap, float aq, T* __restrict__ out,
                                                  int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i >= n) return;
  const float v = ld(z + i);
  st(out + i, v > 0.f ? ap * v * v + 0.5f * v : aq * (expm1f(v) - v) + 0.5f * v);
}

__global__ __launch_bounds__(NT) void softcap_kernel(float* __restrict__ x, float cap, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

// Row of the bigram table for every token: (previous * mul_prev + token * mul_cur) mod buckets, row
// ``buckets`` for a sequence's first token. The previous token of a run's first token is the
// sequence's state; this kernel only reads it (the embedding kernel that follows writes it).
__global__ __launch_bounds__(NT) void bigram_rows_kernel(const int64_t* __restrict__ ids, int T, int64_t buckets,
                                                        int64_t mul_prev, int64_t mul_cur,
                                                        const int* __restrict__ prev_state,
                                                        const int* __restrict__ row_seq,
                                                        const int* __restrict__ seq_start,
                                                        const int* __restrict__ seq_slot,
                                                        const int* __restrict__ seq_init, int* __restrict__ rows) {
  const int t = blockIdx.x * NT + threadIdx.x;
  if (t >= T) return;
  const int s = row_seq[t];
  int64_t prev;
  if (t > seq_start[s]) prev = ids[t - 1];
  else if (seq_init[s]) prev = prev_state[seq_slot[s]];
  else {
    rows[t] = (int)buckets;
    return;
  }
  int64_t r = (prev * mul_prev + ids[t] * mul_cur) % buckets;
  if (r < 0) r += buckets;
  rows[t] = (int)r;
}

// x = table[id] * scale + bigram[row] (fp32) and its copy in the activation type; the workgroup of a
// run's last token writes the token into the sequence's state.
template <typename T>
__global__ __launch_bounds__(NT) void bigram_embed_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                         float scale, int64_t V, const T* __restrict__ bigram,
                                                         const int* __restrict__ rows, int* __restrict__ prev_state,
                                                         const int* __restrict__ row_seq,
                                                         const int* __restrict__ seq_start,
                                                         const int* __restrict__ seq_slot, float* __restrict__ x,
                                                         T* __restrict__ out, int d) {
  const int64_t row = blockIdx.x;
  const int64_t id = min(max(ids[row], (int64_t)0), V - 1);  // a bad id must not read outside the table
  const T* src = table + id * (int64_t)d;
  const T* big = bigram ? bigram + (int64_t)rows[row] * d : nullptr;
  for (int c = threadIdx.x; c < d; c += NT) {
    float v = ld(src + c) * scale;
    if (big) v += ld(big + c);
    x[row * d + c] = v;
    st(out + row * d + c, v);
  }
  if (threadIdx.x == 0 && prev_state != nullptr) {
    const int s = row_seq[row];
    if (row + 1 == seq_start[s + 1]) prev_state[seq_slot[s]] = (int)ids[row];
  }
}

// x += rms_norm(a y + b y2 + bias) * wp;  out = x (activation type) or rms_norm(x) * wn
template <typename T>
__global__ __launch_bounds__(NT) void post_norm_add_kernel(const T* __restrict__ y, int64_t y_stride,
                                                          const T* __restrict__ y2, int64_t y2_stride, float a,
                                                          float b, const float* __restrict__ bias,
                                                          const T* __restrict__ wp, float* __restrict__ x, float eps,
                                                          const T* __restrict__ wn, T* __restrict__ out, int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  const T* y2r = y2 ? y2 + row * y2_stride : nullptr;
  float* xr = x + row * d;
  auto val = [&](int c) {
    float v = a * ld(yr + c);
    if (y2r) v += b * ld(y2r + c);
    if (bias) v += bias[c];
    return v;
  };
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = val(c);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = xr[c] + val(c) * inv * ld(wp + c);
    xr[c] = v;
    s2 += v * v;
    if (wn == nullptr) st(out + row * d + c, v);
  }
  if (wn == nullptr) return;
  s2 = block_sum<NT>(s2, red);
  const float inv2 = 1.f / sqrtf(s2 / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, xr[c] * inv2 * ld(wn + c));
}

// The same for bf16 rows of d = 8 n <= 8 * NT * NCH elements with 16-byte accesses: a thread keeps its
// NCH chunks of eight elements in registers from the first pass to the last, so y is read once, x read
// and written once and out written once; a small step's rows are a few loads deep instead of d / NT.
template <int NCH>
__global__ __launch_bounds__(NT) void post_norm_add_vec_kernel(const bf16_t* __restrict__ y, int64_t y_stride,
                                                              const bf16_t* __restrict__ y2, int64_t y2_stride,
                                                              float a, float b, const float* __restrict__ bias,
                                                              const bf16_t* __restrict__ wp, float* __restrict__ x,
                                                              float eps, const bf16_t* __restrict__ wn,
                                                              bf16_t* __restrict__ out, int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  auto ld8 = [](const bf16_t* p, float* v) {
    const uint4 q = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
    v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
    v[4] = __uint_as_float(q.z << 16); v[5] = __uint_as_float(q.z & 0xffff0000u);
    v[6] = __uint_as_float(q.w << 16); v[7] = __uint_as_float(q.w & 0xffff0000u);
  };
  auto ldf8 = [](const float* p, float* v) {
    const float4 q0 = *reinterpret_cast<const float4*>(p), q1 = *reinterpret_cast<const float4*>(p + 4);
    v[0] = q0.x; v[1] = q0.y; v[2] = q0.z; v[3] = q0.w; v[4] = q1.x; v[5] = q1.y; v[6] = q1.z; v[7] = q1.w;
  };
  auto pack = [](float lo_, float hi_) {
    const __bf16 l16 = (__bf16)lo_, h16 = (__bf16)hi_;
    return (uint32_t)__builtin_bit_cast(uint16_t, l16) | ((uint32_t)__builtin_bit_cast(uint16_t, h16) << 16);
  };
  float v[NCH][8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (k * NT + threadIdx.x) * 8;
    if (c < d) {
      ld8(y + row * y_stride + c, v[k]);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[k][i] *= a;
      if (y2) {
        float t[8];
        ld8(y2 + row * y2_stride + c, t);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[k][i] += b * t[i];
      }
      if (bias) {
        float t[8];
        ldf8(bias + c, t);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[k][i] += t[i];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[k][i] * v[k][i];
    }
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  float s2 = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (k * NT + threadIdx.x) * 8;
    if (c < d) {
      float xv[8], w[8];
      ldf8(x + row * d + c, xv);
      ld8(wp + c, w);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[k][i] = xv[i] + v[k][i] * inv * w[i];
        s2 += v[k][i] * v[k][i];
      }
      float* xr = x + row * d + c;
      *reinterpret_cast<float4*>(xr) = make_float4(v[k][0], v[k][1], v[k][2], v[k][3]);
      *reinterpret_cast<float4*>(xr + 4) = make_float4(v[k][4], v[k][5], v[k][6], v[k][7]);
    }
  }
  float inv2 = 1.f;
  if (wn != nullptr) {
    s2 = block_sum<NT>(s2, red);
    inv2 = 1.f / sqrtf(s2 / (float)d + eps);
  }
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (k * NT + threadIdx.x) * 8;
    if (c < d) {
      float w[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
      if (wn != nullptr) ld8(wn + c, w);
      uint4 o;
      o.x = pack(v[k][0] * inv2 * w[0], v[k][1] * inv2 * w[1]);
      o.y = pack(v[k][2] * inv2 * w[2], v[k][3] * inv2 * w[3]);
      o.z = pack(v[k][4] * inv2 * w[4], v[k][5] * inv2 * w[5]);
      o.w = pack(v[k][6] * inv2 * w[6], v[k][7] * inv2 * w[7]);
      *reinterpret_cast<uint4*>(out + row * d + c) = o;
    }
  }
}

// x = table[id] (fp32 residual);  out = x / rms(x) * w
template <typename T>
__global__ __launch_bounds__(NT) void embed_norm_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                       int64_t V, const T* __restrict__ w, float eps,
                                                       float* __restrict__ x, T* __restrict__ out, int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  const int64_t id = min(max(ids[row], (int64_t)0), V - 1);  // a bad id must not read outside the table
  const T* src = table + id * (int64_t)d;
  float* xr = x + row * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = ld(src + c);
    xr[c] = v;
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, ld(src + c) * inv * ld(w + c));
}

// out = y / rms(y) * w over rows of n elements (y may be a column view: y_stride); a wave per row
template <typename T>
__global__ __launch_bounds__(NT) void rms_norm_rows_kernel(const T* __restrict__ y, int64_t y_stride,
                                                          const T* __restrict__ w, float eps, T* __restrict__ out,
                                                          int n, int rows) {
  const int64_t row = (int64_t)blockIdx.x * (NT / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const T* yr = y + row * y_stride;
  float ss = 0.f;
  for (int c = lane; c < n; c += 64) {
    const float v = ld(yr + c);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)n + eps);
  for (int c = lane; c < n; c += 64) st(out + row * n + c, ld(yr + c) * inv * ld(w + c));
}

// the same with a workgroup per row: long rows of small steps
template <typename T>
__global__ __launch_bounds__(NT) void rms_norm_row_block_kernel(const T* __restrict__ y, int64_t y_stride,
                                                               const T* __restrict__ w, float eps,
                                                               T* __restrict__ out, int n) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += NT) {
    const float v = ld(yr + c);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += NT) st(out + row * n + c, ld(yr + c) * inv * ld(w + c));
}

template <typename T>
__global__ __launch_bounds__(NT) void relu2_kernel(const T* __restrict__ z, T* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i >= n) return;
  const float v = fmaxf(ld(z + i), 0.f);
  st(out + i, v * v);
}

// bf16, eight elements per thread (n a multiple of 8, 16-byte aligned)
__global__ __launch_bounds__(NT) void relu2_vec_kernel(const uint4* __restrict__ z, uint4* __restrict__ out, int64_t n8) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i >= n8) return;
  const uint4 t = z[i];
  uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float a = fmaxf(__uint_as_float(w[k] << 16), 0.f), b = fmaxf(__uint_as_float(w[k] & 0xffff0000u), 0.f);
    const __bf16 ha = (__bf16)(a * a), hb = (__bf16)(b * b);
    w[k] = (uint32_t)__builtin_bit_cast(uint16_t, ha) | ((uint32_t)__builtin_bit_cast(uint16_t, hb) << 16);
  }
  out[i] = make_uint4(w[0], w[1], w[2], w[3]);
}

}  // namespace

extern "C" {

void sm_embed_norm(const int64_t* ids, const void* table, int64_t V, const void* w, float eps, float* x, void* out,
                   int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((embed_norm_kernel<float>), dim3(T), dim3(NT), 0, stream, ids, (const float*)table, V,
                       (const float*)w, eps, x, (float*)out, d);
  else
    hipLaunchKernelGGL((embed_norm_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, ids, (const bf16_t*)table, V,
                       (const bf16_t*)w, eps, x, (bf16_t*)out, d);
}

void sm_rms_norm_rows(const void* y, int64_t y_stride, const void* w, float eps, void* out, int rows, int n, int f32,
                      hipStream_t stream) {
  if (rows == 0) return;
  if (n >= 512 && rows <= 16384) {  // a wave would walk a long row alone
    if (f32)
      hipLaunchKernelGGL((rms_norm_row_block_kernel<float>), dim3(rows), dim3(NT), 0, stream, (const float*)y, y_stride,
                         (const float*)w, eps, (float*)out, n);
    else
      hipLaunchKernelGGL((rms_norm_row_block_kernel<bf16_t>), dim3(rows), dim3(NT), 0, stream, (const bf16_t*)y,
                         y_stride, (const bf16_t*)w, eps, (bf16_t*)out, n);
    return;
  }
  const dim3 grid((rows + NT / 64 - 1) / (NT / 64));
  if (f32)
    hipLaunchKernelGGL((rms_norm_rows_kernel<float>), grid, dim3(NT), 0, stream, (const float*)y, y_stride,
                       (const float*)w, eps, (float*)out, n, rows);
  else
    hipLaunchKernelGGL((rms_norm_rows_kernel<bf16_t>), grid, dim3(NT), 0, stream, (const bf16_t*)y, y_stride,
                       (const bf16_t*)w, eps, (bf16_t*)out, n, rows);
}

void sm_relu2(const void* z, void* out, int64_t n, int f32, hipStream_t stream) {
  if (n == 0) return;
  if (f32) {
    hipLaunchKernelGGL((relu2_kernel<float>), dim3((unsigned)((n + NT - 1) / NT)), dim3(NT), 0, stream,
                       (const float*)z, (float*)out, n);
  } else if ((n & 7) == 0 && (((uintptr_t)z | (uintptr_t)out) & 15) == 0) {
    const int64_t n8 = n >> 3;
    hipLaunchKernelGGL(relu2_vec_kernel, dim3((unsigned)((n8 + NT - 1) / NT)), dim3(NT), 0, stream, (const uint4*)z,
                       (uint4*)out, n8);
  } else {
    hipLaunchKernelGGL((relu2_kernel<bf16_t>), dim3((unsigned)((n + NT - 1) / NT)), dim3(NT), 0, stream,
                       (const bf16_t*)z, (bf16_t*)out, n);
  }
}

void sm_bigram_embed(const int64_t* ids, const void* table, float scale, int64_t V, const void* bigram,
                     int64_t buckets, int64_t mul_prev, int64_t mul_cur, int* prev_state, const int* row_seq,
                     const int* seq_start, const int* seq_slot, const int* seq_init, int* rows, float* x, void* out,
                     int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (bigram != nullptr)
    hipLaunchKernelGGL(bigram_rows_kernel, dim3((T + NT - 1) / NT), dim3(NT), 0, stream, ids, T, buckets, mul_prev,
                       mul_cur, prev_state, row_seq, seq_start, seq_slot, seq_init, rows);
  if (f32)
    hipLaunchKernelGGL((bigram_embed_kernel<float>), dim3(T), dim3(NT), 0, stream, ids, (const float*)table, scale, V,
                       (const float*)bigram, rows, prev_state, row_seq, seq_start, seq_slot, x, (float*)out, d);
  else
    hipLaunchKernelGGL((bigram_embed_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, ids, (const bf16_t*)table, scale, V,
                       (const bf16_t*)bigram, rows, prev_state, row_seq, seq_start, seq_slot, x, (bf16_t*)out, d);
}

void sm_post_norm_add(const void* y, int64_t y_stride, const void* y2, int64_t y2_stride, float a, float b,
                      const float* bias, const void* wp, float* x, float eps, const void* wn, void* out, int T, int d,
                      int f32, hipStream_t stream) {
  if (T == 0) return;
  const int nch = (d / 8 + NT - 1) / NT;
  const bool aligned = (((uintptr_t)y | (uintptr_t)y2 | (uintptr_t)bias | (uintptr_t)wp | (uintptr_t)x | (uintptr_t)wn |
                         (uintptr_t)out) & 15) == 0 && y_stride % 8 == 0 && y2_stride % 8 == 0;
  if (!f32 && d % 8 == 0 && nch <= 4 && aligned) {
#define SM_PNA(N)                                                                                                     \
  hipLaunchKernelGGL(post_norm_add_vec_kernel<N>, dim3(T), dim3(NT), 0, stream, (const bf16_t*)y, y_stride,           \
                     (const bf16_t*)y2, y2_stride, a, b, bias, (const bf16_t*)wp, x, eps, (const bf16_t*)wn,          \
                     (bf16_t*)out, d)
    if (nch <= 1) SM_PNA(1);
    else if (nch == 2) SM_PNA(2);
    else if (nch == 3) SM_PNA(3);
    else SM_PNA(4);
#undef SM_PNA
    return;
  }
  if (f32)
    hipLaunchKernelGGL((post_norm_add_kernel<float>), dim3(T), dim3(NT), 0, stream, (const float*)y, y_stride,
                       (const float*)y2, y2_stride, a, b, bias, (const float*)wp, x, eps, (const float*)wn,
                       (float*)out, d);
  else
    hipLaunchKernelGGL((post_norm_add_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, (const bf16_t*)y, y_stride,
                       (const bf16_t*)y2, y2_stride, a, b, bias, (const bf16_t*)wp, x, eps, (const bf16_t*)wn,
                       (bf16_t*)out, d);
}

void sm_embed_scale(const int64_t* ids, const void* table, float scale, float* o0, float* o1, int T, int d,
                    int64_t V, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32) hipLaunchKernelGGL((embed_scale_kernel<float>), dim3(T), dim3(NT), 0, stream, ids, (const float*)table, scale, o0, o1, d, V);
  else hipLaunchKernelGGL((embed_scale_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, ids, (const bf16_t*)table, scale, o0, o1, d, V);
}

void sm_zc_norm(const float* x, const void* w, float eps, void* out, int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32) hipLaunchKernelGGL((zc_norm_kernel<float>), dim3(T), dim3(NT), 0, stream, x, (const float*)w, eps, (float*)out, d);
  else hipLaunchKernelGGL((zc_norm_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, x, (const bf16_t*)w, eps, (bf16_t*)out, d);
}

void sm_add_post_norm(const void* y, int64_t y_stride, const void* wp, const void* ls, float* x, float eps,
                      const void* wn, void* out, int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((add_post_norm_kernel<float>), dim3(T), dim3(NT), 0, stream, (const float*)y, y_stride,
                       (const float*)wp, (const float*)ls, x, eps, (const float*)wn, (float*)out, d);
  else
    hipLaunchKernelGGL((add_post_norm_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, (const bf16_t*)y, y_stride,
                       (const bf16_t*)wp, (const bf16_t*)ls, x, eps, (const bf16_t*)wn, (bf16_t*)out, d);
}

void sm_depth_avg_norm(float* hist, int64_t plane, int n, const float* coef, int dst, const void* w, float eps,
                       void* out, int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((depth_avg_norm_kernel<float>), dim3(T), dim3(NT), 0, stream, hist, plane, n, coef, dst,
                       (const float*)w, eps, (float*)out, d);
  else
    hipLaunchKernelGGL((depth_avg_norm_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, hist, plane, n, coef, dst,
                       (const bf16_t*)w, eps, (bf16_t*)out, d);
}

void sm_xielu(const void* z, float ap, float aq, void* out, int64_t n, int f32, hipStream_t stream) {
  if (n == 0) return;
  const dim3 grid((unsigned)((n + NT - 1) / NT));
  if (f32) hipLaunchKernelGGL((xielu_kernel<float>), grid, dim3(NT), 0, stream, (const float*)z, ap, aq, (float*)out, n);
  else hipLaunchKernelGGL((xielu_kernel<bf16_t>), grid, dim3(NT), 0, stream, (const bf16_t*)z, ap, aq, (bf16_t*)out, n);
}

void sm_softcap(float* x, float cap, int64_t n, hipStream_t stream) {
  if (n == 0) return;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + NT - 1) / NT)), dim3(NT), 0, stream, x, cap, n);
}

}  // extern "C"
