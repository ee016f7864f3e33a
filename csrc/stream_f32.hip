// A residual stream kept in f32 next to bf16 (or f32) sublayer outputs:
//   * token + learned position embedding gather into the f32 stream (and a second copy for models
//     that add the embedding output again later);
//   * fused "stream update + RMSNorm": x += m * (a + b) + e, h = x / sqrt(mean(x^2) + eps) * (off + w)
//     -- the update of a block whose sublayers all read one norm's output and are summed, and the
//     next block's norm, in one pass over the row (a, b, e optional; off = 1 for weights stored
//     around zero); with a row index list it gathers rows instead and leaves the stream alone (the
//     rows that feed the LM head);
//   * soft-capped logits: cap * tanh(z / cap), f32 out.
#include "common.h"
#include "kernels.h"

namespace {

template <typename T>
LK_DEVICE float ldv(const T* p);
template <>
LK_DEVICE float ldv<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <>
LK_DEVICE float ldv<float>(const float* p) { return *p; }
template <typename T>
LK_DEVICE void stv(T* p, float v);
template <>
LK_DEVICE void stv<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }
template <>
LK_DEVICE void stv<float>(float* p, float v) { *p = v; }

__device__ int g_stream_embed_errors = 0;

template <typename T>
__global__ __launch_bounds__(256) void embed_pos_kernel(const int* __restrict__ ids, const int* __restrict__ positions,
                                                        const T* __restrict__ tok, int vocab,
                                                        const T* __restrict__ pos, int max_pos, int W,
                                                        float* __restrict__ x, float* __restrict__ copy) {
  const long row = blockIdx.x;
  const int id = ids[row], ps = positions[row];
  const bool ok = id >= 0 && id < vocab && ps >= 0 && ps < max_pos;
  if (!ok && threadIdx.x == 0) atomicAdd(&g_stream_embed_errors, 1);
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = ok ? ldv<T>(tok + (long)id * W + c) + ldv<T>(pos + (long)ps * W + c) : 0.f;
    x[row * W + c] = v;
    if (copy) copy[row * W + c] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void stream_rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ a, long as,
                                                             const float* __restrict__ ab, const T* __restrict__ b, long bs,
                                                             const float* __restrict__ e, float m,
                                                             const float* __restrict__ w, float woff, float eps,
                                                             const long* __restrict__ idx, T* __restrict__ out, long os,
                                                             int W) {
  __shared__ float red[4];
  const long orow = blockIdx.x, row = idx ? idx[orow] : orow;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = x[row * W + c];
    float d = 0.f;
    if (a) d += ldv<T>(a + row * as + c) + (ab ? ab[c] : 0.f);
    if (b) d += ldv<T>(b + row * bs + c);
    v += m * d;
    if (e) v += e[row * W + c];
    if (!idx && (a || b || e)) x[row * W + c] = v;
    ss += v * v;
  }
  ss = block_sum<4>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) {
    float v;
    if (!idx) {
      v = x[row * W + c];  // this thread's own store above (or the untouched stream)
    } else {
      v = x[row * W + c];
      float d = 0.f;
      if (a) d += ldv<T>(a + row * as + c) + (ab ? ab[c] : 0.f);
      if (b) d += ldv<T>(b + row * bs + c);
      v += m * d;
      if (e) v += e[row * W + c];
    }
    stv<T>(out + orow * os + c, v * inv * (w ? woff + w[c] : 1.f));
  }
}

// The same with the row kept in registers and 16-byte (f32) / 8-byte (bf16) accesses: W % 4 == 0,
// W <= 4 * 256 * MAXV, 16-byte aligned rows.  One read of every input, one write of x and of out.
template <typename T, int MAXV>
__global__ __launch_bounds__(256) void stream_rmsnorm_vec_kernel(float* __restrict__ x, const T* __restrict__ a, long as,
                                                                 const float* __restrict__ ab, const T* __restrict__ b,
                                                                 long bs,
                                                                 const float* __restrict__ e, float m,
                                                                 const float* __restrict__ w, float woff, float eps,
                                                                 const long* __restrict__ idx, T* __restrict__ out,
                                                                 long os, int W) {
  __shared__ float red[4];
  const long orow = blockIdx.x, row = idx ? idx[orow] : orow;
  const int nv = W >> 2;
  floatx4 v[MAXV];
  float ss = 0.f;
  auto ld4 = [](const T* p) -> floatx4 {
    if constexpr (sizeof(T) == 2) {
      const short4_t r = *reinterpret_cast<const short4_t*>(p);
      return floatx4{bf2f((bf16_t)r[0]), bf2f((bf16_t)r[1]), bf2f((bf16_t)r[2]), bf2f((bf16_t)r[3])};
    } else {
      return *reinterpret_cast<const floatx4*>(p);
    }
  };
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      floatx4 t = *reinterpret_cast<const floatx4*>(x + row * W + 4 * c);
      floatx4 d = {0.f, 0.f, 0.f, 0.f};
      if (a) d += ld4(a + row * as + 4 * c);
      if (a && ab) d += *reinterpret_cast<const floatx4*>(ab + 4 * c);
      if (b) d += ld4(b + row * bs + 4 * c);
      t += m * d;
      if (e) t += *reinterpret_cast<const floatx4*>(e + row * W + 4 * c);
      if (!idx && (a || b || e)) *reinterpret_cast<floatx4*>(x + row * W + 4 * c) = t;
      v[i] = t;
      ss += t[0] * t[0] + t[1] * t[1] + t[2] * t[2] + t[3] * t[3];
    }
  }
  ss = block_sum<4>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      floatx4 g = {1.f, 1.f, 1.f, 1.f};
      if (w) g = *reinterpret_cast<const floatx4*>(w + 4 * c) + woff;
      const floatx4 r = v[i] * inv * g;
      T* o = out + orow * os + 4 * c;
      if constexpr (sizeof(T) == 2) {
        short4_t q = {(short)f2bf(r[0]), (short)f2bf(r[1]), (short)f2bf(r[2]), (short)f2bf(r[3])};
        *reinterpret_cast<short4_t*>(o) = q;
      } else {
        *reinterpret_cast<floatx4*>(o) = r;
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softcap_kernel(const T* __restrict__ in, long is, float cap, float* __restrict__ out,
                                                      long os, int V) {
  const long row = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < V; c += 256 * gridDim.y) {
    const float z = ldv<T>(in + row * is + c);
    out[row * os + c] = cap > 0.f ? cap * tanhf(z / cap) : z;
  }
}

// out[r][c] = silu(x[r][c]) * x[r][I + c] for f32 rows [gate | up] (the bf16 case is the GEMM's epilogue)
__global__ __launch_bounds__(256) void silu_mul_f32_kernel(const float* __restrict__ x, long xs, float* __restrict__ out,
                                                           long os, int I) {
  const long row = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < I; c += 256 * gridDim.y) {
    const float g = x[row * xs + c];
    out[row * os + c] = g / (1.f + expf(-g)) * x[row * xs + I + c];
  }
}

}  // namespace

int lk_silu_mul_f32(const float* x, long xs, float* out, long os, long rows, int I, hipStream_t st) {
  if (rows <= 0) return 0;
  silu_mul_f32_kernel<<<dim3((unsigned)rows, (unsigned)((I + 2047) / 2048)), 256, 0, st>>>(x, xs, out, os, I);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_stream_embed_errors() {
  int v = 0;
  if (hipMemcpyFromSymbol(&v, HIP_SYMBOL(g_stream_embed_errors), sizeof(int)) != hipSuccess) return -1;
  return v;
}

int lk_embed_pos(const int* ids, const int* positions, const void* tok, int vocab, const void* pos, int max_pos, long rows,
                 int W, float* x, float* copy, int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  if (esz == 2)
    embed_pos_kernel<bf16_t><<<(unsigned)rows, 256, 0, st>>>(ids, positions, (const bf16_t*)tok, vocab, (const bf16_t*)pos,
                                                             max_pos, W, x, copy);
  else
    embed_pos_kernel<float><<<(unsigned)rows, 256, 0, st>>>(ids, positions, (const float*)tok, vocab, (const float*)pos,
                                                            max_pos, W, x, copy);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_stream_rmsnorm(float* x, const void* a, long as, const float* a_bias, const void* b, long bs, const float* e, float m, const float* w,
                      float woff, float eps, const long* idx, long out_rows, void* out, long os, int W, int esz,
                      hipStream_t st) {
  if (out_rows <= 0) return 0;
  const auto al = [](const void* p, long stride_bytes, int vec_bytes) {
    return p == nullptr || (reinterpret_cast<uintptr_t>(p) % vec_bytes == 0 && stride_bytes % vec_bytes == 0);
  };
  constexpr int kMaxV = 8;
  const int tv = esz == 2 ? 8 : 16;  // bytes of a 4-element access to the activations
  if (W % 4 == 0 && W <= 4 * 256 * kMaxV && al(x, (long)W * 4, 16) && al(e, (long)W * 4, 16) && al(w, 0, 16) && al(a_bias, 0, 16) &&
      al(a, as * (long)esz, tv) && al(b, bs * (long)esz, tv) && al(out, os * (long)esz, tv)) {
    if (esz == 2)
      stream_rmsnorm_vec_kernel<bf16_t, kMaxV><<<(unsigned)out_rows, 256, 0, st>>>(
          x, (const bf16_t*)a, as, a_bias, (const bf16_t*)b, bs, e, m, w, woff, eps, idx, (bf16_t*)out, os, W);
    else
      stream_rmsnorm_vec_kernel<float, kMaxV><<<(unsigned)out_rows, 256, 0, st>>>(
          x, (const float*)a, as, a_bias, (const float*)b, bs, e, m, w, woff, eps, idx, (float*)out, os, W);
    LK_CHECK_LAUNCH();
    return 0;
  }
  if (esz == 2)
    stream_rmsnorm_kernel<bf16_t><<<(unsigned)out_rows, 256, 0, st>>>(x, (const bf16_t*)a, as, a_bias, (const bf16_t*)b, bs, e, m, w,
                                                                      woff, eps, idx, (bf16_t*)out, os, W);
  else
    stream_rmsnorm_kernel<float><<<(unsigned)out_rows, 256, 0, st>>>(x, (const float*)a, as, a_bias, (const float*)b, bs, e, m, w,
                                                                     woff, eps, idx, (float*)out, os, W);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_softcap(const void* in, long is, float cap, float* out, long os, long rows, int V, int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  dim3 grid((unsigned)rows, (unsigned)((V + 2047) / 2048));
  if (esz == 2) softcap_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)in, is, cap, out, os, V);
  else softcap_kernel<float><<<grid, 256, 0, st>>>((const float*)in, is, cap, out, os, V);
  LK_CHECK_LAUNCH();
  return 0;
}
