// Sigmoid attention with a logarithmic distance penalty over a paged K/V cache.
//
//   weight(i, j) = sigmoid(scale * <q_i, k_j> - r1_h * ln(1 + r2_h * (i - j)) + pb_h),  j <= i
//   out_i        = sum_j weight(i, j) * v_j            (no normalisation over the keys)
//
// q and k are unit-RMS per head (lk_unitnorm_kv_write does that in f32 and files k / v into the
// cache), the score, the penalty and the weight are f32.  Nothing couples the keys of a row (no
// running maximum, no denominator), so a key range can be cut anywhere and the pieces summed:
// the decode kernel splits a context over waves and workgroups and adds the parts in a fixed
// order.
//
// Layouts: K cache [blocks, G, BS, dim]; V cache TRANSPOSED per block [blocks, G, vdim, BS], so
// that both MFMA operands are contiguous along their contraction index (dim for q.k, keys for
// p.v) and every fragment is one 16-byte (K) or 8/16-byte (V) load straight from the cache: no
// LDS staging, no barriers.  Waves of a workgroup that share a kv head hit the same lines in L1.
//
// One wave = 16 "columns" (queries) against a run of 16-key tiles:
//   S^T (16 keys x 16 columns) = K . Q^T     A = K rows, B = the columns' q kept in registers
//   O^T (vdim x 16 columns)   += V^T . P^T   A = V^T rows, B = P^T taken from the S^T accumulators
// bf16: v_mfma_f32_16x16x32_bf16; f32: v_mfma_f32_16x16x4_f32 (true 32-bit products), same
// accumulator layout (lane = column l % 16, rows 4 * (l / 16) + j).  The order in which the
// contraction index is walked is permuted identically on both operands where that saves shuffles.
// Prefill: the columns are 16 consecutive queries of one head; decode: the columns are the query
// heads of one kv group (all at the last position).
#include "common.h"
#include "kernels.h"
#include "attn_frag.h"

namespace {

struct SigParams {
  const void* q;   // rows of [H * dim] (+ anything behind them), unit-RMS per head
  long qs;         // row stride in elements
  const void* kc;  // [NB, G, BS, dim]
  const void* vc;  // [NB, G, vdim, BS]
  const int* bt;   // [B, bt_stride] cache blocks of each sequence
  int bt_stride;
  int H, G, dim, vdim, BS;
  float scale;
  const float* r1;  // [H]
  const float* r2;  // [H]
  const float* pb;  // [H]
};

template <bool EXACT>
LK_DEVICE float sig_weight(float s, float r1, float r2, float pb, int d) {
  if constexpr (EXACT) {
    const float x = s - r1 * logf(1.f + r2 * (float)d) + pb;
    return 1.f / (1.f + expf(-x));
  } else {
    const float x = s - r1 * __logf(1.f + r2 * (float)d) + pb;
    return __builtin_amdgcn_rcpf(1.f + __expf(-x));
  }
}

// The columns of this wave against the 32-key steps step0, step0 + stride, ... of keys [k0, k1):
// k0 is a multiple of 32; k1 <= the sequence's context.  Column n = lane % 16 sits at position
// qpos and sees keys <= qpos.
//
// Key order inside a step: row m of S^T tile t is key 8 (m / 4) + 4 t + m % 4, so after both tiles
// lane group g holds the weights of the 8 CONSECUTIVE keys 8g .. 8g + 7 -- one 16-byte piece of a
// V^T row (bf16), and exactly the k-slots 8g .. 8g + 7 of the P.V MFMA's B operand.  Keys at or
// past k1 are read from the last valid key / key run (always allocated, finite) and weigh zero.
// bf16: the next step's K fragments are requested as soon as this step's Q.K MFMAs have
// consumed the current ones, and this step's V fragments before the weights are computed, so
// both fly under the transcendental-heavy weight arithmetic.
template <typename T, int PAD>
LK_DEVICE void sig_run(const SigParams& p, const uint4_t (&qf)[PAD / (4 * El<T>::V)], int kvh, const int* bt, int k0,
                       int k1, int step0, int stride, bool cvalid, int qpos, float r1, float r2, float pb,
                       floatx4 (&o)[PAD / 16]) {
  constexpr int EV = El<T>::V, KS = PAD / (4 * EV), VT = PAD / 16;
  constexpr bool PIPE = sizeof(T) == 2;
  const int lane = threadIdx.x & 63, n16 = lane & 15, g = lane >> 4;
  const T* kc = reinterpret_cast<const T*>(p.kc);
  const T* vc = reinterpret_cast<const T*>(p.vc);
  const int krow = 8 * (n16 >> 2) + (n16 & 3);  // this lane's K row inside a step (+ 4 t)
  auto load_k = [&](int kb, uint4_t (&kf)[2][KS]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = min(kb + krow + 4 * t, k1 - 1);
      const T* kr = kc + (((long)bt[key / p.BS] * p.G + kvh) * p.BS + key % p.BS) * p.dim;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = s * 4 * EV + g * EV;
        kf[t][s] = d0 < p.dim ? ld16(kr + d0) : uint4_t{0u, 0u, 0u, 0u};
      }
    }
  };
  uint4_t kf[2][KS];
  int kb = k0 + 32 * step0;
  if (PIPE && kb < k1) load_k(kb, kf);
  for (; kb < k1; kb += 32 * stride) {
    if (!PIPE) load_k(kb, kf);
    floatx4 c[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      c[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; ++s)
        if (s * 4 * EV < p.dim) c[t] = mma_qk<T>(kf[t][s], qf[s], c[t]);
    }
    // this lane group's run of 8 keys of V^T (a masked run re-reads the last valid one)
    const int vk = kb + 8 * g < k1 ? kb + 8 * g : ((k1 - 1) & ~7);
    const T* vrow = vc + ((long)bt[vk / p.BS] * p.G + kvh) * p.vdim * p.BS + vk % p.BS;
    uint4_t vf[PIPE ? VT : 1];
    if constexpr (PIPE) {
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        const int vd = vt * 16 + n16;
        vf[vt] = (vt * 16 < p.vdim && vd < p.vdim) ? ld16(vrow + (long)vd * p.BS) : uint4_t{0u, 0u, 0u, 0u};
      }
      const int kn = kb + 32 * stride;
      if (kn < k1) load_k(kn, kf);
    }
    float pw[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = kb + 8 * g + 4 * t + j, d = qpos - key;
        pw[t][j] = (cvalid && d >= 0 && key < k1) ? sig_weight<sizeof(T) == 4>(c[t][j] * p.scale, r1, r2, pb, d) : 0.f;
      }
    if constexpr (PIPE) {
      short8 pbits;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pbits[j] = (short)f2bf(pw[0][j]);
        pbits[4 + j] = (short)f2bf(pw[1][j]);
      }
#pragma unroll
      for (int vt = 0; vt < VT; ++vt)
        if (vt * 16 < p.vdim)
          o[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(short8, vf[vt]), pbits, o[vt], 0, 0, 0);
    } else {
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        if (vt * 16 < p.vdim) {
          const int vd = vt * 16 + n16;
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            floatx4 a = {0.f, 0.f, 0.f, 0.f};
            if (vd < p.vdim) a = *reinterpret_cast<const floatx4*>(vrow + (long)vd * p.BS + 4 * t);
#pragma unroll
            for (int j = 0; j < 4; ++j) o[vt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], pw[t][j], o[vt], 0, 0, 0);
          }
        }
      }
    }
  }
}

template <typename T, int PAD>
LK_DEVICE void load_q(const SigParams& p, const T* qrow, bool cvalid, uint4_t (&qf)[PAD / (4 * El<T>::V)]) {
  constexpr int EV = El<T>::V, KS = PAD / (4 * EV);
  const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int d0 = s * 4 * EV + g * EV;
    qf[s] = (cvalid && d0 < p.dim) ? ld16(qrow + d0) : uint4_t{0u, 0u, 0u, 0u};
  }
}

// Sum of the 4 waves' O^T accumulators in wave order through LDS; afterwards wave 0 holds the total.
template <int VT>
LK_DEVICE void sum_waves(floatx4 (&o)[VT], float (&red)[3][VT][64][4]) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (w > 0) {
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) red[w - 1][vt][lane][j] = o[vt][j];
  }
  __syncthreads();
  if (w == 0) {
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) o[vt][j] = ((o[vt][j] + red[0][vt][lane][j]) + red[1][vt][lane][j]) + red[2][vt][lane][j];
  }
}

// ---- prefill: workgroup = one 16-query tile of one head; its 4 waves take every fourth 32-key
// step of the tile's causal key range and are summed through LDS.  (Four heads per workgroup, one
// wave each, left a long row's 30-odd dependent steps on one wave: the kernel was bound by that
// chain, not by arithmetic.)  blockIdx.x = head, so the heads of a kv group that read the same K / V
// run side by side; blockIdx.y walks the host's tile list, heaviest tiles first.
template <typename T, int PAD>
__global__ __launch_bounds__(256) void sigattn_prefill_kernel(SigParams p, const int* __restrict__ cu_q,
                                                              const int* __restrict__ ctx_lens,
                                                              const int* __restrict__ tile_seq,
                                                              const int* __restrict__ tile_q0, T* __restrict__ out,
                                                              long os) {
  constexpr int VT = PAD / 16;
  __shared__ float red[3][VT][64][4];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, n16 = lane & 15, g = lane >> 4;
  const int head = blockIdx.x;
  const int b = tile_seq[blockIdx.y], q0 = tile_q0[blockIdx.y];
  const int qbeg = cu_q[b], qlen = cu_q[b + 1] - qbeg, ctx = ctx_lens[b], past = ctx - qlen;
  const int qi = q0 + n16;
  const bool cvalid = qi < qlen;
  const int qpos = past + qi;
  const T* qrow = reinterpret_cast<const T*>(p.q) + (long)(qbeg + min(qi, qlen - 1)) * p.qs + (long)head * p.dim;
  uint4_t qf[PAD / (4 * El<T>::V)];
  load_q<T, PAD>(p, qrow, cvalid, qf);
  floatx4 o[VT];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) o[vt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int k1 = min(ctx, past + q0 + 16);
  sig_run<T, PAD>(p, qf, head / (p.H / p.G), p.bt + (long)b * p.bt_stride, 0, k1, w, 4, cvalid, qpos, p.r1[head],
                  p.r2[head], p.pb[head], o);
  sum_waves<VT>(o, red);
  if (w == 0 && cvalid) {
    T* orow = out + (long)(qbeg + qi) * os + (long)head * p.vdim;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int vd = vt * 16 + 4 * g + j;
        if (vd < p.vdim) El<T>::st(orow + vd, o[vt][j]);
      }
  }
}

// ---- decode: workgroup = (sequence, up to 16 heads of one kv group, key split z); its 4 waves
// take every fourth 32-key step of the split and are summed through LDS in wave order ------------
template <typename T, int PAD>
__global__ __launch_bounds__(256) void sigattn_decode_kernel(SigParams p, const int* __restrict__ ctx_lens, int Z,
                                                             T* __restrict__ out, long os,
                                                             float* __restrict__ part) {
  constexpr int VT = PAD / 16;
  __shared__ float red[3][VT][64][4];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, n16 = lane & 15, g = lane >> 4;
  const int rep = p.H / p.G, ngr = (rep + 15) / 16;
  const int b = blockIdx.x, kvh = blockIdx.y / ngr, sub = blockIdx.y % ngr, z = blockIdx.z;
  const int ctx = ctx_lens[b];
  const int hn = sub * 16 + n16;
  const bool cvalid = hn < rep;
  const int head = kvh * rep + min(hn, rep - 1);
  const T* qrow = reinterpret_cast<const T*>(p.q) + (long)b * p.qs + (long)head * p.dim;
  uint4_t qf[PAD / (4 * El<T>::V)];
  load_q<T, PAD>(p, qrow, cvalid, qf);
  floatx4 o[VT];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) o[vt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int nsteps = (ctx + 31) / 32, spz = (nsteps + Z - 1) / Z;
  const int s0 = z * spz, s1 = min(nsteps, s0 + spz);
  if (s0 < s1)
    sig_run<T, PAD>(p, qf, kvh, p.bt + (long)b * p.bt_stride, 32 * s0, min(ctx, 32 * s1), w, 4, cvalid, ctx - 1,
                    p.r1[head], p.r2[head], p.pb[head], o);
  sum_waves<VT>(o, red);
  if (w == 0 && cvalid) {
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int vd = vt * 16 + 4 * g + j;
        if (vd < p.vdim) {
          if (Z == 1) El<T>::st(out + (long)b * os + (long)head * p.vdim + vd, o[vt][j]);
          else part[(((long)b * p.H + head) * Z + z) * p.vdim + vd] = o[vt][j];
        }
      }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void sigattn_reduce_kernel(const float* __restrict__ part, int Z, int H, int vdim,
                                                             T* __restrict__ out, long os) {
  const int b = blockIdx.x, head = blockIdx.y;
  const float* pp = part + ((long)b * H + head) * Z * vdim;
  for (int vd = threadIdx.x; vd < vdim; vd += 256) {
    float s = 0.f;
    for (int z = 0; z < Z; ++z) s += pp[(long)z * vdim + vd];
    El<T>::st(out + (long)b * os + (long)head * vdim + vd, s);
  }
}

// ---- unit-RMS q / k per head, k and v into the paged cache --------------------------------------
// One workgroup per token; its 4 waves take the H + 2G (head, kind) jobs in turn.  The mean of the
// squares is over the head's first norm_dim elements' worth (norm_dim <= dim: heads padded with
// zero columns up to the kernels' vector width keep their true size as the divisor).
template <typename T>
__global__ __launch_bounds__(256) void unitnorm_kv_write_kernel(T* __restrict__ qkv, long qs, int H, int G, int dim,
                                                                int vdim, int norm_dim, float eps, T* __restrict__ kc,
                                                                T* __restrict__ vc, const int* __restrict__ slots,
                                                                int BS, const T* __restrict__ bias) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int slot = slots[t];
  T* row = qkv + t * qs;
  const long blk = slot >= 0 ? slot / BS : 0;
  const int off = slot >= 0 ? slot % BS : 0;
  for (int job = w; job < H + 2 * G; job += 4) {
    if (job < H + G) {  // a q or k head: x / sqrt(mean(x^2) + eps)
      T* x = row + (long)job * dim;
      const T* bb = bias ? bias + (long)job * dim : nullptr;  // the projection's bias, added here in f32
      float ss = 0.f;
      for (int c = lane; c < dim; c += 64) {
        const float v = El<T>::ld(x + c) + (bb ? El<T>::ld(bb + c) : 0.f);
        ss += v * v;
      }
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)norm_dim + eps);
      if (job < H) {
        for (int c = lane; c < dim; c += 64) El<T>::st(x + c, (El<T>::ld(x + c) + (bb ? El<T>::ld(bb + c) : 0.f)) * inv);
      } else if (slot >= 0) {
        T* dst = kc + ((blk * G + (job - H)) * BS + off) * dim;
        for (int c = lane; c < dim; c += 64) El<T>::st(dst + c, (El<T>::ld(x + c) + (bb ? El<T>::ld(bb + c) : 0.f)) * inv);
      }
    } else if (slot >= 0) {  // a v head, filed key-contiguous
      const int gh = job - H - G;
      const T* x = row + (long)(H + G) * dim + (long)gh * vdim;
      const T* bb = bias ? bias + (long)(H + G) * dim + (long)gh * vdim : nullptr;
      T* dst = vc + (blk * G + gh) * (long)vdim * BS + off;
      for (int c = lane; c < vdim; c += 64) El<T>::st(dst + (long)c * BS, El<T>::ld(x + c) + (bb ? El<T>::ld(bb + c) : 0.f));
    }
  }
}

int pad_of(int dim, int vdim) {
  const int m = dim > vdim ? dim : vdim;
  return m <= 64 ? 64 : m <= 96 ? 96 : m <= 128 ? 128 : m <= 192 ? 192 : m <= 256 ? 256 : 0;
}

bool shape_ok(int H, int G, int dim, int vdim, int BS, int esz) {
  const int ev = 16 / esz;
  return H > 0 && G > 0 && H % G == 0 && dim > 0 && vdim > 0 && dim % ev == 0 && vdim % ev == 0 && BS % 16 == 0 &&
         pad_of(dim, vdim) != 0;
}

template <typename T, int PAD>
int launch_prefill(const SigParams& p, const int* cu_q, const int* ctx, const int* ts, const int* tq, int ntiles,
                   void* out, long os, hipStream_t st) {
  if (ntiles > 65535) return -2;
  dim3 grid(p.H, ntiles);
  sigattn_prefill_kernel<T, PAD><<<grid, 256, 0, st>>>(p, cu_q, ctx, ts, tq, reinterpret_cast<T*>(out), os);
  LK_CHECK_LAUNCH();
  return 0;
}

template <typename T, int PAD>
int launch_decode(const SigParams& p, const int* ctx, int B, int Z, void* out, long os, float* part, hipStream_t st) {
  const int rep = p.H / p.G;
  dim3 grid(B, p.G * ((rep + 15) / 16), Z);
  sigattn_decode_kernel<T, PAD><<<grid, 256, 0, st>>>(p, ctx, Z, reinterpret_cast<T*>(out), os, part);
  LK_CHECK_LAUNCH();
  if (Z > 1) {
    sigattn_reduce_kernel<T><<<dim3(B, p.H), 256, 0, st>>>(part, Z, p.H, p.vdim, reinterpret_cast<T*>(out), os);
    LK_CHECK_LAUNCH();
  }
  return 0;
}

#define LK_SIG_DISPATCH(FN, ...)                       \
  switch (pad) {                                       \
    case 64: return FN<T, 64>(__VA_ARGS__);            \
    case 96: return FN<T, 96>(__VA_ARGS__);            \
    case 128: return FN<T, 128>(__VA_ARGS__);          \
    case 192: return FN<T, 192>(__VA_ARGS__);          \
    case 256: return FN<T, 256>(__VA_ARGS__);          \
    default: return -1;                                \
  }

template <typename T>
int prefill_t(const SigParams& p, const int* cu_q, const int* ctx, const int* ts, const int* tq, int ntiles, void* out,
              long os, hipStream_t st) {
  const int pad = pad_of(p.dim, p.vdim);
  LK_SIG_DISPATCH(launch_prefill, p, cu_q, ctx, ts, tq, ntiles, out, os, st)
}

template <typename T>
int decode_t(const SigParams& p, const int* ctx, int B, int Z, void* out, long os, float* part, hipStream_t st) {
  const int pad = pad_of(p.dim, p.vdim);
  LK_SIG_DISPATCH(launch_decode, p, ctx, B, Z, out, os, part, st)
}

SigParams make_params(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride, int H, int G,
                      int dim, int vdim, int BS, float scale, const float* r1, const float* r2, const float* pb) {
  SigParams p;
  p.q = q; p.qs = qs; p.kc = kc; p.vc = vc; p.bt = bt; p.bt_stride = bt_stride;
  p.H = H; p.G = G; p.dim = dim; p.vdim = vdim; p.BS = BS; p.scale = scale; p.r1 = r1; p.r2 = r2; p.pb = pb;
  return p;
}

}  // namespace

int lk_sigattn_supported(int H, int G, int dim, int vdim, int BS, int esz) { return shape_ok(H, G, dim, vdim, BS, esz); }

int lk_unitnorm_kv_write(void* qkv, long qs, long T, int H, int G, int dim, int vdim, int norm_dim, float eps, void* kc, void* vc,
                         const int* slots, int BS, const void* bias, int esz, hipStream_t st) {
  if (T <= 0) return 0;
  if (!shape_ok(H, G, dim, vdim, BS, esz) || norm_dim < 1 || norm_dim > dim) return -1;
  if (esz == 2)
    unitnorm_kv_write_kernel<bf16_t><<<(unsigned)T, 256, 0, st>>>((bf16_t*)qkv, qs, H, G, dim, vdim, norm_dim, eps, (bf16_t*)kc,
                                                                  (bf16_t*)vc, slots, BS, (const bf16_t*)bias);
  else
    unitnorm_kv_write_kernel<float><<<(unsigned)T, 256, 0, st>>>((float*)qkv, qs, H, G, dim, vdim, norm_dim, eps, (float*)kc,
                                                                 (float*)vc, slots, BS, (const float*)bias);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_sigattn_prefill(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride,
                       const int* cu_q, const int* ctx_lens, const int* tile_seq, const int* tile_q0, int ntiles, int H,
                       int G, int dim, int vdim, int BS, float scale, const float* r1, const float* r2, const float* pb,
                       void* out, long os, int esz, hipStream_t st) {
  if (ntiles <= 0) return 0;
  if (!shape_ok(H, G, dim, vdim, BS, esz)) return -1;
  const SigParams p = make_params(q, qs, kc, vc, bt, bt_stride, H, G, dim, vdim, BS, scale, r1, r2, pb);
  return esz == 2 ? prefill_t<bf16_t>(p, cu_q, ctx_lens, tile_seq, tile_q0, ntiles, out, os, st)
                  : prefill_t<float>(p, cu_q, ctx_lens, tile_seq, tile_q0, ntiles, out, os, st);
}

int lk_sigattn_decode(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride,
                      const int* ctx_lens, int B, int Z, int H, int G, int dim, int vdim, int BS, float scale,
                      const float* r1, const float* r2, const float* pb, void* out, long os, float* part, int esz,
                      hipStream_t st) {
  if (B <= 0) return 0;
  if (!shape_ok(H, G, dim, vdim, BS, esz) || Z < 1 || (Z > 1 && part == nullptr)) return -1;
  const SigParams p = make_params(q, qs, kc, vc, bt, bt_stride, H, G, dim, vdim, BS, scale, r1, r2, pb);
  return esz == 2 ? decode_t<bf16_t>(p, ctx_lens, B, Z, out, os, part, st)
                  : decode_t<float>(p, ctx_lens, B, Z, out, os, part, st);
}
