// Kernels of the transformer blocks that surround the MoE layer
// (vmoe/nn/vit_moe.py:151-184): the residual add fused with the layer norm that
// follows it, and softmax attention over one image's tokens.
#include <hip/hip_runtime.h>

#include "vmoe_common.h"
#include "vmoe_hip.h"

namespace vmoe {
namespace {

constexpr int kLnThreads = 256;
constexpr int kLnWaves = kLnThreads / 64;

template <typename T> struct Vec4;
template <> struct Vec4<float> {
  __device__ static __forceinline__ float4 load(const float* p) {
    return *reinterpret_cast<const float4*>(p);
  }
  __device__ static __forceinline__ float4 load_stream(const float* p) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    const f32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
    return make_float4(t.x, t.y, t.z, t.w);
  }
  __device__ static __forceinline__ void store(float* p, float4 v) {
    *reinterpret_cast<float4*>(p) = v;
  }
  // For data that is not read again soon (the residual stream between two blocks'
  // norms: another few hundred MB pass through the caches first).
  __device__ static __forceinline__ void store_stream(float* p, float4 v) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    f32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<f32x4_t*>(p));
  }
};
template <> struct Vec4<bf16_t> {
  __device__ static __forceinline__ float4 load(const bf16_t* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(bf_lo(u.x), bf_hi(u.x), bf_lo(u.y), bf_hi(u.y));
  }
  __device__ static __forceinline__ float4 load_stream(const bf16_t* p) {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    const u32x2_t u = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
    return make_float4(bf_lo(u.x), bf_hi(u.x), bf_lo(u.y), bf_hi(u.y));
  }
  __device__ static __forceinline__ void store(bf16_t* p, float4 v) {
    uint2 u;
    u.x = pack_bf16x2(v.x, v.y);
    u.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// One wave per row, the row held in registers (NV float4 per lane, D <= 256 * NV):
//   x = residual (+ branch);  residual_out = x;
//   norm_out = (x - mean) * rsqrt(var + eps) * scale + bias,  var = E[x^2] - E[x]^2
// which is flax.linen.LayerNorm's arithmetic (float32 statistics, "fast variance").
// Every element is read once and written once: HBM-bound.
template <typename TB, typename TO, int NV>
__global__ __launch_bounds__(kLnThreads) void add_layer_norm_kernel(
    const float* residual, const TB* __restrict__ branch,
    const float* __restrict__ scale, const float* __restrict__ bias,
    float* residual_out, TO* __restrict__ norm_out, long rows, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const int chunks = D >> 2;
  float4 sc[NV], bi[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + 64 * i;
    sc[i] = make_float4(1.f, 1.f, 1.f, 1.f);
    bi[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < chunks) {
      if (scale != nullptr) sc[i] = Vec4<float>::load(scale + 4 * c);
      if (bias != nullptr) bi[i] = Vec4<float>::load(bias + 4 * c);
    }
  }
  const float inv_d = 1.0f / (float)D;
  const long stride = (long)gridDim.x * kLnWaves;
  for (long row = (long)blockIdx.x * kLnWaves + (threadIdx.x >> 6); row < rows; row += stride) {
    const size_t base = (size_t)row * D;
    float4 v[NV];
    float s = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + 64 * i;
      v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (c < chunks) {
        v[i] = Vec4<float>::load_stream(residual + base + 4 * c);
        if (branch != nullptr) {
          const float4 b = Vec4<TB>::load_stream(branch + base + 4 * c);
          v[i].x += b.x; v[i].y += b.y; v[i].z += b.z; v[i].w += b.w;
        }
        if (residual_out != nullptr) Vec4<float>::store_stream(residual_out + base + 4 * c, v[i]);
      }
      s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
      s2 += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
    }
    if (norm_out == nullptr) continue;
    const float mean = wave_sum(s) * inv_d;
    const float var = fmaxf(wave_sum(s2) * inv_d - mean * mean, 0.f);
    const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + 64 * i;
      if (c < chunks) {
        float4 y;
        y.x = (v[i].x - mean) * (rstd * sc[i].x) + bi[i].x;
        y.y = (v[i].y - mean) * (rstd * sc[i].y) + bi[i].y;
        y.z = (v[i].z - mean) * (rstd * sc[i].z) + bi[i].z;
        y.w = (v[i].w - mean) * (rstd * sc[i].w) + bi[i].w;
        Vec4<TO>::store(norm_out + base + 4 * c, y);
      }
    }
  }
}

// Any width: one wave per row, the row read again for each pass (it stays in L2).
template <typename TB, typename TO>
__global__ __launch_bounds__(kLnThreads) void add_layer_norm_generic_kernel(
    const float* residual, const TB* __restrict__ branch,
    const float* __restrict__ scale, const float* __restrict__ bias,
    float* residual_out, TO* __restrict__ norm_out, long rows, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const float inv_d = 1.0f / (float)D;
  const long stride = (long)gridDim.x * kLnWaves;
  for (long row = (long)blockIdx.x * kLnWaves + (threadIdx.x >> 6); row < rows; row += stride) {
    const size_t base = (size_t)row * D;
    float s = 0.f, s2 = 0.f;
    for (int j = lane; j < D; j += 64) {
      float x = residual[base + j];
      if (branch != nullptr) x += Elt<TB>::load(branch + base + j);
      s += x;
      s2 += x * x;
    }
    const float mean = wave_sum(s) * inv_d;
    const float var = fmaxf(wave_sum(s2) * inv_d - mean * mean, 0.f);
    const float rstd = 1.0f / sqrtf(var + eps);
    for (int j = lane; j < D; j += 64) {
      float x = residual[base + j];
      if (branch != nullptr) x += Elt<TB>::load(branch + base + j);
      if (norm_out != nullptr) {
        const float g = scale != nullptr ? scale[j] : 1.f;
        const float b = bias != nullptr ? bias[j] : 0.f;
        Elt<TO>::store(norm_out + base + j, (x - mean) * (rstd * g) + b);
      }
      // Written last: residual_out may be the residual itself.
      if (residual_out != nullptr) residual_out[base + j] = x;
    }
  }
}

template <typename TB, typename TO>
int launch_add_layer_norm(const VmoeAddLayerNormParams* p, hipStream_t stream) {
  const long rows = (long)p->rows;
  const int D = p->D;
  long blocks = (rows + kLnWaves - 1) / kLnWaves;
  if (blocks > 256 * 16) blocks = 256 * 16;
  const dim3 grid((unsigned)blocks), block(kLnThreads);
  const float* res = p->residual;
  const TB* br = static_cast<const TB*>(p->branch);
  TO* out = static_cast<TO*>(p->norm_out);
  const bool vec = (D % 4 == 0) && D <= 2048 && aligned16(res) && aligned16(p->residual_out) &&
                   aligned16(p->scale) && aligned16(p->bias) &&
                   (reinterpret_cast<uintptr_t>(br) & 7u) == 0 &&
                   (reinterpret_cast<uintptr_t>(out) & 7u) == 0 &&
                   (sizeof(TB) == 2 || aligned16(br)) && (sizeof(TO) == 2 || aligned16(out));
#define VMOE_LN_CASE(NV)                                                                      \
  hipLaunchKernelGGL((add_layer_norm_kernel<TB, TO, NV>), grid, block, 0, stream, res, br,    \
                     p->scale, p->bias, p->residual_out, out, rows, D, p->eps)
  if (!vec) {
    hipLaunchKernelGGL((add_layer_norm_generic_kernel<TB, TO>), grid, block, 0, stream, res, br,
                       p->scale, p->bias, p->residual_out, out, rows, D, p->eps);
  } else if (D <= 256) {
    VMOE_LN_CASE(1);
  } else if (D <= 512) {
    VMOE_LN_CASE(2);
  } else if (D <= 768) {
    VMOE_LN_CASE(3);
  } else if (D <= 1024) {
    VMOE_LN_CASE(4);
  } else if (D <= 1536) {
    VMOE_LN_CASE(6);
  } else {
    VMOE_LN_CASE(8);
  }
#undef VMOE_LN_CASE
  return launch_status();
}


// --------------------------------------------------------------------------- attention
// softmax(Q K^T * scale) V per (image, head), head size 64, bfloat16 in and out,
// float32 logits, statistics and accumulation (flax dot_product_attention as called
// by MultiHeadDotProductAttention, vmoe/nn/vit_moe.py:166-174, without mask/dropout).
//
// One workgroup per (image, head); its keys and values sit in LDS for the whole
// kernel (K row-major, V transposed), each wave owns tiles of 32 queries.
// The logits are produced transposed, S^T = K Q^T, so that a lane holds one
// query's logits for 16 of the 32 keys of a tile: row maxima and sums are
// lane-local plus one exchange with lane ^ 32.  The exponentials, packed to
// bfloat16 in the order they already have in the accumulator, are directly the
// second operand of O^T = V^T P^T; only V^T's fragment follows that key order
// (two 8-byte reads).  Keys are walked tile by tile with a running maximum
// ("online" softmax), so the registers do not grow with the sequence length.
constexpr int kHd = 64;
constexpr int kAttnMaxWaves = 8;
constexpr int kKRow = kHd + 8;        // K row in LDS: 144 bytes, conflict-free 16-byte fragment reads
constexpr int kStageRow = 32 + 8;     // output staging row: 32 head columns + pad (80 bytes)

__global__ __launch_bounds__(kAttnMaxWaves * 64) void attention_bf16_kernel(
    const bf16_t* __restrict__ Q, const bf16_t* __restrict__ Kp, const bf16_t* __restrict__ Vp,
    bf16_t* __restrict__ O, int H, int Sq, int Sk, long q_sb, long q_ss, long k_sb, long k_ss,
    long v_sb, long v_ss, float scale_log2e, int sk_pad) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __align__(16) unsigned char smem[];
  const int vt_row = sk_pad + 8;
  bf16_t* Ks = reinterpret_cast<bf16_t*>(smem);
  bf16_t* Vt = Ks + (size_t)sk_pad * kKRow;
  bf16_t* stage_all = Vt + (size_t)kHd * vt_row;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int b = blockIdx.x / H, head = blockIdx.x - b * H;
  const bf16_t* Kb = Kp + (size_t)b * k_sb + (size_t)head * kHd;
  const bf16_t* Vb = Vp + (size_t)b * v_sb + (size_t)head * kHd;
  const bf16_t* Qb = Q + (size_t)b * q_sb + (size_t)head * kHd;

  const int ql = lane & 31, hh = lane >> 5;
  const int q_tiles = (Sq + 31) >> 5, k_tiles = sk_pad >> 5;
  // The first query tile's fragments are requested before anything else.
  bf16x8 qf[4];
  {
    const int q = wave * 32 + ql;
    const int qc = q < Sq ? q : Sq - 1;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      qf[c] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
          Qb + (size_t)qc * q_ss + 16 * c + 8 * hh));
  }
  // Stage K row-major; keys past Sk are zero.  Four chunks in flight per thread.
  for (int c0 = tid; c0 < sk_pad * 8; c0 += 4 * nthreads) {
    uint4 kv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + u * nthreads;
      const int key = c >> 3, part = c & 7;
      kv[u] = make_uint4(0, 0, 0, 0);
      if (key < Sk) kv[u] = *reinterpret_cast<const uint4*>(Kb + (size_t)key * k_ss + part * 8);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + u * nthreads;
      if (c < sk_pad * 8)
        *reinterpret_cast<uint4*>(Ks + (c >> 3) * kKRow + (c & 7) * 8) = kv[u];
    }
  }
  // Stage V transposed: a thread takes 8 keys x 8 head columns, transposes the
  // block in registers and writes each head column's 8 keys as one 16-byte chunk.
  // Consecutive lanes take consecutive key blocks of one column group, so 16 lanes
  // write 2 x 128 contiguous bytes that fall in disjoint banks.
  const int kblocks = sk_pad >> 3;
  for (int id = tid; id < kblocks * 8; id += nthreads) {
    const int part = id / kblocks, kb = id - part * kblocks;
    uint32_t w[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = kb * 8 + i;
      uint4 r = make_uint4(0, 0, 0, 0);
      if (key < Sk) r = *reinterpret_cast<const uint4*>(Vb + (size_t)key * v_ss + part * 8);
      w[i][0] = r.x; w[i][1] = r.y; w[i][2] = r.z; w[i][3] = r.w;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
      uint4 o4;
      o4.x = __builtin_amdgcn_perm(w[1][j >> 1], w[0][j >> 1], sel);
      o4.y = __builtin_amdgcn_perm(w[3][j >> 1], w[2][j >> 1], sel);
      o4.z = __builtin_amdgcn_perm(w[5][j >> 1], w[4][j >> 1], sel);
      o4.w = __builtin_amdgcn_perm(w[7][j >> 1], w[6][j >> 1], sel);
      *reinterpret_cast<uint4*>(Vt + (part * 8 + j) * vt_row + kb * 8) = o4;
    }
  }
  __syncthreads();

  bf16_t* stage = stage_all + (size_t)wave * 32 * kStageRow;
  for (int qt = wave; qt < q_tiles; qt += nwaves) {
    if (qt != wave) {
      const int q = qt * 32 + ql;
      const int qc = q < Sq ? q : Sq - 1;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        qf[c] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
            Qb + (size_t)qc * q_ss + 16 * c + 8 * hh));
    }
    floatx16 o[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 16; ++j) o[i][j] = 0.f;
    float m = 0.f, l = 0.f;
    for (int kt = 0; kt < k_tiles; ++kt) {
      floatx16 sacc;
#pragma unroll
      for (int j = 0; j < 16; ++j) sacc[j] = 0.f;
      const bf16_t* krow = Ks + (kt * 32 + ql) * kKRow + 8 * hh;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bf16x8 kf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(krow + 16 * c));
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[c], sacc, 0, 0, 0);
      }
      // sacc[4 * g + t] is the logit of key kt * 32 + 8 * g + 4 * hh + t for query ql.
      float p[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) p[j] = sacc[j];
      if (kt == k_tiles - 1 && Sk < sk_pad) {      // only the last tile holds padding keys
        const int key0 = kt * 32 + 4 * hh;
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (key0 + 8 * g + t >= Sk) p[4 * g + t] = -INFINITY;
      }
      float tmax = p[0];
#pragma unroll
      for (int j = 1; j < 16; ++j) tmax = fmaxf(tmax, p[j]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64)) * scale_log2e;   // scale > 0
      // The running maximum only has to bound the exponents: it is raised when a
      // tile exceeds it by more than 2^8, which keeps every term below 2^8 and
      // makes the rescaling of the accumulators rare (wave-uniform branch).
      if (kt == 0) {
        m = tmax;
      } else {
        const bool raise = tmax > m + 8.0f;
        if (__any(raise)) {
          const float m_new = raise ? tmax : m;
          const float alpha = __builtin_amdgcn_exp2f(m - m_new);
          l *= alpha;
          m = m_new;
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) o[i][j] *= alpha;
        }
      }
      float lsum = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(p[j], scale_log2e, -m));
        lsum += p[j];
      }
      l += lsum;
#pragma unroll
      for (int c2 = 0; c2 < 2; ++c2) {
        uint4 pk;
        pk.x = pack_bf16x2(p[8 * c2 + 0], p[8 * c2 + 1]);
        pk.y = pack_bf16x2(p[8 * c2 + 2], p[8 * c2 + 3]);
        pk.z = pack_bf16x2(p[8 * c2 + 4], p[8 * c2 + 5]);
        pk.w = pack_bf16x2(p[8 * c2 + 6], p[8 * c2 + 7]);
        const bf16x8 pf = __builtin_bit_cast(bf16x8, pk);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          // Reduction slots 0..3 / 4..7 of this lane: keys 16*c2 + 4*hh + t and + 8.
          const bf16_t* vrow = Vt + (32 * i + ql) * vt_row + kt * 32 + 16 * c2 + 4 * hh;
          const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
          const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 8);
          const bf16x8 vf = __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
          o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, o[i], 0, 0, 0);
        }
      }
    }
    mfma_result_fence();
    l += __shfl_xor(l, 32, 64);
    const float inv = 1.0f / l;
    // o[i][4 * g + t]: head column 32 * i + 8 * g + 4 * hh + t of query ql.
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 w;
        w.x = pack_bf16x2(o[i][4 * g] * inv, o[i][4 * g + 1] * inv);
        w.y = pack_bf16x2(o[i][4 * g + 2] * inv, o[i][4 * g + 3] * inv);
        *reinterpret_cast<uint2*>(stage + ql * kStageRow + 8 * g + 4 * hh) = w;
      }
      // A wave's LDS operations complete in order: it reads back what it just wrote.
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int id = lane + 64 * r;
        const int row = id >> 2, part = id & 3;
        const uint4 v = *reinterpret_cast<const uint4*>(stage + row * kStageRow + part * 8);
        const int qo = qt * 32 + row;
        if (qo < Sq)
          *reinterpret_cast<uint4*>(O + ((size_t)b * Sq + qo) * ((size_t)H * kHd) + head * kHd +
                                    32 * i + part * 8) = v;
      }
    }
  }
#endif
}

}  // namespace
}  // namespace vmoe

using namespace vmoe;

extern "C" int vmoe_add_layer_norm(const VmoeAddLayerNormParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->residual == nullptr) return VMOE_E_NULL;
  if (p->residual_out == nullptr && p->norm_out == nullptr) return VMOE_E_NULL;
  if (p->rows < 1 || p->D < 1) return VMOE_E_SHAPE;
  if ((p->branch_dtype != VMOE_F32 && p->branch_dtype != VMOE_BF16) ||
      (p->out_dtype != VMOE_F32 && p->out_dtype != VMOE_BF16))
    return VMOE_E_DTYPE;
  hipStream_t s = as_stream(stream);
  const bool bb = p->branch_dtype == VMOE_BF16, ob = p->out_dtype == VMOE_BF16;
  if (bb && ob) return launch_add_layer_norm<bf16_t, bf16_t>(p, s);
  if (bb) return launch_add_layer_norm<bf16_t, float>(p, s);
  if (ob) return launch_add_layer_norm<float, bf16_t>(p, s);
  return launch_add_layer_norm<float, float>(p, s);
}

extern "C" int vmoe_attention(const VmoeAttentionParams* p, vmoe_stream_t stream) {
  if (p == nullptr || p->q == nullptr || p->k == nullptr || p->v == nullptr || p->out == nullptr)
    return VMOE_E_NULL;
  if (p->B < 1 || p->H < 1 || p->Sq < 1 || p->Sk < 1) return VMOE_E_SHAPE;
  if (p->dtype != VMOE_BF16 || p->head_dim != kHd || !(p->scale > 0.f)) return VMOE_E_UNSUPPORTED;
  if ((int64_t)p->B * p->H >= INT32_MAX) return VMOE_E_OVERFLOW;
  const int64_t strides[6] = {p->q_stride_b, p->q_stride_s, p->k_stride_b,
                              p->k_stride_s, p->v_stride_b, p->v_stride_s};
  for (int64_t s : strides)
    if (s % 8 != 0) return VMOE_E_ALIGN;
  if (!aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->out))
    return VMOE_E_ALIGN;
  const int sk_pad = (p->Sk + 31) / 32 * 32;
  int waves = (p->Sq + 31) / 32;
  if (waves > kAttnMaxWaves) waves = kAttnMaxWaves;
  const size_t lds = (size_t)sk_pad * kKRow * 2 + (size_t)kHd * (sk_pad + 8) * 2 +
                     (size_t)waves * 32 * kStageRow * 2;
  if (lds > 160 * 1024) return VMOE_E_UNSUPPORTED;
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(attention_bf16_kernel), lds);
  if (e != hipSuccess) return (int)e;
  const float scale_log2e = p->scale * 1.4426950408889634f;
  hipLaunchKernelGGL(attention_bf16_kernel, dim3((unsigned)(p->B * p->H)), dim3(waves * 64), lds,
                     as_stream(stream), (const bf16_t*)p->q, (const bf16_t*)p->k,
                     (const bf16_t*)p->v, (bf16_t*)p->out, p->H, p->Sq, p->Sk, (long)p->q_stride_b,
                     (long)p->q_stride_s, (long)p->k_stride_b, (long)p->k_stride_s,
                     (long)p->v_stride_b, (long)p->v_stride_s, scale_log2e, sk_pad);
  return launch_status();
}
