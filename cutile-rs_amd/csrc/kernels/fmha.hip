// Fused multi-head attention forward for gfx950 (bf16 or f16 in/out, f32
// softmax statistics and accumulation).
//
// Tile program being implemented (cutile-examples/examples/flash_attention_causal.rs:19-134,
// cutile-benchmarks/benches/fmha.rs:20-145): one tile block per (batch*head, BM
// query rows); for each KV tile j < tc:
//   qk = Q·K_jᵀ · (qk_scale / ln 2)  (+ -inf where masked, for tiles j >= mask_start)
//   m' = max(m, rowmax(qk)); p = exp2(qk - m'); α = exp2(m - m')
//   l = l·α + rowsum(p); acc = acc·α + p·V_j; m = m'
// and finally out = acc / l.  Key j is visible to query i iff i + input_pos >= j
// (causal) and j < k_seqlen; tc = ceil(min(input_pos + (q_tile+1)·BM, k_seqlen) / BN).
//
// Mapping to CDNA4.  Everything is computed transposed: Sᵀ = K·Qᵀ and
// Oᵀ = Vᵀ·Pᵀ with v_mfma_f32_32x32x16.  In the MFMA result layout a lane owns
// one column, so with the transposed product each lane owns ONE QUERY ROW:
//  * row max / row sum are reductions over a lane's own registers plus a single
//    exchange with lane^32 — no cross-lane trees, no LDS;
//  * α and 1/l are per-lane scalars;
//  * the f32 Sᵀ accumulators, converted to 16-bit in place, ARE the second
//    operand (Pᵀ) of the next MFMA — P never moves between lanes;
//  * Qᵀ is an MFMA operand straight from global memory (d-contiguous), K is
//    d-contiguous in LDS (ds_read_b128), and Vᵀ is formed by the LDS transpose
//    read ds_read_b64_tr_b16 from V stored as it is in memory.
// K and V tiles are staged through LDS, double buffered, one barrier per KV
// tile, with the next tile's global loads in flight during the current tile's
// matrix work.  One wavefront owns 32 query rows; a workgroup is BM/32 waves.
#include <hip/hip_runtime.h>

#include "kernel_args.h"

using namespace cutile;

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define LDS_PTR(T) __attribute__((address_space(3))) T*

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

template <typename T>
struct Elem;
template <>
struct Elem<__bf16> {
  using vec8 = bf16x8;
  __device__ static __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{lo, hi}, b2));  // v_cvt_pk_bf16_f32, RNE
  }
};
template <>
struct Elem<_Float16> {
  using vec8 = f16x8;
  __device__ static __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{lo, hi}, h2));  // v_cvt_pk_f16_f32
  }
};

template <typename T, int BM, int BN, int D>
struct Fmha {
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  static constexpr int kWaves = BM / 32;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int kUnitsPerRow = D / 8;               // 16-byte units per K/V row
  static constexpr int kTileUnits = BN * kUnitsPerRow;
  static constexpr int kLoads = kTileUnits / kThreads;
  static constexpr int kTileBytes = BN * D * 2;
  static constexpr int kStageBytes = 2 * kTileBytes;        // K then V
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static constexpr int SB = BN / 32;                        // 32-row blocks of Sᵀ
  static constexpr int DB = D / 32;                         // 32-row blocks of Oᵀ
  static_assert(D % 32 == 0 && BN % 32 == 0 && BM % 32 == 0, "tile shape");
  static_assert(kTileUnits % kThreads == 0, "tile must split evenly over the workgroup");

  // K tile [BN][D]: unit u of row r at u ^ (r & (kUnitsPerRow-1) & 15).
  __device__ static __forceinline__ int k_off(int r, int u) {
    return r * (D * 2) + ((u ^ (r & (kUnitsPerRow - 1) & 15)) << 4);
  }
  // V tile [BN][D]: unit u of row r at u ^ ((r & 3) << 2) (transpose reads take 4 rows at once);
  // with 8 units per row (D = 64) only one row bit fits, with 4 (D = 32) none.
  __device__ static __forceinline__ int v_off(int r, int u) {
    constexpr int mask = kUnitsPerRow >= 16 ? 3 : (kUnitsPerRow >= 8 ? 1 : 0);
    return r * (D * 2) + ((u ^ ((r & mask) << 2)) << 4);
  }

  __device__ static void run(const PartitionArg<3>& out, const TensorArg<4>& q, const TensorArg<4>& k,
                             const TensorArg<4>& v, float qk_scale, int32_t input_pos,
                             int32_t group_size, int32_t causal, const TileGrid& g) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int l32 = lane & 31, half = lane >> 5;
    const int grp = lane >> 4, l16 = lane & 15;

    const int32_t H = q.shape[1];
    const int32_t bh = blockIdx.x;
    // Heaviest causal tiles (largest query index) are dispatched first.
    const int32_t q_tile = causal ? (int32_t)(g.y - 1 - blockIdx.y) : (int32_t)blockIdx.y;
    const int32_t batch = bh / H, head = bh % H, kv_head = head / group_size;
    const int32_t q_len = q.shape[2], k_len = k.shape[2];
    const int32_t q0 = q_tile * BM + wave * 32;   // first query row of this wavefront

    const T* qb = (const T*)q.ptr + (int64_t)batch * q.strides[0] + (int64_t)head * q.strides[1];
    const T* kb = (const T*)k.ptr + (int64_t)batch * k.strides[0] + (int64_t)kv_head * k.strides[1];
    const T* vb = (const T*)v.ptr + (int64_t)batch * v.strides[0] + (int64_t)kv_head * v.strides[1];
    const int32_t q_ld = q.strides[2], k_ld = k.strides[2], v_ld = v.strides[2];
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(qb, (uint32_t)(((int64_t)(q_len - 1) * q_ld + D) * 2));
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(kb, (uint32_t)(((int64_t)(k_len - 1) * k_ld + D) * 2));
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(vb, (uint32_t)(((int64_t)(k_len - 1) * v_ld + D) * 2));
    constexpr uint32_t kOob = 0x80000000u;

    // Qᵀ operand: lane holds query row q0 + l32, d = ks*16 + half*8 .. +7.
    vec8 qf[D / 16];
    {
      const int32_t qr = q0 + l32;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        uint32_t off = qr < q_len ? (uint32_t)(((int64_t)qr * q_ld + ks * 16 + half * 8) * 2) : kOob;
        qf[ks] = __builtin_bit_cast(vec8, __builtin_amdgcn_raw_buffer_load_b128(rq, off, 0, 0));
      }
    }

    // Loop bounds (flash_attention_causal.rs:60-69).
    int32_t tc = (k_len + BN - 1) / BN;
    int32_t mask_start = k_len / BN;
    if (causal) {
      const int32_t m_end = input_pos + (q_tile + 1) * BM;
      mask_start = min((input_pos + q_tile * BM) / BN, k_len / BN);
      tc = (min(m_end, k_len) + BN - 1) / BN;
    }

    int ld_row[kLoads], ld_unit[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      int c = tid + i * kThreads;
      ld_row[i] = c / kUnitsPerRow;
      ld_unit[i] = c % kUnitsPerRow;
    }
    u32x4 k_reg[kLoads], v_reg[kLoads];
    auto load_global = [&](int32_t j) {
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        int32_t r = j * BN + ld_row[i];
        uint32_t ko = r < k_len ? (uint32_t)(((int64_t)r * k_ld + ld_unit[i] * 8) * 2) : kOob;
        uint32_t vo = r < k_len ? (uint32_t)(((int64_t)r * v_ld + ld_unit[i] * 8) * 2) : kOob;
        k_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rk, ko, 0, 0);
        v_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rv, vo, 0, 0);
      }
    };
    auto store_lds = [&](int stage) {
      unsigned char* sk = lds + stage * kStageBytes;
      unsigned char* sv = sk + kTileBytes;
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        *reinterpret_cast<u32x4*>(sk + k_off(ld_row[i], ld_unit[i])) = k_reg[i];
        *reinterpret_cast<u32x4*>(sv + v_off(ld_row[i], ld_unit[i])) = v_reg[i];
      }
    };

    f32x16 o_acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
    float m_i = -INFINITY, l_i = 0.0f;
    const float c = qk_scale * kLog2e;  // qk_scale / ln 2
    const int32_t q_pos = q0 + l32 + input_pos;  // this lane's query position for the causal rule

    if (tc > 0) {
      load_global(0);
      store_lds(0);
    }
    __syncthreads();

    for (int32_t j = 0; j < tc; ++j) {
      const int cur = j & 1;
      if (j + 1 < tc) load_global(j + 1);
      const unsigned char* sk = lds + cur * kStageBytes;
      const unsigned char* sv = sk + kTileBytes;

      // Sᵀ = K_j · Qᵀ : SB blocks of 32 kv rows x 32 query columns.
      f32x16 s[SB];
#pragma unroll
      for (int sb = 0; sb < SB; ++sb) {
#pragma unroll
        for (int e = 0; e < 16; ++e) s[sb][e] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          vec8 kf = *reinterpret_cast<const vec8*>(sk + k_off(sb * 32 + l32, ks * 2 + half));
          s[sb] = E::mfma(kf, qf[ks], s[sb]);
        }
      }
      // s[sb][e] belongs to kv = j*BN + sb*32 + (e/4)*8 + half*4 + e%4, query = this lane's.
      if (j >= mask_start) {
#pragma unroll
        for (int sb = 0; sb < SB; ++sb)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            int32_t kv = j * BN + sb * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
            bool visible = kv < k_len && (!causal || q_pos >= kv);
            s[sb][e] = visible ? s[sb][e] : -INFINITY;
          }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < SB; ++sb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[sb][e]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // Statistics are kept in the scaled log2 domain: m = c * rowmax(raw).  The
      // reference point m only has to bound the exponents, not equal the maximum:
      // it moves (and the accumulators are rescaled) only when some row's maximum
      // rose by more than kSlack, so p stays below 2^kSlack and after the first
      // tiles the rescale is skipped almost always.
      constexpr float kSlack = 8.0f;
      const float m_cand = fmaxf(m_i, mx * c);
      const bool moved = __builtin_amdgcn_ballot_w64(m_cand > m_i + kSlack) != 0;   // wavefront-uniform
      const float m_new = moved ? m_cand : m_i;
      const float m_use = m_new == -INFINITY ? 0.0f : m_new;  // fully masked so far: keep exp2 finite
      float rs = 0.0f;
      vec8 pf[BN / 16];
#pragma unroll
      for (int sb = 0; sb < SB; ++sb) {
        float p[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[sb][e], c, -m_use));
          rs += p[e];
        }
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          u32x4 w;
          w.x = E::pack2(p[hh * 8 + 0], p[hh * 8 + 1]);
          w.y = E::pack2(p[hh * 8 + 2], p[hh * 8 + 3]);
          w.z = E::pack2(p[hh * 8 + 4], p[hh * 8 + 5]);
          w.w = E::pack2(p[hh * 8 + 6], p[hh * 8 + 7]);
          pf[sb * 2 + hh] = __builtin_bit_cast(vec8, w);
        }
      }
      rs += __shfl_xor(rs, 32, 64);
      if (moved) {
        const float alpha = __builtin_amdgcn_exp2f(m_i - m_use);
        l_i *= alpha;
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
          for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;
        m_i = m_new;
      }
      l_i += rs;

      // Oᵀ += V_jᵀ · Pᵀ.  MFMA step t covers kv rows 16t..16t+15 of the tile; slot
      // (half, jj) of a lane's operand is kv = 16t + 8*(jj/4) + 4*half + jj%4, which is
      // exactly the order the Sᵀ accumulators come in.
#pragma unroll
      for (int t = 0; t < BN / 16; ++t) {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int dcol = db * 32 + (grp & 1) * 16 + (l16 & 3) * 4;  // first of 4 d-columns addressed
          const int kr = t * 16 + (grp >> 1) * 4 + (l16 >> 2);
          const unsigned char* p0 = sv + v_off(kr, dcol >> 3) + (dcol & 7) * 2;
          const unsigned char* p1 = sv + v_off(kr + 8, dcol >> 3) + (dcol & 7) * 2;
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p0);
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p1);
          s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          o_acc[db] = E::mfma(__builtin_bit_cast(vec8, both), pf[t], o_acc[db]);
        }
      }
      if (j + 1 < tc) store_lds(cur ^ 1);
      __syncthreads();
    }

    // out[bh, q, d] = acc / l.  o_acc[db][e]: d = db*32 + (e/4)*8 + half*4 + e%4.
    const int32_t qr = q0 + l32;
    if (qr < out.shape[1] && qr < q_len) {
      T* orow = (T*)out.ptr + (int64_t)bh * out.strides[0] + (int64_t)qr * out.strides[1];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const int d = db * 32 + qd * 8 + half * 4;
          u32x2 w;
          w.x = E::pack2(o_acc[db][qd * 4 + 0] / l_i, o_acc[db][qd * 4 + 1] / l_i);
          w.y = E::pack2(o_acc[db][qd * 4 + 2] / l_i, o_acc[db][qd * 4 + 3] / l_i);
          *reinterpret_cast<u32x2*>(orow + d) = w;
        }
    }
  }
};

}  // namespace

#define FMHA_KERNEL(NAME, T, BM, BN, D)                                                           \
  extern "C" __global__ void __launch_bounds__((BM / 32) * 64)                                   \
      fmha_entry__##NAME##_##BM##x##BN##x##D(PartitionArg<3> out, TensorArg<4> q, TensorArg<4> k, \
                                             TensorArg<4> v, float qk_scale, int32_t input_pos,   \
                                             int32_t query_group_size, int32_t causal, TileGrid g) { \
    Fmha<T, BM, BN, D>::run(out, q, k, v, qk_scale, input_pos, query_group_size, causal, g);     \
  }

FMHA_KERNEL(bf16, __bf16, 128, 64, 128)
FMHA_KERNEL(bf16, __bf16, 128, 128, 128)
FMHA_KERNEL(bf16, __bf16, 256, 64, 128)
FMHA_KERNEL(bf16, __bf16, 128, 64, 64)
FMHA_KERNEL(bf16, __bf16, 64, 64, 64)
FMHA_KERNEL(bf16, __bf16, 64, 32, 32)
FMHA_KERNEL(bf16, __bf16, 32, 32, 32)
FMHA_KERNEL(f16, _Float16, 128, 64, 128)
FMHA_KERNEL(f16, _Float16, 128, 64, 64)
FMHA_KERNEL(f16, _Float16, 32, 32, 32)
