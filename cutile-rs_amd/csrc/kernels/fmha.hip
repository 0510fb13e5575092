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

#include <type_traits>
#include <utility>

#include "kernel_args.h"
#include "lane_exchange.h"

using namespace cutile;

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define LDS_PTR(T) __attribute__((address_space(3))) T*

constexpr float kLog2e = 1.4426950408889634f;

// Bytes from the first element of row 0 to the last of row rows - 1 (16-bit elements, `row_stride`
// elements apart, `d` per row); nothing for an empty range, so that every access is out of range.
__device__ __forceinline__ uint32_t rows_extent_bytes(int32_t rows, int32_t row_stride, int32_t d) {
  return rows > 0 ? (uint32_t)(((int64_t)(rows - 1) * row_stride + d) * 2) : 0u;
}
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

// The two lanes that own one query row are 32 apart: their maximum and sum go through v_permlane32_swap, and the
// four lanes of a head in the matrix-core decode kernel through v_permlane16_swap first (lane_exchange.h), inside the
// vector ALU, where a lane-indexed permute would cost a trip through the LDS crossbar and a wait of its own in the middle
// of every softmax segment.
__device__ __forceinline__ float max_across_halves(float v) { return lanes::across_halves<lanes::Max>(v); }
__device__ __forceinline__ float sum_across_halves(float v) { return lanes::across_halves<lanes::Sum>(v); }
__device__ __forceinline__ float max_across_rows(float v) { return lanes::across_rows<lanes::Max>(v); }
__device__ __forceinline__ float sum_across_rows(float v) { return lanes::across_rows<lanes::Sum>(v); }

// (batch*head, query tile) of this workgroup.  Workgroups are dealt round-robin to
// the 8 XCDs in dispatch order; every query tile of one head is given to the same
// XCD, consecutively, so that the head's K and V (read by each of its query
// tiles) stay in that XCD's L2 instead of being fetched from HBM once per tile.
// Causal launches do the same with a few heads side by side per XCD, heaviest tiles
// first (see below); one head at a time measured slower than the plain order because the
// last head's long tiles start late.
__device__ __forceinline__ void head_and_tile(uint32_t n_bh, uint32_t n_qt, int32_t causal, uint32_t group, int32_t* bh, int32_t* q_tile) {
  constexpr uint32_t kNumXcd = 8;
  const uint32_t id = blockIdx.x + gridDim.x * blockIdx.y;
  uint32_t b, t;
  constexpr uint32_t kCusPerXcd = 32;
  uint32_t side = n_qt >= kCusPerXcd ? 1 : kCusPerXcd / n_qt;     // heads an XCD works on side by side
  // Query heads that share a KV head (consecutive, `group` of them) run side by side on one XCD, tile for tile, so
  // that the K/V rows one of them fetches serve all of them.
  if (group > 1) side = (side + group - 1) / group * group;
  if (n_bh % kNumXcd == 0 && !causal && group <= 1) {
    const uint32_t xcd = id % kNumXcd, slot = id / kNumXcd;
    b = (slot / n_qt) * kNumXcd + xcd;
    t = slot % n_qt;
  } else if (n_bh % (kNumXcd * side) == 0 && (causal || group > 1)) {
    // Causal tiles differ n_qt-fold in length.  An XCD takes `side` heads at a time (their K/V fit its L2) and
    // walks their tiles heaviest first, heads interleaved: the compute units that drew the short tiles of one
    // group free up first and draw the long tiles of the next, so lengths pair up (n_qt + 1 per two tiles).
    const uint32_t xcd = id % kNumXcd, slot = id / kNumXcd, per_group = side * n_qt;
    b = xcd * (n_bh / kNumXcd) + (slot / per_group) * side + (slot % per_group) % side;
    t = (slot % per_group) / side;
  } else {   // plain order: every (head, tile) still covered exactly once
    b = id % n_bh;
    t = id / n_bh;
  }
  *bh = (int32_t)b;
  *q_tile = causal ? (int32_t)(n_qt - 1 - t) : (int32_t)t;
}

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
    int32_t bh, q_tile;
    head_and_tile(g.x, g.y, causal, (uint32_t)group_size, &bh, &q_tile);
    const int32_t batch = bh / H, head = bh % H, kv_head = head / group_size;
    const int32_t q_len = q.shape[2], k_len = k.shape[2];
    const int32_t q0 = q_tile * BM + wave * 32;   // first query row of this wavefront

    const T* qb = (const T*)q.ptr + (int64_t)batch * q.strides[0] + (int64_t)head * q.strides[1];
    const T* kb = (const T*)k.ptr + (int64_t)batch * k.strides[0] + (int64_t)kv_head * k.strides[1];
    const T* vb = (const T*)v.ptr + (int64_t)batch * v.strides[0] + (int64_t)kv_head * v.strides[1];
    const int32_t q_ld = q.strides[2], k_ld = k.strides[2], v_ld = v.strides[2];
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(qb, rows_extent_bytes(q_len, q_ld, D));
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(kb, rows_extent_bytes(k_len, k_ld, D));
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(vb, rows_extent_bytes(k_len, v_ld, D));
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
    const int32_t last_visible = (causal ? min(q_pos, k_len - 1) : k_len - 1) - half * 4;   // last key the lane may see

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
      if (j >= mask_start) {   // visible iff the key's lane-independent index in the tile is <= lim: a compare and a select
        const int32_t lim = last_visible - j * BN;
#pragma unroll
        for (int sb = 0; sb < SB; ++sb)
#pragma unroll
          for (int e = 0; e < 16; ++e) s[sb][e] = (sb * 32 + (e >> 2) * 8 + (e & 3)) <= lim ? s[sb][e] : -INFINITY;
      }
      float mx = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < SB; ++sb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[sb][e]);
      mx = max_across_halves(mx);
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
      if (moved) {   // (l_i and rs are this half's share of the row sum; the halves are added after the last tile)
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
    // A row that saw no key at all (an empty key range) has l = 0 and becomes 0, as in the
    // production kernels (l_safe = max(l, 1e-8), cutile-kernels/src/attention.rs:383-386); any other row has l >= 1.
    l_i = fmaxf(sum_across_halves(l_i), 1.0e-8f);
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

// ---- ping-pong variant (BM = 256, eight wavefronts) --------------------------------------
// The kernel above keeps all wavefronts of a workgroup in the same phase: they
// multiply together (matrix pipes busy, vector ALUs idle) and then run the
// softmax together (the reverse).  Per KV tile a wavefront needs about as many
// vector-ALU cycles for the softmax as matrix-pipe cycles for its 32 MFMAs, so
// here the two wavefronts that share a SIMD (w and w+4) run half a tile apart:
//   interval:        I0      I1      I2          I3          I4
//   waves 0..3:      S0      soft0   PV0,S1      soft1       PV1,S2 ...
//   waves 4..7:      -       S0      soft0       PV0,S1      soft1  ...
// with one workgroup barrier between intervals, so that on every SIMD one
// wavefront feeds the matrix pipe while the other feeds the vector ALU.
//  * K and V tiles go global -> LDS directly (16 bytes per lane), two buffers
//    each; a buffer is refilled in the interval after both halves of the
//    workgroup have read it and is waited for two intervals later;
//  * operand fragments are read from LDS three MFMAs ahead of their use;
//  * the two 32-row blocks of S^T (and the four of O^T) are independent
//    accumulators and are issued alternately, so no MFMA waits on the previous one;
//  * the output leaves through LDS as 16-byte stores of whole 256-byte rows.
template <typename T, int BN, int D>
struct FmhaPingPong {
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  static constexpr int BM = 256;
  static constexpr int kWaves = BM / 32;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int kUnitsPerRow = D / 8;
  static constexpr int kTileBytes = BN * D * 2;
  static constexpr int kRowsPerInstr = 1024 / (D * 2);
  static constexpr int kInstr = kTileBytes / 1024 / kWaves;    // direct loads per wavefront per tile
  static constexpr int SB = BN / 32, DB = D / 32, KS = D / 16, TS = BN / 16;
  static constexpr int kLdsBytes = 4 * kTileBytes;
  static_assert(D == 128 && BN % 32 == 0, "tile shape");
  static_assert(kInstr >= 1 && kTileBytes % (1024 * kWaves) == 0, "tile must split evenly over the workgroup");
  static_assert(kWaves * 32 * D * 2 <= kLdsBytes, "the output bands must fit the tile buffers");

  // Same layouts as Fmha: K unit u of row r at u ^ (r & 15); V unit u at u ^ ((r & 3) << 2).
  __device__ static __forceinline__ int k_off(int r, int u) { return r * (D * 2) + ((u ^ (r & 15)) << 4); }
  __device__ static __forceinline__ int v_off(int r, int u) { return r * (D * 2) + ((u ^ ((r & 3) << 2)) << 4); }

  __device__ static void run(const PartitionArg<3>& out, const TensorArg<4>& q, const TensorArg<4>& k,
                             const TensorArg<4>& v, float qk_scale, int32_t input_pos,
                             int32_t group_size, int32_t causal, const TileGrid& g) {
    // Separately named buffers: the compiler can tell a refill of one from reads of another.
    __shared__ __attribute__((aligned(1024))) unsigned char kb0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char kb1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char vb0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char vb1[kTileBytes];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // The half of the workgroup that runs one interval behind.  Causal: the upper rows (wavefronts 0-3), which see
    // fewer keys: they finish their last tile while the lower rows still have diagonal tiles to do, and what is left
    // of the workgroup's run is the leading half's alone (see tc_h below).
    const bool late = causal ? wave < kWaves / 2 : wave >= kWaves / 2;
    const int l32 = lane & 31, half = lane >> 5;
    const int grp = lane >> 4, l16 = lane & 15;

    const int32_t H = q.shape[1];
    int32_t bh, q_tile;
    head_and_tile(g.x, g.y, causal, (uint32_t)group_size, &bh, &q_tile);
    const int32_t batch = bh / H, head = bh % H, kv_head = head / group_size;
    const int32_t q_len = q.shape[2], k_len = k.shape[2];
    const int32_t q0 = q_tile * BM + wave * 32;

    const T* qb = (const T*)q.ptr + (int64_t)batch * q.strides[0] + (int64_t)head * q.strides[1];
    const T* kb = (const T*)k.ptr + (int64_t)batch * k.strides[0] + (int64_t)kv_head * k.strides[1];
    const T* vb = (const T*)v.ptr + (int64_t)batch * v.strides[0] + (int64_t)kv_head * v.strides[1];
    const int32_t q_ld = q.strides[2], k_ld = k.strides[2], v_ld = v.strides[2];
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(qb, rows_extent_bytes(q_len, q_ld, D));
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(kb, rows_extent_bytes(k_len, k_ld, D));
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(vb, rows_extent_bytes(k_len, v_ld, D));
    constexpr uint32_t kOob = 0x80000000u;

    vec8 qf[KS];
    {
      const int32_t qr = q0 + l32;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        uint32_t off = qr < q_len ? (uint32_t)(((int64_t)qr * q_ld + ks * 16 + half * 8) * 2) : kOob;
        qf[ks] = __builtin_bit_cast(vec8, __builtin_amdgcn_raw_buffer_load_b128(rq, off, 0, 0));
      }
    }
    // The scores are wanted in the log2 domain, c * (q . k) with c = qk_scale * log2(e).  Q is multiplied by c once,
    // here (rounded back to T: a relative 2^-9 per element for bf16, below the rounding of P), and the reference
    // point of the softmax rides in the accumulator the S^T products start from (see neg_ref), so that the
    // MFMAs deliver c * s - m directly and the softmax spends no multiply-add per score.
    const float c = qk_scale * kLog2e;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = E::pack2((float)qf[ks][2 * e] * c, (float)qf[ks][2 * e + 1] * c);
      qf[ks] = __builtin_bit_cast(vec8, w);
    }

    // tc: KV tiles the workgroup fetches.  tc_h: those this half of it (128 query rows) multiplies; under a causal mask
    // the upper half's rows end up to two tiles of keys before the lower half's, and a tile whose keys no row of the
    // half sees adds nothing to it.  mask_start: the first tile in which some key is hidden from some row of the half.
    int32_t tc = (k_len + BN - 1) / BN, tc_h = tc;
    int32_t mask_start = k_len / BN;
    if (causal) {
      const int32_t m_end = input_pos + (q_tile + 1) * BM;
      tc = (min(m_end, k_len) + BN - 1) / BN;
      const int32_t h0 = input_pos + q_tile * BM + (wave / (kWaves / 2)) * (BM / 2);   // position of the half's first query
      mask_start = min(h0 / BN, k_len / BN);
      tc_h = (min(h0 + BM / 2, k_len) + BN - 1) / BN;
    }

    // Global side of the tile fetches: the LDS side of a direct load is lane
    // contiguous, so a lane fetches the unit that belongs at its LDS position.
    int32_t ld_row[kInstr];
    uint32_t k_goff[kInstr], v_goff[kInstr];
#pragma unroll
    for (int i = 0; i < kInstr; ++i) {
      const int r = (wave * kInstr + i) * kRowsPerInstr + lane / kUnitsPerRow;
      const int up = lane % kUnitsPerRow;
      ld_row[i] = r;
      k_goff[i] = (uint32_t)(((int64_t)r * k_ld + (up ^ (r & 15)) * 8) * 2);
      v_goff[i] = (uint32_t)(((int64_t)r * v_ld + (up ^ ((r & 3) << 2)) * 8) * 2);
    }
    // Tile j of K (V) into `buf`; rows at or beyond k_len, and every row when
    // !wanted, use an out-of-range offset and read zeros.
    auto fetch_k = [&](unsigned char* buf, int32_t j, bool wanted = true) {
      const int32_t row0 = wanted ? j * BN : 0;
#pragma unroll
      for (int i = 0; i < kInstr; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (LDS_PTR(void))(buf + (wave * kInstr + i) * 1024), 16,
                                                 wanted && row0 + ld_row[i] < k_len ? k_goff[i] : kOob,
                                                 row0 * k_ld * 2, 0, 0);
    };
    auto fetch_v = [&](unsigned char* buf, int32_t j) {
#pragma unroll
      for (int i = 0; i < kInstr; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (LDS_PTR(void))(buf + (wave * kInstr + i) * 1024), 16,
                                                 j * BN + ld_row[i] < k_len ? v_goff[i] : kOob, j * BN * v_ld * 2, 0, 0);
    };

    // LDS side of the operand reads.
    int k_addr[KS], v_addr[DB];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_addr[ks] = k_off(l32, ks * 2 + half);          // + sb * 32 rows
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int dcol = db * 32 + (grp & 1) * 16 + (l16 & 3) * 4;
      const int kr = (grp >> 1) * 4 + (l16 >> 2);                                   // + t * 16 (+ 8) rows
      v_addr[db] = v_off(kr, dcol >> 3) + (dcol & 7) * 2;
    }
    auto read_k = [&](const unsigned char* buf, int n) -> vec8 {   // step n of S^T: ks = n / SB, sb = n % SB
      return *reinterpret_cast<const vec8*>(buf + k_addr[n / SB] + (n % SB) * 32 * (D * 2));
    };
    auto read_v = [&](const unsigned char* buf, int n) -> vec8 {   // step n of O^T: t = n / DB, db = n % DB
      const unsigned char* p = buf + v_addr[n % DB] + (n / DB) * 16 * (D * 2);
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p);
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p + 8 * (D * 2)));
      return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    f32x16 o_acc[DB], s[SB];
    vec8 pf[TS];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
    float m_i = -INFINITY, l_i = 0.0f;
    // Every S^T block starts from -m_ref in all 16 accumulators of the lane (a lane owns one query), m_ref being the
    // row's reference point (0 until the first tile has set one).
    f32x16 neg_ref;
#pragma unroll
    for (int e = 0; e < 16; ++e) neg_ref[e] = 0.0f;
    const int32_t q_pos = q0 + l32 + input_pos;
    // Last key this lane may see, less the part of a key's index inside a tile that depends on the lane (half * 4).
    const int32_t last_visible = (causal ? min(q_pos, k_len - 1) : k_len - 1) - half * 4;

    // Matrix segments.  Fragments are read kAhead steps before the MFMA that uses
    // them; sched_barrier(0) after every step keeps reads and MFMAs in this order.
    constexpr int kAhead = 3, kRing = kAhead + 1;
    constexpr int NS = SB * KS, NO = TS * DB;   // MFMAs of S^T and of O^T per tile
    // O^T += V_j^T P_j^T from `vbuf`, then (WITH_S) S^T = K_{j+1} Q^T from `kbuf`.
    auto matrix_segment = [&](const unsigned char* vbuf, const unsigned char* kbuf, auto with_s) {
      constexpr int total = NO + (decltype(with_s)::value ? NS : 0);
      vec8 ring[kRing];
      auto read_step = [&](int n) -> vec8 { return n < NO ? read_v(vbuf, n) : read_k(kbuf, n - NO); };
#pragma unroll
      for (int n = 0; n < kAhead; ++n) ring[n % kRing] = read_step(n);
#pragma unroll
      for (int n = 0; n < total; ++n) {
        if (n + kAhead < total) ring[(n + kAhead) % kRing] = read_step(n + kAhead);
        if (n < NO) {
          o_acc[n % DB] = E::mfma(ring[n % kRing], pf[n / DB], o_acc[n % DB]);
        } else {
          const int m = n - NO;
          s[m % SB] = E::mfma(ring[n % kRing], qf[m / SB], m < SB ? neg_ref : s[m % SB]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // S^T = K_0 Q^T alone (first segment).
    auto first_segment = [&](const unsigned char* kbuf) {
      vec8 ring[kRing];
#pragma unroll
      for (int n = 0; n < kAhead; ++n) ring[n % kRing] = read_k(kbuf, n);
#pragma unroll
      for (int m = 0; m < NS; ++m) {
        if (m + kAhead < NS) ring[(m + kAhead) % kRing] = read_k(kbuf, m + kAhead);
        s[m % SB] = E::mfma(ring[m % kRing], qf[m / SB], m < SB ? neg_ref : s[m % SB]);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // Softmax segment of tile j: s -> pf, running statistics.  s holds c * score - m_ref (m_ref = m_i, or 0 before the
    // first tile).  The reference point moves only when some row's maximum rises more than 2^kSlack above it; then
    // (and on the first tile) the scores are shifted to the new reference and O, l are rescaled.  Otherwise p = 2^s.
    auto softmax_segment = [&](int32_t j) {
      if (j >= mask_start) {
        // Key sb*32 + (e>>2)*8 + half*4 + (e&3) of this tile is visible iff it is <= last_visible: one compare
        // against a constant and one select per element.
        const int32_t lim = last_visible - j * BN;
#pragma unroll
        for (int sb = 0; sb < SB; ++sb)
#pragma unroll
          for (int e = 0; e < 16; ++e) s[sb][e] = (sb * 32 + (e >> 2) * 8 + (e & 3)) <= lim ? s[sb][e] : -INFINITY;
      }
      float mx = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < SB; ++sb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[sb][e]);
      mx = max_across_halves(mx);
      constexpr float kSlack = 8.0f;
      const float m_ref = m_i == -INFINITY ? 0.0f : m_i;       // what the accumulators started from
      const float m_cand = fmaxf(m_i, mx + m_ref);
      const bool moved = __builtin_amdgcn_ballot_w64(m_cand > m_i + kSlack) != 0;
      if (moved) {
        const float m_use = m_cand == -INFINITY ? 0.0f : m_cand;
        const float shift = m_use - m_ref;
#pragma unroll
        for (int sb = 0; sb < SB; ++sb)
#pragma unroll
          for (int e = 0; e < 16; ++e) s[sb][e] -= shift;
        const float alpha = __builtin_amdgcn_exp2f(m_i - m_use);   // 0 on the first tile (m_i = -inf)
        l_i *= alpha;
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
          for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;
        m_i = m_cand;
#pragma unroll
        for (int e = 0; e < 16; ++e) neg_ref[e] = -m_use;
      }
      float rs = 0.0f;
#pragma unroll
      for (int sb = 0; sb < SB; ++sb) {
        float p[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          p[e] = __builtin_amdgcn_exp2f(s[sb][e]);
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
      l_i += rs;   // this half's share of the row sum: every rescaling multiplies both halves' shares by the same
                   // alpha, so the halves are added once, after the last tile
    };
    auto interval_end = [&]() {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    };
    auto wait_fetches = [&]() { __builtin_amdgcn_s_waitcnt(0); };   // own fetches landed, own LDS reads done
    // The two halves of the workgroup run the same segments one interval apart;
    // each gets its own straight-line copy of the loop.  Tile j: K_j in kc, V_j in
    // vc, K_{j+1} in kn; refills K_{j+2} -> kc and V_{j+1} -> vn are issued in the
    // interval after both halves have read those buffers (the early half at the
    // start of its matrix segment, the late half at the start of its softmax) and
    // waited for at the end of the following interval.
    auto pipeline = [&](auto late_tag) {
      constexpr bool LATE = decltype(late_tag)::value;
      auto tile = [&](int32_t j, unsigned char* kc, unsigned char* kn, unsigned char* vc, unsigned char* vn,
                      auto last_tag) {
        constexpr bool LAST = decltype(last_tag)::value;
        auto refill = [&]() {
          fetch_k(kc, j + 2, j + 2 < tc);
          fetch_v(vn, j + 1);
        };
        // (the late half's last tile may not be the workgroup's: its share of the fetches goes on)
        const bool fetch_on = !LAST || (LATE && j + 1 < tc);
        if (LATE && fetch_on) refill();
        softmax_segment(j);
        if (!LATE) wait_fetches();
        interval_end();
        if (!LATE && !LAST) refill();
        matrix_segment(vc, kn, std::integral_constant<bool, !LAST>{});
        if (LATE && fetch_on) wait_fetches();
        interval_end();
      };
      // A tile the late half fetches its share of and does not multiply: the same requests, waits and barriers.
      auto idle_tile = [&](int32_t j, unsigned char* kc, unsigned char* vn) {
        const bool fetch_on = j + 1 < tc;
        if (fetch_on) {
          fetch_k(kc, j + 2, j + 2 < tc);
          fetch_v(vn, j + 1);
        }
        interval_end();
        if (fetch_on) wait_fetches();
        interval_end();
      };
      fetch_k(kb1, 1, tc > 1);
      fetch_v(vb0, 0);
      if (LATE) interval_end();          // this half sits out the first interval
      first_segment(kb0);
      if (LATE) wait_fetches();
      interval_end();
      const int32_t mine = LATE ? tc_h : tc;   // the leading half's rows reach the workgroup's last tile
      int32_t j = 0;
      for (; j + 2 < mine; j += 2) {
        tile(j, kb0, kb1, vb0, vb1, std::false_type{});
        tile(j + 1, kb1, kb0, vb1, vb0, std::false_type{});
      }
      if (mine - j == 2) {
        tile(j, kb0, kb1, vb0, vb1, std::false_type{});
        tile(j + 1, kb1, kb0, vb1, vb0, std::true_type{});
      } else {
        tile(j, kb0, kb1, vb0, vb1, std::true_type{});
      }
      if (LATE) {
        for (j = mine; j < tc; ++j) {
          if (j & 1) idle_tile(j, kb1, vb0); else idle_tile(j, kb0, vb1);
        }
      }
      if (!LATE) interval_end();         // pairs with the late half's last interval
    };
    if (tc > 0) {
      fetch_k(kb0, 0);
      wait_fetches();
      interval_end();
      if (late)
        pipeline(std::true_type{});
      else
        pipeline(std::false_type{});
    }
    interval_end();                      // nobody reads the tile buffers any more

    // out[bh, q, d] = acc / l through LDS: this wavefront's 32 rows x D as T, 16-byte
    // chunk c of row r at chunk c ^ (r & 15); then whole rows leave as 16-byte stores.
    unsigned char* band = (wave < 2 ? kb0 : wave < 4 ? kb1 : wave < 6 ? vb0 : vb1) + (wave & 1) * (32 * D * 2);
    l_i = sum_across_halves(l_i);
    const float inv_l = 1.0f / fmaxf(l_i, 1.0e-8f);   // l = 0 only for an empty key range: the row becomes 0
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int chunk = db * 4 + qd;   // d = chunk*8 + half*4 .. +3
        u32x2 w;
        w.x = E::pack2(o_acc[db][qd * 4 + 0] * inv_l, o_acc[db][qd * 4 + 1] * inv_l);
        w.y = E::pack2(o_acc[db][qd * 4 + 2] * inv_l, o_acc[db][qd * 4 + 3] * inv_l);
        *reinterpret_cast<u32x2*>(band + l32 * (D * 2) + ((chunk ^ (l32 & 15)) << 4) + half * 8) = w;
      }
    constexpr int kLanesPerRow = D * 2 / 16, kRowsPerPass = 64 / kLanesPerRow;
    const int rd_row = lane / kLanesPerRow, rd_chunk = lane % kLanesPerRow;
#pragma unroll
    for (int pass = 0; pass < 32 / kRowsPerPass; ++pass) {
      const int r = pass * kRowsPerPass + rd_row;
      const int32_t qr = q0 + r;
      u32x4 w = *reinterpret_cast<const u32x4*>(band + r * (D * 2) + ((rd_chunk ^ (r & 15)) << 4));
      if (qr < out.shape[1] && qr < q_len)
        *reinterpret_cast<u32x4*>((T*)out.ptr + (int64_t)bh * out.strides[0] + (int64_t)qr * out.strides[1] + rd_chunk * 8) = w;
    }
  }
};

// ---- decode attention: split over the KV sequence, then merge ---------------------------------
// fmha_decode_gqa_split / splitk_reduce_merge (cutile-kernels/src/attention.rs:737-902, 917-1013).
// One new token: the GROUP query heads that share KV head h attend to keys
// 0..input_pos of that head's cache.  A workgroup takes one (KV head, split) and
// streams its share of the cache once.  This is bandwidth work (every K and V
// byte feeds only GROUP dot products), so it runs on the vector ALUs, arranged
// to spend few instructions per byte:
//  * a cache row of D halves is spread over the 16 lanes of one DPP row (D/16
//    halves each); a wavefront holds four such rows side by side ("slots") and
//    each lane works on R rows per pass, so a pass of the workgroup covers 16 R keys;
//  * q.k partial sums use the packed-half dot instruction; the R*GROUP partial
//    sums of a lane are reduced over the 16 lanes by a reduce-scatter butterfly
//    (N-1 cross-lane adds instead of 4 N).  To make the butterfly free of
//    selects every lane computes its partial sums in a lane-dependent order:
//    register j holds the sum with index j ^ p(lane), which only changes the
//    addresses of the K rows and q rows the lane loads;
//  * after the butterfly one lane owns one (row, head) score; the online
//    softmax (log2 domain, p rounded to f16 as in the tile program) runs on that
//    single value, and the probabilities return to all lanes as f16 pairs by
//    row broadcasts;
//  * p.V uses the packed-half dot again on (row 2i, row 2i+1) pairs, f32 accumulators;
//    the accumulators are rescaled only in passes where some running maximum moved.
// The partial result is normalised and stored with lse = m + log2(l), as the merge
// kernel expects; a split with no keys stores att = 0 and lse = -1e30 + log2(BN)
// (the tile program's untouched initial state).
namespace decode {
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
  return __builtin_bit_cast(float, dpp_u<CTRL>(__builtin_bit_cast(uint32_t, x)));
}
// The four pairings of the butterfly inside a row of 16 lanes: i^8, 7-i within
// each group of 8, i^2, i^1.  Pairing 1 flips bits 2, 1 and 0 of the lane number together,
// which is why the index a lane ends up owning is lane ^ (bit 2 ? 3 : 0) (see owner()).
template <int STEP>
__device__ __forceinline__ uint32_t partner_u(uint32_t x) {
  static_assert(STEP >= 0 && STEP < 4, "butterfly step");
  if constexpr (STEP == 0) return dpp_u<0x128>(x);        // row_ror:8
  else if constexpr (STEP == 1) return dpp_u<0x141>(x);   // row_half_mirror
  else if constexpr (STEP == 2) return dpp_u<0x4E>(x);    // quad_perm:[2,3,0,1]
  else return dpp_u<0xB1>(x);                             // quad_perm:[1,0,3,2]
}
template <int STEP>
__device__ __forceinline__ float partner_f(float x) {
  return __builtin_bit_cast(float, partner_u<STEP>(__builtin_bit_cast(uint32_t, x)));
}
__host__ __device__ constexpr int owner(int index4) { return index4 ^ (((index4 >> 2) & 1) * 3); }   // an involution
template <int LANE>
__device__ __forceinline__ uint32_t row_bcast_u(uint32_t x) { return dpp_u<0x150 + LANE>(x); }        // row_newbcast
template <int LANE>
__device__ __forceinline__ float row_bcast_f(float x) { return dpp_f<0x150 + LANE>(x); }

// x[0..N): reduce over the 16 lanes of the row.  While more than one value is left each step halves
// them (a lane keeps the lower half and adds its partner's upper half); then plain all-reduce steps.
template <int N, int STEP = 0>
__device__ __forceinline__ void reduce_scatter(float* x) {
  if constexpr (STEP < 4) {
    if constexpr (N > 1) {
#pragma unroll
      for (int i = 0; i < N / 2; ++i) x[i] += partner_f<STEP>(x[i + N / 2]);
      reduce_scatter<N / 2, STEP + 1>(x);
    } else {
      x[0] += partner_f<STEP>(x[0]);
      reduce_scatter<1, STEP + 1>(x);
    }
  }
}
// all-reduce over the first STEPS pairings (the lanes that own the same head but different rows)
template <int STEPS, bool MAX, int STEP = 0>
__device__ __forceinline__ float reduce_rows(float x) {
  if constexpr (STEP < STEPS) {
    const float o = partner_f<STEP>(x);
    return reduce_rows<STEPS, MAX, STEP + 1>(MAX ? fmaxf(x, o) : x + o);
  } else {
    return x;
  }
}
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
// K and V rows are read once per launch by one workgroup: streamed past the caches (nontemporal).
template <int W>
__device__ __forceinline__ void load_row(const _Float16* p, uint32_t (&dst)[W]) {
  if constexpr (W == 2) {
    const u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    dst[0] = t[0], dst[1] = t[1];
  } else {
#pragma unroll
    for (int i = 0; i < W / 4; ++i) {
      const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + i * 8));
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[i * 4 + e] = t[e];
    }
  }
}
constexpr int ilog2(int v) { return v <= 1 ? 0 : 1 + ilog2(v / 2); }
constexpr int kNontemporal = 2;     // cache-policy operand of buffer loads: the nt bit
}  // namespace decode

template <int G, int D>
__device__ __forceinline__ void decode_split(const TensorArg<3>& q, const TensorArg<3>& k, const TensorArg<3>& v,
                                             const PartitionArg<3>& att_out, const PartitionArg<2>& lse_out,
                                             float qk_scale, const uint32_t* pos_dev, int32_t bn, const TileGrid& g) {
  using namespace decode;
  constexpr int E = D / 16, W = E / 2;           // halves / dwords of a row held by one lane
  constexpr int R = G * E > 64 ? 2 : 4;          // rows per lane and pass
  constexpr int N = R * G;                       // partial sums per lane and pass
  constexpr int NF = N > 16 ? N / 16 : 1;        // scores a lane owns after the butterfly
  constexpr int LOGR = ilog2(R), LOGG = ilog2(G), LOGN = LOGR + LOGG;
  constexpr int kWaves = 4, kSlots = 4, kRowsPerWave = kSlots * R;
  static_assert(D % 32 == 0 && (G & (G - 1)) == 0 && N <= 32 && NF <= G, "decode tile");
  __shared__ float sm[kWaves][G], sl[kWaves][G];
  __shared__ __attribute__((aligned(16))) float sacc[kWaves][G][D];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int slot = lane >> 4, dl = lane & 15;
  // index bits this lane ends up owning: the top LOGN bits of owner(dl) (all four and one in-lane bit when N = 32)
  const int own = owner(dl);
  const int p = N <= 16 ? own >> (4 - (LOGN > 4 ? 4 : LOGN)) : own << 1;
  const int pr = p >> LOGG, pg = p & (G - 1);
  const int32_t head = blockIdx.x, split = blockIdx.y, splits = (int32_t)g.y;
  const int32_t max_seq = min(k.shape[1], v.shape[1]);
  const int32_t s_kv = min((int32_t)pos_dev[0] + 1, max_seq);
  const int32_t tiles = (s_kv + bn - 1) / bn, per_split = (tiles + splits - 1) / splits;
  const int32_t r0 = split * per_split * bn;
  const int32_t r1 = min(min((split + 1) * per_split, tiles) * bn, s_kv);
  const float c = qk_scale * kLog2e;

  uint32_t qh[G][W];                             // register g' holds head g' ^ pg
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
    load_row<W>((const _Float16*)q.ptr + (int64_t)head * q.strides[0] + (int64_t)(gi ^ pg) * q.strides[1] + dl * E, qh[gi]);
  float m[NF], l[NF], acc[G][E];
#pragma unroll
  for (int i = 0; i < NF; ++i) m[i] = -1.0e30f, l[i] = 0.0f;
#pragma unroll
  for (int gi = 0; gi < G; ++gi)
#pragma unroll
    for (int e = 0; e < E; ++e) acc[gi][e] = 0.0f;
  const _Float16* kb = (const _Float16*)k.ptr + (int64_t)head * k.strides[0] + dl * E;
  const _Float16* vb = (const _Float16*)v.ptr + (int64_t)head * v.strides[0] + dl * E;
  // which half of an f16 pair this lane's probability is: rows 2i (low) and 2i+1 (high)
  const uint32_t pair_sel = (pr & 1) ? 0x05040100u : 0x01000504u;

  for (int32_t base = r0 + wave * kRowsPerWave; base < r1; base += kWaves * kRowsPerWave) {   // wavefront-uniform
    uint32_t kr[R][W], vr[R][W];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      // rows past the end of the split re-read its last row: their scores are masked below, so p = 0
      const int32_t krow = min(base + (r ^ pr) * kSlots + slot, r1 - 1), vrow = min(base + r * kSlots + slot, r1 - 1);
      load_row<W>(kb + (int64_t)krow * k.strides[1], kr[r]);
      load_row<W>(vb + (int64_t)vrow * v.strides[1], vr[r]);
    }
    float x[N];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int gi = 0; gi < G; ++gi) {
        float d = 0.0f;
#pragma unroll
        for (int w = 0; w < W; ++w)
          d = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, kr[r][w]), __builtin_bit_cast(h2, qh[gi][w]), d, false);
        x[r * G + gi] = d;
      }
    reduce_scatter<N>(x);
    // this lane now owns the scores of row pr, heads pg .. pg + NF - 1
    const bool valid = base + pr * kSlots + slot < r1;
    uint32_t pair[NF];
    float alpha[NF];
    bool moved = false;
#pragma unroll
    for (int i = 0; i < NF; ++i) {
      const float sc = valid ? x[i] * c : -INFINITY;
      const float m_new = fmaxf(m[i], reduce_rows<LOGR, true>(sc));
      alpha[i] = __builtin_amdgcn_exp2f(m[i] - m_new);
      const float pv = __builtin_amdgcn_exp2f(sc - m_new);
      l[i] = l[i] * alpha[i] + reduce_rows<LOGR, false>(pv);
      moved |= m_new != m[i];
      m[i] = m_new;
      const uint32_t mine = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)pv);
      pair[i] = __builtin_amdgcn_perm(mine, partner_u<LOGR - 1>(mine), pair_sel);
    }
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
      static_for<G>([&](auto gi) {
        constexpr int t = gi.value;                                          // row 0, head gi
        constexpr int src = owner(N <= 16 ? t << (4 - (LOGN > 4 ? 4 : LOGN)) : t >> 1);
        const float a = row_bcast_f<src>(alpha[N <= 16 ? 0 : t & 1]);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[gi.value][e] *= a;
      });
    }
    static_for<R / 2>([&](auto rp) {
      uint32_t lo[W], hi[W];
#pragma unroll
      for (int w = 0; w < W; ++w) {
        lo[w] = __builtin_amdgcn_perm(vr[2 * rp.value + 1][w], vr[2 * rp.value][w], 0x05040100u);
        hi[w] = __builtin_amdgcn_perm(vr[2 * rp.value + 1][w], vr[2 * rp.value][w], 0x07060302u);
      }
      static_for<G>([&](auto gi) {
        constexpr int t = 2 * rp.value * G + gi.value;                       // row 2 rp, head gi
        constexpr int src = owner(N <= 16 ? t << (4 - (LOGN > 4 ? 4 : LOGN)) : t >> 1);
        const h2 pp = __builtin_bit_cast(h2, row_bcast_u<src>(pair[N <= 16 ? 0 : t & 1]));
#pragma unroll
        for (int w = 0; w < W; ++w) {
          acc[gi.value][2 * w] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, lo[w]), pp, acc[gi.value][2 * w], false);
          acc[gi.value][2 * w + 1] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, hi[w]), pp, acc[gi.value][2 * w + 1], false);
        }
      });
    });
  }
  // running maximum and sum of every head, back in all lanes of the slot
  float mg[G], lg[G];
  static_for<G>([&](auto gi) {
    constexpr int t = gi.value;
    constexpr int src = owner(N <= 16 ? t << (4 - (LOGN > 4 ? 4 : LOGN)) : t >> 1);
    mg[gi.value] = row_bcast_f<src>(m[N <= 16 ? 0 : t & 1]);
    lg[gi.value] = row_bcast_f<src>(l[N <= 16 ? 0 : t & 1]);
  });
  // merge the four slots of this wavefront ...
#pragma unroll
  for (int o = 16; o < 64; o <<= 1) {
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
      const float mo = __shfl_xor(mg[gi], o, 64), lo = __shfl_xor(lg[gi], o, 64);
      const float m_new = fmaxf(mg[gi], mo);
      const float fs = __builtin_amdgcn_exp2f(mg[gi] - m_new), fo = __builtin_amdgcn_exp2f(mo - m_new);
      lg[gi] = lg[gi] * fs + lo * fo;
#pragma unroll
      for (int e = 0; e < E; ++e) acc[gi][e] = acc[gi][e] * fs + __shfl_xor(acc[gi][e], o, 64) * fo;
      mg[gi] = m_new;
    }
  }
  // ... and the wavefronts through LDS
  if (slot == 0) {
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
      if (dl == 0) {
        sm[wave][gi] = mg[gi];
        sl[wave][gi] = lg[gi];
      }
#pragma unroll
      for (int e = 0; e < E; ++e) sacc[wave][gi][dl * E + e] = acc[gi][e];
    }
  }
  __syncthreads();
  if (wave == 0 && slot == 0) {
    _Float16* ab = (_Float16*)att_out.ptr + (int64_t)head * att_out.strides[0] + dl * E;
    float* lb = (float*)lse_out.ptr + (int64_t)head * lse_out.strides[0];
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
      float mt = sm[0][gi];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) mt = fmaxf(mt, sm[w][gi]);
      float lt = 0.0f, at[E] = {};
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        const float f = __builtin_amdgcn_exp2f(sm[w][gi] - mt);
        lt += sl[w][gi] * f;
#pragma unroll
        for (int e = 0; e < E; ++e) at[e] += sacc[w][gi][dl * E + e] * f;
      }
      if (r0 >= r1) lt = (float)bn;   // no keys in this split: the tile program's untouched l = 1 per lane
      const float safe = fmaxf(lt, 1.0e-8f);
      const int64_t orow = (int64_t)split * G + gi;
      _Float16* dst = ab + orow * att_out.strides[1];
#pragma unroll
      for (int e = 0; e < E; e += 4) {
        f16x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = (_Float16)(at[e + j] / safe);
        *reinterpret_cast<f16x4*>(dst + e) = o;
      }
      if (dl == 0) lb[orow * lse_out.strides[1]] = mt + __builtin_log2f(safe);
    }
  }
}

// ---- decode attention on the matrix cores ----------------------------------------------------
// With GROUP >= 4 the vector ALUs no longer keep up with HBM (two dot products per cached value
// and head), and at D = 64 they do not for any group.  Here a wavefront takes 32 keys at a time and uses v_mfma_f32_16x16x32_f16 with
// the query heads as the 16-wide N dimension (heads beyond GROUP are zero):
//   S^T [16 keys x 16 heads]  = K [16 keys x D]   . Q^T [D x 16 heads]     (two blocks of 16 keys)
//   O^T [D x 16 heads]       += V^T [D x 32 keys]  . P^T [32 keys x 16 heads]
// so that every lane owns ONE head (column) in both products: running maximum, sum and the
// rescale factor are per-lane scalars, and the f32 scores a lane holds after the first product
// (4 keys of each block) ARE, converted to f16, its 8 values of the second product's B operand —
// the 32 keys of the slab are simply taken in the order in which the lanes already hold them.
// K rows are MFMA A operands straight from global memory (a lane loads 16 bytes of one key).
// V must be read transposed (8 keys of one column per lane): each wavefront streams its V rows
// into a private LDS stage with 16-byte direct loads (chunk c of row r at chunk c ^ 2(r & 3),
// so the transposing reads of 4 rows x 2 chunks are conflict-free) and reads them back with
// ds_read_b64_tr_b16.  Two stages, one 32-key slab ahead; wavefront-private, so the loop has no
// barrier.  Slabs past the end of the split re-read its last row and are masked (p = 0).
// What one workgroup works on: the queries of one KV head, keys [r0, r1) of its cache, and where the partial
// result of query head c goes (att + c * att_row_stride, lse + c * lse_row_stride).
struct DecodeSplitView {
  const _Float16* q;
  const _Float16* k;
  const _Float16* v;
  _Float16* att;
  float* lse;
  int64_t q_row_stride, k_row_stride, v_row_stride, att_row_stride, lse_row_stride;
  int32_t v_rows;      // rows of v that exist (extent of its buffer descriptor)
  int32_t r0, r1;
  float empty_sum;     // what a split without keys reports: its sum (the output is 0 / sum) and its lse
  float empty_lse;
};

template <int G, int D>
__device__ __forceinline__ void decode_split_mfma_view(const DecodeSplitView& w, float qk_scale) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  constexpr int kWaves = 4, kSlab = 32;
  constexpr int QS = D / 32;                 // K slices of the first product
  constexpr int OS = D / 16;                 // 16-row slices of O^T
  constexpr int CP = D / 8;                  // 16-byte chunks per V row
  constexpr int kRowsPerInstr = 64 / CP;     // V rows one direct load covers
  constexpr int kVInstr = kSlab / kRowsPerInstr;
  constexpr int kStageBytes = kSlab * D * 2;
  static_assert(G <= 16 && D % 32 == 0 && CP <= 64 && 64 % CP == 0, "decode tile");
  __shared__ __attribute__((aligned(1024))) unsigned char vst[kWaves][2][kStageBytes];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, quad = lane >> 4;           // head (column) and key group of this lane
  const int32_t r0 = w.r0, r1 = w.r1;
  const float c = qk_scale * kLog2e;

  // Q^T operands: column = head, 8 consecutive d per lane and slice
  f16x8 qf[QS];
#pragma unroll
  for (int sidx = 0; sidx < QS; ++sidx) {
    f16x8 t = {};
    if (col < G) t = *reinterpret_cast<const f16x8*>(w.q + (int64_t)col * w.q_row_stride + sidx * 32 + quad * 8);
    qf[sidx] = t;
  }
  const _Float16* kb = w.k;
  const int64_t k_row_stride = w.k_row_stride, v_row_stride = w.v_row_stride;
  const __amdgpu_buffer_rsrc_t rv = make_rsrc(w.v, (uint32_t)(((int64_t)(w.v_rows - 1) * v_row_stride + D) * 2));
  unsigned char* my_stage[2] = {vst[wave][0], vst[wave][1]};

  // LDS side of the transposing reads: lane i of a 16-lane group supplies row (i >> 2), columns 4 (i & 3) .. + 3
  int tr_off[2];
  {
    const int i16 = lane & 15;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const int row = blk * 16 + quad * 4 + (i16 >> 2);
      const int cc = (i16 & 3) * 4;                    // column inside the 16-column slice
      tr_off[blk] = row * (D * 2) + ((((cc >> 3)) ^ ((row & 3) << 1)) << 4) + (cc & 7) * 2;
    }
  }
  auto request_slab = [&](int32_t base, f16x8 (&kreg)[2][QS], unsigned char* stage) {
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const int32_t row = min(base + blk * 16 + col, r1 - 1);
#pragma unroll
      for (int sidx = 0; sidx < QS; ++sidx)
        kreg[blk][sidx] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(kb + (int64_t)row * k_row_stride + sidx * 32 + quad * 8));
    }
#pragma unroll
    for (int i = 0; i < kVInstr; ++i) {
      const int lrow = i * kRowsPerInstr + lane / CP;
      const int chunk = (lane % CP) ^ ((lrow & 3) << 1);
      const int32_t row = min(base + lrow, r1 - 1);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (LDS_PTR(void))(stage + i * 1024), 16,
                                               (uint32_t)(((int64_t)row * v_row_stride + chunk * 8) * 2), 0, 0, decode::kNontemporal);
    }
  };

  float m = -1.0e30f, l = 0.0f;
  f32x4 oacc[OS];
#pragma unroll
  for (int i = 0; i < OS; ++i) oacc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  auto slab = [&](int32_t base, const f16x8 (&kreg)[2][QS], const unsigned char* stage) {
    f32x4 sc[2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      sc[blk] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int sidx = 0; sidx < QS; ++sidx) sc[blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[blk][sidx], qf[sidx], sc[blk], 0, 0, 0);
    }
    // this lane: head `col`, keys base + 16 blk + 4 quad + i
    float sv[8], mx = -INFINITY;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool valid = base + blk * 16 + quad * 4 + i < r1;
        sv[blk * 4 + i] = valid ? sc[blk][i] * c : -INFINITY;
        mx = fmaxf(mx, sv[blk * 4 + i]);
      }
    mx = max_across_rows(mx);
    const float m_new = fmaxf(m, mx);
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    float rs = 0.0f;
    f16x8 pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pv = __builtin_amdgcn_exp2f(sv[e] - m_new);
      rs += pv;
      pf[e] = (_Float16)pv;
    }
    rs = sum_across_rows(rs);
    l = l * alpha + rs;
    if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {
#pragma unroll
      for (int i = 0; i < OS; ++i) oacc[i] *= alpha;
    }
    m = m_new;
    // this slab's V rows (requested one slab ago) have landed once at most the 2 QS + kVInstr loads
    // of the slab requested after them are outstanding
    __builtin_amdgcn_s_waitcnt(0x0f70 | ((2 * QS + kVInstr) & 15) | ((((2 * QS + kVInstr) >> 4) & 3) << 14));
#pragma unroll
    for (int i = 0; i < OS; ++i) {
      // slice i lies 2 i chunks further; chunk numbers are XOR-swizzled, so the offset is an XOR too
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(stage + (tr_off[0] ^ (i << 5))));
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(stage + (tr_off[1] ^ (i << 5))));
      const f16x8 vt = __builtin_bit_cast(f16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      oacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vt, pf, oacc[i], 0, 0, 0);
    }
  };

  f16x8 ka[2][QS], kbuf[2][QS];
  const int32_t first = r0 + wave * kSlab, stride = kWaves * kSlab;
  if (first < r1) {
    request_slab(first, ka, my_stage[0]);
    for (int32_t base = first; base < r1; base += 2 * stride) {      // wavefront-uniform; slabs past r1 are masked
      request_slab(base + stride, kbuf, my_stage[1]);
      slab(base, ka, my_stage[0]);
      request_slab(base + 2 * stride, ka, my_stage[0]);
      slab(base + stride, kbuf, my_stage[1]);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();     // every wavefront is done with its stages: they now carry the partial results

  float* sm = reinterpret_cast<float*>(&vst[0][0][0]);            // [kWaves][16]
  float* sl = sm + kWaves * 16;                                   // [kWaves][16]
  float* sacc = sl + kWaves * 16;                                 // [kWaves][G][D]
  static_assert((2 * kWaves * 16 + kWaves * G * D) * 4 <= kWaves * 2 * kStageBytes, "partials fit the stages");
  if (col < G) {
    if (quad == 0) {
      sm[wave * 16 + col] = m;
      sl[wave * 16 + col] = l;
    }
#pragma unroll
    for (int i = 0; i < OS; ++i)
      *reinterpret_cast<f32x4*>(sacc + ((wave * G + col) * D + i * 16 + quad * 4)) = oacc[i];
  }
  __syncthreads();
  if (wave == 0 && col < G) {
    float mt = sm[col];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mt = fmaxf(mt, sm[w * 16 + col]);
    float lt = 0.0f, f[kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      f[w] = __builtin_amdgcn_exp2f(sm[w * 16 + col] - mt);
      lt += sl[w * 16 + col] * f[w];
    }
    if (r0 >= r1) lt = w.empty_sum;   // no keys in this split: the tile program's untouched l = 1 per lane
    const float safe = fmaxf(lt, 1.0e-8f);
    _Float16* dst = w.att + (int64_t)col * w.att_row_stride;
#pragma unroll
    for (int i = 0; i < OS; ++i) {
      f32x4 a = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int w = 0; w < kWaves; ++w) a += *reinterpret_cast<const f32x4*>(sacc + ((w * G + col) * D + i * 16 + quad * 4)) * f[w];
      f16x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (_Float16)(a[j] / safe);
      *reinterpret_cast<f16x4*>(dst + i * 16 + quad * 4) = o;
    }
    if (quad == 0) w.lse[(int64_t)col * w.lse_row_stride] = r0 >= r1 ? w.empty_lse : mt + __builtin_log2f(safe);
  }
}

// fmha_decode_gqa_split: q [kv_heads, GROUP, D], k and v [kv_heads, max_seq, D], partial results at row
// split * GROUP + c of att_out [kv_heads, splits * GROUP, D] and lse_out [kv_heads, splits * GROUP]; the tiles of
// `bn` keys are dealt to the splits in equal runs.
template <int G, int D>
__device__ __forceinline__ void decode_split_mfma(const TensorArg<3>& q, const TensorArg<3>& k, const TensorArg<3>& v,
                                                  const PartitionArg<3>& att_out, const PartitionArg<2>& lse_out,
                                                  float qk_scale, const uint32_t* pos_dev, int32_t bn, const TileGrid& g) {
  const int32_t head = blockIdx.x, split = blockIdx.y, splits = (int32_t)g.y;
  const int32_t max_seq = min(k.shape[1], v.shape[1]);
  const int32_t s_kv = min((int32_t)pos_dev[0] + 1, max_seq);
  const int32_t tiles = (s_kv + bn - 1) / bn, per_split = (tiles + splits - 1) / splits;
  DecodeSplitView w;
  w.r0 = split * per_split * bn;
  w.r1 = min(min((split + 1) * per_split, tiles) * bn, s_kv);
  w.q = (const _Float16*)q.ptr + (int64_t)head * q.strides[0];
  w.k = (const _Float16*)k.ptr + (int64_t)head * k.strides[0];
  w.v = (const _Float16*)v.ptr + (int64_t)head * v.strides[0];
  w.q_row_stride = q.strides[1], w.k_row_stride = k.strides[1], w.v_row_stride = v.strides[1];
  w.v_rows = max_seq;
  const int64_t orow = (int64_t)split * G;
  w.att = (_Float16*)att_out.ptr + (int64_t)head * att_out.strides[0] + orow * att_out.strides[1];
  w.lse = (float*)lse_out.ptr + (int64_t)head * lse_out.strides[0] + orow * lse_out.strides[1];
  w.att_row_stride = att_out.strides[1], w.lse_row_stride = lse_out.strides[1];
  w.empty_sum = (float)bn;
  w.empty_lse = -1.0e30f + __builtin_log2f((float)bn);
  decode_split_mfma_view<G, D>(w, qk_scale);
}

// attention_decode_kernel_grouped (cutile-kernels/src/experimental/attention.rs:385-846): the same partial attention in
// batched layouts.  q [B, kv_heads, GROUP, D]; k, v [B, kv_heads, S, D]; att [B, kv_heads, GROUP, splits, D];
// lse [B, kv_heads, GROUP, splits]; innermost strides 1, the others given in elements.  Split t takes keys
// [t * kv_len_per_split, min((t + 1) * kv_len_per_split, *s_kv)) (attention.rs:629-633, with kv_len_per_split a
// multiple of the key tile); a split without keys writes zeros and lse = -inf (attention.rs:775-780, 806-807).
// Workgroup (batch, kv head, split) as in the reference's grid (attention.rs:597-601).
struct GroupedDecodeArgs {
  const void* q;
  const void* k;
  const void* v;
  void* att;
  void* lse;
  const int32_t* s_kv;
  int32_t q_strides[3], k_strides[3], v_strides[3], att_strides[4], lse_strides[3];
  int32_t k_rows, v_rows, kv_len_per_split;
  float softmax_scale;
};

template <int G, int D>
__device__ __forceinline__ void decode_grouped(const GroupedDecodeArgs& a, const TileGrid& g) {
  const int32_t batch = blockIdx.x, head = blockIdx.y, split = blockIdx.z;
  if (batch >= (int32_t)g.x || head >= (int32_t)g.y || split >= (int32_t)g.z) return;
  const int32_t s_kv = min(a.s_kv[0], min(a.k_rows, a.v_rows));
  DecodeSplitView w;
  w.r0 = split * a.kv_len_per_split;
  w.r1 = min(w.r0 + a.kv_len_per_split, s_kv);
  w.q = (const _Float16*)a.q + (int64_t)batch * a.q_strides[0] + (int64_t)head * a.q_strides[1];
  w.k = (const _Float16*)a.k + (int64_t)batch * a.k_strides[0] + (int64_t)head * a.k_strides[1];
  w.v = (const _Float16*)a.v + (int64_t)batch * a.v_strides[0] + (int64_t)head * a.v_strides[1];
  w.q_row_stride = a.q_strides[2], w.k_row_stride = a.k_strides[2], w.v_row_stride = a.v_strides[2];
  w.v_rows = a.v_rows;
  w.att = (_Float16*)a.att + (int64_t)batch * a.att_strides[0] + (int64_t)head * a.att_strides[1] + (int64_t)split * a.att_strides[3];
  w.lse = (float*)a.lse + (int64_t)batch * a.lse_strides[0] + (int64_t)head * a.lse_strides[1] + split;
  w.att_row_stride = a.att_strides[2], w.lse_row_stride = a.lse_strides[2];
  w.empty_sum = 1.0f;
  w.empty_lse = -INFINITY;
  decode_split_mfma_view<G, D>(w, a.softmax_scale);
}

// out[h, g, :] = sum_s w[g, s] att[h, s*GROUP + g, :], w = exp2(lse - max_s lse) / max(sum, 1e-8).
// One workgroup per (KV head, query head of the group).  The weights come from two
// workgroup-wide reductions over the splits; then the rows of the partial results are
// streamed 256 / lanes-per-row at a time (16 bytes per lane when the layout allows it)
// and the row groups are summed through LDS.
__device__ __forceinline__ float block_reduce(float x, bool take_max, float* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float y = __shfl_xor(x, o, 64);
    x = take_max ? fmaxf(x, y) : x + y;
  }
  __syncthreads();                       // scratch may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = x;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < (int)(blockDim.x >> 6); ++w) r = take_max ? fmaxf(r, scratch[w]) : r + scratch[w];
  return r;
}

__device__ __forceinline__ void splitk_merge(const TensorArg<3>& att, const TensorArg<2>& lse, const PartitionArg<3>& out) {
  constexpr int kThreads = 256;
  __shared__ float red[4];
  __shared__ __attribute__((aligned(16))) float part[kThreads * 8];
  const int32_t group = out.shape[1], d = out.shape[2];
  const int32_t head = blockIdx.x / group, gi = blockIdx.x % group;
  const int32_t splits = att.shape[1] / group;
  const int tid = threadIdx.x;
  const _Float16* ab = (const _Float16*)att.ptr + (int64_t)head * att.strides[0] + (int64_t)gi * att.strides[1];
  const float* lb = (const float*)lse.ptr + (int64_t)head * lse.strides[0] + (int64_t)gi * lse.strides[1];
  _Float16* ob = (_Float16*)out.ptr + (int64_t)head * out.strides[0] + (int64_t)gi * out.strides[1];
  const int64_t att_step = (int64_t)group * att.strides[1], lse_step = (int64_t)group * lse.strides[1];

  float mx = -INFINITY;
  for (int32_t sidx = tid; sidx < splits; sidx += kThreads) mx = fmaxf(mx, lb[sidx * lse_step]);
  mx = block_reduce(mx, true, red);
  float sum = 0.0f;
  for (int32_t sidx = tid; sidx < splits; sidx += kThreads) sum += __builtin_amdgcn_exp2f(lb[sidx * lse_step] - mx);
  sum = block_reduce(sum, false, red);
  const float inv = 1.0f / fmaxf(sum, 1.0e-8f);

  const bool vec = d % 8 == 0 && att.strides[2] == 1 && out.strides[2] == 1 && att.strides[1] % 8 == 0 && att.strides[0] % 8 == 0 &&
                   out.strides[1] % 8 == 0 && out.strides[0] % 8 == 0 && ((uintptr_t)att.ptr & 15) == 0 && ((uintptr_t)out.ptr & 15) == 0;
  const int epl = vec ? 8 : 1;                               // elements per lane
  const int32_t chunks = d / epl;
  int lpr = 1;
  while (lpr < chunks && lpr < kThreads) lpr <<= 1;          // lanes per row (a power of two)
  const int rows_par = kThreads / lpr, my_row = tid / lpr, my_c = tid % lpr;
  for (int32_t c0 = 0; c0 < chunks; c0 += lpr) {             // one trip unless D > 2048 (256 without 16-byte accesses)
    const int32_t cidx = c0 + my_c;
    float a[8] = {};
    if (cidx < chunks) {
      for (int32_t sidx = my_row; sidx < splits; sidx += rows_par) {
        const float w = __builtin_amdgcn_exp2f(lb[sidx * lse_step] - mx) * inv;
        const _Float16* src = ab + sidx * att_step;
        if (vec) {
          const f16x8 t = *reinterpret_cast<const f16x8*>(src + cidx * 8);
#pragma unroll
          for (int e = 0; e < 8; ++e) a[e] = __builtin_fmaf((float)t[e], w, a[e]);
        } else {
          a[0] = __builtin_fmaf((float)src[(int64_t)cidx * att.strides[2]], w, a[0]);
        }
      }
    }
    __syncthreads();                                         // part[] of the previous trip has been consumed
#pragma unroll
    for (int e = 0; e < 8; ++e) part[(my_row * lpr + my_c) * 8 + e] = a[e];
    __syncthreads();
    if (my_row == 0 && cidx < chunks) {
      for (int r = 1; r < rows_par; ++r)
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] += part[(r * lpr + my_c) * 8 + e];
      if (vec) {
        f16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (_Float16)a[e];
        *reinterpret_cast<f16x8*>(ob + cidx * 8) = o;
      } else {
        ob[(int64_t)cidx * out.strides[2]] = (_Float16)a[0];
      }
    }
  }
}

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
FMHA_KERNEL(bf16, __bf16, 128, 32, 256)
FMHA_KERNEL(f16, _Float16, 128, 32, 256)

// The sequence-layout attention kernels of cutile-kernels whose position lives in device memory
// (flash_attn_causal_seq_dynpos_f16 attention.rs:128-231, fmha_causal :598-726): q and out
// [q_len, q_heads, D], k and v [kv_heads, max_seq, D], handed over as permuted views of the layout
// above.  query_start = *position_start; with `kv_len_from_position` only keys 0 .. position are read
// (the dynpos form), otherwise every key of the view.
#define FMHA_SEQ_KERNEL(NAME, T, BM, BN, D)                                                       \
  extern "C" __global__ void __launch_bounds__((BM / 32) * 64)                                   \
      fmha_seq_entry__##NAME##_##BM##x##BN##x##D(PartitionArg<3> out, TensorArg<4> q, TensorArg<4> k, \
                                                 TensorArg<4> v, float qk_scale,                  \
                                                 const uint32_t* position_start,                  \
                                                 int32_t kv_len_from_position,                    \
                                                 int32_t query_group_size, int32_t causal, TileGrid g) { \
    const int32_t pos = (int32_t)min(position_start[0], 0x3fffffffu);                             \
    TensorArg<4> kk = k, vv = v;                                                                  \
    if (kv_len_from_position) kk.shape[2] = vv.shape[2] = min(min(k.shape[2], v.shape[2]), pos + 1); \
    Fmha<T, BM, BN, D>::run(out, q, kk, vv, qk_scale, pos, query_group_size, causal, g);         \
  }
FMHA_SEQ_KERNEL(f16, _Float16, 128, 64, 128)
FMHA_SEQ_KERNEL(f16, _Float16, 128, 64, 64)
FMHA_SEQ_KERNEL(f16, _Float16, 32, 32, 32)
FMHA_SEQ_KERNEL(f16, _Float16, 128, 32, 256)

#define FMHA_PINGPONG_KERNEL(NAME, T, BN, D)                                                       \
  extern "C" __global__ void __launch_bounds__(512)                                               \
      fmha_entry__##NAME##_256x##BN##x##D##_pp(PartitionArg<3> out, TensorArg<4> q, TensorArg<4> k, \
                                               TensorArg<4> v, float qk_scale, int32_t input_pos,  \
                                               int32_t query_group_size, int32_t causal, TileGrid g) { \
    FmhaPingPong<T, BN, D>::run(out, q, k, v, qk_scale, input_pos, query_group_size, causal, g);  \
  }

FMHA_PINGPONG_KERNEL(bf16, __bf16, 64, 128)
FMHA_PINGPONG_KERNEL(f16, _Float16, 64, 128)

// fmha_decode_gqa_split<GROUP, BN, D, NUM_KV_SPLITS>(q, k, v, att_out: [1,GROUP,D] tiles, lse_out: [1,GROUP] tiles,
//                                                   qk_scale, position_start); grid (kv_heads, NUM_KV_SPLITS)
#define DECODE_SPLIT_KERNEL(G, D)                                                                  \
  extern "C" __global__ void __launch_bounds__(256)                                               \
      fmha_decode_gqa_split_entry__f16_g##G##_d##D(TensorArg<3> q, TensorArg<3> k, TensorArg<3> v, \
                                                   PartitionArg<3> att_out, PartitionArg<2> lse_out, \
                                                   float qk_scale, const uint32_t* position_start, \
                                                   int32_t bn, TileGrid g) {                       \
    decode_split<G, D>(q, k, v, att_out, lse_out, qk_scale, position_start, bn, g);               \
  }
#define DECODE_SPLIT_GROUPS(D) DECODE_SPLIT_KERNEL(1, D) DECODE_SPLIT_KERNEL(2, D) DECODE_SPLIT_KERNEL(4, D) DECODE_SPLIT_KERNEL(8, D)
DECODE_SPLIT_GROUPS(64)
DECODE_SPLIT_GROUPS(128)
DECODE_SPLIT_GROUPS(256)

#define DECODE_SPLIT_MFMA_KERNEL(G, D)                                                             \
  extern "C" __global__ void __launch_bounds__(256)                                               \
      fmha_decode_gqa_split_entry__f16_g##G##_d##D##_mfma(TensorArg<3> q, TensorArg<3> k, TensorArg<3> v, \
                                                          PartitionArg<3> att_out, PartitionArg<2> lse_out, \
                                                          float qk_scale, const uint32_t* position_start, \
                                                          int32_t bn, TileGrid g) {                \
    decode_split_mfma<G, D>(q, k, v, att_out, lse_out, qk_scale, position_start, bn, g);          \
  }
DECODE_SPLIT_MFMA_KERNEL(1, 64)
DECODE_SPLIT_MFMA_KERNEL(1, 128)
DECODE_SPLIT_MFMA_KERNEL(1, 256)
DECODE_SPLIT_MFMA_KERNEL(2, 64)
DECODE_SPLIT_MFMA_KERNEL(2, 128)
DECODE_SPLIT_MFMA_KERNEL(2, 256)
DECODE_SPLIT_MFMA_KERNEL(4, 64)
DECODE_SPLIT_MFMA_KERNEL(4, 128)
DECODE_SPLIT_MFMA_KERNEL(4, 256)
DECODE_SPLIT_MFMA_KERNEL(8, 64)
DECODE_SPLIT_MFMA_KERNEL(8, 128)
DECODE_SPLIT_MFMA_KERNEL(8, 256)
DECODE_SPLIT_MFMA_KERNEL(16, 64)
DECODE_SPLIT_MFMA_KERNEL(16, 128)
DECODE_SPLIT_MFMA_KERNEL(16, 256)

#define DECODE_GROUPED_KERNEL(G, D)                                                                \
  extern "C" __global__ void __launch_bounds__(256)                                               \
      attention_decode_grouped_entry__f16_g##G##_d##D(GroupedDecodeArgs a, TileGrid g) {           \
    decode_grouped<G, D>(a, g);                                                                   \
  }
#define DECODE_GROUPED_GROUPS(D) \
  DECODE_GROUPED_KERNEL(1, D) DECODE_GROUPED_KERNEL(2, D) DECODE_GROUPED_KERNEL(4, D) DECODE_GROUPED_KERNEL(8, D) DECODE_GROUPED_KERNEL(16, D)
DECODE_GROUPED_GROUPS(64)
DECODE_GROUPED_GROUPS(128)
DECODE_GROUPED_GROUPS(256)

// splitk_reduce_merge<GROUP, D, CHUNK_D, NUM_KV_SPLITS, ..>(att_partial, lse_partial, out: [1,GROUP,CHUNK_D] tiles)
extern "C" __global__ void __launch_bounds__(256)
    splitk_reduce_merge_entry__f16(TensorArg<3> att_partial, TensorArg<2> lse_partial, PartitionArg<3> out, TileGrid g) {
  splitk_merge(att_partial, lse_partial, out);
}
