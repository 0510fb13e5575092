// MX block-scaled fp8 GEMM for gfx950:
//   z[M,N] = alpha * sum_k (x[i,k] * sx[i,k/32]) * (y[j,k] * sy[j,k/32])
// x [M,K] and y [N,K] are fp8 e4m3fn bytes (both K-contiguous), sx [M,K/32] and
// sy [N,K/32] are e8m0 scale bytes (2^(b-127)), accumulation is f32.
//
// Tile program being implemented (cutile-examples/examples/mxfp8.rs:34-64): per
// [BM,BN] output tile, for each K tile: tile_z = mmaf_scaled(x, yᵀ, tile_z, sx, syᵀ);
// then z.store(tile_z * alpha).  The op contract is cutile/src/_core.rs:2283-2311.
//
// Mapping to CDNA4: v_mfma_scale_f32_32x32x64_f8f6f4 multiplies a 32x64 by a
// 64x32 fp8 block and scales each 32-wide K block of every row by an e8m0 byte,
// so the scales never touch the data path: no dequantisation, no extra
// multiplies.  Operand layout (measured on gfx950): a lane (row r = lane%32,
// half h = lane/32) holds 32 bytes; its first 16 belong to the instruction's K
// block 0 (bytes 16h..16h+15 of it) and its last 16 to K block 1; lanes with
// h = 0 supply the scale of block 0 for their row and lanes with h = 1 the scale
// of block 1, as byte 0 of the scale VGPR.  The
// four scale bytes a row needs for a 128-wide K tile are fetched as one aligned
// dword straight from global memory (they are 1/32 of the data) and shifted so
// that the lane's own block sits in the byte the instruction reads.
// Data tiles go through LDS exactly like the bf16 GEMM's x tile (both operands
// are K-contiguous here, so there is no transpose at all): double buffered,
// XOR-swizzled 16-byte units, one barrier per K tile, buffer-descriptor loads
// for branch-free zero padding, transposed MFMA issue for 4-column-per-lane
// stores, XCD-aware grouped tile order.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gemm_common.h"
#include "kernel_args.h"

using namespace cutile;
using namespace cutile::gemm;

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));

template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT>
struct MxGemm {
  static constexpr int BK = 128;  // fp8 elements (= bytes) per K tile: four MX blocks
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int kUnitsPerRow = BK / 16;
  static constexpr int kALoads = BM * kUnitsPerRow / kThreads;
  static constexpr int kBLoads = BN * kUnitsPerRow / kThreads;
  static constexpr int kABytes = BM * BK, kBBytes = BN * BK;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert((BM * kUnitsPerRow) % kThreads == 0 && (BN * kUnitsPerRow) % kThreads == 0, "split");

  __device__ static __forceinline__ int lds_off(int r, int u) {
    return r * BK + ((u ^ ((r >> 1) & 7)) << 4);
  }

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             const TensorArg<2>& xs, const TensorArg<2>& ys, float alpha,
                             const TileGrid& g) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, khalf = lane >> 5;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[0], K = min(x.shape[1], y.shape[1]);
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t ldsa = xs.strides[0], ldsb = ys.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;

    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)((int64_t)(M - 1) * lda + x.shape[1]));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)((int64_t)(N - 1) * ldb + y.shape[1]));
    const __amdgpu_buffer_rsrc_t rsa = make_rsrc(xs.ptr, (uint32_t)((int64_t)(xs.shape[0] - 1) * ldsa + xs.shape[1]));
    const __amdgpu_buffer_rsrc_t rsb = make_rsrc(ys.ptr, (uint32_t)((int64_t)(ys.shape[0] - 1) * ldsb + ys.shape[1]));
    constexpr uint32_t kOob = 0x80000000u;

    int a_row[kALoads], a_unit[kALoads], b_row[kBLoads], b_unit[kBLoads];
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      int c = tid + i * kThreads;
      a_row[i] = c / kUnitsPerRow;
      a_unit[i] = c % kUnitsPerRow;
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      int c = tid + i * kThreads;
      b_row[i] = c / kUnitsPerRow;
      b_unit[i] = c % kUnitsPerRow;
    }
    u32x4 a_reg[kALoads], b_reg[kBLoads];
    uint32_t sa_reg[TM], sb_reg[TN];  // one dword = the 4 scale bytes of this lane's row for a K tile
    auto load_global = [&](int32_t k0) {
#pragma unroll
      for (int i = 0; i < kALoads; ++i) {
        int32_t r = row0 + a_row[i], kk = k0 + a_unit[i] * 16;
        uint32_t off = (r < M && kk < K) ? (uint32_t)((int64_t)r * lda + kk) : kOob;
        a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, off, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) {
        int32_t r = col0 + b_row[i], kk = k0 + b_unit[i] * 16;
        uint32_t off = (r < N && kk < K) ? (uint32_t)((int64_t)r * ldb + kk) : kOob;
        b_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, off, 0, 0);
      }
    };
    auto load_scales = [&](int32_t k0) {
      // Rows beyond the tensor read scale byte 0 (2^-127) against all-zero data: contributes 0.
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        int32_t r = row0 + wm * WM + tm * 32 + l32;
        uint32_t off = r < M ? (uint32_t)((int64_t)r * ldsa + k0 / 32) : kOob;
        sa_reg[tm] = __builtin_amdgcn_raw_buffer_load_b32(rsa, off, 0, 0);
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        int32_t r = col0 + wn * WN + tn * 32 + l32;
        uint32_t off = r < N ? (uint32_t)((int64_t)r * ldsb + k0 / 32) : kOob;
        sb_reg[tn] = __builtin_amdgcn_raw_buffer_load_b32(rsb, off, 0, 0);
      }
    };
    auto store_lds = [&](int stage) {
      unsigned char* sa = lds + stage * kStageBytes;
      unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int i = 0; i < kALoads; ++i) *reinterpret_cast<u32x4*>(sa + lds_off(a_row[i], a_unit[i])) = a_reg[i];
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) *reinterpret_cast<u32x4*>(sb + lds_off(b_row[i], b_unit[i])) = b_reg[i];
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

    const int k_tiles = K / BK;
    uint32_t sa_cur[TM], sb_cur[TN];
    if (k_tiles > 0) {
      load_global(0);
      load_scales(0);
      store_lds(0);
    }
    __syncthreads();

    for (int kt = 0; kt < k_tiles; ++kt) {
      const int cur = kt & 1;
      // This lane's four scale bytes for the current K tile (MX blocks 4kt..4kt+3).
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) sa_cur[tm] = sa_reg[tm];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) sb_cur[tn] = sb_reg[tn];
      if (kt + 1 < k_tiles) {
        load_global((kt + 1) * BK);
        load_scales((kt + 1) * BK);
      }
      const unsigned char* sa = lds + cur * kStageBytes;
      const unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        i32x8 af[TM], bfr[TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          int r = wm * WM + tm * 32 + l32;
          u32x4 lo = *reinterpret_cast<const u32x4*>(sa + lds_off(r, ks * 4 + khalf));
          u32x4 hi = *reinterpret_cast<const u32x4*>(sa + lds_off(r, ks * 4 + 2 + khalf));
          af[tm] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          int r = wn * WN + tn * 32 + l32;
          u32x4 lo = *reinterpret_cast<const u32x4*>(sb + lds_off(r, ks * 4 + khalf));
          u32x4 hi = *reinterpret_cast<const u32x4*>(sb + lds_off(r, ks * 4 + 2 + khalf));
          bfr[tn] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) {
            // MFMA step ks covers MX blocks 2ks and 2ks+1 of the K tile; lanes 0-31 supply
            // the scale of the first, lanes 32-63 of the second, moved to byte 0.
            acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                bfr[tn], af[tm], acc[tn][tm], 0, 0, 0, (int)(sb_cur[tn] >> (8 * (2 * ks + khalf))), 0,
                (int)(sa_cur[tm] >> (8 * (2 * ks + khalf))));
          }
      }
      if (kt + 1 < k_tiles) store_lds(cur ^ 1);
      __syncthreads();
    }

    OutT* zp = (OutT*)z.ptr;
    const int32_t ldz = z.strides[0];
    const int32_t zM = z.shape[0], zN = z.shape[1];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int32_t r = row0 + wm * WM + tm * 32 + l32;
      if (r >= zM) continue;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int32_t c = col0 + wn * WN + tn * 32 + q * 8 + khalf * 4;
          if (c >= zN) continue;
          OutT* dst = zp + (int64_t)r * ldz + c;
          float v0 = acc[tn][tm][q * 4 + 0] * alpha, v1 = acc[tn][tm][q * 4 + 1] * alpha;
          float v2 = acc[tn][tm][q * 4 + 2] * alpha, v3 = acc[tn][tm][q * 4 + 3] * alpha;
          if constexpr (sizeof(OutT) == 2) {
            u32x2 o;
            o.x = pack_bf16x2(v0, v1);
            o.y = pack_bf16x2(v2, v3);
            *reinterpret_cast<u32x2*>(dst) = o;
          } else {
            f32x4 o = {v0, v1, v2, v3};
            *reinterpret_cast<f32x4*>(dst) = o;
          }
        }
    }
  }
};

// ---- pipelined variant: global -> LDS directly, scales through LDS too ---------------------
// Same pipeline as the bf16 GEMM's direct variant, adapted to 32-byte operands:
//  * data tiles AND the tile's scale dwords are fetched with buffer loads that
//    write straight into LDS (data: 16 bytes per lane with the swizzle applied on
//    the global side; scales: one dword per row, 256 bytes per instruction), two
//    stages, refilled one K tile ahead;
//  * an fp8 operand fragment is 8 registers, so there is one set of fragments,
//    not two: each fragment is reloaded for the next 64-wide K step right after
//    the last MFMA that reads it, at least three MFMAs (192 matrix-pipe cycles)
//    before its next use.  The MFMAs of a step run outer-fragment-major so that
//    the outer fragments free up one by one and the inner ones during the last
//    outer iteration;
//  * the stage hand-over sits after the third MFMA of a tile's second K step: by
//    then every read of the current stage has completed without being waited for;
//  * memory instructions are dealt out between MFMAs, sched_barrier(0) keeps
//    the written order; the epilogue is the shared LDS-staged one.
template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT>
struct MxGemmDirect {
  static constexpr int BK = 128;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int kAInstr = BM / 8 / kWaves, kBInstr = BN / 8 / kWaves;   // 1 KiB = 8 rows of 128 bytes
  static constexpr int kSInstr = (BM + BN) / 64 / kWaves;                     // 1 KiB = 64 rows x 16 scale bytes
  static constexpr int kABytes = BM * BK, kBBytes = BN * BK;
  static constexpr int kScaleBytes = (BM + BN) * 16;                          // 4 K tiles of scales per row
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes + 2 * kScaleBytes;
  static constexpr bool kOuterIsN = TN <= TM;          // the operand with fewer fragments is the outer one
  static constexpr int NO = kOuterIsN ? TN : TM, NI = kOuterIsN ? TM : TN;
  static constexpr int NB = TM * TN;
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0 && (BM + BN) % (64 * kWaves) == 0 && BM % 64 == 0,
                "tile must split evenly");
  static_assert(NI >= 3 && NB >= 6, "the reload distance assumes at least three inner fragments");
  static_assert(kWaves / 2 * kEpilogueBytesPerWave<WN> <= kStageBytes, "the output bands must fit the stages");

  __device__ static __forceinline__ int lds_off(int r, int u) { return r * BK + ((u ^ ((r >> 1) & 7)) << 4); }

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             const TensorArg<2>& xs, const TensorArg<2>& ys, float alpha, const TileGrid& g) {
    __shared__ __attribute__((aligned(1024))) unsigned char stage0[kStageBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char stage1[kStageBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char scales0[kScaleBytes];   // scale blocks 0, 2, 4 ...
    __shared__ __attribute__((aligned(1024))) unsigned char scales1[kScaleBytes];   // scale blocks 1, 3, 5 ...
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, khalf = lane >> 5;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[0], K = min(x.shape[1], y.shape[1]);
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t ldsa = xs.strides[0], ldsb = ys.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)((int64_t)(M - 1) * lda + x.shape[1]));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)((int64_t)(N - 1) * ldb + y.shape[1]));
    const __amdgpu_buffer_rsrc_t rsa = make_rsrc(xs.ptr, (uint32_t)((int64_t)(xs.shape[0] - 1) * ldsa + xs.shape[1]));
    const __amdgpu_buffer_rsrc_t rsb = make_rsrc(ys.ptr, (uint32_t)((int64_t)(ys.shape[0] - 1) * ldsb + ys.shape[1]));
    constexpr uint32_t kOob = 0x80000000u;
    const int k_tiles = K / BK;

    // Global side of the fetches (per lane, K tile 0; the K advance is scalar).
    uint32_t a_goff[kAInstr], b_goff[kBInstr], s_goff[kSInstr];
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) {
      const int r = (wave * kAInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      a_goff[i] = (row0 + r < M) ? (uint32_t)((int64_t)(row0 + r) * lda + u * 16) : kOob;
    }
#pragma unroll
    for (int i = 0; i < kBInstr; ++i) {
      const int r = (wave * kBInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      b_goff[i] = (col0 + r < N) ? (uint32_t)((int64_t)(col0 + r) * ldb + u * 16) : kOob;
    }
    // Scale rows: instruction s covers 64 rows; the first BM/64 instructions are x rows.
    // Rows beyond the tensor read scale byte 0 (2^-127) against all-zero data: they contribute 0.
#pragma unroll
    for (int i = 0; i < kSInstr; ++i) {
      const int sidx = wave * kSInstr + i;
      const bool is_x = sidx < BM / 64;
      const int r = (is_x ? sidx : sidx - BM / 64) * 64 + lane;
      s_goff[i] = is_x ? ((row0 + r < M) ? (uint32_t)((int64_t)(row0 + r) * ldsa) : kOob)
                       : ((col0 + r < N) ? (uint32_t)((int64_t)(col0 + r) * ldsb) : kOob);
    }
    // Fetch instruction i of tile kt into `stage`: x data, then y data; with
    // WITH_SCALES also this wavefront's share of the scale block of tile kt (the
    // 16 scale bytes per row that cover tiles kt..kt+3, kt a multiple of 4).  One
    // dword per row per tile would touch a separate cache line per lane every
    // tile; a block of four tiles costs the same lines once.
    constexpr int NF = kAInstr + kBInstr;
    auto scale_block = [&](int32_t tile) -> unsigned char* { return ((tile >> 2) & 1) ? scales1 : scales0; };
    auto fetch_one = [&](unsigned char* stage, int32_t kt, int i) {
      const bool wanted = kt < k_tiles;   // past the last tile: out-of-range offsets, zeros
      const int32_t k0 = wanted ? kt * BK : 0;
      if (i < kAInstr) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(stage + (wave * kAInstr + i) * 1024), 16,
                                                 wanted ? a_goff[i] : kOob, k0, 0, 0);
      } else if (i < kAInstr + kBInstr) {
        const int b = i - kAInstr;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(stage + kABytes + (wave * kBInstr + b) * 1024), 16,
                                                 wanted ? b_goff[b] : kOob, k0, 0, 0);
      } else {
        const int si = i - kAInstr - kBInstr;
        const int sidx = wave * kSInstr + si;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(sidx < BM / 64 ? rsa : rsb,
                                                 (LDS_PTR(void))(scale_block(kt) + sidx * 1024), 16,
                                                 wanted ? s_goff[si] : kOob, k0 / 32, 0, 0);
      }
    };

    // LDS side of the operand reads: a fragment of K step ks is units ks*4+khalf and ks*4+2+khalf.
    int a_addr[2][2], b_addr[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        a_addr[ks][h] = lds_off(wm * WM + l32, ks * 4 + 2 * h + khalf);                 // + tm * 32 rows
        b_addr[ks][h] = kABytes + lds_off(wn * WN + l32, ks * 4 + 2 * h + khalf);       // + tn * 32 rows
      }
    const int sa_addr = (wm * WM + l32) * 16;                                           // + tm * 32 rows, + 4 * (tile % 4)
    const int sb_addr = BM * 16 + (wn * WN + l32) * 16;                                 // + tn * 32 rows
    auto read_a = [&](const unsigned char* stage, int ks, int tm) -> i32x8 {
      u32x4 lo = *reinterpret_cast<const u32x4*>(stage + a_addr[ks][0] + tm * 32 * BK);
      u32x4 hi = *reinterpret_cast<const u32x4*>(stage + a_addr[ks][1] + tm * 32 * BK);
      return i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    };
    auto read_b = [&](const unsigned char* stage, int ks, int tn) -> i32x8 {
      u32x4 lo = *reinterpret_cast<const u32x4*>(stage + b_addr[ks][0] + tn * 32 * BK);
      u32x4 hi = *reinterpret_cast<const u32x4*>(stage + b_addr[ks][1] + tn * 32 * BK);
      return i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

    i32x8 af[TM], bfr[TN];               // the one set of operand fragments
    // A row's 16 scale bytes for the four K tiles of a scale block, read once per block as one 16-byte LDS read
    // (rows are 16 bytes apart: a wavefront's read is one contiguous 512-byte run, free of bank conflicts, where a
    // dword per row and tile puts rows r and r+16 on the same bank); component p belongs to tile 4q + p.
    u32x4 sa_blk[TM], sb_blk[TN];
    int sas[TM], sbs[TN];                // scales of a tile's second K step, already moved to byte 0
    // K step ks covers MX blocks 2ks and 2ks+1 of the tile; lanes 0-31 supply the scale
    // of the first, lanes 32-63 of the second, in byte 0 of the scale operand.
    const int sh0 = 8 * khalf, sh1 = 8 * (2 + khalf);
    auto read_scale_block = [&](int32_t tile) {      // tile: a multiple of 4
      const unsigned char* blk = scale_block(tile);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) sa_blk[tm] = *reinterpret_cast<const u32x4*>(blk + sa_addr + tm * 32 * 16);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) sb_blk[tn] = *reinterpret_cast<const u32x4*>(blk + sb_addr + tn * 32 * 16);
    };
    // MFMA j of a K step (outer-major) and, after it, the reload of whatever fragment it used last.
    auto mfma_step = [&](int j, int ks, auto phase) {
      constexpr int PH = decltype(phase)::value;
      const int o = j / NI, i = j % NI;
      const int tn = kOuterIsN ? o : i, tm = kOuterIsN ? i : o;
      const int sb = ks == 0 ? (int)(sb_blk[tn][PH] >> sh0) : sbs[tn];
      const int sa = ks == 0 ? (int)(sa_blk[tm][PH] >> sh0) : sas[tm];
      acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0, sb, 0, sa);
    };
    auto reload_after = [&](int j, const unsigned char* stage, int ks) {
      const int o = j / NI, i = j % NI;
      if (i == NI - 1) {        // outer fragment o is done
        if (kOuterIsN) bfr[o] = read_b(stage, ks, o); else af[o] = read_a(stage, ks, o);
      }
      if (o == NO - 1) {        // inner fragment i is done
        if (kOuterIsN) af[i] = read_a(stage, ks, i); else bfr[i] = read_b(stage, ks, i);
      }
    };

    // Prologue: tile 0 (and 1) on their way, first fragments and scales in registers.
    if (k_tiles > 0) {
#pragma unroll
      for (int i = 0; i < NF + kSInstr; ++i) fetch_one(stage0, 0, i);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
#pragma unroll
      for (int i = 0; i < NF; ++i) fetch_one(stage1, 1, i);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) af[tm] = read_a(stage0, 0, tm);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) bfr[tn] = read_b(stage0, 0, tn);
      read_scale_block(0);
    }
    constexpr int kHandOverAt = 3;   // MFMAs of the second K step issued before the hand-over
    // `with_scales`: tile kt+2 opens a scale block (kt + 2 is a multiple of 4).
    // `phase` = kt % 4 (the tile's place in its scale block), known where the call is written.
    auto k_tile = [&](unsigned char* cur, const unsigned char* nxt, int kt, auto with_scales, auto phase) {
      constexpr int PH = decltype(phase)::value;
      constexpr int NFT = NF + (decltype(with_scales)::value ? kSInstr : 0);
      // K step 0; fragments of step 1 are reloaded from `cur` as they free up.
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        mfma_step(j, 0, phase);
        __builtin_amdgcn_sched_barrier(0);   // the reload must follow the last reader, or it needs registers of its own
        reload_after(j, cur, 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      // K step 1; after the hand-over, fragments and scales of tile kt+1 come from
      // `nxt` and tile kt+2 is fetched into `cur`.
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) sas[tm] = (int)(sa_blk[tm][PH] >> sh1);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) sbs[tn] = (int)(sb_blk[tn][PH] >> sh1);
#pragma unroll
      for (int j = 0; j < kHandOverAt; ++j) {
        mfma_step(j, 1, phase);
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_waitcnt(0);   // own reads of `cur` done, own share of tile kt+1 landed
      __syncthreads();
      if constexpr (PH == 3) read_scale_block(kt + 1);   // the next tile opens a scale block; this tile's second K step has its scales in sas / sbs
#pragma unroll
      for (int j = kHandOverAt; j < NB; ++j) {
#pragma unroll
        for (int i = 0; i < NFT; ++i)
          if (i * (NB - kHandOverAt) / NFT == j - kHandOverAt) fetch_one(cur, kt + 2, i);
        mfma_step(j, 1, phase);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jj = 0; jj < NB; ++jj)   // reloads that fell before the hand-over are issued with the first MFMA after it
          if ((jj < kHandOverAt && j == kHandOverAt) || jj == j) reload_after(jj, nxt, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // Whole pairs in the loop, an odd last tile after it: with the second tile
    // under a condition inside the loop the compiler would have to assume, at the
    // top of the loop, a refill of stage0 in flight and wait for it before every read.
    int kt = 0;
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    using P2 = std::integral_constant<int, 2>;
    using P3 = std::integral_constant<int, 3>;
    for (; kt + 4 <= k_tiles; kt += 4) {
      k_tile(stage0, stage1, kt, std::false_type{}, P0{});
      k_tile(stage1, stage0, kt + 1, std::false_type{}, P1{});
      k_tile(stage0, stage1, kt + 2, std::true_type{}, P2{});
      k_tile(stage1, stage0, kt + 3, std::false_type{}, P3{});
    }
    if (kt < k_tiles) k_tile(stage0, stage1, kt, std::false_type{}, P0{});
    if (kt + 1 < k_tiles) k_tile(stage1, stage0, kt + 1, std::false_type{}, P1{});
    if (kt + 2 < k_tiles) k_tile(stage0, stage1, kt + 2, std::true_type{}, P2{});

    // Every wavefront is past its operand reads and every fetch has landed: the
    // stages are free to carry the output.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] *= alpha;
    unsigned char* band = (wave < kWaves / 2 ? stage0 : stage1) + (wave % (kWaves / 2)) * kEpilogueBytesPerWave<WN>;
    store_tile_staged<TM, TN, OutT>(acc, band, (OutT*)z.ptr, z.strides[0], z.shape[0], z.shape[1], row0 + wm * WM,
                                    col0 + wn * WN, lane, 0);
  }
};

// ---- the direct pipeline on v_mfma_scale_f32_16x16x128_f8f6f4 ("e") ------------------------------------
// The matrix kernels here run against the chip's power limit, and per flop the 16 x 16 x 128 form writes half as many
// accumulator values as 32 x 32 x 64: a loop of nothing but scaled fp8 MFMAs on random operand bits sustains 4250
// TFLOP/s with it against 3810 (equal, 4960 - 4990, on constant operands).  Operand layout (measured on gfx950 with
// one-hot products): a lane (row r = lane % 16, group g = lane / 16) holds 32 bytes of its row; the first 16 are K
// positions 16 g .. 16 g + 15 of the instruction's 128, the last 16 are 64 + 16 g .. 64 + 16 g + 15; lane group s
// supplies, in byte 0 of its scale register, the scale of K block s (positions 32 s .. 32 s + 31) of its row.  The
// result is laid out like v_mfma_f32_16x16x32's.
// One instruction covers a whole K tile, so a tile is 32 MFMAs (4 x row blocks by 8 y row blocks of 16): for each y
// block in turn, the four x blocks.  Registers hold the four x fragments and two y fragments (slot = y block % 2): a
// y fragment is reloaded with y block tn + 2 as its last MFMA issues, the x fragments with the next tile's during the
// last y block, four MFMAs (the other wavefront of the SIMD issues as many in between) before their next use.
// Hand-over of the stages five MFMAs before the end of the tile; the refill of the stage just drained is dealt out over
// those MFMAs.
template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT>
struct MxGemmDirect16 {
  static constexpr int BK = 128;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 16, TN = WN / 16;
  static constexpr int kAInstr = BM / 8 / kWaves, kBInstr = BN / 8 / kWaves;   // 1 KiB = 8 rows of 128 bytes
  static constexpr int kSInstr = (BM + BN) / 64 / kWaves;                     // 1 KiB = 64 rows x 16 scale bytes
  static constexpr int kABytes = BM * BK, kBBytes = BN * BK;
  static constexpr int kScaleBytes = (BM + BN) * 16;                          // 4 K tiles of scales per row
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes + 2 * kScaleBytes;
  static constexpr int NB = TM * TN;
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0 && (BM + BN) % (64 * kWaves) == 0 && BM % 64 == 0,
                "tile must split evenly");
  static_assert(TN % 2 == 0 && TN >= 4 && TM >= 2, "two y fragment slots: an even number of y blocks keeps a block in its slot from tile to tile");

  __device__ static __forceinline__ int lds_off(int r, int u) { return r * BK + ((u ^ ((r >> 1) & 7)) << 4); }

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             const TensorArg<2>& xs, const TensorArg<2>& ys, float alpha, const TileGrid& g) {
    // The y stages come first in LDS (the larger alignment sorts them to the front): every y fragment read then
    // reaches its 16 rows through the instruction's 16-bit offset from ONE pair of per-lane addresses, whichever the
    // stage.  The x stages lie beyond that reach; their four fragments per tile add the stage's address to the lane's
    // offset at each read (an opaque copy keeps the compiler from carrying one address register per fragment and stage).
    __shared__ __attribute__((aligned(4096))) unsigned char ys0[kBBytes];
    __shared__ __attribute__((aligned(4096))) unsigned char ys1[kBBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs0[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs1[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char scales0[kScaleBytes];   // scale blocks 0, 2, 4 ...
    __shared__ __attribute__((aligned(1024))) unsigned char scales1[kScaleBytes];   // scale blocks 1, 3, 5 ...
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l16 = lane & 15, grp = lane >> 4;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[0], K = min(x.shape[1], y.shape[1]);
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t ldsa = xs.strides[0], ldsb = ys.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)((int64_t)(M - 1) * lda + x.shape[1]));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)((int64_t)(N - 1) * ldb + y.shape[1]));
    const __amdgpu_buffer_rsrc_t rsa = make_rsrc(xs.ptr, (uint32_t)((int64_t)(xs.shape[0] - 1) * ldsa + xs.shape[1]));
    const __amdgpu_buffer_rsrc_t rsb = make_rsrc(ys.ptr, (uint32_t)((int64_t)(ys.shape[0] - 1) * ldsb + ys.shape[1]));
    constexpr uint32_t kOob = 0x80000000u;
    const int k_tiles = K / BK;

    // Global side of the fetches: as in MxGemmDirect (per lane, K tile 0; the K advance is scalar).
    uint32_t a_goff[kAInstr], b_goff[kBInstr], s_goff[kSInstr];
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) {
      const int r = (wave * kAInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      a_goff[i] = (row0 + r < M) ? (uint32_t)((int64_t)(row0 + r) * lda + u * 16) : kOob;
    }
#pragma unroll
    for (int i = 0; i < kBInstr; ++i) {
      const int r = (wave * kBInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      b_goff[i] = (col0 + r < N) ? (uint32_t)((int64_t)(col0 + r) * ldb + u * 16) : kOob;
    }
#pragma unroll
    for (int i = 0; i < kSInstr; ++i) {
      const int sidx = wave * kSInstr + i;
      const bool is_x = sidx < BM / 64;
      const int r = (is_x ? sidx : sidx - BM / 64) * 64 + lane;
      s_goff[i] = is_x ? ((row0 + r < M) ? (uint32_t)((int64_t)(row0 + r) * ldsa) : kOob)
                       : ((col0 + r < N) ? (uint32_t)((int64_t)(col0 + r) * ldsb) : kOob);
    }
    constexpr int NF = kAInstr + kBInstr;
    auto scale_block = [&](int32_t tile) -> unsigned char* { return ((tile >> 2) & 1) ? scales1 : scales0; };
    auto fetch_one = [&](unsigned char* xs, unsigned char* ys, int32_t kt, int i) {
      const bool wanted = kt < k_tiles;   // past the last tile: out-of-range offsets, zeros
      const int32_t k0 = wanted ? kt * BK : 0;
      if (i < kAInstr) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(xs + (wave * kAInstr + i) * 1024), 16,
                                                 wanted ? a_goff[i] : kOob, k0, 0, 0);
      } else if (i < kAInstr + kBInstr) {
        const int b = i - kAInstr;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(ys + (wave * kBInstr + b) * 1024), 16,
                                                 wanted ? b_goff[b] : kOob, k0, 0, 0);
      } else {
        const int si = i - kAInstr - kBInstr;
        const int sidx = wave * kSInstr + si;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(sidx < BM / 64 ? rsa : rsb,
                                                 (LDS_PTR(void))(scale_block(kt) + sidx * 1024), 16,
                                                 wanted ? s_goff[si] : kOob, k0 / 32, 0, 0);
      }
    };

    // LDS side: the lane's two 16-byte units of its row (K positions 16 g .. and 64 + 16 g ..) and its scale byte.
    const int a_lo = lds_off(wm * WM + l16, grp), a_hi = lds_off(wm * WM + l16, 4 + grp);               // + tm * 16 rows
    const int b_lo = lds_off(wn * WN + l16, grp), b_hi = lds_off(wn * WN + l16, 4 + grp);                 // + tn * 16 rows
    const int sa_addr = (wm * WM + l16) * 16 + grp;                                 // + tm * 16 rows, + 4 * (tile % 4)
    const int sb_addr = BM * 16 + (wn * WN + l16) * 16 + grp;                       // + tn * 16 rows
    auto read_frag = [&](const unsigned char* stage, int lo, int hi, int blk, bool far) -> i32x8 {
      if (far) asm volatile("" : "+v"(lo), "+v"(hi));
      u32x4 l = *reinterpret_cast<const u32x4*>(stage + lo + blk * 16 * BK);
      u32x4 h = *reinterpret_cast<const u32x4*>(stage + hi + blk * 16 * BK);
      return i32x8{(int)l.x, (int)l.y, (int)l.z, (int)l.w, (int)h.x, (int)h.y, (int)h.z, (int)h.w};
    };

    f32x4_acc acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[tn][tm][v] = 0.0f;

    i32x8 af[TM], bfr[2];       // x fragments of the tile; y fragments (slot = y block % 2)
    int sa[TM], sb[2];          // their scales (byte 0)
    // A fragment's scale is one byte read straight from the staged scale rows (lane group g reads byte g of the row's
    // dword for the tile: no shift) by an instruction the compiler does not see as a memory access: the scale rows
    // sit in two buffers picked at run time, and a visible read of "either" would be made to wait for every fetch in
    // flight.  The reads are ordered by the hand-over like all the others, and each is issued in front of its
    // fragment's own reads, whose wait covers it.  `base` = the scale block's LDS address plus the lane's row and
    // byte; the row block and the tile's place in the scale block are the instruction's offset.
    // (The four lane groups read four bytes of one dword, which the LDS counts as a bank conflict, two cycles a read;
    // reading the dwords instead, all twelve of a tile behind the hand-over, packed with v_perm_b32 and picked by the
    // MFMA's op_sel, was built and measured slower: the same conflicts, and a tile's worth of LDS latency exposed.)
    auto read_scale = [&](uint32_t base, int off) -> int {
      int v;
      asm volatile("ds_read_u8 %0, %1 offset:%2" : "=v"(v) : "v"(base), "n"(off));
      return v;
    };
    auto scale_base = [&](const unsigned char* blk, int lane_addr) -> uint32_t { return (uint32_t)(uintptr_t)blk + (uint32_t)lane_addr; };
    auto load_a = [&](const unsigned char* xs, uint32_t sbase, int ph, int tm) {
      sa[tm] = read_scale(sbase, tm * 16 * 16 + 4 * ph);
      af[tm] = read_frag(xs, a_lo, a_hi, tm, true);
    };
    auto load_b = [&](const unsigned char* ys, uint32_t sbase, int ph, int tn) {
      sb[tn & 1] = read_scale(sbase, tn * 16 * 16 + 4 * ph);
      bfr[tn & 1] = read_frag(ys, b_lo, b_hi, tn, false);
    };

    // Prologue: tile 0 (and 1) on their way, the first fragments and scales in registers.
    if (k_tiles > 0) {
#pragma unroll
      for (int i = 0; i < NF + kSInstr; ++i) fetch_one(xs0, ys0, 0, i);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
#pragma unroll
      for (int i = 0; i < NF; ++i) fetch_one(xs1, ys1, 1, i);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) load_a(xs0, scale_base(scales0, sa_addr), 0, tm);
#pragma unroll
      for (int tn = 0; tn < 2; ++tn) load_b(ys0, scale_base(scales0, sb_addr), 0, tn);
    }
    // The hand-over sits before the last MFMA of the last y block but one: the reload behind that MFMA is the first
    // read of the next tile's stage, and the last read of the current one (y block TN - 1, requested behind the MFMAs of
    // block TN - 3) has had a block's MFMAs to complete, so the wait in front of the barrier finds it done.
    constexpr int kHandOverAt = (TN - 1) * TM - 1;
    constexpr int kFetchSlots = NB - kHandOverAt;
    // `with_scales`: tile kt+2 opens a scale block (kt + 2 is a multiple of 4).
    // `phase` = kt % 4 (the tile's place in its scale block), known where the call is written.
    auto k_tile = [&](unsigned char* x_cur, unsigned char* y_cur, const unsigned char* x_nxt, const unsigned char* y_nxt, int kt,
                      auto with_scales, auto phase) {
      constexpr int PH = decltype(phase)::value;
      constexpr int NFT = NF + (decltype(with_scales)::value ? kSInstr : 0);
      constexpr int PHN = (PH + 1) & 3;
      const uint32_t sb_cur = scale_base(scale_block(kt), sb_addr);
      const uint32_t sa_nxt = scale_base(scale_block(kt + 1), sa_addr), sb_nxt = scale_base(scale_block(kt + 1), sb_addr);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          const int j = tn * TM + tm;
          if (j == kHandOverAt) {
            __builtin_amdgcn_s_waitcnt(0);   // own reads of `cur` done, own share of tile kt+1 landed
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
          }
          if (j >= kHandOverAt) {
#pragma unroll
            for (int i = 0; i < NFT; ++i)
              if (i * kFetchSlots / NFT == j - kHandOverAt) fetch_one(x_cur, y_cur, kt + 2, i);
          }
          acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bfr[tn & 1], af[tm], acc[tn][tm], 0, 0, 0, sb[tn & 1], 0, sa[tm]);
          __builtin_amdgcn_sched_barrier(0);   // a reload must follow the last reader, or it needs registers of its own
          if (tn == TN - 1) load_a(x_nxt, sa_nxt, PHN, tm);       // x block tm has done its last MFMA of this tile
          if (tm == TM - 1) {                                       // so has y block tn: its slot takes y block tn + 2
            if (tn + 2 < TN) load_b(y_cur, sb_cur, PH, tn + 2);
            else load_b(y_nxt, sb_nxt, PHN, tn + 2 - TN);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };
    int kt = 0;
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    using P2 = std::integral_constant<int, 2>;
    using P3 = std::integral_constant<int, 3>;
    for (; kt + 4 <= k_tiles; kt += 4) {
      k_tile(xs0, ys0, xs1, ys1, kt, std::false_type{}, P0{});
      k_tile(xs1, ys1, xs0, ys0, kt + 1, std::false_type{}, P1{});
      k_tile(xs0, ys0, xs1, ys1, kt + 2, std::true_type{}, P2{});
      k_tile(xs1, ys1, xs0, ys0, kt + 3, std::false_type{}, P3{});
    }
    if (kt < k_tiles) k_tile(xs0, ys0, xs1, ys1, kt, std::false_type{}, P0{});
    if (kt + 1 < k_tiles) k_tile(xs1, ys1, xs0, ys0, kt + 1, std::false_type{}, P1{});
    if (kt + 2 < k_tiles) k_tile(xs0, ys0, xs1, ys1, kt + 2, std::true_type{}, P2{});

    // Every wavefront is past its operand reads and every fetch has landed: the stages are free to carry the output.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[tn][tm][v] *= alpha;
    static_assert(kWaves == 8 && 2 * kEpilogueBytesPerWave<WN> <= kABytes && 2 * kEpilogueBytesPerWave<WN> <= kBBytes, "two output bands per stage array");
    unsigned char* band = (wave < 2 ? ys0 : wave < 4 ? ys1 : wave < 6 ? xs0 : xs1) + (wave & 1) * kEpilogueBytesPerWave<WN>;
    store_tile_staged16<TM, TN, OutT>(acc, band, (OutT*)z.ptr, z.strides[0], z.shape[0], z.shape[1], row0 + wm * WM,
                                      col0 + wn * WN, lane, 0);
  }
};

}  // namespace

#define MX_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                                   \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                     \
      linear_tile_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, TensorArg<2> xs, \
                                TensorArg<2> ys, float alpha, TileGrid g) {                        \
    MxGemm<BM, BN, WVM, WVN, OUT_T>::run(z, x, y, xs, ys, alpha, g);                               \
  }

MX_KERNEL(mxfp8_bf16_256x256x128_w2x2, 256, 256, 2, 2, __bf16)
MX_KERNEL(mxfp8_bf16_256x256x128_w2x4, 256, 256, 2, 4, __bf16)
MX_KERNEL(mxfp8_bf16_128x128x128_w2x2, 128, 128, 2, 2, __bf16)
MX_KERNEL(mxfp8_f32_256x256x128_w2x2, 256, 256, 2, 2, float)
MX_KERNEL(mxfp8_f32_128x128x128_w2x2, 128, 128, 2, 2, float)
MX_KERNEL(mxfp8_f32_32x32x128_w1x1, 32, 32, 1, 1, float)
MX_KERNEL(mxfp8_f32_64x64x128_w1x1, 64, 64, 1, 1, float)

#define MX_DIRECT_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                            \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                     \
      linear_tile_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, TensorArg<2> xs, \
                                TensorArg<2> ys, float alpha, TileGrid g) {                        \
    MxGemmDirect<BM, BN, WVM, WVN, OUT_T>::run(z, x, y, xs, ys, alpha, g);                         \
  }

MX_DIRECT_KERNEL(mxfp8_bf16_256x256x128_d2x4, 256, 256, 2, 4, __bf16)
MX_DIRECT_KERNEL(mxfp8_bf16_256x256x128_d4x2, 256, 256, 4, 2, __bf16)
MX_DIRECT_KERNEL(mxfp8_f32_256x256x128_d2x4, 256, 256, 2, 4, float)

#define MX_DIRECT16_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                          \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                     \
      linear_tile_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, TensorArg<2> xs, \
                                TensorArg<2> ys, float alpha, TileGrid g) {                        \
    MxGemmDirect16<BM, BN, WVM, WVN, OUT_T>::run(z, x, y, xs, ys, alpha, g);                       \
  }

MX_DIRECT16_KERNEL(mxfp8_bf16_256x256x128_e4x2, 256, 256, 4, 2, __bf16)
MX_DIRECT16_KERNEL(mxfp8_f32_256x256x128_e4x2, 256, 256, 4, 2, float)
