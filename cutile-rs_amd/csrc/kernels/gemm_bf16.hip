// Tiled bf16 GEMM for gfx950: z[M,N] (+)= x[M,K] · y[K,N], f32 accumulation on
// the matrix cores, bf16 (or f32) output.
//
// Tile program being implemented (cutile-benchmarks/benches/gemm.rs:20-41,
// cutile-examples/examples/gemm.rs:20-36): one tile block per [BM,BN] output
// tile; acc = z.load() (or 0); for i in 0..K/BK: acc = mma(x[pid0,i], y[i,pid1], acc);
// z.store(acc).  Loads outside a tensor read 0, stores outside z are dropped.
//
// Mapping to CDNA4:
//  * one workgroup per output tile, WAVES_M x WAVES_N wavefronts, each owning a
//    WM x WN sub-tile built from v_mfma_f32_32x32x16_bf16 (64-lane wavefronts,
//    8 K-values per lane per operand);
//  * x and y tiles are staged through LDS, double buffered, one barrier per
//    K-step; the next tile's global loads are issued before the current tile's
//    MFMAs so HBM/L2 latency hides under matrix work;
//  * x is K-contiguous, which is what an MFMA operand wants (ds_read_b128 per
//    lane).  y is N-contiguous; its operand is formed with ds_read_b64_tr_b16,
//    the LDS transpose read of gfx950, so no transposed copy of y is ever made;
//  * both LDS tiles are XOR-swizzled in 16-byte units so operand reads spread
//    over the banks;
//  * the MFMA is issued with y's fragment as its first operand and x's as the
//    second, i.e. it produces the transposed tile: each lane then holds 4
//    consecutive N-columns of one output row, which turns the epilogue into
//    8-byte stores instead of 2-byte ones;
//  * global reads go through buffer descriptors, whose out-of-range reads return
//    0 — exactly the tile program's zero padding, with no branches;
//  * workgroup ids are remapped so that each XCD (own L2) works on a compact
//    band of output tiles, walked in groups of GROUP_M tile rows.
#include <hip/hip_runtime.h>

#include "gemm_common.h"
#include "mapped_partition.h"
#include "kernel_args.h"

using namespace cutile;
using namespace cutile::gemm;

namespace {

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, typename OutT>
struct Gemm {
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int kAChunksPerRow = BK / 8;          // 16-byte units per x-tile row
  static constexpr int kBChunksPerRow = BN / 8;          // 16-byte units per y-tile row
  static constexpr int kAChunks = BM * kAChunksPerRow;
  static constexpr int kBChunks = BK * kBChunksPerRow;
  static constexpr int kALoads = kAChunks / kThreads;
  static constexpr int kBLoads = kBChunks / kThreads;
  static constexpr int kABytes = BM * BK * 2, kBBytes = BK * BN * 2;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert(BK == 64, "the x-tile swizzle assumes 8 sixteen-byte units per row");
  static_assert(kAChunks % kThreads == 0 && kBChunks % kThreads == 0, "tile must split evenly");
  static_assert(kBChunksPerRow >= 16, "the y-tile swizzle needs at least 16 units per row");

  // x tile: row-major [BM][BK]; unit u of row r lives at unit (u ^ ((r >> 1) & 7)).
  __device__ static __forceinline__ int a_lds_off(int r, int u) {
    return r * (BK * 2) + ((u ^ ((r >> 1) & 7)) << 4);
  }
  // y tile: row-major [BK][BN]; unit u of k-row r lives at unit (u ^ ((r & 3) << 2)).
  __device__ static __forceinline__ int b_lds_off(int r, int u) {
    return r * (BN * 2) + ((u ^ ((r & 3) << 2)) << 4);
  }

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             int32_t k_total, const TileGrid& g, int32_t accumulate) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[1];
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;
    // K actually readable from both operands and asked for; beyond it tiles read 0.
    const int32_t k_valid = min(min(x.shape[1], y.shape[0]), k_total);

    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)(((int64_t)(M - 1) * lda + x.shape[1]) * 2));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)(((int64_t)(y.shape[0] - 1) * ldb + N) * 2));
    constexpr uint32_t kOob = 0x80000000u;  // beyond any descriptor -> reads 0

    // Per-thread global -> LDS assignments (fixed over the K loop except for k0).
    int a_row[kALoads], a_unit[kALoads], b_row[kBLoads], b_unit[kBLoads];
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      int c = tid + i * kThreads;
      a_row[i] = c / kAChunksPerRow;
      a_unit[i] = c % kAChunksPerRow;
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      int c = tid + i * kThreads;
      b_row[i] = c / kBChunksPerRow;
      b_unit[i] = c % kBChunksPerRow;
    }

    u32x4 a_reg[kALoads], b_reg[kBLoads];
    auto load_global = [&](int32_t k0) {
#pragma unroll
      for (int i = 0; i < kALoads; ++i) {
        int32_t r = row0 + a_row[i], kk = k0 + a_unit[i] * 8;
        uint32_t off = (r < M && kk < k_valid) ? (uint32_t)(((int64_t)r * lda + kk) * 2) : kOob;
        a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, off, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) {
        int32_t kk = k0 + b_row[i], c = col0 + b_unit[i] * 8;
        uint32_t off = (kk < k_valid && c < N) ? (uint32_t)(((int64_t)kk * ldb + c) * 2) : kOob;
        b_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, off, 0, 0);
      }
    };
    auto store_lds = [&](int stage) {
      unsigned char* sa = lds + stage * kStageBytes;
      unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int i = 0; i < kALoads; ++i) *reinterpret_cast<u32x4*>(sa + a_lds_off(a_row[i], a_unit[i])) = a_reg[i];
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) *reinterpret_cast<u32x4*>(sb + b_lds_off(b_row[i], b_unit[i])) = b_reg[i];
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

    // Lane roles inside the operand reads.
    const int l32 = lane & 31, khalf = lane >> 5;          // x operand: row l32, k-units khalf
    const int grp = lane >> 4, l16 = lane & 15;            // y operand: transpose-read groups
    const int tr_row = l16 >> 2, tr_col = (l16 & 3) * 4;   // address role inside a 4x16 block
    const int b_n_half = (grp & 1) * 16, b_k_half = (grp >> 1) * 8;

    const int k_tiles = (k_total + BK - 1) / BK;
    if (k_tiles > 0) {
      load_global(0);
      store_lds(0);
    }
    __syncthreads();

    for (int kt = 0; kt < k_tiles; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < k_tiles) load_global((kt + 1) * BK);
      const unsigned char* sa = lds + cur * kStageBytes;
      const unsigned char* sb = sa + kABytes;
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        bf16x8 af[TM], bfr[TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          int r = wm * WM + tm * 32 + l32;
          af[tm] = *reinterpret_cast<const bf16x8*>(sa + a_lds_off(r, ks * 2 + khalf));
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          int n = wn * WN + tn * 32 + b_n_half + tr_col;  // first of the 4 columns this lane addresses
          int kr = ks * 16 + b_k_half + tr_row;
          const unsigned char* p0 = sb + b_lds_off(kr, n >> 3) + (n & 7) * 2;
          const unsigned char* p1 = sb + b_lds_off(kr + 4, n >> 3) + (n & 7) * 2;
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p0);
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p1);
          typedef short s16x8 __attribute__((ext_vector_type(8)));
          s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          bfr[tn] = __builtin_bit_cast(bf16x8, both);
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm)
            acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
      }
      if (kt + 1 < k_tiles) store_lds(cur ^ 1);
      __syncthreads();
    }

    // Epilogue.  acc[tn][tm][v]: output row = tm*32 + l32, columns
    // tn*32 + (v/4)*8 + khalf*4 + (v%4): four consecutive columns per v-quad.
    OutT* zp = (OutT*)z.ptr;
    const int32_t ldz = z.strides[0];
    const int32_t zM = z.shape[0], zN = z.shape[1];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int32_t r = row0 + wm * WM + tm * 32 + l32;
      if (r >= zM) continue;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int32_t c = col0 + wn * WN + tn * 32 + q * 8 + khalf * 4;
          if (c >= zN) continue;
          OutT* dst = zp + (int64_t)r * ldz + c;
          float v0 = acc[tn][tm][q * 4 + 0], v1 = acc[tn][tm][q * 4 + 1];
          float v2 = acc[tn][tm][q * 4 + 2], v3 = acc[tn][tm][q * 4 + 3];
          if constexpr (sizeof(OutT) == 2) {
            if (accumulate) {
              u32x2 old = *reinterpret_cast<const u32x2*>(dst);
              v0 += __builtin_bit_cast(float, old.x << 16);
              v1 += __builtin_bit_cast(float, old.x & 0xffff0000u);
              v2 += __builtin_bit_cast(float, old.y << 16);
              v3 += __builtin_bit_cast(float, old.y & 0xffff0000u);
            }
            u32x2 o;
            o.x = pack_bf16x2(v0, v1);
            o.y = pack_bf16x2(v2, v3);
            *reinterpret_cast<u32x2*>(dst) = o;
          } else {
            f32x4 o = {v0, v1, v2, v3};
            if (accumulate) o += *reinterpret_cast<const f32x4*>(dst);
            *reinterpret_cast<f32x4*>(dst) = o;
          }
        }
      }
    }
  }
};


// ---- pipelined variant: global -> LDS without passing through registers ------------------
// Differences from Gemm above:
//  * tiles are fetched with buffer loads that write straight into LDS (16 bytes
//    per lane, 1 KiB per wavefront instruction).  The XOR swizzle is applied by
//    choosing WHICH global unit a lane fetches, because the LDS side of such a
//    load is always lane-contiguous;
//  * two LDS stages, and the hand-over point sits before the LAST MFMA block of
//    a K tile: by then every wavefront holds that tile's last operands in
//    registers, so after one barrier the stage can be refilled with tile kt+2
//    while the first operands of tile kt+1 are read under the remaining MFMAs.
//    A tile's loads are thus in flight for a whole K tile, and neither the
//    barrier nor LDS latency is exposed;
//  * operands are read one MFMA block ahead (register double buffering);
//  * the K advance of the global addresses rides in the scalar offset of the
//    buffer instruction: no per-iteration address arithmetic in vector registers.
template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT, typename InT = __bf16>
struct GemmDirect {
  static constexpr int BK = 64;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int UB = BN / 8;                         // 16-byte units per y-tile row
  static constexpr int kAInstr = BM / 8 / kWaves;           // 1 KiB = 8 x-tile rows
  static constexpr int kBRowsPerInstr = 64 / UB;
  static constexpr int kBInstr = BK / kBRowsPerInstr / kWaves;
  static constexpr int kABytes = BM * BK * 2, kBBytes = BK * BN * 2;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert(BM % (8 * kWaves) == 0 && BK % (kBRowsPerInstr * kWaves) == 0, "tile must split evenly");
  static_assert(UB >= 16 && UB <= 64, "y-tile row must be 16..64 units");

  __device__ static __forceinline__ int a_lds_off(int r, int u) { return r * (BK * 2) + ((u ^ ((r >> 1) & 7)) << 4); }
  __device__ static __forceinline__ int b_lds_off(int r, int u) { return r * (BN * 2) + ((u ^ ((r & 3) << 2)) << 4); }

  struct Frags {
    bf16x8 a[TM], b[TN];
  };

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             int32_t k_total, const TileGrid& g, int32_t accumulate) {
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    run_tile(z, x, y, k_total, pm, pn, accumulate);
  }

  // gemm_persistent (cutile-examples/examples/persistent_gemm.rs:35-59): workgroup b computes the
  // tiles of stream items b, b + gridDim.x, ... of the mapped output partition, from zero
  // accumulators.  Workgroups are dealt round-robin to the XCDs, so item i is first sent to
  // position (i % 8) * (total / 8) + i / 8 of the schedule (a bijection when 8 divides the
  // total): each XCD then walks one contiguous eighth of the grouped order and its L2 sees
  // neighbouring tiles, as in the one-tile-per-workgroup launch.
  __device__ static void run_persistent(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                        const MappedArg& m) {
    for (uint32_t item = blockIdx.x; item < m.total; item += gridDim.x) {
      const uint32_t pos = m.total % kNumXcd == 0 ? (item % kNumXcd) * (m.total / kNumXcd) + item / kNumXcd : item;
      uint32_t bid[3];
      mapped_index(m, pos, bid);
      run_tile(z, x, y, x.shape[1], bid[0], bid[1], 0);
      __syncthreads();   // the output bands live in the stages that the next tile refills
    }
  }

  __device__ static __forceinline__ void run_tile(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                                  int32_t k_total, uint32_t pm, uint32_t pn, int32_t accumulate) {
    // Two separately named stages so that the compiler can tell a refill of one
    // from operand reads of the other.
    __shared__ __attribute__((aligned(1024))) unsigned char stage0[kStageBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char stage1[kStageBytes];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int32_t M = x.shape[0], N = y.shape[1];
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;
    const int32_t k_valid = min(min(x.shape[1], y.shape[0]), k_total);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)(((int64_t)(M - 1) * lda + x.shape[1]) * 2));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)(((int64_t)(y.shape[0] - 1) * ldb + N) * 2));
    constexpr uint32_t kOob = 0x80000000u;

    // Global side of the tile fetches (per lane, K tile 0; the K advance is scalar).
    uint32_t a_goff[kAInstr], b_goff[kBInstr];
    int32_t a_k[kAInstr], b_k[kBInstr];  // K index (within a tile) this lane fetches: for the K tail
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) {
      const int r = (wave * kAInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      a_k[i] = u * 8;
      a_goff[i] = (row0 + r < M) ? (uint32_t)(((int64_t)(row0 + r) * lda + u * 8) * 2) : kOob;
    }
#pragma unroll
    for (int i = 0; i < kBInstr; ++i) {
      const int r = (wave * kBInstr + i) * kBRowsPerInstr + lane / UB;
      const int u = (lane % UB) ^ ((r & 3) << 2);
      b_k[i] = r;
      b_goff[i] = (col0 + u * 8 < N) ? (uint32_t)(((int64_t)r * ldb + col0 + u * 8) * 2) : kOob;
    }
    auto fetch_tile = [&](unsigned char* stage, int32_t k0) {
      if (k0 + BK > k_valid) {  // uniform; only the last tile can be short: lanes beyond K fetch zeros
#pragma unroll
        for (int i = 0; i < kAInstr; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(stage + (wave * kAInstr + i) * 1024), 16,
                                                   k0 + a_k[i] >= k_valid ? kOob : a_goff[i], k0 * 2, 0, 0);
#pragma unroll
        for (int i = 0; i < kBInstr; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(stage + kABytes + (wave * kBInstr + i) * 1024),
                                                   16, k0 + b_k[i] >= k_valid ? kOob : b_goff[i], k0 * ldb * 2, 0, 0);
      } else {
#pragma unroll
        for (int i = 0; i < kAInstr; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(stage + (wave * kAInstr + i) * 1024), 16,
                                                   a_goff[i], k0 * 2, 0, 0);
#pragma unroll
        for (int i = 0; i < kBInstr; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(stage + kABytes + (wave * kBInstr + i) * 1024),
                                                   16, b_goff[i], k0 * ldb * 2, 0, 0);
      }
    };

    // LDS side of the operand reads (byte offsets inside a stage).
    const int l32 = lane & 31, khalf = lane >> 5;
    const int grp = lane >> 4, l16 = lane & 15;
    const int tr_row = l16 >> 2, tr_col = (l16 & 3) * 4;
    int a_addr[TM][4], b_addr[TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) a_addr[tm][ks] = a_lds_off(wm * WM + tm * 32 + l32, ks * 2 + khalf);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int n = wn * WN + tn * 32 + (grp & 1) * 16 + tr_col;
      const int kr = (grp >> 1) * 8 + tr_row;  // (kr & 3) does not depend on ks: the swizzle term is fixed
      b_addr[tn] = kABytes + b_lds_off(kr, n >> 3) + (n & 7) * 2;
    }
    auto read_frags = [&](const unsigned char* stage, int ks, Frags& f) {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) f.a[tm] = *reinterpret_cast<const bf16x8*>(stage + a_addr[tm][ks]);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const unsigned char* p = stage + b_addr[tn] + ks * 16 * (BN * 2);
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p);
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p + 4 * (BN * 2)));
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        f.b[tn] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;
    auto mfma_block = [&](const Frags& f) {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          acc[tn][tm] = mfma_32x32x16<InT>(f.b[tn], f.a[tm], acc[tn][tm]);
    };

    const int k_tiles = (k_total + BK - 1) / BK;
    Frags f0, f1;
    if (k_tiles > 0) {
      fetch_tile(stage0, 0);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (k_tiles > 1) fetch_tile(stage1, BK);
      read_frags(stage0, 0, f0);
    }

    // ---- steady state: one memory instruction group per MFMA ----------------------------
    // A wavefront issues in order and an MFMA holds the issue slot until the matrix
    // pipe accepts it, so whatever follows a run of MFMAs starts late and whatever
    // precedes it delays the pipe.  Operand reads (one MFMA block ahead) and the
    // refill of the stage just released are therefore dealt out between the MFMAs,
    // at most two per MFMA; sched_barrier(0) after every step keeps that order.
    constexpr int NB = TM * TN;          // MFMAs per block (one 16-wide K step)
    constexpr int NR = TM + TN;          // operand fragments per block, issue order b0, a0..a(TM-1), b1..
    auto read_operand = [&](const unsigned char* stage, int ks, Frags& f, int r) {
      if (r >= 1 && r <= TM) {
        f.a[r - 1] = *reinterpret_cast<const bf16x8*>(stage + a_addr[r - 1][ks]);
      } else {
        const int tn = r == 0 ? 0 : r - TM;
        const unsigned char* p = stage + b_addr[tn] + ks * 16 * (BN * 2);
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p);
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p + 4 * (BN * 2)));
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        f.b[tn] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };
    auto fetch_one = [&](unsigned char* stage, int32_t k0, int i) {
      if (i < kAInstr)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(stage + (wave * kAInstr + i) * 1024), 16,
                                                 a_goff[i], k0 * 2, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(stage + kABytes + (wave * kBInstr + (i - kAInstr)) * 1024),
                                                 16, b_goff[i - kAInstr], k0 * ldb * 2, 0, 0);
    };
    // MFMAs of one block on `use`, with the fragments of (rd_stage, rd_ks) read into
    // `into` during the first READ_SLOTS MFMAs and, if REFILL, tile k0 fetched into
    // `fill` during the first FETCH_SLOTS.
    constexpr int READ_SLOTS = NB / 2 > 0 ? NB / 2 : 1;
    constexpr int NF = kAInstr + kBInstr;
    constexpr int FETCH_SLOTS = NB / 2 > 0 ? NB / 2 : 1;
    auto block = [&](const unsigned char* rd_stage, int rd_ks, Frags& into, const Frags& use, bool refill,
                     unsigned char* fill, int32_t k0) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        if (refill) {
#pragma unroll
          for (int i = 0; i < NF; ++i)
            if (i * FETCH_SLOTS / NF == j) fetch_one(fill, k0, i);
        }
#pragma unroll
        for (int r = 0; r < NR; ++r)
          if (r * READ_SLOTS / NR == j) read_operand(rd_stage, rd_ks, into, r);
        acc[j / TM][j % TM] =
            mfma_32x32x16<InT>(use.b[j / TM], use.a[j % TM], acc[j / TM][j % TM]);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    auto k_tile_fast = [&](unsigned char* cur, unsigned char* nxt, int kt) {
      block(cur, 1, f1, f0, false, nullptr, 0);
      block(cur, 2, f0, f1, false, nullptr, 0);
      block(cur, 3, f1, f0, false, nullptr, 0);
      // Hand-over: all of `cur` is in registers, this wavefront's share of tile
      // kt+1 has landed in `nxt`.
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      block(nxt, 0, f0, f1, true, cur, (kt + 2) * BK);
    };

    // One K tile, any position: `cur` is being multiplied, `nxt` holds (or is
    // receiving) tile kt+1.  Used for the last tiles, where the refill may be short
    // or absent.
    auto k_tile = [&](unsigned char* cur, unsigned char* nxt, int kt) {
      read_frags(cur, 1, f1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_block(f0);
      __builtin_amdgcn_sched_barrier(0);
      read_frags(cur, 2, f0);
      __builtin_amdgcn_sched_barrier(0);
      mfma_block(f1);
      __builtin_amdgcn_sched_barrier(0);
      read_frags(cur, 3, f1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_block(f0);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (kt + 2 < k_tiles) fetch_tile(cur, (kt + 2) * BK);
      if (kt + 1 < k_tiles) read_frags(nxt, 0, f0);
      __builtin_amdgcn_sched_barrier(0);
      mfma_block(f1);
      __builtin_amdgcn_sched_barrier(0);
    };
    // Tiles whose refill (tile kt+2) lies wholly inside K take the fast path.
    const int fast_end = k_valid / BK - 2;  // kt < fast_end  <=>  (kt + 3) * BK <= k_valid
    int kt = 0;
    for (; kt + 1 < fast_end; kt += 2) {
      k_tile_fast(stage0, stage1, kt);
      k_tile_fast(stage1, stage0, kt + 1);
    }
    for (; kt < k_tiles; kt += 2) {
      k_tile(stage0, stage1, kt);
      if (kt + 1 < k_tiles) k_tile(stage1, stage0, kt + 1);
    }

    // Every wavefront is past its operand reads and every fetch has landed: the
    // stages are free to carry the output.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    static_assert(kWaves / 2 * kEpilogueBytesPerWave<WN> <= kStageBytes, "the output bands must fit the stages");
    unsigned char* band = (wave < kWaves / 2 ? stage0 : stage1) + (wave % (kWaves / 2)) * kEpilogueBytesPerWave<WN>;
    store_tile_staged<TM, TN, OutT>(acc, band, (OutT*)z.ptr, z.strides[0],
                                    z.shape[0], z.shape[1], row0 + wm * WM, col0 + wn * WN, lane, accumulate);
  }
};

// ---- ring variant: three x stages, two y stages released by halves -----------------------
// The two-stage pipeline above gives a tile's loads one K tile of time to land,
// and the matrix pipes were measured waiting on them for about a quarter of the
// run.  Here every load has at least one and a half K tiles:
//  * the x tile (K-contiguous rows, consumed by column slices) can only be
//    released as a whole, so it gets three stages: tile kt+3 is fetched when
//    tile kt is released, two tiles before its first use;
//  * the y tile is consumed by rows, so its two stages are released by halves:
//    K rows 0..31 after the first MFMA block of a tile, K rows 32..63 at the
//    hand-over before the last block; each half is refilled at once with the
//    same half of tile kt+2;
//  * loads complete in issue order, so both barriers of a K tile wait with
//    vmcnt(kAInstr + kBInstr): exactly the loads needed next have landed, one
//    tile's worth of younger ones stays in flight;
//  * fetches past the end of K read zeros through the descriptor's range check,
//    so the loop has one shape for every tile, including a ragged last one.
// LDS: 3 * BM*BK*2 + 2 * BK*BN*2 bytes (160 KiB for 256x256).
template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT, typename InT = __bf16>
struct GemmRing {
  static constexpr int BK = 64;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int UB = BN / 8;                         // 16-byte units per y-tile row
  static constexpr int kAInstr = BM / 8 / kWaves;           // 1 KiB = 8 x-tile rows
  static constexpr int kBRowsPerInstr = 64 / UB;
  static constexpr int kBInstr = BK / kBRowsPerInstr / kWaves;
  static constexpr int kABytes = BM * BK * 2, kBBytes = BK * BN * 2;
  static constexpr int kLdsBytes = 3 * kABytes + 2 * kBBytes;
  static_assert(BM % (8 * kWaves) == 0 && BK % (kBRowsPerInstr * kWaves) == 0, "tile must split evenly");
  static_assert(UB >= 16 && UB <= 64, "y-tile row must be 16..64 units");
  static_assert(kBInstr % 2 == 0, "each wavefront fetches the same share of both y halves");
  static_assert(kAInstr + kBInstr <= 15, "the wait count must fit the low vmcnt field");

  __device__ static __forceinline__ int a_lds_off(int r, int u) { return r * (BK * 2) + ((u ^ ((r >> 1) & 7)) << 4); }
  __device__ static __forceinline__ int b_lds_off(int r, int u) { return r * (BN * 2) + ((u ^ ((r & 3) << 2)) << 4); }

  struct Frags {
    bf16x8 a[TM], b[TN];
  };

  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             int32_t k_total, const TileGrid& g, int32_t accumulate) {
    // Separately named stages: the compiler can then tell a refill of one from
    // operand reads of another and adds no waits of its own.
    __shared__ __attribute__((aligned(1024))) unsigned char xs0[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs1[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs2[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char ys0a[kBBytes / 2];  // y stage 0, K rows 0..31
    __shared__ __attribute__((aligned(1024))) unsigned char ys0b[kBBytes / 2];  //            K rows 32..63
    __shared__ __attribute__((aligned(1024))) unsigned char ys1a[kBBytes / 2];
    __shared__ __attribute__((aligned(1024))) unsigned char ys1b[kBBytes / 2];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    const int32_t M = x.shape[0], N = y.shape[1];
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;
    const int32_t k_valid = min(min(x.shape[1], y.shape[0]), k_total);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)(((int64_t)(M - 1) * lda + x.shape[1]) * 2));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)(((int64_t)(y.shape[0] - 1) * ldb + N) * 2));
    constexpr uint32_t kOob = 0x80000000u;

    // Global side of the fetches (per lane, K tile 0; the K advance is scalar).
    // y instruction i of this wavefront covers K rows of half i / (kBInstr/2).
    uint32_t a_goff[kAInstr], b_goff[kBInstr];
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) {
      const int r = (wave * kAInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      a_goff[i] = (row0 + r < M) ? (uint32_t)(((int64_t)(row0 + r) * lda + u * 8) * 2) : kOob;
    }
#pragma unroll
    for (int i = 0; i < kBInstr; ++i) {
      const int r = (i * kWaves + wave) * kBRowsPerInstr + lane / UB;
      const int u = (lane % UB) ^ ((r & 3) << 2);
      b_goff[i] = (col0 + u * 8 < N) ? (uint32_t)(((int64_t)r * ldb + col0 + u * 8) * 2) : kOob;
    }
    // K is a whole number of tiles here (the launcher sends ragged K to the
    // two-stage variant), so a tile is either wholly inside K or wholly beyond it;
    // beyond it every lane's offset is out of range and the fetch reads zeros.
    auto fetch_a = [&](unsigned char* stage, int32_t k0, int i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(stage + (wave * kAInstr + i) * 1024), 16,
                                               k0 < k_valid ? a_goff[i] : kOob, k0 * 2, 0, 0);
    };
    // `half` = the y half-stage receiving K rows 32*h..32*h+31, h = i / (kBInstr/2)
    auto fetch_b = [&](unsigned char* half, int32_t k0, int i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(half + ((i % (kBInstr / 2)) * kWaves + wave) * 1024),
                                               16, k0 < k_valid ? b_goff[i] : kOob, k0 * ldb * 2, 0, 0);
    };

    // LDS side of the operand reads (byte offsets inside a stage).
    const int l32 = lane & 31, khalf = lane >> 5;
    const int grp = lane >> 4, l16 = lane & 15;
    const int tr_row = l16 >> 2, tr_col = (l16 & 3) * 4;
    int a_addr[TM][4], b_addr[TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) a_addr[tm][ks] = a_lds_off(wm * WM + tm * 32 + l32, ks * 2 + khalf);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int n = wn * WN + tn * 32 + (grp & 1) * 16 + tr_col;
      const int kr = (grp >> 1) * 8 + tr_row;  // (kr & 3) does not depend on ks: the swizzle term is fixed
      b_addr[tn] = b_lds_off(kr, n >> 3) + (n & 7) * 2;
    }
    constexpr int NB = TM * TN;  // MFMAs per block (one 16-wide K step)
    constexpr int NR = TM + TN;  // operand fragments per block, issue order b0, a0..a(TM-1), b1..
    // `yh` = the y half-stage holding K step ks (rows 16*ks..16*ks+15 of the tile)
    auto read_operand = [&](const unsigned char* xs, const unsigned char* yh, int ks, Frags& f, int r) {
      if (r >= 1 && r <= TM) {
        f.a[r - 1] = *reinterpret_cast<const bf16x8*>(xs + a_addr[r - 1][ks]);
      } else {
        const int tn = r == 0 ? 0 : r - TM;
        const unsigned char* p = yh + b_addr[tn] + (ks & 1) * 16 * (BN * 2);
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p);
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p + 4 * (BN * 2)));
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        f.b[tn] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

    // One MFMA block on `use`.  Dealt out between its MFMAs, at most two per
    // MFMA and in this order: refill instructions first..last of the x stage
    // `fill_x` (if any) and of the y stage `fill_y` (instructions fb0..fb1-1),
    // then the reads of (rd_x, rd_y, rd_ks) into `into`.  A wavefront issues in
    // order and an MFMA holds the issue slot until the matrix pipe takes it, so
    // memory work placed after a run of MFMAs would start late; sched_barrier(0)
    // after every step keeps the order written here.
    constexpr int SLOTS = NB / 2 > 0 ? NB / 2 : 1;
    auto block = [&](const Frags& use, const unsigned char* rd_x, const unsigned char* rd_y, int rd_ks, Frags& into,
                     unsigned char* fill_x, unsigned char* fill_y, int fb0, int fb1, int32_t k0_x, int32_t k0_y) {
      const int n_fill = (fill_x ? kAInstr : 0) + (fb1 - fb0);
#pragma unroll
      for (int j = 0; j < NB; ++j) {
#pragma unroll
        for (int i = 0; i < kAInstr + kBInstr; ++i) {
          if (i < n_fill && i * SLOTS / n_fill == j) {
            if (fill_x && i < kAInstr)
              fetch_a(fill_x, k0_x, i);
            else
              fetch_b(fill_y, k0_y, fb0 + i - (fill_x ? kAInstr : 0));
          }
        }
#pragma unroll
        for (int r = 0; r < NR; ++r)
          if (r * SLOTS / NR == j) read_operand(rd_x, rd_y, rd_ks, into, r);
        acc[j / TM][j % TM] =
            mfma_32x32x16<InT>(use.b[j / TM], use.a[j % TM], acc[j / TM][j % TM]);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // s_waitcnt immediate of gfx9: vmcnt [3:0] (and [15:14]), expcnt [6:4], lgkmcnt [11:8].
    constexpr int kWaitOlderLoads = (kAInstr + kBInstr) | (7 << 4) | (0 << 8);
    constexpr int kWaitPrologue = ((2 * kAInstr + 3 * kBInstr / 2) & 15) | (7 << 4) | (0 << 8) | (((2 * kAInstr + 3 * kBInstr / 2) >> 4) << 14);

    const int k_tiles = (k_total + BK - 1) / BK;
    Frags f0, f1;
    // Prologue, in the issue order the steady state would have produced.
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs0, 0, i);
#pragma unroll
    for (int i = 0; i < kBInstr / 2; ++i) fetch_b(ys0a, 0, i);
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs1, BK, i);
#pragma unroll
    for (int i = kBInstr / 2; i < kBInstr; ++i) fetch_b(ys0b, 0, i);
#pragma unroll
    for (int i = 0; i < kBInstr / 2; ++i) fetch_b(ys1a, BK, i);
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs2, 2 * BK, i);
#pragma unroll
    for (int i = kBInstr / 2; i < kBInstr; ++i) fetch_b(ys1b, BK, i);
    __builtin_amdgcn_s_waitcnt(kWaitPrologue);  // x tile 0 and the first y half of tile 0 have landed
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < NR; ++r) read_operand(xs0, ys0a, 0, f0, r);

    // Tile kt lives in x_cur and the y halves (ya_cur, yb_cur); tile kt+1 in x_nxt, ya_nxt.
    auto k_tile = [&](unsigned char* x_cur, unsigned char* ya_cur, unsigned char* yb_cur, const unsigned char* x_nxt,
                      const unsigned char* ya_nxt, int kt) {
      block(f0, x_cur, ya_cur, 1, f1, nullptr, nullptr, 0, 0, 0, 0);
      // First y half of tile kt is in registers everywhere; its second half has landed.
      __builtin_amdgcn_s_waitcnt(kWaitOlderLoads);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      block(f1, x_cur, yb_cur, 2, f0, nullptr, ya_cur, 0, kBInstr / 2, 0, (kt + 2) * BK);
      block(f0, x_cur, yb_cur, 3, f1, nullptr, nullptr, 0, 0, 0, 0);
      // Hand-over: all of tile kt is in registers; x tile kt+1 and its first y half have landed.
      __builtin_amdgcn_s_waitcnt(kWaitOlderLoads);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      block(f1, x_nxt, ya_nxt, 0, f0, x_cur, yb_cur, kBInstr / 2, kBInstr, (kt + 3) * BK, (kt + 2) * BK);
    };
    // The stage names repeat every 6 tiles (3 x stages, 2 y stages).
    int kt = 0;
    for (; kt + 6 <= k_tiles; kt += 6) {
      k_tile(xs0, ys0a, ys0b, xs1, ys1a, kt);
      k_tile(xs1, ys1a, ys1b, xs2, ys0a, kt + 1);
      k_tile(xs2, ys0a, ys0b, xs0, ys1a, kt + 2);
      k_tile(xs0, ys1a, ys1b, xs1, ys0a, kt + 3);
      k_tile(xs1, ys0a, ys0b, xs2, ys1a, kt + 4);
      k_tile(xs2, ys1a, ys1b, xs0, ys0a, kt + 5);
    }
    const int rest = k_tiles - kt;
    if (rest > 0) k_tile(xs0, ys0a, ys0b, xs1, ys1a, kt);
    if (rest > 1) k_tile(xs1, ys1a, ys1b, xs2, ys0a, kt + 1);
    if (rest > 2) k_tile(xs2, ys0a, ys0b, xs0, ys1a, kt + 2);
    if (rest > 3) k_tile(xs0, ys1a, ys1b, xs1, ys0a, kt + 3);
    if (rest > 4) k_tile(xs1, ys0a, ys0b, xs2, ys1a, kt + 4);
    __builtin_amdgcn_s_waitcnt(0);  // trailing (zero-filling) fetches must not outlive the workgroup's LDS

    // Every wavefront is past its operand reads and every fetch has landed: the
    // stages are free to carry the output (two wavefronts share an x stage, the
    // last two take the y stages).
    __syncthreads();
    static_assert(2 * kEpilogueBytesPerWave<WN> <= kABytes && kEpilogueBytesPerWave<WN> <= kBBytes / 2 && kWaves <= 10,
                  "the output bands must fit the stages");
    unsigned char* band = wave < 2 ? xs0 : wave < 4 ? xs1 : wave < 6 ? xs2 : wave == 6 ? ys0a : wave == 7 ? ys0b : wave == 8 ? ys1a : ys1b;
    if (wave < 6) band += (wave & 1) * kEpilogueBytesPerWave<WN>;
    store_tile_staged<TM, TN, OutT>(acc, band, (OutT*)z.ptr, z.strides[0], z.shape[0], z.shape[1], row0 + wm * WM,
                                    col0 + wn * WN, lane, accumulate);
  }
};

// ---- the ring variant on v_mfma_f32_16x16x32 -----------------------------------------------
// Same stages, fetches, barriers and wait counts as GemmRing; the matrix instruction is the 16 x 16 x 32 form.
// On this chip the matrix kernels run against the power limit, and per flop the 16 x 16 x 32 form writes half as
// many accumulator values as 32 x 32 x 16: a loop of nothing but MFMAs on random bf16 operands sustains
// 2093 TFLOP/s with it against 1854 (equal, 2463 - 2481, on constant operands).  A block is 16 MFMAs (half of the
// sub-tile's rows by all of its columns, one 32-wide K step) and lasts as long as a block of GemmRing; the y
// fragments of a K step serve two blocks, so LDS traffic is unchanged.
template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT, typename InT = __bf16>
struct GemmRing16 {
  static constexpr int BK = 64;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 16, TN = WN / 16;   // 16 x 16 accumulator blocks of the wavefront's sub-tile
  static constexpr int TMH = TM / 2;                   // x fragments of one MFMA block (half the sub-tile's rows)
  static_assert(TM % 2 == 0, "a block takes half of the sub-tile's rows");
  static constexpr int UB = BN / 8;                         // 16-byte units per y-tile row
  static constexpr int kAInstr = BM / 8 / kWaves;           // 1 KiB = 8 x-tile rows
  static constexpr int kBRowsPerInstr = 64 / UB;
  static constexpr int kBInstr = BK / kBRowsPerInstr / kWaves;
  static constexpr int kABytes = BM * BK * 2, kBBytes = BK * BN * 2;
  static constexpr int kLdsBytes = 3 * kABytes + 2 * kBBytes;
  static_assert(BM % (8 * kWaves) == 0 && BK % (kBRowsPerInstr * kWaves) == 0, "tile must split evenly");
  static_assert(UB >= 16 && UB <= 64, "y-tile row must be 16..64 units");
  static_assert(kBInstr % 2 == 0, "each wavefront fetches the same share of both y halves");
  static_assert(kAInstr + kBInstr <= 15, "the wait count must fit the low vmcnt field");

  __device__ static __forceinline__ int a_lds_off(int r, int u) { return r * (BK * 2) + ((u ^ ((r >> 1) & 7)) << 4); }
  // y rows 8 apart are read by neighbouring lane groups of one transposing read: bit 3 of the row moves them 32 bytes apart
  __device__ static __forceinline__ int b_swizzle(int r) { return ((r & 3) << 2) | (((r >> 3) & 1) << 1); }
  __device__ static __forceinline__ int b_lds_off(int r, int u) { return r * (BN * 2) + ((u ^ b_swizzle(r)) << 4); }


  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                             int32_t k_total, const TileGrid& g, int32_t accumulate) {
    uint32_t pm, pn;
    tile_coords(g.x, g.y, &pm, &pn);
    run_tile(z, x, y, k_total, pm, pn, accumulate);
  }

  // gemm_persistent: workgroup b computes the tiles of stream items b, b + gridDim.x, ... of the mapped output
  // partition from zero accumulators, in the XCD-contiguous order of GemmDirect::run_persistent.
  __device__ static void run_persistent(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                        const MappedArg& m) {
    for (uint32_t item = blockIdx.x; item < m.total; item += gridDim.x) {
      const uint32_t pos = m.total % kNumXcd == 0 ? (item % kNumXcd) * (m.total / kNumXcd) + item / kNumXcd : item;
      uint32_t bid[3];
      mapped_index(m, pos, bid);
      run_tile(z, x, y, x.shape[1], bid[0], bid[1], 0);
      __syncthreads();   // the output bands live in the stages that the next tile refills
    }
  }

  // gemm launched with one workgroup per compute unit ("p"): workgroup b walks the tiles b, b + gridDim.x, ... of the
  // launch's XCD-contiguous, M-grouped order, tile after tile with the full tile body (any extents, any K, z as the
  // initial accumulator or not).  Against one workgroup per tile it saves the workgroup starts and keeps each XCD on
  // one contiguous eighth of the order round by round.
  __device__ static void run_walk(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y, int32_t k_total,
                                  const TileGrid& g, int32_t accumulate) {
    const uint32_t total = g.x * g.y;
    for (uint32_t item = blockIdx.x; item < total; item += gridDim.x) {
      uint32_t pm, pn;
      tile_of_id(item, g.x, g.y, gridDim.x, &pm, &pn);
      run_tile(z, x, y, k_total, pm, pn, accumulate);
      __syncthreads();   // the output bands live in the stages that the next tile refills
    }
  }

  __device__ static __forceinline__ void run_tile(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                                  int32_t k_total, uint32_t pm, uint32_t pn, int32_t accumulate) {
    // Separately named stages: the compiler can then tell a refill of one from
    // operand reads of another and adds no waits of its own.
    __shared__ __attribute__((aligned(1024))) unsigned char xs0[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs1[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs2[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char ys0a[kBBytes / 2];  // y stage 0, K rows 0..31
    __shared__ __attribute__((aligned(1024))) unsigned char ys0b[kBBytes / 2];  //            K rows 32..63
    __shared__ __attribute__((aligned(1024))) unsigned char ys1a[kBBytes / 2];
    __shared__ __attribute__((aligned(1024))) unsigned char ys1b[kBBytes / 2];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int32_t M = x.shape[0], N = y.shape[1];
    const int32_t lda = x.strides[0], ldb = y.strides[0];
    const int32_t row0 = pm * BM, col0 = pn * BN;
    const int32_t k_valid = min(min(x.shape[1], y.shape[0]), k_total);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)(((int64_t)(M - 1) * lda + x.shape[1]) * 2));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)(((int64_t)(y.shape[0] - 1) * ldb + N) * 2));
    constexpr uint32_t kOob = 0x80000000u;

    // Global side of the fetches (per lane, K tile 0; the K advance is scalar).
    // y instruction i of this wavefront covers K rows of half i / (kBInstr/2).
    // A lane fetches K positions k0 + 8 u .. + 7 of an x row and K row k0 + r of y: past the end of K (a ragged last
    // tile, or a trailing fetch beyond the last one) its offset is out of range and the fetch brings zeros.  K is a
    // multiple of 8, so a 16-byte unit is wholly inside K or wholly beyond it.
    uint32_t a_goff[kAInstr], b_goff[kBInstr];
    int32_t a_klim[kAInstr];      // k0 < a_klim[i]  <=>  the lane's unit of instruction i lies inside K
    const int32_t b_klim = k_valid - (int32_t)(lane / UB);   // k0 + (first row of the instruction) < b_klim  <=>  the lane's row does
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) {
      const int r = (wave * kAInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      a_goff[i] = (row0 + r < M) ? (uint32_t)(((int64_t)(row0 + r) * lda + u * 8) * 2) : kOob;
      a_klim[i] = k_valid - u * 8;
    }
#pragma unroll
    for (int i = 0; i < kBInstr; ++i) {
      const int r = (i * kWaves + wave) * kBRowsPerInstr + lane / UB;
      const int u = (lane % UB) ^ b_swizzle(r);
      b_goff[i] = (col0 + u * 8 < N) ? (uint32_t)(((int64_t)r * ldb + col0 + u * 8) * 2) : kOob;
    }
    auto fetch_a = [&](unsigned char* stage, int32_t k0, int i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(stage + (wave * kAInstr + i) * 1024), 16,
                                               k0 < a_klim[i] ? a_goff[i] : kOob, k0 * 2, 0, 0);
    };
    // `half` = the y half-stage receiving K rows 32*h..32*h+31, h = i / (kBInstr/2)
    auto fetch_b = [&](unsigned char* half, int32_t k0, int i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(half + ((i % (kBInstr / 2)) * kWaves + wave) * 1024),
                                               16, k0 + (i * kWaves + wave) * kBRowsPerInstr < b_klim ? b_goff[i] : kOob,
                                               k0 * ldb * 2, 0, 0);
    };

    // LDS side of the operand reads (byte offsets inside a stage).  v_mfma_f32_16x16x32: a lane holds 8 consecutive K
    // values (group lane / 16 of the 32-wide K step) of row lane % 16 of its operand.
    const int grp = lane >> 4, l16 = lane & 15;
    const int tr_row = l16 >> 2, tr_col = (l16 & 3) * 4;
    // x: the swizzle term of row r + 16 tm is that of row r, so one address per K step serves all row blocks
    // (16 rows = 16 * BK * 2 bytes further on, an immediate offset of the read)
    int a_addr[2], b_addr[TN];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) a_addr[ks] = a_lds_off(wm * WM + l16, ks * 4 + grp);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int n = wn * WN + tn * 16 + tr_col;
      const int kr = grp * 8 + tr_row;         // row inside the y half-stage that holds this K step; the swizzle of kr + 4 is the same
      b_addr[tn] = b_lds_off(kr, n >> 3) + (n & 7) * 2;
    }
    constexpr int NB = TMH * TN;  // MFMAs per block: half the sub-tile's rows, one 32-wide K step
    // x fragments i of rows [mh * TMH * 16, ..) at K step ks of stage xs
    auto read_a = [&](const unsigned char* xs, int ks, int mh, bf16x8 (&into)[TMH], int i) {
      into[i] = *reinterpret_cast<const bf16x8*>(xs + a_addr[ks] + (mh * TMH + i) * (16 * BK * 2));
    };
    // y fragment tn of the K step held by the half-stage yh
    auto read_b = [&](const unsigned char* yh, bf16x8 (&into)[TN], int tn) {
      const unsigned char* p = yh + b_addr[tn];
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p);
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p + 4 * (BN * 2)));
      into[tn] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    f32x4 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[tn][tm][v] = 0.0f;

    // One MFMA block: rows [mh * TMH * 16, ..) of the sub-tile times all its columns, on the x fragments `a` and the
    // y fragments `ub`, row block by row block.  Dealt out between its MFMAs in this
    // order: refill instructions first..last of the x stage `fill_x` (if any) and of the y stage `fill_y`
    // (instructions fb0..fb1-1), then, if rd_y, the reads of the next K step's y fragments into `ib`.  The x
    // fragments are one set: as soon as the last MFMA on a row block has issued, its fragment is read again for the
    // next block (rd_x, rd_ks, rd_mh) — three row blocks of MFMAs before it is used.  A wavefront issues in order
    // and an MFMA holds the issue slot until the matrix pipe takes it, so memory work placed after a run of MFMAs
    // would start late; sched_barrier(0) after every step keeps the order written here.
    constexpr int SLOTS = NB;   // memory instructions spread over all the block's MFMAs: one per MFMA at most (measured +3 % over the first half only)
    // (what a block does besides its MFMAs is said by the flags with_y / with_fill_x and the range fb0..fb1: a null
    // test of an LDS pointer is a run-time test, address 0 being a valid one)
    auto block = [&](bf16x8 (&a)[TMH], const bf16x8 (&ub)[TN], int mh, const unsigned char* rd_x, int rd_ks, int rd_mh,
                     bool with_y, const unsigned char* rd_y, bf16x8 (&ib)[TN], bool with_fill_x, unsigned char* fill_x,
                     unsigned char* fill_y, int fb0, int fb1, int32_t k0_x, int32_t k0_y) {
      const int n_fill = (with_fill_x ? kAInstr : 0) + (fb1 - fb0);
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int tm = j / TN, tn = j % TN;
#pragma unroll
        for (int i = 0; i < kAInstr + kBInstr; ++i) {
          if (i < n_fill && i * SLOTS / n_fill == j) {
            if (with_fill_x && i < kAInstr)
              fetch_a(fill_x, k0_x, i);
            else
              fetch_b(fill_y, k0_y, fb0 + i - (with_fill_x ? kAInstr : 0));
          }
        }
        if (with_y) {
#pragma unroll
          for (int q = 0; q < TN; ++q)
            if (q * SLOTS / TN == j) read_b(rd_y, ib, q);
        }
        acc[tn][mh * TMH + tm] = mfma_16x16x32<InT>(ub[tn], a[tm], acc[tn][mh * TMH + tm]);
        if (tn == TN - 1) read_a(rd_x, rd_ks, rd_mh, a, tm);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // s_waitcnt immediate of gfx9: vmcnt [3:0] (and [15:14]), expcnt [6:4], lgkmcnt [11:8].
    constexpr int kWaitOlderLoads = (kAInstr + kBInstr) | (7 << 4) | (0 << 8);
    constexpr int kWaitPrologue = ((2 * kAInstr + 3 * kBInstr / 2) & 15) | (7 << 4) | (0 << 8) | (((2 * kAInstr + 3 * kBInstr / 2) >> 4) << 14);

    const int k_tiles = (k_total + BK - 1) / BK;
    bf16x8 af[TMH], b0[TN], b1[TN];
    // Prologue, in the issue order the steady state would have produced.
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs0, 0, i);
#pragma unroll
    for (int i = 0; i < kBInstr / 2; ++i) fetch_b(ys0a, 0, i);
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs1, BK, i);
#pragma unroll
    for (int i = kBInstr / 2; i < kBInstr; ++i) fetch_b(ys0b, 0, i);
#pragma unroll
    for (int i = 0; i < kBInstr / 2; ++i) fetch_b(ys1a, BK, i);
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs2, 2 * BK, i);
#pragma unroll
    for (int i = kBInstr / 2; i < kBInstr; ++i) fetch_b(ys1b, BK, i);
    __builtin_amdgcn_s_waitcnt(kWaitPrologue);  // x tile 0 and the first y half of tile 0 have landed
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) read_b(ys0a, b0, tn);
#pragma unroll
    for (int i = 0; i < TMH; ++i) read_a(xs0, 0, 0, af, i);

    // Tile kt lives in x_cur and the y halves (ya_cur, yb_cur); tile kt+1 in x_nxt, ya_nxt.
    auto k_tile = [&](unsigned char* x_cur, unsigned char* ya_cur, unsigned char* yb_cur, const unsigned char* x_nxt,
                      const unsigned char* ya_nxt, int kt) {
      // blocks: (K step 0, upper rows) (K step 0, lower rows) (K step 1, upper) (K step 1, lower); every block reads
      // the next block's x fragments, the second and the fourth also the next K step's y fragments
      block(af, b0, 0, x_cur, 0, 1, false, x_cur, b1, false, x_cur, x_cur, 0, 0, 0, 0);
      // First y half of tile kt is in registers everywhere; its second half has landed.
      __builtin_amdgcn_s_waitcnt(kWaitOlderLoads);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      block(af, b0, 1, x_cur, 1, 0, true, yb_cur, b1, false, x_cur, ya_cur, 0, kBInstr / 2, 0, (kt + 2) * BK);
      block(af, b1, 0, x_cur, 1, 1, false, x_cur, b0, false, x_cur, x_cur, 0, 0, 0, 0);
      // Hand-over: all of tile kt is in registers; x tile kt+1 and its first y half have landed.
      __builtin_amdgcn_s_waitcnt(kWaitOlderLoads);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      block(af, b1, 1, x_nxt, 0, 0, true, ya_nxt, b0, true, x_cur, yb_cur, kBInstr / 2, kBInstr, (kt + 3) * BK, (kt + 2) * BK);
    };
    // The stage names repeat every 6 tiles (3 x stages, 2 y stages).
    int kt = 0;
    for (; kt + 6 <= k_tiles; kt += 6) {
      k_tile(xs0, ys0a, ys0b, xs1, ys1a, kt);
      k_tile(xs1, ys1a, ys1b, xs2, ys0a, kt + 1);
      k_tile(xs2, ys0a, ys0b, xs0, ys1a, kt + 2);
      k_tile(xs0, ys1a, ys1b, xs1, ys0a, kt + 3);
      k_tile(xs1, ys0a, ys0b, xs2, ys1a, kt + 4);
      k_tile(xs2, ys1a, ys1b, xs0, ys0a, kt + 5);
    }
    const int rest = k_tiles - kt;
    if (rest > 0) k_tile(xs0, ys0a, ys0b, xs1, ys1a, kt);
    if (rest > 1) k_tile(xs1, ys1a, ys1b, xs2, ys0a, kt + 1);
    if (rest > 2) k_tile(xs2, ys0a, ys0b, xs0, ys1a, kt + 2);
    if (rest > 3) k_tile(xs0, ys1a, ys1b, xs1, ys0a, kt + 3);
    if (rest > 4) k_tile(xs1, ys0a, ys0b, xs2, ys1a, kt + 4);
    __builtin_amdgcn_s_waitcnt(0);  // trailing (zero-filling) fetches must not outlive the workgroup's LDS

    // Every wavefront is past its operand reads and every fetch has landed: the
    // stages are free to carry the output (two wavefronts share an x stage, the
    // last two take the y stages).
    __syncthreads();
    static_assert(2 * kEpilogueBytesPerWave<WN> <= kABytes && kEpilogueBytesPerWave<WN> <= kBBytes / 2 && kWaves <= 10,
                  "the output bands must fit the stages");
    unsigned char* band = wave < 2 ? xs0 : wave < 4 ? xs1 : wave < 6 ? xs2 : wave == 6 ? ys0a : wave == 7 ? ys0b : wave == 8 ? ys1a : ys1b;
    if (wave < 6) band += (wave & 1) * kEpilogueBytesPerWave<WN>;
    store_tile_staged16<TM, TN, OutT>(acc, band, (OutT*)z.ptr, z.strides[0], z.shape[0], z.shape[1], row0 + wm * WM,
                                    col0 + wn * WN, lane, accumulate);
  }
};

// ---- the 16 x 16 x 32 ring as one stream over many output tiles ------------------------------
// A workgroup that computes several output tiles one after another (four per compute unit at 8192^3) pays, per tile
// of GemmRing16, for an epilogue through LDS, a barrier because the output bands live in the operand stages, and a
// prologue whose first fetch nothing hides.  Here the operand ring never stops:
//  * the K tiles of a workgroup's output tiles form ONE sequence; the fetch two / three tiles ahead simply runs on
//    into the next output tile's first K tiles (tile origin and K position are both in the scalar offset of the
//    fetch, the per-lane offsets do not depend on the tile), so when the last MFMA of an output tile issues, the
//    next tile's first three x tiles and two y tiles are in LDS or in flight;
//  * the epilogue uses no LDS, so it needs no barrier and leaves the stages alone: two in-ALU exchanges
//    (v_permlane32_swap, v_permlane16_swap) turn the accumulator layout of v_mfma_f32_16x16x32 (a lane: 4
//    consecutive columns of one row, the four lane groups side by side, 16-column blocks in registers) into 8
//    consecutive columns per lane with the four lane groups side by side — each store instruction then writes 16
//    rows of 64 contiguous bytes, and the old z for `accumulate` is read in that same shape, two row blocks ahead;
// Needs whole tiles in M, N and K (the launcher checks; everything else runs GemmRing16) and at least three K tiles.
template <int BM, int BN, int WAVES_M, int WAVES_N, typename OutT, typename InT = __bf16>
struct GemmStream16 {
  static_assert(sizeof(OutT) == 2, "16-bit outputs");
  static constexpr int BK = 64;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 16, TN = WN / 16;
  static constexpr int TMH = TM / 2;
  static_assert(TM % 2 == 0 && TN % 2 == 0, "row blocks by halves, column blocks by pairs");
  static constexpr int UB = BN / 8;
  static constexpr int kAInstr = BM / 8 / kWaves;
  static constexpr int kBRowsPerInstr = 64 / UB;
  static constexpr int kBInstr = BK / kBRowsPerInstr / kWaves;
  static constexpr int kABytes = BM * BK * 2, kBBytes = BK * BN * 2;
  static constexpr int kLdsBytes = 3 * kABytes + 2 * kBBytes;
  static_assert(BM % (8 * kWaves) == 0 && BK % (kBRowsPerInstr * kWaves) == 0, "tile must split evenly");
  static_assert(UB >= 16 && UB <= 64, "y-tile row must be 16..64 units");
  static_assert(kBInstr % 2 == 0, "each wavefront fetches the same share of both y halves");
  static_assert(kAInstr + kBInstr <= 15, "the wait count must fit the low vmcnt field");

  __device__ static __forceinline__ int a_lds_off(int r, int u) { return r * (BK * 2) + ((u ^ ((r >> 1) & 7)) << 4); }
  __device__ static __forceinline__ int b_swizzle(int r) { return ((r & 3) << 2) | (((r >> 3) & 1) << 1); }
  __device__ static __forceinline__ int b_lds_off(int r, int u) { return r * (BN * 2) + ((u ^ b_swizzle(r)) << 4); }

  // The register that held `a` holds zeros afterwards (a tied operand: to the compiler the same value lives on, so the
  // loop that follows accumulates where the last tile did and no second set of accumulator registers appears).
  __device__ static __forceinline__ void clear_in_place(f32x4& a) {
    asm volatile("v_mov_b32 %0, 0\n\tv_mov_b32 %1, 0\n\tv_mov_b32 %2, 0\n\tv_mov_b32 %3, 0"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));
  }
  // upper 32 lanes of a <-> lower 32 lanes of b, component by component.  (Inline assembly on purpose: through the
  // compiler's builtin for this instruction the second result came back as a copy of the first in this kernel.)
  __device__ static __forceinline__ void swap_halves(f32x4& a, f32x4& b) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float p = a[c], q = b[c];
      asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(p), "+v"(q));
      a[c] = p, b[c] = q;
    }
  }
  // odd rows of 16 lanes of a <-> even rows of b
  __device__ static __forceinline__ void swap_rows(f32x4& a, f32x4& b) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float p = a[c], q = b[c];
      asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(p), "+v"(q));
      a[c] = p, b[c] = q;
    }
  }

  // `tile_of(j, &pm, &pn)`: the tile of this workgroup's j-th item, j < n_mine.  ACCUMULATE and STREAM (z read and
  // written past the caches) are compile-time: under a run-time flag the compiler cannot pair the epilogue's loads
  // with their uses and waits for everything in flight, the ring's fetches included.  One instantiation per kernel:
  // the stages below are static arrays of this function.
  template <bool ACCUMULATE, bool STREAM, class TileOf>
  __device__ static __forceinline__ void run_items(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                                   int32_t k_total, uint32_t n_mine, TileOf tile_of) {
    // Separately named stages: the compiler can then tell a refill of one from operand reads of another and adds no
    // waits of its own.
    __shared__ __attribute__((aligned(1024))) unsigned char xs0[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs1[kABytes];
    __shared__ __attribute__((aligned(1024))) unsigned char xs2[kABytes];
    // (the larger alignment puts the y stages first: all four then lie inside the 64 KiB that the immediate offset
    // of an LDS read spans, so one address register per column block serves them all)
    __shared__ __attribute__((aligned(4096))) unsigned char ys0a[kBBytes / 2];
    __shared__ __attribute__((aligned(4096))) unsigned char ys0b[kBBytes / 2];
    __shared__ __attribute__((aligned(4096))) unsigned char ys1a[kBBytes / 2];
    __shared__ __attribute__((aligned(4096))) unsigned char ys1b[kBBytes / 2];
    constexpr bool accumulate = ACCUMULATE, stream = STREAM;
    if (n_mine == 0) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int32_t lda = x.strides[0], ldb = y.strides[0], ldz = z.strides[0];
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(x.ptr, (uint32_t)(((int64_t)(x.shape[0] - 1) * lda + x.shape[1]) * 2));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(y.ptr, (uint32_t)(((int64_t)(y.shape[0] - 1) * ldb + y.shape[1]) * 2));
    const int k_tiles = k_total / BK;

    // Per-lane side of the fetches: the lane's place inside ANY x tile / y tile.  Where the tile lies (its first row
    // or column, its K position) and which of the wavefront's fetch instructions it is go into the scalar offset.
    // x instruction i covers rows (wave * kAInstr + i) * 8 + lane / 8: the swizzle term ((row >> 1) & 7) of a lane
    // repeats with i & 1, so two per-lane offsets serve all of them; y instruction i covers K rows
    // (i * kWaves + wave) * kBRowsPerInstr + lane / UB, whose swizzle term does not depend on i at all: one offset.
    static_assert(kAInstr % 2 == 0 && (kWaves * kBRowsPerInstr) % 16 == 0, "fetch offsets repeat as assumed");
    uint32_t a_voff[2], b_voff;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = (wave * kAInstr + i) * 8 + (lane >> 3);
      const int u = (lane & 7) ^ ((r >> 1) & 7);
      a_voff[i] = (uint32_t)(((int64_t)((wave * kAInstr) * 8 + (lane >> 3)) * lda + u * 8) * 2);   // row of instruction 0: the row step is scalar
    }
    {
      const int r = wave * kBRowsPerInstr + lane / UB;
      const int u = (lane % UB) ^ b_swizzle(r);
      b_voff = (uint32_t)(((int64_t)r * ldb + u * 8) * 2);
    }
    const uint32_t a_istep = (uint32_t)(8 * lda * 2), b_istep = (uint32_t)(kWaves * kBRowsPerInstr * ldb * 2);
    auto fetch_a = [&](unsigned char* stage, uint32_t soff, int i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (LDS_PTR(void))(stage + (wave * kAInstr + i) * 1024), 16, a_voff[i & 1],
                                               (int32_t)(soff + (uint32_t)i * a_istep), 0, 0);
    };
    auto fetch_b = [&](unsigned char* half, uint32_t soff, int i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (LDS_PTR(void))(half + ((i % (kBInstr / 2)) * kWaves + wave) * 1024), 16, b_voff,
                                               (int32_t)(soff + (uint32_t)i * b_istep), 0, 0);
    };

    const int grp = lane >> 4, l16 = lane & 15;
    const int tr_row = l16 >> 2, tr_col = (l16 & 3) * 4;
    // x: the address of K step 1 is that of K step 0 with bit 6 flipped (the K step is bit 2 of the 16-byte unit, which
    // the swizzle only XORs); it is formed where it is used, one instruction per block, instead of living in a register
    // of its own per 64 KiB window of LDS for the whole kernel.
    int a_addr0, b_addr[TN];
    a_addr0 = a_lds_off(wm * WM + l16, grp);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int n = wn * WN + tn * 16 + tr_col;
      const int kr = grp * 8 + tr_row;
      b_addr[tn] = b_lds_off(kr, n >> 3) + (n & 7) * 2;
    }
    constexpr int NB = TMH * TN;
    auto read_a = [&](const unsigned char* xs, int a_at, int mh, bf16x8 (&into)[TMH], int i) {
      into[i] = *reinterpret_cast<const bf16x8*>(xs + a_at + (mh * TMH + i) * (16 * BK * 2));
    };
    auto a_addr_of = [&](int ks) {
      int at = a_addr0;
      if (ks == 1) asm volatile("v_xor_b32 %0, 64, %1" : "=v"(at) : "v"(a_addr0));
      return at;
    };
    auto read_b = [&](const unsigned char* yh, bf16x8 (&into)[TN], int tn) {
      const unsigned char* p = yh + b_addr[tn];
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p);
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p + 4 * (BN * 2)));
      into[tn] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    f32x4 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[tn][tm][v] = 0.0f;

    // One MFMA block, as in GemmRing16 (memory instructions dealt out one per MFMA at most); so_x / so_y are the
    // scalar offsets of the x tile and the y tile being fetched.
    constexpr int SLOTS = NB;
    auto block = [&](bf16x8 (&a)[TMH], const bf16x8 (&ub)[TN], int mh, const unsigned char* rd_x, int rd_ks, int rd_mh,
                     bool with_y, const unsigned char* rd_y, bf16x8 (&ib)[TN], bool with_fill_x, unsigned char* fill_x,
                     unsigned char* fill_y, int fb0, int fb1, uint32_t so_x, uint32_t so_y) {
      const int n_fill = (with_fill_x ? kAInstr : 0) + (fb1 - fb0);
      const int rd_at = a_addr_of(rd_ks);
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int tm = j / TN, tn = j % TN;
#pragma unroll
        for (int i = 0; i < kAInstr + kBInstr; ++i) {
          if (i < n_fill && i * SLOTS / n_fill == j) {
            if (with_fill_x && i < kAInstr)
              fetch_a(fill_x, so_x, i);
            else
              fetch_b(fill_y, so_y, fb0 + i - (with_fill_x ? kAInstr : 0));
          }
        }
        if (with_y) {
#pragma unroll
          for (int q = 0; q < TN; ++q)
            if (q * SLOTS / TN == j) read_b(rd_y, ib, q);
        }
        acc[tn][mh * TMH + tm] = mfma_16x16x32<InT>(ub[tn], a[tm], acc[tn][mh * TMH + tm]);
        if (tn == TN - 1) read_a(rd_x, rd_at, rd_mh, a, tm);
        __builtin_amdgcn_sched_barrier(0);
      }
    };

    // Where the current output tile and the next one lie (scalar): byte offsets of the tile's first x row / y column.
    uint32_t pm, pn;
    tile_of(0u, &pm, &pn);
    uint32_t a_cur = (uint32_t)((int64_t)pm * BM * lda * 2), b_cur = pn * (BN * 2);
    uint32_t z_row = pm * BM, z_col = pn * BN;
    uint32_t a_nxt = a_cur, b_nxt = b_cur, z_row_nxt = z_row, z_col_nxt = z_col;
    auto look_ahead = [&](uint32_t j) {      // the tile after item j, or item j's own once more (fetched, never used)
      if (j + 1 < n_mine) {
        uint32_t qm, qn;
        tile_of(j + 1, &qm, &qn);
        a_nxt = (uint32_t)((int64_t)qm * BM * lda * 2), b_nxt = qn * (BN * 2);
        z_row_nxt = qm * BM, z_col_nxt = qn * BN;
      }
    };
    look_ahead(0);
    const uint32_t y_step = (uint32_t)(BK * ldb * 2);
    // x tile / y tile number kf counted from the current output tile's first: past its last, the next tile's
    auto so_x = [&](int kf) { return kf < k_tiles ? a_cur + (uint32_t)kf * (BK * 2) : a_nxt + (uint32_t)(kf - k_tiles) * (BK * 2); };
    auto so_y = [&](int kf) { return kf < k_tiles ? b_cur + (uint32_t)kf * y_step : b_nxt + (uint32_t)(kf - k_tiles) * y_step; };

    bf16x8 af[TMH], b0[TN], b1[TN];
    // Prologue of the first output tile, in the issue order the steady state would have produced.
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs0, so_x(0), i);
#pragma unroll
    for (int i = 0; i < kBInstr / 2; ++i) fetch_b(ys0a, so_y(0), i);
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs1, so_x(1), i);
#pragma unroll
    for (int i = kBInstr / 2; i < kBInstr; ++i) fetch_b(ys0b, so_y(0), i);
#pragma unroll
    for (int i = 0; i < kBInstr / 2; ++i) fetch_b(ys1a, so_y(1), i);
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) fetch_a(xs2, so_x(2), i);
#pragma unroll
    for (int i = kBInstr / 2; i < kBInstr; ++i) fetch_b(ys1b, so_y(1), i);
    constexpr int kPrologueLeft = 2 * kAInstr + 3 * kBInstr / 2;
    __builtin_amdgcn_s_waitcnt((kPrologueLeft & 15) | (7 << 4) | (0 << 8) | ((kPrologueLeft >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) read_b(ys0a, b0, tn);
#pragma unroll
    for (int i = 0; i < TMH; ++i) read_a(xs0, a_addr0, 0, af, i);

    // K tile kt of the current output tile: GemmRing16's, with the fetches' scalar offsets running on into the next
    // output tile.  Stores and loads share the wavefront's in-order memory counter, so in the first K tile after an
    // epilogue these waits also wait for the older half of the epilogue's stores — by then a K tile's worth of matrix
    // work old.  (Waits with a larger count in that K tile were built: behind a branch the compiler's own
    // bookkeeping of what is in flight turns inexact and it adds waits of its own in front of the operand reads;
    // as a second straight-line copy of the K tile the register allocation falls apart.)
    constexpr int kWaitOlderLoads = (kAInstr + kBInstr) | (7 << 4) | (0 << 8);
    auto k_tile = [&](unsigned char* x_cur, unsigned char* ya_cur, unsigned char* yb_cur, const unsigned char* x_nxt,
                      const unsigned char* ya_nxt, int kt) {
      block(af, b0, 0, x_cur, 0, 1, false, x_cur, b1, false, x_cur, x_cur, 0, 0, 0, 0);
      __builtin_amdgcn_s_waitcnt(kWaitOlderLoads);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      block(af, b0, 1, x_cur, 1, 0, true, yb_cur, b1, false, x_cur, ya_cur, 0, kBInstr / 2, 0, so_y(kt + 2));
      block(af, b1, 0, x_cur, 1, 1, false, x_cur, b0, false, x_cur, x_cur, 0, 0, 0, 0);
      __builtin_amdgcn_s_waitcnt(kWaitOlderLoads);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      block(af, b1, 1, x_nxt, 0, 0, true, ya_nxt, b0, true, x_cur, yb_cur, kBInstr / 2, kBInstr, so_x(kt + 3), so_y(kt + 2));
    };

    // Epilogue of the tile at (z_row, z_col): registers only.  After the two exchanges lane (grp, l16) holds, for row
    // block tm and column pair kp, the 8 consecutive columns kp * 32 + grp * 8 .. + 7 of row tm * 16 + l16.  z is
    // addressed like the operands: one per-lane offset for every access, the rest in the scalar offset.
    const __amdgpu_buffer_rsrc_t rz = make_rsrc(z.ptr, (uint32_t)(((int64_t)(z.shape[0] - 1) * ldz + z.shape[1]) * 2));
    const uint32_t z_voff = (uint32_t)(((int64_t)l16 * ldz + grp * 8) * 2);
    constexpr int kAux = stream ? 2 : 0;      // nt: past the caches
    // row blocks per chunk of old z (a chunk ahead is in flight while one is added): two where the registers allow it;
    // the f16 kernels have four registers fewer to spare and would spill in the K loop
    constexpr int CH = __is_same(OutT, _Float16) ? 1 : 2;
    constexpr int KP = TN / 2;
    auto epilogue = [&]() {
      // scalar offset of row block tm, column pair kp of this wavefront's part of the tile
      auto z_soff = [&](int tm, int kp) {
        return (uint32_t)(((int64_t)(z_row + wm * WM + tm * 16) * ldz + z_col + wn * WN + kp * 32) * 2);
      };
      u32x4 old[2][CH][KP];
      auto load_chunk = [&](int c, u32x4 (&o)[CH][KP]) {
#pragma unroll
        for (int t = 0; t < CH; ++t)
#pragma unroll
          for (int kp = 0; kp < KP; ++kp)
            o[t][kp] = __builtin_amdgcn_raw_buffer_load_b128(rz, z_voff, z_soff(c * CH + t, kp), kAux);
      };
      if (accumulate) load_chunk(0, old[0]);
#pragma unroll
      for (int c = 0; c < TM / CH; ++c) {
        if (accumulate && c + 1 < TM / CH) load_chunk(c + 1, old[(c + 1) & 1]);
#pragma unroll
        for (int t = 0; t < CH; ++t) {
          const int tm = c * CH + t;
#pragma unroll
          for (int kp = 0; kp < KP; ++kp) {
            f32x4 lo = acc[2 * kp][tm], hi = acc[2 * kp + 1][tm];
            swap_halves(lo, hi);
            swap_rows(lo, hi);
            if (accumulate) {
              const u32x4 o = old[c & 1][t][kp];
              lo[0] += stored_lo<OutT>(o.x), lo[1] += stored_hi<OutT>(o.x), lo[2] += stored_lo<OutT>(o.y), lo[3] += stored_hi<OutT>(o.y);
              hi[0] += stored_lo<OutT>(o.z), hi[1] += stored_hi<OutT>(o.z), hi[2] += stored_lo<OutT>(o.w), hi[3] += stored_hi<OutT>(o.w);
            }
            const u32x4 w = {pack_out2<OutT>(lo[0], lo[1]), pack_out2<OutT>(lo[2], lo[3]), pack_out2<OutT>(hi[0], hi[1]),
                             pack_out2<OutT>(hi[2], hi[3])};
            __builtin_amdgcn_raw_buffer_store_b128(w, rz, z_voff, z_soff(tm, kp), kAux);
            // A 16-byte store reads its data registers for a few cycles after it issues, and the compiler, which knows this
            // hazard only for stores without a scalar offset, reuses them at once (the next block's exchange operands
            // are moved in): two idle cycles keep the new values out of the store.
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_nop 1");
            __builtin_amdgcn_sched_barrier(0);
            // zero for the next tile, in place: the accumulators of the next tile are the same registers
            clear_in_place(acc[2 * kp][tm]);
            clear_in_place(acc[2 * kp + 1][tm]);
          }
        }
      }
    };

    // The stage names repeat every 6 K tiles (3 x stages, 2 y stages); an output tile may end after any of them.
    // After the workgroup's last tile the wavefront ends right there (this body is the whole kernel): six loop exits
    // would be routed through one block in front of the loop header, and the compiler's bookkeeping of the fetches in
    // flight would then see every phase's end state arrive at the first phase and add waits of its own there.
    int left = k_tiles;       // K tiles of the current output tile still to run
    uint32_t item = 0;
    auto tile_end = [&]() {
      epilogue();
      if (++item == n_mine) {
        __builtin_amdgcn_s_waitcnt(0);  // the look-ahead fetches must not outlive the workgroup's LDS
        __builtin_amdgcn_endpgm();
      }
      a_cur = a_nxt, b_cur = b_nxt, z_row = z_row_nxt, z_col = z_col_nxt;
      look_ahead(item);
      left = k_tiles;
    };
    for (;;) {
      k_tile(xs0, ys0a, ys0b, xs1, ys1a, k_tiles - left);
      if (--left == 0) tile_end();
      k_tile(xs1, ys1a, ys1b, xs2, ys0a, k_tiles - left);
      if (--left == 0) tile_end();
      k_tile(xs2, ys0a, ys0b, xs0, ys1a, k_tiles - left);
      if (--left == 0) tile_end();
      k_tile(xs0, ys1a, ys1b, xs1, ys0a, k_tiles - left);
      if (--left == 0) tile_end();
      k_tile(xs1, ys0a, ys0b, xs2, ys1a, k_tiles - left);
      if (--left == 0) tile_end();
      k_tile(xs2, ys1a, ys1b, xs0, ys0a, k_tiles - left);
      if (--left == 0) tile_end();
    }
  }

  // gemm: workgroup b takes the tiles b, b + gridDim.x, ... of the launch's XCD-contiguous, M-grouped order
  template <bool ACCUMULATE, bool STREAM>
  __device__ static void run(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y, int32_t k_total,
                             const TileGrid& g) {
    const uint32_t total = g.x * g.y;
    const uint32_t n_mine = blockIdx.x < total ? (total - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    run_items<ACCUMULATE, STREAM>(z, x, y, k_total, n_mine, [&](uint32_t j, uint32_t* pm, uint32_t* pn) {
      tile_of_id(blockIdx.x + j * gridDim.x, g.x, g.y, gridDim.x, pm, pn);
    });
  }
  // gemm_persistent: the stream items of the mapped partition, from zero accumulators
  template <bool STREAM>
  __device__ static void run_persistent(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                        const MappedArg& m) {
    const uint32_t n_mine = blockIdx.x < m.total ? (m.total - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    run_items<false, STREAM>(z, x, y, x.shape[1], n_mine, [&](uint32_t j, uint32_t* pm, uint32_t* pn) {
      const uint32_t it = blockIdx.x + j * gridDim.x;
      const uint32_t pos = m.total % kNumXcd == 0 ? (it % kNumXcd) * (m.total / kNumXcd) + it / kNumXcd : it;
      uint32_t bid[3];
      mapped_index(m, pos, bid);
      *pm = bid[0], *pn = bid[1];
    });
  }
};

// ---- any-layout variant ---------------------------------------------------------------------
// The tile program for arbitrary tile shapes, element types (bf16, f16, f32),
// strides and extents — what the pipelined variants cannot take (rows that are
// not 16-byte aligned, N or K not a multiple of 8, tile shapes without a
// precompiled kernel, e.g. the reference tests' 16x16x8).  It computes the same
// function directly: z[r,c] (+)= sum_k x[r,k] * y[k,c] over the region the launch
// grid covers, reads outside a tensor contributing 0, f32 accumulation in K
// order, one rounding on store.  64x64 outputs per workgroup of 256 lanes, 4x4
// per lane, operands staged through LDS as f32.  Correctness path, not a fast one.
template <typename T>
__device__ __forceinline__ float elem_to_f32(T v) { return (float)v; }

// One block of at most 64x64 outputs with its top-left corner at (row0, col0); stores
// are limited to rows < row_end and columns < col_end.
template <typename InT, typename OutT>
__device__ __forceinline__ void any_layout_block(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                                 int32_t k_total, int64_t row0, int64_t col0, int64_t row_end,
                                                 int64_t col_end, int32_t accumulate) {
  constexpr int TS = 64, KS = 16;
  __shared__ float xs[TS][KS + 1];
  __shared__ float ys[KS][TS + 1];
  const int tid = threadIdx.x;
  const int tr = tid / 16, tc = tid % 16;             // this lane's 4x4 block inside the 64x64 tile
  const int32_t k_valid = min(min(x.shape[1], y.shape[0]), k_total);
  const InT* xp = (const InT*)x.ptr;
  const InT* yp = (const InT*)y.ptr;
  float acc[4][4] = {};
  for (int32_t k0 = 0; k0 < k_valid; k0 += KS) {
    for (int i = tid; i < TS * KS; i += 256) {
      const int r = i / KS, kk = i % KS;
      const int64_t gr = row0 + r;
      xs[r][kk] = (gr < x.shape[0] && k0 + kk < k_valid)
                      ? elem_to_f32(xp[gr * x.strides[0] + (int64_t)(k0 + kk) * x.strides[1]]) : 0.0f;
    }
    for (int i = tid; i < KS * TS; i += 256) {
      const int kk = i / TS, c = i % TS;
      const int64_t gc = col0 + c;
      ys[kk][c] = (gc < y.shape[1] && k0 + kk < k_valid)
                      ? elem_to_f32(yp[(int64_t)(k0 + kk) * y.strides[0] + gc * y.strides[1]]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[tr * 4 + i][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ys[kk][tc * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  OutT* zp = (OutT*)z.ptr;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t gr = row0 + tr * 4 + i, gc = col0 + tc * 4 + j;
      if (gr < row_end && gc < col_end) {
        OutT* dst = zp + gr * z.strides[0] + gc * z.strides[1];
        float v = acc[i][j];
        if (accumulate) v += elem_to_f32(*dst);
        *dst = (OutT)v;
      }
    }
}

template <typename InT, typename OutT>
__device__ void gemm_any_layout(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                int32_t k_total, const TileGrid& g, int32_t accumulate) {
  const int64_t cover_m = min((int64_t)g.x * z.pshape[0], (int64_t)z.shape[0]);
  const int64_t cover_n = min((int64_t)g.y * z.pshape[1], (int64_t)z.shape[1]);
  any_layout_block<InT, OutT>(z, x, y, k_total, (int64_t)blockIdx.x * 64, (int64_t)blockIdx.y * 64, cover_m, cover_n, accumulate);
}

// The persistent form for any tile shape: stream items in the reference's order, each
// [BM, BN] tile of the partition covered by 64x64 blocks.
template <typename InT, typename OutT>
__device__ void gemm_any_layout_persistent(const PartitionArg<2>& z, const TensorArg<2>& x, const TensorArg<2>& y,
                                           const MappedArg& m) {
  const int64_t bm = z.pshape[0], bn = z.pshape[1];
  for (uint32_t item = blockIdx.x; item < m.total; item += gridDim.x) {
    uint32_t bid[3];
    mapped_index(m, item, bid);
    const int64_t r_end = min((int64_t)(bid[0] + 1) * bm, (int64_t)z.shape[0]);
    const int64_t c_end = min((int64_t)(bid[1] + 1) * bn, (int64_t)z.shape[1]);
    for (int64_t r = (int64_t)bid[0] * bm; r < r_end; r += 64)
      for (int64_t c = (int64_t)bid[1] * bn; c < c_end; c += 64)
        any_layout_block<InT, OutT>(z, x, y, x.shape[1], r, c, r_end, c_end, 0);
  }
}

}  // namespace

// gemm<bf16, BM, BN, BK>(z, x, y, k) with trailing launch metadata.
#define GEMM_KERNEL(NAME, BM, BN, BK, WVM, WVN, OUT_T)                                          \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    Gemm<BM, BN, BK, WVM, WVN, OUT_T>::run(z, x, y, k, g, accumulate);                          \
  }

GEMM_KERNEL(bf16_256x256x64_w2x2, 256, 256, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_256x256x64_w2x4, 256, 256, 64, 2, 4, __bf16)
GEMM_KERNEL(bf16_256x256x64_w4x2, 256, 256, 64, 4, 2, __bf16)
GEMM_KERNEL(bf16_256x128x64_w2x2, 256, 128, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_128x256x64_w2x2, 128, 256, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_128x128x64_w2x2, 128, 128, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16_64x128x64_w2x2, 64, 128, 64, 2, 2, __bf16)
GEMM_KERNEL(bf16f32_128x128x64_w2x2, 128, 128, 64, 2, 2, float)
GEMM_KERNEL(bf16f32_256x256x64_w2x2, 256, 256, 64, 2, 2, float)

#define GEMM_DIRECT_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                        \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    GemmDirect<BM, BN, WVM, WVN, OUT_T>::run(z, x, y, k, g, accumulate);                        \
  }

GEMM_DIRECT_KERNEL(bf16_256x256x64_d4x2, 256, 256, 4, 2, __bf16)
GEMM_DIRECT_KERNEL(bf16_256x256x64_d2x4, 256, 256, 2, 4, __bf16)
GEMM_DIRECT_KERNEL(bf16_128x128x64_d2x2, 128, 128, 2, 2, __bf16)

// the same pipelines on f16 operands (v_mfma_f32_32x32x16_f16), f16 z
#define GEMM_DIRECT_F16_KERNEL(NAME, BM, BN, WVM, WVN)                                            \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    GemmDirect<BM, BN, WVM, WVN, _Float16, _Float16>::run(z, x, y, k, g, accumulate);           \
  }                                                                                             \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_persistent_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, MappedArg m) { \
    GemmDirect<BM, BN, WVM, WVN, _Float16, _Float16>::run_persistent(z, x, y, m);               \
  }
GEMM_DIRECT_F16_KERNEL(f16_256x256x64_d4x2, 256, 256, 4, 2)
GEMM_DIRECT_F16_KERNEL(f16_128x128x64_d2x2, 128, 128, 2, 2)

// group_gemm_f16_nt_desc<BM, BN, BK, NUM_SM>(a_ptrs, b_ptrs, c_ptrs: [groups] i64; a_metas, b_metas, c_metas:
// [groups, 8] i32 = (rows, cols, row stride, ...); num_groups) — cutile-kernels/src/experimental/moe.rs:67-128.
// Group g multiplies A_g [m, k] by B_g [k, n] into C_g [m, n] (f16, f32 accumulation); the tiles of all groups form
// one sequence, group after group and row-major inside a group, and workgroup w computes tiles w, w + grid, ...
// (:82-83, 106-124).  The descriptors are read from device memory by every workgroup; as in the reference they are
// trusted: pointers 16-byte aligned, rows and columns multiples of 16, row strides multiples of 8 (:24, 47-55).
template <typename G, int BM, int BN>
__device__ __forceinline__ void group_gemm_desc(const TensorArg<1>& a_ptrs, const TensorArg<1>& b_ptrs, const TensorArg<1>& c_ptrs,
                                                const TensorArg<2>& a_metas, const TensorArg<2>& b_metas,
                                                const TensorArg<2>& c_metas, int32_t num_groups) {
  auto uniform = [](int32_t v) { return __builtin_amdgcn_readfirstlane(v); };
  auto describe = [&](const TensorArg<1>& ptrs, const TensorArg<2>& metas, int32_t g, TensorArg<2>* t) {
    const uint32_t* pp = reinterpret_cast<const uint32_t*>((const int64_t*)ptrs.ptr + (int64_t)g * ptrs.strides[0]);
    const int32_t* mp = (const int32_t*)metas.ptr + (int64_t)g * metas.strides[0];
    const uint64_t addr = (uint64_t)(uint32_t)uniform((int32_t)pp[0]) | ((uint64_t)(uint32_t)uniform((int32_t)pp[1]) << 32);
    t->ptr = (void*)addr;
    t->shape[0] = uniform(mp[0]);
    t->shape[1] = uniform(mp[metas.strides[1]]);
    t->strides[0] = uniform(mp[2 * metas.strides[1]]);
    t->strides[1] = 1;
  };
  uint32_t tile_idx = blockIdx.x, group_start = 0;
  for (int32_t g = 0; g < num_groups; ++g) {
    TensorArg<2> a, b, c;
    describe(a_ptrs, a_metas, g, &a);
    describe(b_ptrs, b_metas, g, &b);
    describe(c_ptrs, c_metas, g, &c);
    const int32_t m = a.shape[0], k = a.shape[1], n = b.shape[1];
    const uint32_t tiles_n = (uint32_t)((n + BN - 1) / BN);
    const uint32_t tiles = (uint32_t)((m + BM - 1) / BM) * tiles_n;
    PartitionArg<2> z;
    z.ptr = c.ptr;
    z.shape[0] = c.shape[0], z.shape[1] = c.shape[1];
    z.strides[0] = z.pstrides[0] = c.strides[0], z.strides[1] = z.pstrides[1] = 1;
    z.pshape[0] = BM, z.pshape[1] = BN;
    while (tile_idx >= group_start && tile_idx < group_start + tiles) {
      const uint32_t in_group = tile_idx - group_start;
      // (consecutive positions run on different XCDs; with a tile row of 8 or 16 tiles every XCD keeps meeting the same
      // one or two B panels, which measured better than handing each XCD a contiguous eighth of the group: 3.8 against 5.8 GB)
      G::run_tile(z, a, b, k, in_group / tiles_n, in_group % tiles_n, 0);
      __syncthreads();   // the output bands live in the stages that the next tile refills
      tile_idx += gridDim.x;
    }
    group_start += tiles;
  }
}
#define GROUP_GEMM_KERNEL(NAME, BM, BN, WVM, WVN)                                                 \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      group_gemm_nt_desc_entry__##NAME(TensorArg<1> a_ptrs, TensorArg<1> b_ptrs, TensorArg<1> c_ptrs, TensorArg<2> a_metas, \
                                       TensorArg<2> b_metas, TensorArg<2> c_metas, int32_t num_groups) { \
    group_gemm_desc<GemmDirect<BM, BN, WVM, WVN, _Float16, _Float16>, BM, BN>(a_ptrs, b_ptrs, c_ptrs, a_metas, b_metas, c_metas, num_groups); \
  }
GROUP_GEMM_KERNEL(f16_256x256x64_d2x4, 256, 256, 2, 4)
GROUP_GEMM_KERNEL(f16_128x128x64_d2x2, 128, 128, 2, 2)

#define GEMM_RING_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                          \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    GemmRing<BM, BN, WVM, WVN, OUT_T>::run(z, x, y, k, g, accumulate);                          \
  }

GEMM_RING_KERNEL(bf16_256x256x64_r2x4, 256, 256, 2, 4, __bf16)
GEMM_RING_KERNEL(bf16_256x256x64_r4x2, 256, 256, 4, 2, __bf16)
GEMM_RING_KERNEL(bf16_128x128x64_r2x2, 128, 128, 2, 2, __bf16)
#define GEMM_RING_KERNEL_F16(NAME, BM, BN, WVM, WVN)                                            \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    GemmRing<BM, BN, WVM, WVN, _Float16, _Float16>::run(z, x, y, k, g, accumulate);            \
  }
GEMM_RING_KERNEL_F16(f16_256x256x64_r2x4, 256, 256, 2, 4)
GEMM_RING_KERNEL_F16(f16_256x256x64_r4x2, 256, 256, 4, 2)

// the ring pipeline on v_mfma_f32_16x16x32 ("q")
#define GEMM_RING16_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T, IN_T)                                  \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    GemmRing16<BM, BN, WVM, WVN, OUT_T, IN_T>::run(z, x, y, k, g, accumulate);                  \
  }
GEMM_RING16_KERNEL(bf16_256x256x64_q2x4, 256, 256, 2, 4, __bf16, __bf16)
GEMM_RING16_KERNEL(f16_256x256x64_q2x4, 256, 256, 2, 4, _Float16, _Float16)
// 128 x 128 tiles on four wavefronts: 80 KiB of stages, so two workgroups share a compute unit and one's main loop
// runs under the other's prologue and epilogue (for launches of about one 256 x 256 tile per compute unit)
GEMM_RING16_KERNEL(bf16_128x128x64_q2x2, 128, 128, 2, 2, __bf16, __bf16)
GEMM_RING16_KERNEL(f16_128x128x64_q2x2, 128, 128, 2, 2, _Float16, _Float16)
#define GEMM_RING16_PERSISTENT_KERNEL(NAME, BM, BN, WVM, WVN, T)                                 \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_persistent_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, MappedArg m) { \
    GemmRing16<BM, BN, WVM, WVN, T, T>::run_persistent(z, x, y, m);                             \
  }
extern "C" __global__ void __launch_bounds__(512)
    group_gemm_nt_desc_entry__f16_256x256x64_q2x4(TensorArg<1> a_ptrs, TensorArg<1> b_ptrs, TensorArg<1> c_ptrs, TensorArg<2> a_metas,
                                                  TensorArg<2> b_metas, TensorArg<2> c_metas, int32_t num_groups) {
  group_gemm_desc<GemmRing16<256, 256, 2, 4, _Float16, _Float16>, 256, 256>(a_ptrs, b_ptrs, c_ptrs, a_metas, b_metas, c_metas, num_groups);
}
#define GEMM_RING16_WALK_KERNEL(NAME, BM, BN, WVM, WVN, T)                                        \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                         int32_t accumulate) {                                                  \
    GemmRing16<BM, BN, WVM, WVN, T, T>::run_walk(z, x, y, k, g, accumulate);                    \
  }
GEMM_RING16_WALK_KERNEL(bf16_256x256x64_p2x4, 256, 256, 2, 4, __bf16)
GEMM_RING16_WALK_KERNEL(f16_256x256x64_p2x4, 256, 256, 2, 4, _Float16)
GEMM_RING16_PERSISTENT_KERNEL(bf16_256x256x64_q2x4, 256, 256, 2, 4, __bf16)
GEMM_RING16_PERSISTENT_KERNEL(f16_256x256x64_q2x4, 256, 256, 2, 4, _Float16)

// the 16 x 16 x 32 ring streaming over a workgroup's output tiles ("s"): gemm launched with one workgroup per compute
// unit, and the persistent GEMM over a mapped partition.  One kernel per (z read as the initial accumulator or not,
// z past the caches or through them): the launcher picks; `accumulate` is part of the signature all the same.
#define GEMM_STREAM16_KERNEL(NAME, SUFFIX, ACC, NT, BM, BN, WVM, WVN, T)                         \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_entry__##NAME##SUFFIX(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, TileGrid g, \
                                 int32_t accumulate) {                                          \
    GemmStream16<BM, BN, WVM, WVN, T, T>::template run<ACC, NT>(z, x, y, k, g);                 \
  }
#define GEMM_STREAM16_PERSISTENT_KERNEL(NAME, SUFFIX, NT, BM, BN, WVM, WVN, T)                   \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_persistent_entry__##NAME##SUFFIX(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, MappedArg m) { \
    GemmStream16<BM, BN, WVM, WVN, T, T>::template run_persistent<NT>(z, x, y, m);              \
  }
#define GEMM_STREAM16_FAMILY(NAME, T)                                                            \
  GEMM_STREAM16_KERNEL(NAME, , true, true, 256, 256, 2, 4, T)                                    \
  GEMM_STREAM16_KERNEL(NAME, _cached, true, false, 256, 256, 2, 4, T)                            \
  GEMM_STREAM16_KERNEL(NAME, _new, false, true, 256, 256, 2, 4, T)                               \
  GEMM_STREAM16_KERNEL(NAME, _new_cached, false, false, 256, 256, 2, 4, T)                       \
  GEMM_STREAM16_PERSISTENT_KERNEL(NAME, , true, 256, 256, 2, 4, T)                               \
  GEMM_STREAM16_PERSISTENT_KERNEL(NAME, _cached, false, 256, 256, 2, 4, T)
GEMM_STREAM16_FAMILY(bf16_256x256x64_s2x4, __bf16)
GEMM_STREAM16_FAMILY(f16_256x256x64_s2x4, _Float16)

#define GEMM_ANY_LAYOUT_KERNEL(NAME, IN_T, OUT_T)                                                \
  extern "C" __global__ void __launch_bounds__(256)                                            \
      gemm_entry__##NAME##_generic(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, int32_t k, \
                                   TileGrid g, int32_t accumulate) {                            \
    gemm_any_layout<IN_T, OUT_T>(z, x, y, k, g, accumulate);                                    \
  }

GEMM_ANY_LAYOUT_KERNEL(bf16, __bf16, __bf16)
GEMM_ANY_LAYOUT_KERNEL(bf16f32, __bf16, float)
GEMM_ANY_LAYOUT_KERNEL(f16, _Float16, _Float16)
GEMM_ANY_LAYOUT_KERNEL(f32, float, float)

// gemm_persistent<T, BM, BN, BK, MAP_SHAPE>(z: mapped [BM,BN] tiles, x, y): grid (num_tile_blocks, 1, 1)
#define GEMM_PERSISTENT_KERNEL(NAME, BM, BN, WVM, WVN, OUT_T)                                    \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      gemm_persistent_entry__##NAME(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, MappedArg m) { \
    GemmDirect<BM, BN, WVM, WVN, OUT_T>::run_persistent(z, x, y, m);                            \
  }

GEMM_PERSISTENT_KERNEL(bf16_256x256x64_d4x2, 256, 256, 4, 2, __bf16)
GEMM_PERSISTENT_KERNEL(bf16_256x256x64_d2x4, 256, 256, 2, 4, __bf16)
GEMM_PERSISTENT_KERNEL(bf16_128x128x64_d2x2, 128, 128, 2, 2, __bf16)

#define GEMM_PERSISTENT_ANY_LAYOUT_KERNEL(NAME, IN_T, OUT_T)                                     \
  extern "C" __global__ void __launch_bounds__(256)                                            \
      gemm_persistent_entry__##NAME##_generic(PartitionArg<2> z, TensorArg<2> x, TensorArg<2> y, MappedArg m) { \
    gemm_any_layout_persistent<IN_T, OUT_T>(z, x, y, m);                                        \
  }

GEMM_PERSISTENT_ANY_LAYOUT_KERNEL(bf16, __bf16, __bf16)
GEMM_PERSISTENT_ANY_LAYOUT_KERNEL(f16, _Float16, _Float16)
GEMM_PERSISTENT_ANY_LAYOUT_KERNEL(f32, float, float)

// batch_matmul<E, BM, BN, BK, K>(c: [1, BM, BN] tiles of [batches, M, N], a: [batches, M, K], b: [batches, K, N]) —
// cutile-examples/examples/batch_matmul.rs:16-44: c[p] = a[p] · b[p] from zero accumulators over K / BK whole K tiles,
// every batch in one launch.  A workgroup takes its batch from one grid axis, cuts the three rank-2 slices out of the
// operands and runs the tile body of the plain GEMM on them; a batch that a or b does not have reads as zeros.
template <typename T>
__device__ __forceinline__ void batch_slices(const PartitionArg<3>& c, const TensorArg<3>& a, const TensorArg<3>& b,
                                             uint32_t batch, PartitionArg<2>* z, TensorArg<2>* x, TensorArg<2>* y) {
  z->ptr = (T*)c.ptr + (int64_t)batch * c.strides[0];
  x->ptr = (T*)a.ptr + (int64_t)batch * a.strides[0];
  y->ptr = (T*)b.ptr + (int64_t)batch * b.strides[0];
  for (int d = 0; d < 2; ++d) {
    z->shape[d] = c.shape[d + 1], z->strides[d] = c.strides[d + 1];
    z->pshape[d] = c.pshape[d + 1], z->pstrides[d] = c.pstrides[d + 1];
    x->shape[d] = a.shape[d + 1], x->strides[d] = a.strides[d + 1];
    y->shape[d] = b.shape[d + 1], y->strides[d] = b.strides[d + 1];
  }
  if (batch >= (uint32_t)a.shape[0] || batch >= (uint32_t)b.shape[0]) {   // zero padding of the missing batch
    x->ptr = a.ptr, y->ptr = b.ptr;
    x->shape[1] = 0, y->shape[0] = 0;
  }
}
// tile grid (batches, M tiles, N tiles); HIP grid (M tiles * N tiles, batches, 1)
#define BATCH_MATMUL_KERNEL(NAME, T, BM, BN, WVM, WVN) BATCH_MATMUL_KERNEL_OF(GemmDirect, NAME, T, BM, BN, WVM, WVN)
#define BATCH_MATMUL_KERNEL_OF(BODY, NAME, T, BM, BN, WVM, WVN)                                  \
  extern "C" __global__ void __launch_bounds__(WVM* WVN * 64)                                  \
      batch_matmul_entry__##NAME(PartitionArg<3> c, TensorArg<3> a, TensorArg<3> b, int32_t k, TileGrid g) { \
    PartitionArg<2> z;                                                                         \
    TensorArg<2> x, y;                                                                         \
    batch_slices<T>(c, a, b, blockIdx.y, &z, &x, &y);                                          \
    const TileGrid tiles = {g.y, g.z, 1, 0};                                                   \
    BODY<BM, BN, WVM, WVN, T, T>::run(z, x, y, k, tiles, 0);                                   \
  }
// the ring-pipelined bodies first (they fetch whole K tiles only: K % 64 == 0)
BATCH_MATMUL_KERNEL_OF(GemmRing16, bf16_256x256x64_q2x4, __bf16, 256, 256, 2, 4)
BATCH_MATMUL_KERNEL_OF(GemmRing16, f16_256x256x64_q2x4, _Float16, 256, 256, 2, 4)
BATCH_MATMUL_KERNEL_OF(GemmRing, bf16_256x256x64_r2x4, __bf16, 256, 256, 2, 4)
BATCH_MATMUL_KERNEL_OF(GemmRing, f16_256x256x64_r2x4, _Float16, 256, 256, 2, 4)
BATCH_MATMUL_KERNEL(bf16_256x256x64_d2x4, __bf16, 256, 256, 2, 4)
BATCH_MATMUL_KERNEL(bf16_128x128x64_d2x2, __bf16, 128, 128, 2, 2)
BATCH_MATMUL_KERNEL(f16_256x256x64_d4x2, _Float16, 256, 256, 4, 2)
BATCH_MATMUL_KERNEL(f16_128x128x64_d2x2, _Float16, 128, 128, 2, 2)
// any tile shape, strides and extents: HIP grid (64-row blocks, 64-column blocks, batches)
#define BATCH_MATMUL_ANY_LAYOUT_KERNEL(NAME, T)                                                  \
  extern "C" __global__ void __launch_bounds__(256)                                            \
      batch_matmul_entry__##NAME##_generic(PartitionArg<3> c, TensorArg<3> a, TensorArg<3> b, int32_t k, TileGrid g) { \
    PartitionArg<2> z;                                                                         \
    TensorArg<2> x, y;                                                                         \
    batch_slices<T>(c, a, b, blockIdx.z, &z, &x, &y);                                          \
    const TileGrid tiles = {g.y, g.z, 1, 0};                                                   \
    gemm_any_layout<T, T>(z, x, y, k, tiles, 0);                                               \
  }
BATCH_MATMUL_ANY_LAYOUT_KERNEL(bf16, __bf16)
BATCH_MATMUL_ANY_LAYOUT_KERNEL(f16, _Float16)
BATCH_MATMUL_ANY_LAYOUT_KERNEL(f32, float)
