// Hand-written CDNA4 (gfx950) GEMM main loop for the fused GEMM/BMM +
// epilogue-visitor-tree kernels.
//
// Role in the reference (apuaaChen/EVT_AE): this replaces the un-vendored
// CUTLASS sm80 `GemmUniversalWithVisitor` main loop that FusedGEMM / FusedBMM
// instantiate (python/gtl/compiler/passes/evt_fuser.py:481-518, :605-642).
// It is not derived from it: the design is wave64 / MFMA / LDS-DMA native.
//
//   * one workgroup computes a BM x BN tile of D = A*B with WM x WN waves,
//     each wave a (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks
//     (v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulators in registers);
//   * A and B tiles of depth BK are staged in LDS, STAGES deep.  The fast path
//     moves them with buffer_load_dwordx4 ... lds (global -> LDS DMA, no
//     VGPR round trip); out-of-range chunks read as zero through the buffer
//     range check.  The safe path (any alignment, any shape) gathers elements
//     through registers;
//   * a K-contiguous operand tile is stored row by row with an XOR swizzle of
//     its 16-byte chunks and read back with ds_read_b128; an operand whose
//     other dimension is contiguous is stored k-row by k-row and read back
//     with ds_read_b64_tr_b16, which transposes it into MFMA operand order;
//   * workgroup ids are remapped so that each XCD (own L2) owns a compact
//     block of output tiles.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace evt {

#define EVT_DEV __device__ __forceinline__

typedef _Float16 f16;
typedef __bf16 bf16;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;

constexpr int kNumXcd = 8;            // MI355X: 8 XCDs, workgroups dealt round-robin
constexpr uint32_t kOobOffset = 0x80000000u;   // > any num_records we set
constexpr uint32_t kRsrcFlags = 0x00020000u;   // raw buffer, 32-bit data format
constexpr uint32_t kRsrcRange = 0x7fffffffu;

struct GemmArgs {
  int M, N, K, L;
  const char* A;
  int64_t lda, bsA;   // elements
  const char* B;
  int64_t ldb, bsB;   // elements
  int tiles_m, tiles_n;
  char* workspace;
};

// Compile-time description of one kernel variant.
template <int BM_, int BN_, int BK_, int WM_, int WN_, bool A_KC_, bool B_KC_,
          bool DMA_, int STAGES_, bool BF16_, int GROUP_M_>
struct GemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr bool A_KC = A_KC_, B_KC = B_KC_, DMA = DMA_, BF16 = BF16_;
  static constexpr int STAGES = STAGES_, GROUP_M = GROUP_M_;
  static constexpr int WAVES = WM * WN;
  static constexpr int THREADS = WAVES * 64;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int MI = TM / 32, NI = TN / 32;
  static constexpr int KS = BK / 16;
  // Layout of each operand tile in LDS: K-contiguous rows, or k-rows.
  static constexpr bool A_LDS_KC = A_KC || !DMA;
  static constexpr bool B_LDS_KC = B_KC || !DMA;
  // With a K-contiguous B tile the rows (= output columns) can be permuted for
  // free while loading, so every lane ends up owning NI adjacent columns.
  static constexpr bool INTERLEAVE = B_LDS_KC && (NI > 1);
  static constexpr int A_BYTES = BM * BK * 2;
  static constexpr int B_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  static_assert(BK == 32 || BK == 64, "BK must be 32 or 64");
  static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be 32-aligned");
  static_assert(STAGES >= 2 && STAGES <= 4, "2..4 stages");
};

// ---------------------------------------------------------------------------
// LDS slot functions.  A "slot" is one 16-byte chunk (8 elements).
// ---------------------------------------------------------------------------

// K-contiguous tile: logical (row r, chunk q of BK/8) -> slot.  The chunk index
// is XOR-ed with low row bits and one row bit is flipped so that 8 as well as
// 16 consecutive rows at equal q land in distinct 16-byte bank groups.
template <int CH>
EVT_DEV int kc_slot(int r, int q) {
  if constexpr (CH == 8) {
    const int rho = r ^ ((r >> 3) & 1);
    return rho * 8 + (q ^ (r & 7));
  } else {
    const int rho = r ^ (((r >> 3) & 1) << 1);
    return rho * 4 + (q ^ ((r >> 1) & 3));
  }
}

template <int CH>
EVT_DEV void kc_unslot(int slot, int& r, int& q) {
  if constexpr (CH == 8) {
    const int rho = slot >> 3, qq = slot & 7;
    r = rho ^ ((rho >> 3) & 1);
    q = qq ^ (r & 7);
  } else {
    const int rho = slot >> 2, qq = slot & 3;
    r = rho ^ (((rho >> 3) & 1) << 1);
    q = qq ^ ((r >> 1) & 3);
  }
}

// k-row tile (the non-K dimension is contiguous): logical (k, chunk c of
// ROWS/8) -> slot; chunk index XOR-ed with (k & 3) * 4.
template <int RC>
EVT_DEV int nc_swz(int k) { return ((k & 3) << 2) & (RC - 1); }

EVT_DEV __amdgpu_buffer_rsrc_t make_rsrc(const char* p) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, kRsrcRange, kRsrcFlags);
}

// wait until at most n vector-memory operations of this wave are outstanding
template <int N>
EVT_DEV void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

// ---------------------------------------------------------------------------
// One GEMM operand (A or B) of a workgroup tile: global -> LDS movement and
// LDS -> MFMA-fragment reads.
//   ROWS     tile extent in the non-K dimension (BM for A, BN for B)
//   SRC_KC   the source matrix is contiguous along K
//   PERM_NI  >1: LDS row (w*PERM_TN + f*32 + j) holds global row
//            (w*PERM_TN + j*PERM_NI + f)  (column interleave, B only)
// ---------------------------------------------------------------------------
template <int ROWS, int BK, bool SRC_KC, bool DMA, int THREADS, int PERM_NI, int PERM_TN>
struct Operand {
  static constexpr bool LDS_KC = SRC_KC || !DMA;
  static constexpr int CH = BK / 8;
  static constexpr int RC = ROWS / 8;
  static constexpr int CHUNKS = ROWS * BK / 8;
  static constexpr int NLOAD = CHUNKS / THREADS;
  static_assert(CHUNKS % THREADS == 0 && NLOAD >= 1, "tile too small for the workgroup");
  static_assert(!(PERM_NI > 1) || LDS_KC, "row permutation needs a K-contiguous LDS tile");

  const char* base;        // start of this tile's rows / columns at k = 0 (bytes)
  int64_t ld;              // elements
  int rows_left;           // valid rows from the tile origin (may exceed ROWS)
  int K;
  uint32_t voff[NLOAD];    // byte offset of my chunk inside the tile, or kOobOffset
  int kin[NLOAD];          // first k (within a tile) my chunk covers

  static EVT_DEV int grow(int r) {
    if constexpr (PERM_NI > 1) {
      const int w = r / PERM_TN, x = r % PERM_TN;
      return w * PERM_TN + (x & 31) * PERM_NI + (x >> 5);
    } else {
      return r;
    }
  }

  EVT_DEV void init(const char* base_, int64_t ld_, int rows_left_, int K_, int tid) {
    base = base_; ld = ld_; rows_left = rows_left_; K = K_;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int slot = i * THREADS + tid;
      if constexpr (LDS_KC) {
        int r, q;
        kc_unslot<CH>(slot, r, q);
        const int g = grow(r);
        kin[i] = q * 8;
        if constexpr (SRC_KC) {
          voff[i] = (g < rows_left) ? (uint32_t)(g * ld * 2 + q * 16) : kOobOffset;
        } else {
          voff[i] = (uint32_t)g;   // safe path only: row index, guarded per element
        }
      } else {
        const int k = slot / RC, cs = slot % RC;
        const int c = cs ^ nc_swz<RC>(k);
        kin[i] = k;
        voff[i] = (c * 8 < rows_left) ? (uint32_t)(k * ld * 2 + c * 16) : kOobOffset;
      }
    }
  }

  // ---- fast path: global -> LDS DMA of k-tile `kt` into `lds` -------------
  EVT_DEV void dma(int kt, char* lds, int wave) const {
    const int64_t adv = SRC_KC ? (int64_t)kt * BK * 2 : (int64_t)kt * BK * ld * 2;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(base + adv);
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const uint32_t v = (k0 + kin[i] < K) ? voff[i] : kOobOffset;
      char* dst = lds + (i * THREADS + wave * 64) * 16;   // wave-uniform; lane*16 added by hardware
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)dst, 16, v, 0, 0, 0);
    }
  }

  // ---- safe path: element-wise guarded gather through registers ----------
  EVT_DEV void fetch(int kt, u32x4 (&regs)[NLOAD], int tid) const {
    const uint16_t* src = (const uint16_t*)base;
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      int r, q;
      kc_unslot<CH>(i * THREADS + tid, r, q);
      const int g = grow(r);
      const bool rok = g < rows_left;
      uint16_t e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + q * 8 + j;
        const bool ok = rok && (k < K);
        const int64_t off = SRC_KC ? ((int64_t)g * ld + k) : ((int64_t)k * ld + g);
        e[j] = ok ? src[off] : (uint16_t)0;
      }
      regs[i].x = e[0] | ((uint32_t)e[1] << 16);
      regs[i].y = e[2] | ((uint32_t)e[3] << 16);
      regs[i].z = e[4] | ((uint32_t)e[5] << 16);
      regs[i].w = e[6] | ((uint32_t)e[7] << 16);
    }
  }

  EVT_DEV void commit(const u32x4 (&regs)[NLOAD], char* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      *(u32x4*)(lds + (i * THREADS + tid) * 16) = regs[i];
    }
  }
};

// Per-lane LDS read addressing of MFMA operand fragments (32 rows x 16 k).
template <int ROWS, int BK, bool LDS_KC, int NFRAG>
struct FragReader {
  static constexpr int CH = BK / 8;
  static constexpr int RC = ROWS / 8;
  uint32_t off[LDS_KC ? (BK / 16) : NFRAG];

  EVT_DEV void init(int wave_row_base, int lane) {
    if constexpr (LDS_KC) {
      // lane reads row (base + lane % 32), chunk 2*ks + lane / 32
      const int r = wave_row_base + (lane & 31);
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) off[ks] = kc_slot<CH>(r, 2 * ks + (lane >> 5)) * 16;
    } else {
      // transposing read: each group of 16 lanes covers 4 k-rows x 16 rows
      const int u = lane >> 4, s = lane & 15;
      const int kl = 8 * (u >> 1) + (s >> 2);
      const int i0 = wave_row_base + 16 * (u & 1) + 4 * (s & 3);
#pragma unroll
      for (int f = 0; f < NFRAG; ++f) {
        const int i = i0 + f * 32;
        off[f] = (kl * RC + ((i >> 3) ^ nc_swz<RC>(kl))) * 16 + (i & 7) * 2;
      }
    }
  }

  // fragment f at k-substep ks of the tile at `lds`
  EVT_DEV u32x4 read(const char* lds, int f, int ks) const {
    if constexpr (LDS_KC) {
      return *(const u32x4*)(lds + off[ks] + f * (32 * CH * 16));
    } else {
      const char* p = lds + off[f] + ks * (16 * RC * 16);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p);
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * RC * 16));
      u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      u32x4 r;
      r.x = l2.x; r.y = l2.y; r.z = h2.x; r.w = h2.y;
      return r;
    }
  }
};

template <bool BF16>
EVT_DEV f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
}

// Workgroup id -> (batch, tile_m, tile_n).  Consecutive ids are dealt
// round-robin to the XCDs by the hardware; undo that so each XCD gets a
// contiguous range of logical ids, then walk tiles in groups of GROUP_M rows
// so a range covers a compact block of the output (shared A and B panels stay
// in that XCD's L2).
template <int GROUP_M>
EVT_DEV void tile_coords(int pid, int nblocks, int tiles_m, int tiles_n, int& batch, int& tm, int& tn) {
  const int per = nblocks / kNumXcd;
  int lid = pid;
  if (pid < per * kNumXcd) lid = (pid % kNumXcd) * per + pid / kNumXcd;
  const int per_batch = tiles_m * tiles_n;
  batch = lid / per_batch;
  const int t = lid - batch * per_batch;
  const int gsz_full = GROUP_M * tiles_n;
  const int group = t / gsz_full;
  const int first_m = group * GROUP_M;
  const int gm = min(tiles_m - first_m, GROUP_M);
  const int in = t - group * gsz_full;
  tm = first_m + in % gm;
  tn = in / gm;
}

// The main loop: acc[mi][ni] += A_tile * B_tile over all k-tiles.
template <class Cfg>
struct Mainloop {
  using OpA = Operand<Cfg::BM, Cfg::BK, Cfg::A_KC, Cfg::DMA, Cfg::THREADS, 0, 0>;
  using OpB = Operand<Cfg::BN, Cfg::BK, Cfg::B_KC, Cfg::DMA, Cfg::THREADS,
                      Cfg::INTERLEAVE ? Cfg::NI : 0, Cfg::TN>;
  using RdA = FragReader<Cfg::BM, Cfg::BK, Cfg::A_LDS_KC, Cfg::MI>;
  using RdB = FragReader<Cfg::BN, Cfg::BK, Cfg::B_LDS_KC, Cfg::NI>;
  static constexpr int LPS = OpA::NLOAD + OpB::NLOAD;   // DMA ops per thread per stage

  static EVT_DEV void compute(const char* lds, const RdA& ra, const RdB& rb,
                              f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
    const char* la = lds;
    const char* lb = lds + Cfg::A_BYTES;
#pragma unroll
    for (int ks = 0; ks < Cfg::KS; ++ks) {
      u32x4 af[Cfg::MI], bf[Cfg::NI];
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi) af[mi] = ra.read(la, mi, ks);
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni) bf[ni] = rb.read(lb, ni, ks);
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < Cfg::NI; ++ni)
          acc[mi][ni] = mfma32<Cfg::BF16>(af[mi], bf[ni], acc[mi][ni]);
    }
  }

  static EVT_DEV void run(const GemmArgs& g, int batch, int m0, int n0, char* smem,
                          f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;

    OpA a;
    OpB b;
    {
      const char* pa = g.A + ((int64_t)batch * g.bsA + (Cfg::A_KC ? (int64_t)m0 * g.lda : (int64_t)m0)) * 2;
      const char* pb = g.B + ((int64_t)batch * g.bsB + (Cfg::B_KC ? (int64_t)n0 * g.ldb : (int64_t)n0)) * 2;
      a.init(pa, g.lda, g.M - m0, g.K, tid);
      b.init(pb, g.ldb, g.N - n0, g.K, tid);
    }
    RdA ra;
    RdB rb;
    ra.init(wm * Cfg::TM, lane);
    rb.init(wn * Cfg::TN, lane);

#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;

    const int KT = (g.K + Cfg::BK - 1) / Cfg::BK;

    if constexpr (Cfg::DMA) {
      // prologue: STAGES-1 tiles in flight
#pragma unroll
      for (int s = 0; s < Cfg::STAGES - 1; ++s) {
        if (s < KT) {
          a.dma(s, smem + s * Cfg::STAGE_BYTES, wave);
          b.dma(s, smem + s * Cfg::STAGE_BYTES + Cfg::A_BYTES, wave);
        }
      }
      int stage = 0;
      for (int kt = 0; kt < KT; ++kt) {
        // tile kt has landed once at most (STAGES-2) younger tiles are pending
        if (kt + Cfg::STAGES - 2 < KT) {
          wait_vmcnt<(Cfg::STAGES - 2) * LPS>();
        } else {
          wait_vmcnt<0>();
        }
        __syncthreads();   // tile kt visible to all waves; everyone left tile kt-1
        const int nk = kt + Cfg::STAGES - 1;
        if (nk < KT) {
          int ns = stage + Cfg::STAGES - 1;
          if (ns >= Cfg::STAGES) ns -= Cfg::STAGES;
          a.dma(nk, smem + ns * Cfg::STAGE_BYTES, wave);
          b.dma(nk, smem + ns * Cfg::STAGE_BYTES + Cfg::A_BYTES, wave);
        }
        compute(smem + stage * Cfg::STAGE_BYTES, ra, rb, acc);
        stage = (stage + 1 == Cfg::STAGES) ? 0 : stage + 1;
      }
    } else {
      u32x4 sa[OpA::NLOAD], sb[OpB::NLOAD];
      a.fetch(0, sa, tid);
      b.fetch(0, sb, tid);
      a.commit(sa, smem, tid);
      b.commit(sb, smem + Cfg::A_BYTES, tid);
      __syncthreads();
      for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) {
          a.fetch(kt + 1, sa, tid);
          b.fetch(kt + 1, sb, tid);
        }
        compute(smem + cur * Cfg::STAGE_BYTES, ra, rb, acc);
        if (kt + 1 < KT) {
          a.commit(sa, smem + (cur ^ 1) * Cfg::STAGE_BYTES, tid);
          b.commit(sb, smem + (cur ^ 1) * Cfg::STAGE_BYTES + Cfg::A_BYTES, tid);
        }
        __syncthreads();
      }
    }
  }
};

}  // namespace evt
