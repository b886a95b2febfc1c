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
  // two-level batch index of an operand: batch l starts (l / bdiv) * bs + (l % bdiv) * bs2 elements in
  // (bdiv = 1: one level); a [B, S, H, D] tensor then serves as B * H batches of [S, D] without a copy
  int bdivA, bdivB;
  int64_t bs2A, bs2B;
  int tiles_m, tiles_n;
  char* workspace;
  // phase 2 of a cross-tile reduction runs inside this kernel (last workgroup
  // to arrive) instead of in a separate finalize kernel
  int row_inkernel, col_inkernel;
  // A per-row reduction may also fold batches into one result: row_fold_count
  // batches share a result; with row_fold_mod they are l, l + row_fold_step, ...
  // (result keyed by l % row_fold_step), otherwise row_fold_count consecutive
  // ones (keyed by l / row_fold_count).  (0, 1, 1): every batch on its own.
  int row_fold_mod, row_fold_step, row_fold_count;
  // A per-column reduction may fold the batches that agree modulo col_fold_step (col_fold_count of them) into
  // one result, keyed by l % col_fold_step.  (1, 1): every batch on its own.
  int col_fold_step, col_fold_count;
  // Split-K: `splits` workgroups share an output tile, each over `k_chunk` (a multiple of BK) of the K extent;
  // they leave their accumulators in the workspace and the last one to arrive adds them up in split order and
  // runs the epilogue.  splits == 1: one workgroup per tile, nothing goes through the workspace.
  int splits, k_chunk;
  // Many splits meet in two levels: `split_group` consecutive splits form a group whose last arriver adds the
  // group's tiles up and leaves one tile; the last group to finish adds up the groups' tiles.  The last arriver of a
  // one-level exchange would read every tile alone.  0 or >= splits: one level.
  int split_group;
  // GemmCfg::WALK: a workgroup computes `walk` consecutive tiles of a row block, left to right, and a per-row
  // reduction leaves one partial per workgroup: parts_n = ceil(tiles_n / walk) of them per row.  Elsewhere
  // walk = 1 and parts_n = tiles_n.
  int walk, parts_n;
};

// Compile-time description of one kernel variant.
//   TILE_IO_  the epilogue reads or writes full tensors: worth giving every lane adjacent output columns
//   WALK_     a workgroup walks over several tiles of a row block (GemmArgs::walk), the operand ring running
//             on from one tile into the next (ping-pong loops only)
//   K_EXACT_  K is a multiple of BK in every launch
template <int BM_, int BN_, int BK_, int WM_, int WN_, bool A_KC_, bool B_KC_,
          bool DMA_, int STAGES_, bool BF16_, int GROUP_M_, int PIPE_ = 0, bool TILE_IO_ = true, bool WALK_ = false,
          bool K_EXACT_ = false>
struct GemmCfg {
  // PIPE 0: ring of STAGES tiles, fragments fetched inside each k-tile.
  // PIPE 1: look-ahead ring (STAGES >= 3): tile kt+1 is made visible one
  //         iteration early so the first fragments of the next k-tile are
  //         fetched under the MFMAs of the current one, and the instruction
  //         order (MFMA / LDS read / DMA issue) is pinned.
  // PIPE 2: ping-pong (8 waves, STAGES >= 2): the two waves that share a SIMD
  //         alternate between a phase of back-to-back MFMAs on fragments held
  //         in registers and a phase of LDS fragment reads; a workgroup
  //         barrier ends every phase, so one wave's LDS traffic always runs
  //         under the other wave's MFMAs.
  // PIPE 3: ping-pong with one barrier per k-tile: the barrier between a
  //         group's read phase and its MFMA phase is dropped and wave
  //         priorities keep the two waves of a SIMD out of step.
  // PIPE 4 + flags: PIPE 3 with options (Mainloop::PP_*):
  //         1  group 0 meets the k-tile barrier inside its MFMA phase, a
  //            quarter of its MFMAs still to issue, so the matrix pipe has work
  //            while the barrier resolves and group 1 starts;
  //         2  group 0 issues its global->LDS transfers between the LDS reads
  //            of its read phase instead of between its MFMAs (with two stages:
  //            instead of in one burst in front of the reads);
  //         4  group 1 does the same (STAGES >= 3).
  // PIPE 12: one wave per SIMD (4 waves, STAGES >= 2): each wave alternates MFMAs on the fragments of one k
  //         sub-step with the LDS reads of the next, its transfers spread between them; one barrier per
  //         k-tile.  A 128 x 256 tile then has 64 x 128 wave tiles, a quarter less LDS read traffic per MFMA
  //         than the 64 x 64 wave tiles of eight waves.
  // PIPE 16 + p (p = 2 ... 11): ping-pong loop p with every k-tile split between the two wave groups instead of
  //         the output tile: waves w and w + 4 compute the same (2 TM) x TN block, one on the first half of each
  //         k-tile's depth, the other on the second, and add their accumulators through LDS behind the loop, each
  //         keeping TM of the rows.  A 128 x 256 tile then has 64 x 128 wave tiles in the loop -- three quarters
  //         of the LDS reads per MFMA of the 64 x 64 ones -- and still two waves per SIMD to alternate.
  static constexpr bool KSPLIT = PIPE_ >= 16;
  static constexpr int PIPE = KSPLIT ? PIPE_ - 16 : PIPE_;
  static constexpr bool SOLO = PIPE == 12;
  static constexpr bool PINGPONG = PIPE >= 2 && !SOLO;
  static constexpr bool WALK = WALK_;
  // K is a multiple of BK in every launch (the host refuses others): see Operand
  static constexpr bool K_EXACT = K_EXACT_;
  static_assert(!WALK_ || K_EXACT_, "the carried-over operand ring has no code for a partial k-tile");
  static constexpr int PP_FLAGS = PIPE >= 4 ? PIPE - 4 : 0;
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr bool A_KC = A_KC_, B_KC = B_KC_, DMA = DMA_, BF16 = BF16_;
  static constexpr int STAGES = STAGES_, GROUP_M = GROUP_M_;
  static constexpr int WAVES = WM * WN;
  static constexpr int THREADS = WAVES * 64;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int MI = TM / 32, NI = TN / 32;
  static constexpr int KS = BK / 16;
  // the wave tile of the main loop: as the epilogue's, or twice its rows with a split k-tile
  static constexpr int LTM = KSPLIT ? 2 * TM : TM, LTN = TN;
  static constexpr int LMI = LTM / 32, LNI = NI;
  // which of the epilogue's wave tiles a wave owns.  With a split k-tile wave 4 g + p (group g, position p of the
  // (WM / 2) x WN grid of loop tiles) keeps rows [g TM, (g + 1) TM) of loop tile p.
  static EVT_DEV int epi_wave(int wave) {
    if constexpr (KSPLIT) {
      const int g = wave >> 2, p = wave & 3;
      return ((p / WN) * 2 + g) * WN + p % WN;
    } else {
      return wave;
    }
  }
  // Layout of each operand tile in LDS: K-contiguous rows, or k-rows.
  static constexpr bool A_LDS_KC = A_KC || !DMA;
  static constexpr bool B_LDS_KC = B_KC || !DMA;
  // With a K-contiguous B tile the rows (= output columns) can be permuted for
  // free while loading, so every lane ends up owning NI adjacent columns.
  static constexpr bool INTERLEAVE = B_LDS_KC && (NI > 1);
  // With a k-row B tile the transposing LDS read hands lane j column j of each 32-column block.  The blocks are
  // then laid over the wave's columns in 4-column pieces (piece p of block f covers columns 4 (p NI + f) ...), and
  // after the main loop the four lanes of a quad exchange accumulators so that every lane again owns NI adjacent
  // columns (regroup_columns): the epilogue's vector accesses work for either operand layout.
  static constexpr bool REGROUP = TILE_IO_ && !B_LDS_KC && (NI == 2 || NI == 4);
  static constexpr bool ADJACENT = INTERLEAVE || REGROUP;   // a lane's NI columns are adjacent in the output
  static constexpr int A_BYTES = BM * BK * 2;
  static constexpr int B_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  // One-wave-per-SIMD workgroups whose LDS leaves room for a second workgroup on the CU are compiled for two
  // waves per SIMD (at most 256 registers): two such workgroups then share a CU and run out of step, one's
  // epilogue under the other's main loop.
  static constexpr int MIN_WAVES_PER_SIMD = (SOLO && LDS_BYTES <= 80 * 1024) ? 2 : 1;
  static_assert(BK == 32 || BK == 64, "BK must be 32 or 64");
  static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be 32-aligned");
  static_assert(STAGES >= 1 && STAGES <= 8, "1..8 stages");
  static_assert(PIPE != 1 || (DMA && STAGES >= 3 && (BK / 16) % 2 == 0), "look-ahead needs DMA, >= 3 stages");
  static_assert(!KSPLIT || (PINGPONG && !WALK_ && WM % 2 == 0 && KS % 2 == 0 && LMI * LNI <= 8 &&
                            WM * WN * MI * NI * 4096 <= STAGES * (BM + BN) * BK * 2),
                "split k-tiles: a ping-pong loop, an even number of wave rows, accumulators of 128 registers at most, "
                "and LDS for one exchange of them");
  static_assert(!PINGPONG || (DMA && STAGES >= 2 && WM * WN == 8), "ping-pong needs DMA, >= 2 stages, 8 waves");
  static_assert(PIPE >= 0 && PIPE <= 12 && PIPE_ <= 27, "unknown pipeline");
  static_assert(!SOLO || (DMA && STAGES >= 2 && WM * WN == 4 && (BK / 16) % 2 == 0), "one wave per SIMD: DMA, >= 2 stages, 4 waves");
  static_assert(!WALK || PINGPONG, "walking over tiles is built into the ping-pong loops");
  static_assert(!(PP_FLAGS & 4) || STAGES >= 3, "group 1 can only issue in its read phase with three or more stages");
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

EVT_DEV __amdgpu_buffer_rsrc_t make_rsrc(const char* p, uint32_t num_records = kRsrcRange) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, num_records, kRsrcFlags);
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
//   K_EXACT  K is a multiple of BK (the host checks): no k-tile is partial, so the transfers need no per-lane
//            test against K, and a k-tile past the end reads as zeros through an empty buffer range
// ---------------------------------------------------------------------------
template <int ROWS, int BK, bool SRC_KC, bool DMA, int THREADS, int PERM_NI, int PERM_TN, bool K_EXACT = false>
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
  struct DmaTile {
    __amdgpu_buffer_rsrc_t rsrc;
    int k0;
  };
  EVT_DEV DmaTile dma_begin(int kt) const {
    const int64_t adv = SRC_KC ? (int64_t)kt * BK * 2 : (int64_t)kt * BK * ld * 2;
    if constexpr (K_EXACT) return DmaTile{make_rsrc(base + adv, kt * BK < K ? kRsrcRange : 0u), kt * BK};
    else return DmaTile{make_rsrc(base + adv), kt * BK};
  }
  // transfer number i (of NLOAD) of this thread
  EVT_DEV void dma_chunk(const DmaTile& d, char* lds, int wave, int i) const {
    uint32_t v = voff[i];
    if constexpr (!K_EXACT) v = (d.k0 + kin[i] < K) ? voff[i] : kOobOffset;
    char* dst = lds + (i * THREADS + wave * 64) * 16;   // wave-uniform; lane*16 added by hardware
    __builtin_amdgcn_raw_ptr_buffer_load_lds(d.rsrc, (lds_void_ptr)dst, 16, v, 0, 0, 0);
  }
  EVT_DEV void dma(int kt, char* lds, int wave) const {
    const DmaTile d = dma_begin(kt);
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) dma_chunk(d, lds, wave, i);
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

// LDS reads issued through inline assembly.  The compiler orders every LDS
// access it can see behind all outstanding global->LDS transfers (it cannot
// tell the ring stages apart), which would drain the DMA ring at each k-tile;
// these reads are invisible to that logic.  The caller waits for them with
// lds_wait_all() and then passes every destination through lds_pin().
EVT_DEV u32x4 lds_read_b128(uint32_t addr) {
  u32x4 r;
  asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}
EVT_DEV u32x2 lds_read_tr16_b64(uint32_t addr) {
  u32x2 r;
  asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}
EVT_DEV void lds_wait_all() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
template <class T>
EVT_DEV void lds_pin(T& x) { asm volatile("" : "+v"(x)); }
EVT_DEV uint32_t lds_addr(const char* p) { return (uint32_t)(uintptr_t)p; }

// Per-lane LDS read addressing of MFMA operand fragments (32 rows x 16 k).
//   PIECES  (k-row tiles only) > 0: fragment f takes its 32 rows in 8 pieces of 4, piece p = rows
//           4 (p PIECES + f) ... of the wave's slice (GemmCfg::REGROUP); 0: rows 32 f ...
template <int ROWS, int BK, bool LDS_KC, int NFRAG, int PIECES = 0>
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
      const int i0 = wave_row_base + (PIECES > 0 ? ((u & 1) * 4 + (s & 3)) * 4 * PIECES : 16 * (u & 1) + 4 * (s & 3));
#pragma unroll
      for (int f = 0; f < NFRAG; ++f) {
        const int i = i0 + f * (PIECES > 0 ? 4 : 32);
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

  // All fragments of one k-tile (ping-pong pipeline), read with the inline
  // assembly helpers: issue(), then lds_wait_all(), then pin(), then frag().
  static constexpr int KSN = BK / 16;
  struct Tile {
    u32x4 q[LDS_KC ? KSN * NFRAG : 1];
    u32x2 h[LDS_KC ? 1 : 2 * KSN * NFRAG];
  };
  // number of LDS read instructions of one k-tile, and read number i of them (k-sub-step major)
  static constexpr int NREADS = LDS_KC ? KSN * NFRAG : 2 * KSN * NFRAG;
  EVT_DEV void issue_one(uint32_t lds, Tile& t, int i) const {
    if constexpr (LDS_KC) {
      const int ks = i / NFRAG, f = i % NFRAG;
      t.q[i] = lds_read_b128(lds + off[ks] + f * (32 * CH * 16));
    } else {
      const int pr = i >> 1, ks = pr / NFRAG, f = pr % NFRAG;
      t.h[i] = lds_read_tr16_b64(lds + off[f] + ks * (16 * RC * 16) + (i & 1) * (4 * RC * 16));
    }
  }
  EVT_DEV void issue(uint32_t lds, Tile& t) const {
#pragma unroll
    for (int i = 0; i < NREADS; ++i) issue_one(lds, t, i);
  }
  // The fragments of one k sub-step (one wave per SIMD pipeline): issue_sub() for every i < SUB_READS, then
  // lds_wait_all(), pin_sub(), frag_sub().
  struct Sub {
    u32x4 q[LDS_KC ? NFRAG : 1];
    u32x2 h[LDS_KC ? 1 : 2 * NFRAG];
  };
  static constexpr int SUB_READS = LDS_KC ? NFRAG : 2 * NFRAG;
  EVT_DEV void issue_sub(uint32_t lds, Sub& t, int ks, int i) const {
    if constexpr (LDS_KC) {
      t.q[i] = lds_read_b128(lds + off[ks] + i * (32 * CH * 16));
    } else {
      const int f = i >> 1;
      t.h[i] = lds_read_tr16_b64(lds + off[f] + ks * (16 * RC * 16) + (i & 1) * (4 * RC * 16));
    }
  }
  EVT_DEV void pin_sub(Sub& t) const {
    if constexpr (LDS_KC) {
#pragma unroll
      for (int i = 0; i < NFRAG; ++i) lds_pin(t.q[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 2 * NFRAG; ++i) lds_pin(t.h[i]);
    }
  }
  EVT_DEV u32x4 frag_sub(const Sub& t, int f) const {
    if constexpr (LDS_KC) {
      return t.q[f];
    } else {
      const u32x2 lo = t.h[2 * f], hi = t.h[2 * f + 1];
      u32x4 r;
      r.x = lo.x; r.y = lo.y; r.z = hi.x; r.w = hi.y;
      return r;
    }
  }
  EVT_DEV void pin(Tile& t) const { pin_reads<0, NREADS>(t); }
  // the destinations of reads [LO, HI) (numbered as issue_one numbers them)
  template <int LO, int HI>
  EVT_DEV void pin_reads(Tile& t) const {
    if constexpr (LDS_KC) {
#pragma unroll
      for (int i = LO; i < HI; ++i) lds_pin(t.q[i]);
    } else {
#pragma unroll
      for (int i = LO; i < HI; ++i) lds_pin(t.h[i]);
    }
  }
  EVT_DEV u32x4 frag(const Tile& t, int f, int ks) const {
    if constexpr (LDS_KC) {
      return t.q[ks * NFRAG + f];
    } else {
      const u32x2 lo = t.h[2 * (ks * NFRAG + f)], hi = t.h[2 * (ks * NFRAG + f) + 1];
      u32x4 r;
      r.x = lo.x; r.y = lo.y; r.z = hi.x; r.w = hi.y;
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

// GemmCfg::REGROUP: lane c of a quad holds column c of NI four-column pieces (piece f in acc[.][f]); afterwards
// it holds NI adjacent columns in acc[.][0 .. NI-1].  NI = 4: a 4 x 4 transpose inside the quad, lane c ends up
// with piece c.  NI = 2: one exchange with the neighbouring lane; even lanes end up with columns c, c + 1 of piece
// 0, odd lanes with columns c - 1, c of piece 1 (TileCtx::init has the matching column offsets).
EVT_DEV float quad_xchg1(float x) {   // value of lane ^ 1
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0xB1, 0xf, 0xf, true));
}
EVT_DEV float quad_xchg2(float x) {   // value of lane ^ 2
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x4E, 0xf, 0xf, true));
}
template <class Cfg>
EVT_DEV void regroup_columns(f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
  if constexpr (Cfg::REGROUP) {
    const int lane = threadIdx.x & 63;
    const bool b0 = lane & 1, b1 = lane & 2;
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
#pragma unroll
        for (int f = 0; f < Cfg::NI; f += 2) {   // 2 x 2 transposes between lanes c, c ^ 1 on pieces (f, f + 1)
          const float e0 = acc[mi][f][v], e1 = acc[mi][f + 1][v];
          const float got = quad_xchg1(b0 ? e0 : e1);
          acc[mi][f][v] = b0 ? got : e0;
          acc[mi][f + 1][v] = b0 ? e1 : got;
        }
        if constexpr (Cfg::NI == 4) {            // and between lanes c, c ^ 2 on pieces (f, f + 2)
#pragma unroll
          for (int f = 0; f < 2; ++f) {
            const float e0 = acc[mi][f][v], e1 = acc[mi][f + 2][v];
            const float got = quad_xchg2(b1 ? e0 : e1);
            acc[mi][f][v] = b1 ? got : e0;
            acc[mi][f + 2][v] = b1 ? e1 : got;
          }
        }
      }
    }
  }
}

// The main loop: acc[mi][ni] += A_tile * B_tile over all k-tiles.
template <class Cfg>
struct Mainloop {
  using OpA = Operand<Cfg::BM, Cfg::BK, Cfg::A_KC, Cfg::DMA, Cfg::THREADS, 0, 0, Cfg::K_EXACT>;
  using OpB = Operand<Cfg::BN, Cfg::BK, Cfg::B_KC, Cfg::DMA, Cfg::THREADS,
                      Cfg::INTERLEAVE ? Cfg::LNI : 0, Cfg::LTN, Cfg::K_EXACT>;
  using RdA = FragReader<Cfg::BM, Cfg::BK, Cfg::A_LDS_KC, Cfg::LMI>;
  using RdB = FragReader<Cfg::BN, Cfg::BK, Cfg::B_LDS_KC, Cfg::LNI, Cfg::REGROUP ? Cfg::LNI : 0>;
  static constexpr int LPS = OpA::NLOAD + OpB::NLOAD;   // DMA ops per thread per stage

  // One k-tile: KS sub-steps of MI x NI MFMAs.  Fragments of sub-step ks+1
  // are fetched from LDS into a second register set while the MFMAs of
  // sub-step ks issue.
  static EVT_DEV void compute(const char* lds, const RdA& ra, const RdB& rb,
                              f32x16 (&acc)[Cfg::LMI][Cfg::LNI]) {
    const char* la = lds;
    const char* lb = lds + Cfg::A_BYTES;
    u32x4 af[2][Cfg::LMI], bf[2][Cfg::LNI];
#pragma unroll
    for (int mi = 0; mi < Cfg::LMI; ++mi) af[0][mi] = ra.read(la, mi, 0);
#pragma unroll
    for (int ni = 0; ni < Cfg::LNI; ++ni) bf[0][ni] = rb.read(lb, ni, 0);
#pragma unroll
    for (int ks = 0; ks < Cfg::KS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < Cfg::KS) {
#pragma unroll
        for (int mi = 0; mi < Cfg::LMI; ++mi) af[nxt][mi] = ra.read(la, mi, ks + 1);
#pragma unroll
        for (int ni = 0; ni < Cfg::LNI; ++ni) bf[nxt][ni] = rb.read(lb, ni, ks + 1);
      }
#pragma unroll
      for (int mi = 0; mi < Cfg::LMI; ++mi)
#pragma unroll
        for (int ni = 0; ni < Cfg::LNI; ++ni)
          acc[mi][ni] = mfma32<Cfg::BF16>(af[cur][mi], bf[cur][ni], acc[mi][ni]);
    }
  }

  // ---- look-ahead pipeline (PIPE == 1) -------------------------------------
  struct Frags {
    u32x4 a[Cfg::LMI];
    u32x4 b[Cfg::LNI];
  };
  static constexpr int NMFMA = Cfg::LMI * Cfg::LNI;
  static constexpr int NDSREAD = (Cfg::A_LDS_KC ? Cfg::LMI : 2 * Cfg::LMI) + (Cfg::B_LDS_KC ? Cfg::LNI : 2 * Cfg::LNI);

  static EVT_DEV void load_frags(Frags& f, const char* lds, const RdA& ra, const RdB& rb, int ks) {
#pragma unroll
    for (int mi = 0; mi < Cfg::LMI; ++mi) f.a[mi] = ra.read(lds, mi, ks);
#pragma unroll
    for (int ni = 0; ni < Cfg::LNI; ++ni) f.b[ni] = rb.read(lds + Cfg::A_BYTES, ni, ks);
  }
  static EVT_DEV void mma(const Frags& f, f32x16 (&acc)[Cfg::LMI][Cfg::LNI]) {
#pragma unroll
    for (int mi = 0; mi < Cfg::LMI; ++mi)
#pragma unroll
      for (int ni = 0; ni < Cfg::LNI; ++ni) acc[mi][ni] = mfma32<Cfg::BF16>(f.a[mi], f.b[ni], acc[mi][ni]);
  }
  // Scheduling directive for one sub-step of NMFMA MFMAs: NR LDS reads and NV
  // global->LDS transfers are placed between the MFMAs.  The compiler cannot
  // tell that a transfer and an LDS read touch different stages, so it keeps
  // their program order; reads therefore go first (behind the leading MFMAs)
  // and the transfers behind the trailing MFMAs.
  template <int M, int NR, int NV>
  static EVT_DEV void pin_order() {
    if constexpr (M < NMFMA) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (NV == 0) {
        constexpr int r = (NR * (M + 1)) / NMFMA - (NR * M) / NMFMA;
        if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
      } else {
        constexpr int H = NMFMA / 2;
        if constexpr (M < H) {
          constexpr int r = (NR * (M + 1)) / H - (NR * M) / H;
          if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
        } else {
          constexpr int v = (NV * (M - H + 1)) / H - (NV * (M - H)) / H;
          if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x020, v, 0);
        }
      }
      pin_order<M + 1, NR, NV>();
    }
  }
  template <int N>
  static EVT_DEV void wait_tiles() {   // leave N younger tiles in flight
    wait_vmcnt<N * LPS>();
  }
  static EVT_DEV void wait_tiles_dyn(int n) {
    static_assert((Cfg::STAGES - 2) * LPS < 64, "vmcnt is a 6-bit counter");
    if (n <= 0) wait_tiles<0>();
    else if (n == 1) wait_tiles<1>();
    else if (n == 2) wait_tiles<2>();
    else if (n == 3) wait_tiles<(Cfg::STAGES > 4 ? 3 : 0)>();
    else if (n == 4) wait_tiles<(Cfg::STAGES > 5 ? 4 : 0)>();
    else if (n == 5) wait_tiles<(Cfg::STAGES > 6 ? 5 : 0)>();
    else wait_tiles<(Cfg::STAGES > 7 ? 6 : 0)>();
  }

  template <bool STEADY>
  static EVT_DEV void lookahead_iter(int kt, int KT, int& stage, const OpA& a, const OpB& b, const RdA& ra,
                                     const RdB& rb, char* smem, int wave, Frags (&f)[2],
                                     f32x16 (&acc)[Cfg::LMI][Cfg::LNI]) {
    constexpr int S = Cfg::STAGES, D = S - 1;
    if constexpr (STEADY) {
      wait_tiles<D - 2>();            // tile kt+1 has landed (tiles kt+2.. may be in flight)
    } else {
      const int newest = min(kt + D, KT) - 1;
      if (kt + 1 < KT) wait_tiles_dyn(newest - (kt + 1));
    }
    __syncthreads();                  // tile kt+1 visible to all; everyone is done with tile kt-1
    const char* cur = smem + stage * Cfg::STAGE_BYTES;
    int nstage = stage + 1 == S ? 0 : stage + 1;
    const char* nxt = smem + nstage * Cfg::STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < Cfg::KS; ++ks) {
      if (ks + 1 < Cfg::KS) {
        load_frags(f[(ks + 1) & 1], cur, ra, rb, ks + 1);
      } else if (STEADY || kt + 1 < KT) {
        load_frags(f[0], nxt, ra, rb, 0);
      }
      if constexpr (STEADY) {
        if (ks == Cfg::KS - 1) {   // refill the stage tile kt-1 occupied
          int ds = stage + D;
          if (ds >= S) ds -= S;
          a.dma(kt + D, smem + ds * Cfg::STAGE_BYTES, wave);
          b.dma(kt + D, smem + ds * Cfg::STAGE_BYTES + Cfg::A_BYTES, wave);
        }
      }
      mma(f[ks & 1], acc);
      if constexpr (STEADY) {
        if (ks == Cfg::KS - 1) pin_order<0, NDSREAD, LPS>();
        else pin_order<0, NDSREAD, 0>();
      }
    }
    stage = nstage;
  }

  static EVT_DEV void run_lookahead(const OpA& a, const OpB& b, const RdA& ra, const RdB& rb, char* smem,
                                    int wave, int KT, f32x16 (&acc)[Cfg::LMI][Cfg::LNI]) {
    constexpr int S = Cfg::STAGES, D = S - 1;
#pragma unroll
    for (int s = 0; s < D; ++s) {
      if (s < KT) {
        a.dma(s, smem + s * Cfg::STAGE_BYTES, wave);
        b.dma(s, smem + s * Cfg::STAGE_BYTES + Cfg::A_BYTES, wave);
      }
    }
    wait_tiles_dyn(min(D, KT) - 1);   // tile 0 has landed
    __syncthreads();
    Frags f[2];
    load_frags(f[0], smem, ra, rb, 0);
    int stage = 0;
    int kt = 0;
    for (; kt + D < KT; ++kt) lookahead_iter<true>(kt, KT, stage, a, b, ra, rb, smem, wave, f, acc);
    for (; kt < KT; ++kt) lookahead_iter<false>(kt, KT, stage, a, b, ra, rb, smem, wave, f, acc);
  }

  // ---- ping-pong pipeline (PIPE == 2) --------------------------------------
  // Waves w and w+4 run on the same SIMD.  Group 0 (waves 0-3) and group 1
  // (waves 4-7) each walk the k-tiles with two phases per tile: R(T) reads all
  // fragments of tile T from LDS into registers, C(T) issues the MFMAs of tile
  // T.  A workgroup barrier ends every phase and group 1 runs one phase behind
  // group 0, so at any time one wave of a SIMD is in C and the other in R:
  //
  //   phase      2T          2T+1        2T+2        2T+3
  //   group 0    R(T)        C(T)        R(T+1)      C(T+1)
  //   group 1    C(T-1)      R(T)        C(T)        R(T+1)
  //
  // Tile T is read during phases 2T and 2T+1, so the stage of tile T-1 may be
  // refilled with tile T+STAGES-1 from phase 2T on.  The texture path moves
  // only about 64 bytes per clock, so a wave that issues its transfers in one
  // burst stalls for hundreds of cycles; the transfers are therefore spread
  // between the MFMAs of a C phase: group 1 issues its share in C(T-1) (phase
  // 2T) and, with three or more stages, group 0 its share in C(T) (phase
  // 2T+1).  With two stages group 0 has to issue at the start of R(T) to give
  // the data two phases to land.  Every wave waits for its share of tile T+1
  // before the barrier that ends phase 2T+1.  Both groups execute exactly
  // 1 + 2*KT barriers.  Only the barriers that end the odd phases order memory
  // (tile T+1 visible, stage of tile T free); the ones that end the even phases
  // merely pace the two groups, and PIPE 3 leaves them out: group 1 then runs
  // its MFMA phase at a higher wave priority than group 0, so after each
  // barrier group 1 computes first while group 0 reads, and they swap.
  struct TileFrags {
    typename RdA::Tile a;
    typename RdB::Tile b;
  };
  // With a split k-tile (GemmCfg::KSPLIT) group KH reads and multiplies the k sub-steps [KH KS / 2, (KH + 1) KS / 2)
  // of every tile (the reads of a tile are numbered k-sub-step major), on a wave tile of twice the rows.
  static constexpr int PP_DIV = Cfg::KSPLIT ? 2 : 1;
  static constexpr int PP_KS = Cfg::KS / PP_DIV;
  static constexpr int PP_NM = PP_KS * Cfg::LMI * Cfg::LNI;   // MFMAs per C phase
  static constexpr int PP_KH1 = Cfg::KSPLIT ? 1 : 0;          // the half of a k-tile that group 1 takes
  static constexpr bool PP_MIDC = (Cfg::PP_FLAGS & 1) != 0;
  static constexpr bool PP_G0_IN_R = (Cfg::PP_FLAGS & 2) != 0;
  static constexpr bool PP_G1_IN_R = (Cfg::PP_FLAGS & 4) != 0;
  static constexpr bool PP_G0_IN_C = !PP_G0_IN_R && Cfg::STAGES >= 3;
  static constexpr int PP_REST = PP_MIDC ? (PP_NM / 4 > 0 ? PP_NM / 4 : 1) : 0;   // group 0's MFMAs behind the barrier
  static constexpr int PP_NRA = RdA::NREADS / PP_DIV, PP_NRB = RdB::NREADS / PP_DIV;
  static constexpr int PP_NR = PP_NRA + PP_NRB;             // LDS reads per R phase
  // R phase: all fragments of the tile at `lds` are in registers on return.  With ISSUE the transfers of
  // k-tile `nk` into stage `ds` go between the reads (transfer c behind read number (c * PP_NR) / LPS): a wave
  // that waits for LDS anyway absorbs the pacing of the texture path, and the MFMA phases stay pure.
  template <bool ISSUE, int KH = 0>
  static EVT_DEV void pp_read(TileFrags& f, const char* lds, const RdA& ra, const RdB& rb,
                              const OpA& a, const OpB& b, int nk, char* ds, int wave) {
    typename OpA::DmaTile da;
    typename OpB::DmaTile db;
    if constexpr (ISSUE) {
      da = a.dma_begin(nk);
      db = b.dma_begin(nk);
    }
    const uint32_t la = lds_addr(lds), lb = lds_addr(lds + Cfg::A_BYTES);
#pragma unroll
    for (int i = 0; i < PP_NR; ++i) {
      if (i < PP_NRA) ra.issue_one(la, f.a, KH * PP_NRA + i);
      else rb.issue_one(lb, f.b, KH * PP_NRB + i - PP_NRA);
      if constexpr (ISSUE) {
#pragma unroll
        for (int c = 0; c < LPS; ++c) {
          if ((c * PP_NR) / LPS == i) {
            if (c < OpA::NLOAD) a.dma_chunk(da, ds, wave, c);
            else b.dma_chunk(db, ds + Cfg::A_BYTES, wave, c - OpA::NLOAD);
          }
        }
      }
    }
    lds_wait_all();
    ra.template pin_reads<KH * PP_NRA, (KH + 1) * PP_NRA>(f.a);
    rb.template pin_reads<KH * PP_NRB, (KH + 1) * PP_NRB>(f.b);
  }
  // MFMAs [M, MEND) of a C phase, transfer c (of LPS) behind MFMA number (c * SPREAD) / LPS
  template <int M, int MEND, int SPREAD>
  static EVT_DEV void pp_pin_order() {
    if constexpr (M < MEND) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      constexpr int n = ((M + 1) * LPS + SPREAD - 1) / SPREAD - (M * LPS + SPREAD - 1) / SPREAD;
      if constexpr (n > 0 && M < SPREAD) __builtin_amdgcn_sched_group_barrier(0x020, n, 0);
      pp_pin_order<M + 1, MEND, SPREAD>();
    }
  }
  // MFMAs [M0, M1) of the C phase (numbered k-sub-step major); with ISSUE the transfers of k-tile `nk` into
  // stage `ds` are spread between them
  template <bool ISSUE, int PRIO, int M0, int M1, int KH = 0>
  static EVT_DEV void pp_mma(const TileFrags& f, const RdA& ra, const RdB& rb, f32x16 (&acc)[Cfg::LMI][Cfg::LNI],
                             const OpA& a, const OpB& b, int nk, char* ds, int wave) {
    static_assert(!ISSUE || M0 == 0, "transfers are spread from the first MFMA on");
    typename OpA::DmaTile da;
    typename OpB::DmaTile db;
    if constexpr (ISSUE) {
      da = a.dma_begin(nk);
      db = b.dma_begin(nk);
    }
    __builtin_amdgcn_s_setprio(PRIO);
#pragma unroll
    for (int kk = 0; kk < PP_KS; ++kk) {
      const int ks = KH * PP_KS + kk;
#pragma unroll
      for (int mi = 0; mi < Cfg::LMI; ++mi) {
#pragma unroll
        for (int ni = 0; ni < Cfg::LNI; ++ni) {
          const int m = (kk * Cfg::LMI + mi) * Cfg::LNI + ni;
          if (m < M0 || m >= M1) continue;
          acc[mi][ni] = mfma32<Cfg::BF16>(ra.frag(f.a, mi, ks), rb.frag(f.b, ni, ks), acc[mi][ni]);
          if constexpr (ISSUE) {
#pragma unroll
            for (int c = 0; c < LPS; ++c) {
              if ((c * M1) / LPS == m) {
                if (c < OpA::NLOAD) a.dma_chunk(da, ds, wave, c);
                else b.dma_chunk(db, ds + Cfg::A_BYTES, wave, c - OpA::NLOAD);
              }
            }
          }
        }
      }
    }
    if constexpr (ISSUE) pp_pin_order<M0, M1, M1>();
    __builtin_amdgcn_s_setprio(0);
  }
  // Transfers are issued for every T, also past the last k-tile: a tile index
  // beyond K reads as zeros through the buffer range check (no memory traffic)
  // and lands in a stage nobody reads any more, which keeps the vmcnt
  // bookkeeping uniform and the loop free of a second code path.
  static EVT_DEV char* pp_refill_stage(int stage, char* smem) {   // the stage tile T-1 occupied
    const int ds = stage == 0 ? Cfg::STAGES - 1 : stage - 1;
    return smem + ds * Cfg::STAGE_BYTES;
  }
  static EVT_DEV void pp_issue(int nk, int stage, const OpA& a, const OpB& b, char* smem, int wave) {
    char* ds = pp_refill_stage(stage, smem);
    a.dma(nk, ds, wave);
    b.dma(nk, ds + Cfg::A_BYTES, wave);
  }
  // GemmCfg::WALK: what a workgroup carries from one tile of its walk to the next.  The operand ring does not
  // drain between tiles: while another tile follows (`more`), the transfers issued past the last k-tile fetch
  // the first STAGES-1 k-tiles of that tile (same rows of A, B moved on by BN) instead of zeros, so they are
  // in flight or landed while the epilogue runs, and the next main loop starts as if in steady state.  The
  // stage that held the last k-tile is not refilled before that loop's first iteration: it is the epilogue's
  // LDS (epilogue_lds).
  struct Walk {
    int stage = 0;        // ring stage of k-tile 0 of the coming tile
    bool primed = false;  // its first STAGES-1 k-tiles have been issued
  };
  static EVT_DEV char* epilogue_lds(const Walk& wk, char* smem) {
    if constexpr (Cfg::WALK) return pp_refill_stage(wk.stage, smem);
    else return smem;
  }
  // Phase barriers are bare s_barrier instructions: the only memory traffic of
  // the loop is the DMA (waited for explicitly with vmcnt) and the
  // inline-assembly LDS reads (waited for inside pp_read); a fence here would
  // make the compiler drain the DMA ring at every phase.
  static EVT_DEV void pp_barrier() { __builtin_amdgcn_s_barrier(); }
  static EVT_DEV void run_pingpong(const OpA& a, OpB& b, const RdA& ra, const RdB& rb, char* smem,
                                   int wave, int KT, f32x16 (&acc)[Cfg::LMI][Cfg::LNI],
                                   Walk& wk, bool more, int64_t b_step, int tid) {
    constexpr int S = Cfg::STAGES;
    static_assert((S - 1) * LPS < 64, "vmcnt is a 6-bit counter");
    int stage = 0;
    if constexpr (Cfg::WALK) stage = wk.primed ? wk.stage : 0;
    if (!Cfg::WALK || !wk.primed) {
#pragma unroll
      for (int s = 0; s < S - 1; ++s) {
        a.dma(s, smem + s * Cfg::STAGE_BYTES, wave);
        b.dma(s, smem + s * Cfg::STAGE_BYTES + Cfg::A_BYTES, wave);
      }
    }
    // tile 0 has landed.  In a walk the count also covers what the epilogue in between issued after the
    // transfers (the counter runs in issue order), so this waits for those accesses too.
    wait_tiles<S - 2>();
    __syncthreads();
    TileFrags f;
    const int grp = wave >> 2;
    // k-tile to fetch in iteration T: T + S - 1 of this tile, or, past its end with a tile to follow, of that one
    auto fetch_index = [&](int T) {
      int nk = T + S - 1;
      if constexpr (Cfg::WALK) {
        if (more && nk >= KT) nk -= KT;
      }
      return nk;
    };
    auto move_on = [&](int T) {   // from here on the transfers belong to the next tile: B moves on by BN
      if constexpr (Cfg::WALK) {
        if (more && T + S - 1 == KT) {
          int t2 = tid;
          asm volatile("" : "+v"(t2));   // computed here, once per tile, not ahead of the loop and kept in registers
          b.init(b.base + b_step, b.ld, b.rows_left - Cfg::BN, b.K, t2);
        }
      }
    };
    if (grp == 0) {
      for (int T = 0; T < KT; ++T) {
        move_on(T);
        const int nk = fetch_index(T);
        char* ds = pp_refill_stage(stage, smem);
        if constexpr (!PP_G0_IN_C && !PP_G0_IN_R) pp_issue(nk, stage, a, b, smem, wave);
        pp_read<PP_G0_IN_R>(f, smem + stage * Cfg::STAGE_BYTES, ra, rb, a, b, nk, ds, wave);
        if constexpr (Cfg::PIPE == 2) pp_barrier();   // ends phase 2T
        pp_mma<PP_G0_IN_C, 1, 0, PP_NM - PP_REST>(f, ra, rb, acc, a, b, nk, ds, wave);
        wait_tiles<S - 2>();        // my share of tile T+1 has landed
        pp_barrier();               // ends phase 2T+1
        if constexpr (PP_REST > 0) pp_mma<false, 3, PP_NM - PP_REST, PP_NM>(f, ra, rb, acc, a, b, 0, ds, wave);
        stage = stage + 1 == S ? 0 : stage + 1;
      }
    } else {
      if constexpr (!PP_G1_IN_R) pp_issue(S - 1, stage, a, b, smem, wave);
      for (int T = 0; T < KT; ++T) {
        move_on(T);
        const int nk = fetch_index(T);
        char* ds = pp_refill_stage(stage, smem);
        if (T > 0) pp_mma<!PP_G1_IN_R, 2, 0, PP_NM, PP_KH1>(f, ra, rb, acc, a, b, nk, ds, wave);   // C(T-1)
        if constexpr (Cfg::PIPE == 2) pp_barrier();   // ends phase 2T
        pp_read<PP_G1_IN_R, PP_KH1>(f, smem + stage * Cfg::STAGE_BYTES, ra, rb, a, b, nk, ds, wave);
        wait_tiles<S - 2>();        // my share of tile T+1 has landed
        pp_barrier();               // ends phase 2T+1
        stage = stage + 1 == S ? 0 : stage + 1;
      }
      if (KT > 0) pp_mma<false, 2, 0, PP_NM, PP_KH1>(f, ra, rb, acc, a, b, 0, smem, wave);   // C(KT-1)
    }
    if constexpr (Cfg::WALK) {
      wk.stage = stage;
      wk.primed = more;
      if (!more) wait_vmcnt<0>();   // the zero-fill transfers past the last tile have landed
    } else {
      wait_vmcnt<0>();              // the zero-fill transfers past the last tile have landed
    }
  }

  // ---- one wave per SIMD (PIPE 12) ------------------------------------------
  // Four waves, each alone on its SIMD, so nothing else fills the matrix pipe while a wave reads: every wave
  // works through the k sub-steps (16 wide) of a k-tile with two fragment sets, issuing after each MFMA of
  // sub-step s its share of the LDS reads of sub-step s+1 (of the next k-tile behind the last one) and of the
  // transfers of k-tile T+STAGES-1 into the stage tile T-1 occupied.  The order is pinned instruction by
  // instruction; the reads are waited for once per sub-step, a whole sub-step of MFMAs after they were issued.
  // One barrier per k-tile, in front of the first reads of the next: tile T+1 has landed for every wave, and
  // every wave has the last fragments of tile T in registers, so its stage may be refilled from then on.
  // Sub-steps of two k steps (eight MFMAs on a 64 x 64 wave tile, with the transfers of a k-tile in half as
  // many slots) measured 5-10 % slower, 32-deep k-tiles in rings of 4-6 stages 4-20 % slower; with two stages the
  // transfers of tile T+1 go out less than a k-tile before they are needed, and the loop waits for them.
  struct SubFrags {
    typename RdA::Sub a;
    typename RdB::Sub b;
  };
  static constexpr int SO_NR = RdA::SUB_READS + RdB::SUB_READS;   // LDS reads per sub-step
  static constexpr int SO_NM = Cfg::LMI * Cfg::LNI;                 // MFMAs per sub-step
  static EVT_DEV void so_read_all(SubFrags& f, const char* lds, const RdA& ra, const RdB& rb, int ks) {
    const uint32_t la = lds_addr(lds), lb = lds_addr(lds + Cfg::A_BYTES);
#pragma unroll
    for (int i = 0; i < RdA::SUB_READS; ++i) ra.issue_sub(la, f.a, ks, i);
#pragma unroll
    for (int i = 0; i < RdB::SUB_READS; ++i) rb.issue_sub(lb, f.b, ks, i);
  }
  static EVT_DEV void run_solo(const OpA& a, const OpB& b, const RdA& ra, const RdB& rb, char* smem,
                               int wave, int KT, f32x16 (&acc)[Cfg::LMI][Cfg::LNI]) {
    constexpr int S = Cfg::STAGES, KS = Cfg::KS;
    static_assert((S - 1) * LPS < 64, "vmcnt is a 6-bit counter");
    // transfers past the last k-tile read as zeros (or are switched off lane by lane) and land in stages nobody
    // reads any more: the vmcnt bookkeeping stays uniform
#pragma unroll
    for (int s = 0; s < S - 1; ++s) {
      a.dma(s, smem + s * Cfg::STAGE_BYTES, wave);
      b.dma(s, smem + s * Cfg::STAGE_BYTES + Cfg::A_BYTES, wave);
    }
    wait_tiles<S - 2>();   // my share of tile 0 has landed
    pp_barrier();
    SubFrags f[2];
    so_read_all(f[0], smem, ra, rb, 0);
    int stage = 0;
    for (int T = 0; T < KT; ++T) {
      const int nstage = stage + 1 == S ? 0 : stage + 1;
      const char* cur = smem + stage * Cfg::STAGE_BYTES;
      const char* nxt = smem + nstage * Cfg::STAGE_BYTES;
      char* ds = pp_refill_stage(stage, smem);
      const typename OpA::DmaTile da = a.dma_begin(T + S - 1);
      const typename OpB::DmaTile db = b.dma_begin(T + S - 1);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        SubFrags& now = f[ks & 1];
        SubFrags& next = f[(ks + 1) & 1];
        lds_wait_all();            // the fragments of this sub-step, issued a sub-step ago
        ra.pin_sub(now.a);
        rb.pin_sub(now.b);
        const bool last = ks == KS - 1;
        const uint32_t la = lds_addr(last ? nxt : cur), lb = la + Cfg::A_BYTES;
        const int nks = last ? 0 : ks + 1;
        // Slots: the reads of the next sub-step go out behind the first MFMAs (SO_RD of them), so that they are
        // back long before the sub-step ends; the transfers behind the others.  In the last sub-step of a k-tile
        // the barrier stands behind the first SO_BAR MFMAs -- the matrix pipe has work while it resolves -- and
        // the reads, which are of the next k-tile, follow it.
        constexpr int SO_RD = SO_NM >= 4 ? SO_NM / 2 : SO_NM, SO_BAR = SO_NM >= 4 ? 2 : 1;
        constexpr int PER = (LPS + KS - 2) / (KS - 1);           // transfers per sub-step
#pragma unroll
        for (int m = 0; m < SO_NM; ++m) {
          const int mi = m / Cfg::LNI, ni = m % Cfg::LNI;
          acc[mi][ni] = mfma32<Cfg::BF16>(ra.frag_sub(now.a, mi), rb.frag_sub(now.b, ni), acc[mi][ni]);
          __builtin_amdgcn_sched_barrier(0);
          if (last && m == SO_BAR - 1) {
            wait_tiles<S - 2>();     // my share of tile T+1 has landed
            pp_barrier();            // everybody's has; everybody holds the last fragments of tile T
          }
          const int r0 = last ? SO_BAR - 1 : 0;                  // first slot with reads
#pragma unroll
          for (int i = 0; i < SO_NR; ++i) {
            if (r0 + (i * SO_RD) / SO_NR == m) {
              if (i < RdA::SUB_READS) ra.issue_sub(la, next.a, nks, i);
              else rb.issue_sub(lb, next.b, nks, i - RdA::SUB_READS);
            }
          }
          if (!last) {             // the transfers go out during the first KS-1 sub-steps, behind the barrier of tile T-1
#pragma unroll
            for (int j = 0; j < PER; ++j) {
              const int c = ks * PER + j;
              if (c < LPS && SO_RD % SO_NM + (j * (SO_NM - SO_RD % SO_NM)) / PER == m) {
                if (c < OpA::NLOAD) a.dma_chunk(da, ds, wave, c);
                else b.dma_chunk(db, ds + Cfg::A_BYTES, wave, c - OpA::NLOAD);
              }
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      stage = nstage;
    }
    lds_wait_all();                // the reads issued behind the last tile (nobody uses them)
    wait_vmcnt<0>();               // the transfers past the last tile have landed
  }

  static EVT_DEV void run(const GemmArgs& g, int batch, int m0, int n0, int split, char* smem,
                          f32x16 (&acc)[Cfg::LMI][Cfg::LNI]) {
    Walk wk;
    run(g, batch, m0, n0, split, smem, acc, wk, false);
  }
  // `wk`, `more`: see Walk (WALK kernels call this once per tile of the walk, `more` while another follows)
  static EVT_DEV void run(const GemmArgs& g, int batch, int m0, int n0, int split, char* smem,
                          f32x16 (&acc)[Cfg::LMI][Cfg::LNI], Walk& wk, bool more) {
    int tid = threadIdx.x;
    // In a walk this runs once per tile with the epilogue in between.  Everything below that depends only on
    // the thread index (transfer offsets, fragment addresses) would be hoisted out of the tile loop and then
    // stay live, or spilled, through the epilogue, which needs every register itself; hiding where `tid` comes
    // from makes the compiler derive them afresh for each tile.
    if constexpr (Cfg::WALK) asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // with a split k-tile the two groups share the loop's wave tiles: position wave & 3 of a (WM / 2) x WN grid
    const int wpos = Cfg::KSPLIT ? (wave & 3) : wave;
    const int wm = wpos / Cfg::WN, wn = wpos % Cfg::WN;

    OpA a;
    OpB b;
    {
      // this workgroup's share of K: [k_lo, k_lo + Kw)
      const int k_lo = split * g.k_chunk;
      const int Kw_ = g.K - k_lo < g.k_chunk ? g.K - k_lo : g.k_chunk;
      const int64_t boA = (int64_t)(batch / g.bdivA) * g.bsA + (int64_t)(batch % g.bdivA) * g.bs2A;
      const int64_t boB = (int64_t)(batch / g.bdivB) * g.bsB + (int64_t)(batch % g.bdivB) * g.bs2B;
      const char* pa = g.A + (boA + (Cfg::A_KC ? (int64_t)m0 * g.lda + k_lo : (int64_t)m0 + (int64_t)k_lo * g.lda)) * 2;
      const char* pb = g.B + (boB + (Cfg::B_KC ? (int64_t)n0 * g.ldb + k_lo : (int64_t)n0 + (int64_t)k_lo * g.ldb)) * 2;
      a.init(pa, g.lda, g.M - m0, Kw_, tid);
      b.init(pb, g.ldb, g.N - n0, Kw_, tid);
    }
    const int Kw = (g.K - split * g.k_chunk < g.k_chunk) ? g.K - split * g.k_chunk : g.k_chunk;
    RdA ra;
    RdB rb;
    ra.init(wm * Cfg::LTM, lane);
    rb.init(wn * Cfg::LTN, lane);

#pragma unroll
    for (int mi = 0; mi < Cfg::LMI; ++mi)
#pragma unroll
      for (int ni = 0; ni < Cfg::LNI; ++ni)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;

    const int KT = (Kw + Cfg::BK - 1) / Cfg::BK;

    if constexpr (Cfg::PIPE == 1) {
      run_lookahead(a, b, ra, rb, smem, wave, KT, acc);
    } else if constexpr (Cfg::SOLO) {
      run_solo(a, b, ra, rb, smem, wave, KT, acc);
    } else if constexpr (Cfg::PINGPONG) {
      run_pingpong(a, b, ra, rb, smem, wave, KT, acc, wk, more,
                   Cfg::B_KC ? (int64_t)Cfg::BN * g.ldb * 2 : (int64_t)Cfg::BN * 2, tid);
    } else if constexpr (Cfg::DMA && Cfg::STAGES == 1) {
      // K fits one tile (checked by the host): load it, use it
      a.dma(0, smem, wave);
      b.dma(0, smem + Cfg::A_BYTES, wave);
      wait_vmcnt<0>();
      __syncthreads();
      compute(smem, ra, rb, acc);
    } else if constexpr (Cfg::DMA) {
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
