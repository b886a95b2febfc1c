// Epilogue-visitor building blocks that run on the MFMA accumulator registers.
//
// Role in the reference (apuaaChen/EVT_AE): the node vocabulary and callback
// order of src/cuda/epilogue/threadblock/visitor.hpp:33-113 (begin_epilogue /
// visit / end_row / end_epilogue), visitor_load.hpp (accumulator fetch, scalar,
// row and column broadcast, aux load), visitor_compute.hpp (fp32 compute,
// one-hot, comparisons) and visitor_store.hpp (aux store, per-row and
// per-column reductions).  The code generator emits straight-line C++ that
// calls these helpers; all intermediates are fp32 and each stored value is
// rounded once (visitor.hpp:221-226, visitor_store.hpp:99-112).
//
// Differences by design: reductions do not use atomics into pre-zeroed
// outputs (visitor_store.hpp:293-301, :544-553).  Phase 1: each workgroup
// reduces its tile with wave64 cross-lane operations and LDS and writes one
// partial per (tile, row) or (tile, column) to a workspace.  Phase 2: a small
// finalize kernel combines the partials in a fixed order and evaluates the
// per-row / per-column output expressions, so results are deterministic and
// no output needs pre-zeroing.
#pragma once

#include "evt_gemm.hpp"

namespace evt {

// ---------------------------------------------------------------------------
// elementwise functions (fp32)
// ---------------------------------------------------------------------------
// v_exp_f32 / v_log_f32 / v_rcp_f32 are base-2 / 1-ulp hardware functions; the
// constants fold the base change.  Errors are ~1e-7 relative, far inside the
// 2e-2 / 1e-3 parity contract.
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
EVT_DEV float op_exp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }
// exp(x - m) with m_log2e = m * log2(e) computed once per row: one multiply-add per element in front of the
// exponential instead of a subtraction and a multiplication
EVT_DEV float op_exp_minus(float x, float m_log2e) { return __builtin_amdgcn_exp2f(__builtin_fmaf(x, kLog2e, -m_log2e)); }
EVT_DEV float op_log(float x) { return __builtin_amdgcn_logf(x) * kLn2; }
EVT_DEV float op_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
// sigmoid(x) = 1 / (1 + 2^(-x log2 e)); saturates to 0 / 1 for |x| large
EVT_DEV float op_sigmoid(float x) { return op_rcp(1.f + __builtin_amdgcn_exp2f(-kLog2e * x)); }
EVT_DEV float op_tanh(float x) { return 2.f * op_sigmoid(2.f * x) - 1.f; }
EVT_DEV float op_relu(float x) { return x > 0.f ? x : 0.f; }
// gelu_tanh(x) = 0.5 x (1 + tanh(u)) = x sigmoid(2u),  u = sqrt(2/pi) (x + 0.044715 x^3)
constexpr float kGeluA = -2.f * 0.7978845608028654f * kLog2e;   // -2 sqrt(2/pi) log2(e)
constexpr float kGeluB = kGeluA * 0.044715f;
EVT_DEV float gelu_sig(float x, float x2) {   // sigmoid(2u)
  return op_rcp(1.f + __builtin_amdgcn_exp2f(x * (kGeluA + kGeluB * x2)));
}
EVT_DEV float op_gelu_tanh(float x) { return x * gelu_sig(x, x * x); }
EVT_DEV float op_gelu_erf(float x) { return 0.5f * x * (1.f + erff(x * 0.7071067811865476f)); }
EVT_DEV float op_tanh_backward(float gy, float y) { return gy * (1.f - y * y); }
// d/dx gelu_tanh = s + 2 sqrt(2/pi) x s (1 - s) (1 + 3*0.044715 x^2),  s = sigmoid(2u)
EVT_DEV float op_gelu_backward_tanh(float gy, float x) {
  const float x2 = x * x;
  const float s = gelu_sig(x, x2);
  const float a = (2.f * 0.7978845608028654f) * x * (1.f + (3.f * 0.044715f) * x2);
  return gy * (s + s * (a - a * s));
}
EVT_DEV float op_gelu_backward_erf(float gy, float x) {
  const float cdf = 0.5f * (1.f + erff(x * 0.7071067811865476f));
  const float pdf = 0.3989422804014327f * op_exp(-0.5f * x * x);
  return gy * (cdf + x * pdf);
}

// round-trip through a storage type (models aten.to / _to_copy inside the tree)
template <class T>
EVT_DEV float round_to(float x) { return (float)(T)x; }

// ---------------------------------------------------------------------------
// typed loads / stores
// ---------------------------------------------------------------------------
template <class T>
EVT_DEV float ld_f32(const T* p, int64_t off) { return (float)p[off]; }
template <>
EVT_DEV float ld_f32<bool>(const bool* p, int64_t off) { return p[off] ? 1.f : 0.f; }

template <class T>
EVT_DEV void st_f32(T* p, int64_t off, float v) { p[off] = (T)v; }
template <>
EVT_DEV void st_f32<bool>(bool* p, int64_t off, float v) { p[off] = (v != 0.f); }

// a value as its store would round it, and back (exact): what st_f32 writes for v equals what it writes for
// from_storage(to_storage<T>(v))
template <class T>
EVT_DEV T to_storage(float v) { return (T)v; }
template <>
EVT_DEV bool to_storage<bool>(float v) { return v != 0.f; }
template <class T>
EVT_DEV float from_storage(T v) { return (float)v; }
template <>
EVT_DEV float from_storage<bool>(bool v) { return v ? 1.f : 0.f; }

// ---------------------------------------------------------------------------
// Where this lane's accumulator elements live in the output.
// acc[mi][ni][v] is element (row(mi, v), col(ni)).
// ---------------------------------------------------------------------------
// FULL: the whole workgroup tile lies inside the matrix, so no bound checks.
template <class Cfg, bool FULL_>
struct TileCtx {
  static constexpr bool FULL = FULL_;
  static constexpr int MI = Cfg::MI, NI = Cfg::NI;
  static constexpr bool INTERLEAVE = Cfg::ADJACENT;   // this lane's NI columns are adjacent
  static constexpr int COL_STEP = INTERLEAVE ? 1 : 32;
  int M, N, L;
  int batch, tile_m, tile_n, tiles_m, tiles_n;
  int m0, n0;          // tile origin
  int row0, col0;      // this lane's first row / column
  int row_u, col_u;    // their wave-uniform parts (scalar registers) ...
  int row_l, col_l;    // ... and per-lane parts: row0 = row_u + row_l, col0 = col_u + col_l
  int tid, lane, wm, wn;
  char* smem;
  char* workspace;
  // Per-row reductions: this workgroup's partial is number part_n of parts_n along the row.  Without a walk
  // that is the tile; in a walk (GemmCfg::WALK) the tiles of a workgroup fold into a running state per row,
  // kept in LDS at walk_state, and the partial leaves with the last tile.
  int part_n, parts_n;
  bool walk_first, walk_last;
  float* walk_state;

  EVT_DEV void init(const GemmArgs& g, int batch_, int tm, int tn, char* smem_) {
    M = g.M; N = g.N; L = g.L;
    batch = batch_; tile_m = tm; tile_n = tn; tiles_m = g.tiles_m; tiles_n = g.tiles_n;
    part_n = tn; parts_n = g.tiles_n; walk_first = walk_last = true; walk_state = nullptr;
    m0 = tm * Cfg::BM; n0 = tn * Cfg::BN;
    tid = threadIdx.x;
    // walking kernels run main loop and epilogue in turn: keep this lane's indices from being computed once
    // ahead of the tile loop and carried through every main loop (see Mainloop::run)
    if constexpr (Cfg::WALK) asm volatile("" : "+v"(tid));
    lane = tid & 63;
    const int wave = Cfg::epi_wave(__builtin_amdgcn_readfirstlane(tid >> 6));
    wm = wave / Cfg::WN; wn = wave % Cfg::WN;
    row_u = m0 + wm * Cfg::TM; row_l = 4 * (lane >> 5);
    col_u = n0 + wn * Cfg::TN;
    if constexpr (Cfg::REGROUP && NI == 2) col_l = 8 * ((lane & 31) >> 2) + ((lane & 1) << 2) + (lane & 2);   // see regroup_columns
    else col_l = INTERLEAVE ? (lane & 31) * NI : (lane & 31);
    row0 = row_u + row_l;
    col0 = col_u + col_l;
    smem = smem_; workspace = g.workspace;
  }
  EVT_DEV void set_walk(int part, int parts, bool first, bool last, float* state) {
    part_n = part; parts_n = parts; walk_first = first; walk_last = last; walk_state = state;
  }
  EVT_DEV int row(int mi, int v) const { return row0 + mi * 32 + 8 * (v >> 2) + (v & 3); }
  // row of register (mi, v) relative to row0: a compile-time constant once the loops are unrolled
  static EVT_DEV int row_step(int mi, int v) { return mi * 32 + 8 * (v >> 2) + (v & 3); }
  EVT_DEV int col(int ni) const { return col0 + ni * COL_STEP; }
  EVT_DEV bool col_ok(int ni) const { return FULL || col(ni) < N; }
  EVT_DEV bool row_ok(int r) const { return FULL || r < M; }
  // row / column index local to the workgroup tile
  EVT_DEV int lrow(int mi, int v) const { return row(mi, v) - m0; }
  EVT_DEV int lcol(int ni) const { return col(ni) - n0; }
  // number of valid columns in this wave's slice of the row
  EVT_DEV int wave_cols() const {
    const int left = N - (n0 + wn * Cfg::TN);
    return left < 0 ? 0 : (left > Cfg::TN ? Cfg::TN : left);
  }
};

// Load NI values of one accumulator row from an (l, m, n)-strided tensor, in
// its storage type (the generated code issues the loads of 16 rows together,
// ahead of the arithmetic, because loads may not move above stores by
// themselves).  `off` is the element offset of (batch, row, col(0)).
//   FAST   the workgroup tile is interior and the tensor is unit-stride along
//          n (and aligned for the interleaved vector access): no bound checks,
//          no flag tests -- straight-line code the scheduler can batch.
//   else   `flags` bit 0: unit stride along n; bit 1: aligned so the NI
//          adjacent elements of an interleaved lane move as one access
//          (4, 8 or 16 bytes for NI = 2, 4, 8 columns of a 16-bit type).
template <bool FAST, class T, class Tile>
EVT_DEV void aux_load(const Tile& t, const T* p, int64_t off, int64_t sn, int flags, bool rok,
                      T (&out)[Tile::NI]) {
  constexpr int NI = Tile::NI;
  const T* rp = p + off;
  constexpr bool kVec = Tile::INTERLEAVE && sizeof(T) == 2 && (NI == 2 || NI == 4 || NI == 8);
  if constexpr (kVec) {
    if (FAST || ((flags & 2) && rok && t.col0 + NI <= t.N)) {
      if constexpr (NI == 8) {
        const u32x4 raw = *(const u32x4*)rp;
        const T* e = (const T*)&raw;
#pragma unroll
        for (int ni = 0; ni < 8; ++ni) out[ni] = e[ni];
      } else if constexpr (NI == 4) {
        const u32x2 raw = *(const u32x2*)rp;
        const T* e = (const T*)&raw;
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) out[ni] = e[ni];
      } else {
        const uint32_t raw = *(const uint32_t*)rp;
        const T* e = (const T*)&raw;
        out[0] = e[0]; out[1] = e[1];
      }
      return;
    }
  }
  if constexpr (FAST) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) out[ni] = rp[ni * Tile::COL_STEP];
  } else if (flags & 1) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) out[ni] = (rok && t.col_ok(ni)) ? rp[ni * Tile::COL_STEP] : T(0);
  } else {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
      out[ni] = (rok && t.col_ok(ni)) ? rp[(int64_t)ni * Tile::COL_STEP * sn] : T(0);
  }
}

template <bool FAST, class T, class Tile>
EVT_DEV void aux_store(const Tile& t, T* p, int64_t off, int64_t sn, int flags, bool rok,
                       const float (&val)[Tile::NI]) {
  constexpr int NI = Tile::NI;
  T* rp = p + off;
  constexpr bool kVec = Tile::INTERLEAVE && sizeof(T) == 2 && (NI == 2 || NI == 4 || NI == 8);
  if constexpr (kVec) {
    if (FAST || ((flags & 2) && rok && t.col0 + NI <= t.N)) {
      T e[NI];
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) e[ni] = (T)val[ni];
      if constexpr (NI == 8) {
        *(u32x4*)rp = *(const u32x4*)e;
      } else if constexpr (NI == 4) {
        *(u32x2*)rp = *(const u32x2*)e;
      } else {
        *(uint32_t*)rp = *(const uint32_t*)e;
      }
      return;
    }
  }
  if constexpr (FAST) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) st_f32<T>(rp, ni * Tile::COL_STEP, val[ni]);
  } else if (flags & 1) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
      if (rok && t.col_ok(ni)) st_f32<T>(rp, ni * Tile::COL_STEP, val[ni]);
  } else {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
      if (rok && t.col_ok(ni)) st_f32<T>(rp, (int64_t)ni * Tile::COL_STEP * sn, val[ni]);
  }
}

// Check-free access to one accumulator row of a unit-stride tensor, through buffer instructions: `rs` is a
// buffer resource whose base is this wave's corner of the tile (scalar registers), `voff` this lane's byte offset
// inside a row (one register per tensor, the same for every row) and `soff` the row's byte offset from that corner
// (scalar arithmetic) -- no per-row vector address arithmetic.  The bytes a lane moves per row: NI adjacent
// 16-bit elements as one access of 4, 8 or 16 bytes, anything else element by element.
template <class Tile, class T>
constexpr bool row_is_vector() {
  return Tile::INTERLEAVE && sizeof(T) == 2 && (Tile::NI == 2 || Tile::NI == 4 || Tile::NI == 8);
}
template <class T>
EVT_DEV T buffer_load_elem(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
  if constexpr (sizeof(T) == 4) return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(rs, voff, soff, 0));
  else if constexpr (sizeof(T) == 2) return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b16(rs, voff, soff, 0));
  else return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b8(rs, voff, soff, 0));
}
// One value per row (a column vector of the epilogue) through the buffer path of the check-free epilogue:
// `rs` starts at the wave's first row, voff is this lane's byte offset, soff the row's (wave-uniform).
template <class T>
EVT_DEV float buffer_ld_f32(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
  if constexpr (sizeof(T) == 8) {
    const u32x2 raw = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs, voff, soff, 0));
    return (float)__builtin_bit_cast(T, raw);
  } else if constexpr (sizeof(T) == 1) {   // bool
    return buffer_load_elem<uint8_t>(rs, voff, soff) ? 1.f : 0.f;
  } else {
    return (float)buffer_load_elem<T>(rs, voff, soff);
  }
}

// On a tile that is not whole (Tile::FULL false) the same instructions serve: a lane whose row or columns lie
// outside the matrix gets an offset beyond the buffer's range, which the hardware answers with zeros (loads) or
// drops (stores) -- no branch, no per-element address arithmetic.  The caller has checked that valid columns
// come in whole vectors (N a multiple of NI) where a lane's NI columns move as one access.
template <class Tile, class T>
EVT_DEV void row_load(const Tile& t, bool rok, __amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff, T (&out)[Tile::NI]) {
  constexpr int NI = Tile::NI;
  if constexpr (!Tile::FULL) {
    if (!rok || (row_is_vector<Tile, T>() && t.col0 + NI > t.N)) voff = kOobOffset;
  }
  if constexpr (row_is_vector<Tile, T>() && NI == 8) {
    const u32x4 raw = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, 0);
    const T* e = (const T*)&raw;
#pragma unroll
    for (int ni = 0; ni < 8; ++ni) out[ni] = e[ni];
  } else if constexpr (row_is_vector<Tile, T>() && NI == 4) {
    const u32x2 raw = __builtin_amdgcn_raw_buffer_load_b64(rs, voff, soff, 0);
    const T* e = (const T*)&raw;
#pragma unroll
    for (int ni = 0; ni < 4; ++ni) out[ni] = e[ni];
  } else if constexpr (row_is_vector<Tile, T>() && NI == 2) {
    const uint32_t raw = __builtin_amdgcn_raw_buffer_load_b32(rs, voff, soff, 0);
    const T* e = (const T*)&raw;
    out[0] = e[0]; out[1] = e[1];
  } else {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
      out[ni] = buffer_load_elem<T>(rs, t.col_ok(ni) ? voff + (uint32_t)(ni * Tile::COL_STEP * (int)sizeof(T)) : kOobOffset, soff);
  }
}

// NI elements of a 16-bit type in NI / 2 registers
template <class T, int NI>
struct PackOf {
  typedef T type __attribute__((ext_vector_type(NI)));
};
// NI values of one row held in their storage type until a deferred store: a packed vector for 16-bit types with an
// even count (two per register), a plain array otherwise; both are indexed [ni].
template <class T, int NI, bool PACK = (sizeof(T) == 2 && NI % 2 == 0)>
struct StorageRow {
  struct type {
    T e[NI];
    EVT_DEV T& operator[](int i) { return e[i]; }
    EVT_DEV const T& operator[](int i) const { return e[i]; }
  };
};
template <class T, int NI>
struct StorageRow<T, NI, true> {
  typedef typename PackOf<T, NI>::type type;
};

// Output tiles are written once and not read again by this kernel: their stores carry the device-scope,
// non-temporal cache policy (sc1 nt), which sends the data on to memory as it is written instead of leaving it
// dirty in the L2 until the write-back at the end of the kernel -- the write then runs under the kernel's remaining
// work instead of behind it (measured on the attention-score product: 15.1 -> 10.9 us per launch).
constexpr int kStoreStreaming = 16 | 2;   // sc1 | nt
template <class T>
EVT_DEV void buffer_store_elem(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff, float v) {
  if constexpr (sizeof(T) == 4) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, (T)v), rs, voff, soff, kStoreStreaming);
  } else if constexpr (sizeof(T) == 2) {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, (T)v), rs, voff, soff, kStoreStreaming);
  } else {
    __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(v != 0.f), rs, voff, soff, kStoreStreaming);   // bool
  }
}
template <class Tile, class T>
EVT_DEV void row_store(const Tile& t, bool rok, __amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff,
                       const float (&val)[Tile::NI]) {
  constexpr int NI = Tile::NI;
  if constexpr (!Tile::FULL) {
    if (!rok || (row_is_vector<Tile, T>() && t.col0 + NI > t.N)) voff = kOobOffset;
  }
  if constexpr (row_is_vector<Tile, T>()) {
    T e[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) e[ni] = (T)val[ni];
    if constexpr (NI == 8) __builtin_amdgcn_raw_buffer_store_b128(*(const u32x4*)e, rs, voff, soff, kStoreStreaming);
    else if constexpr (NI == 4) __builtin_amdgcn_raw_buffer_store_b64(*(const u32x2*)e, rs, voff, soff, kStoreStreaming);
    else __builtin_amdgcn_raw_buffer_store_b32(*(const uint32_t*)e, rs, voff, soff, kStoreStreaming);
  } else {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
      buffer_store_elem<T>(rs, t.col_ok(ni) ? voff + (uint32_t)(ni * Tile::COL_STEP * (int)sizeof(T)) : kOobOffset, soff, val[ni]);
  }
}

// ---------------------------------------------------------------------------
// rand_like: counter-based uniform numbers, one Philox4x32-10 block per four
// consecutive elements of the rand_like tensor.  Element e (row-major index in
// that tensor) takes word (e & 3) of
//   Philox4x32-10(counter = (lo32(e >> 2), hi32(e >> 2), lo32(offset), salt),
//                 key = (lo32(seed), hi32(seed)))
// mapped to [0, 1) as (word >> 8) * 2^-24, so the values do not depend on the
// tile configuration.  Takes the place of VisitorRand (curand Philox4_32_10
// with a per-thread subsequence,
// src/cuda/epilogue/threadblock/visitor_load.hpp:79-151).
// ---------------------------------------------------------------------------
EVT_DEV void philox4x32_10(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c[0]), lo0 = 0xD2511F53u * c[0];
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c[2]), lo1 = 0xCD9E8D57u * c[2];
    c[0] = hi1 ^ c[1] ^ k0;
    c[1] = lo1;
    c[2] = hi0 ^ c[3] ^ k1;
    c[3] = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

// NI values of one accumulator row; e0 is the element index of (row, col(0)),
// sn the index step between neighbouring columns.
template <class Tile>
EVT_DEV void rand_row(uint64_t seed, uint32_t offset, uint32_t salt, int64_t e0, int64_t sn, float (&out)[Tile::NI]) {
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  int64_t group = -1;
#pragma unroll
  for (int ni = 0; ni < Tile::NI; ++ni) {
    const int64_t e = e0 + (int64_t)ni * Tile::COL_STEP * sn;
    if (ni == 0 || (e >> 2) != group) {   // neighbouring columns of an interleaved lane share a block
      group = e >> 2;
      w[0] = (uint32_t)group; w[1] = (uint32_t)((uint64_t)group >> 32); w[2] = offset; w[3] = salt;
      philox4x32_10(w, (uint32_t)seed, (uint32_t)(seed >> 32));
    }
    const int sel = (int)(e & 3);
    const uint32_t word = sel == 0 ? w[0] : sel == 1 ? w[1] : sel == 2 ? w[2] : w[3];
    out[ni] = (float)(word >> 8) * 5.9604644775390625e-08f;
  }
}

// 8 values of a row kernel's lane: elements e0, e0 + sn, ... (same stream as rand_row)
EVT_DEV void rand8(uint64_t seed, uint32_t offset, uint32_t salt, int64_t e0, int64_t sn, float (&out)[8]) {
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  int64_t group = -1;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int64_t e = e0 + (int64_t)j * sn;
    if (j == 0 || (e >> 2) != group) {
      group = e >> 2;
      w[0] = (uint32_t)group; w[1] = (uint32_t)((uint64_t)group >> 32); w[2] = offset; w[3] = salt;
      philox4x32_10(w, (uint32_t)seed, (uint32_t)(seed >> 32));
    }
    const int sel = (int)(e & 3);
    const uint32_t word = sel == 0 ? w[0] : sel == 1 ? w[1] : sel == 2 ? w[2] : w[3];
    out[j] = (float)(word >> 8) * 5.9604644775390625e-08f;
  }
}

// ---------------------------------------------------------------------------
// cross-lane exchange inside one 32-lane half of a wave (the 32 lanes that hold
// the 32 columns of one accumulator row).  After the 5 steps every lane of the
// half holds the combined value.
// ---------------------------------------------------------------------------
template <int STEP>
EVT_DEV float half_wave_xchg(float x) {
  static_assert(STEP >= 0 && STEP <= 3, "steps 0..3 stay inside a row of 16 lanes");
  const int xi = __builtin_bit_cast(int, x);
  int r;
  if constexpr (STEP == 0) r = __builtin_amdgcn_mov_dpp(xi, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
  else if constexpr (STEP == 1) r = __builtin_amdgcn_mov_dpp(xi, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
  else if constexpr (STEP == 2) r = __builtin_amdgcn_mov_dpp(xi, 0x141, 0xf, 0xf, true);  // row_half_mirror
  else r = __builtin_amdgcn_mov_dpp(xi, 0x140, 0xf, 0xf, true);                           // row_mirror
  return __builtin_bit_cast(float, r);
}
// Last step, between the two rows of 16 lanes of a half: v_permlane16_swap exchanges the odd rows of its first
// operand with the even rows of its second, so with both equal to x the operands end up holding the even and the
// odd row of each pair in every lane -- a VALU instruction, where ds_swizzle goes through the LDS crossbar and
// costs its latency once per accumulator row.  (Written as assembly, with the two wait states the instruction
// needs after a VALU write of its operands and before a VALU read of its results.)
EVT_DEV void row_pair_split(float x, float& even_row, float& odd_row) {
  even_row = x;
  odd_row = x;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(even_row), "+v"(odd_row));
}

EVT_DEV float half_wave_sum(float x) {
  x += half_wave_xchg<0>(x);
  x += half_wave_xchg<1>(x);
  x += half_wave_xchg<2>(x);
  x += half_wave_xchg<3>(x);
  float a, b;
  row_pair_split(x, a, b);
  return a + b;
}
EVT_DEV float half_wave_max(float x) {
  x = fmaxf(x, half_wave_xchg<0>(x));
  x = fmaxf(x, half_wave_xchg<1>(x));
  x = fmaxf(x, half_wave_xchg<2>(x));
  x = fmaxf(x, half_wave_xchg<3>(x));
  float a, b;
  row_pair_split(x, a, b);
  return fmaxf(a, b);
}

// ---------------------------------------------------------------------------
// workspace layout (bytes): [arrival counters | row partials | column partials]
//   counters        one int per (batch, row block) and per (batch, column block)
//   row partials    [L][parts_n][M][ROW_STATE] floats (only if parts_n > 1; parts_n = tiles_n unless workgroups walk)
//   column partials [L][tiles_m][N][COL_STATE] floats (only if tiles_m > 1)
// The counters must be zero before the first launch (evt_workspace_init); a
// launch leaves them zero.  Partials are written before they are read by
// every launch.
// ---------------------------------------------------------------------------
// Phase 2 inside the GEMM kernel pays for few partials.  The last workgroup of a row block pays a ticket round
// trip, one round trip for the partials and their combination on one CU, while everybody else is done; measured
// on 1024 x 131072 (64 partials of three floats per row, 256 rows per block): 6.7 us slower than the finalize
// kernel, which spreads the same work over the chip.  Column partials are one or two floats and fold cheaply.
constexpr int kMaxInKernelPartials = 64;
constexpr int kMaxInKernelRowPartials = 16;

struct WsLayout {
  int64_t counter_bytes, row_bytes, col_bytes;
  int64_t split_counter_bytes, split_bytes;     // split-K: one arrival counter per tile, one accumulator tile per split
  __host__ __device__ int64_t total() const { return counter_bytes + row_bytes + col_bytes + split_counter_bytes + split_bytes; }
};

// a per-row reduction goes through the workspace when several tiles span the
// row or several batches fold into one result
__host__ __device__ inline bool row_uses_workspace(const GemmArgs& g) { return g.parts_n > 1 || g.row_fold_count > 1; }

template <int ROW_STATE, int COL_STATE>
__host__ __device__ inline WsLayout ws_layout(const GemmArgs& g) {
  WsLayout w;
  const bool row = ROW_STATE > 0 && row_uses_workspace(g);
  const bool col = COL_STATE > 0 && (g.tiles_m > 1 || g.col_fold_count > 1);
  const int64_t ncnt = (row ? (int64_t)g.L * g.tiles_m : 0) + (col ? (int64_t)g.L * g.tiles_n : 0);
  w.counter_bytes = (ncnt * 4 + 255) / 256 * 256;
  w.row_bytes = row ? ((int64_t)g.L * g.parts_n * g.M * ROW_STATE * 4 + 255) / 256 * 256 : 0;
  w.col_bytes = col ? ((int64_t)g.L * g.tiles_m * g.N * COL_STATE * 4 + 255) / 256 * 256 : 0;
  w.split_counter_bytes = w.split_bytes = 0;
  return w;
}
// number of groups of a two-level split-K exchange (GemmArgs::split_group), 0 for one level
__host__ __device__ inline int split_groups(const GemmArgs& g) {
  return (g.split_group > 1 && g.split_group < g.splits) ? (g.splits + g.split_group - 1) / g.split_group : 0;
}
// with the split-K regions, which need the tile size
template <class Cfg, int ROW_STATE, int COL_STATE>
__host__ __device__ inline WsLayout ws_layout_split(const GemmArgs& g) {
  WsLayout w = ws_layout<ROW_STATE, COL_STATE>(g);
  if (g.splits > 1) {
    const int64_t tiles = (int64_t)g.L * g.tiles_m * g.tiles_n;
    const int groups = split_groups(g);      // 0: one level
    w.split_counter_bytes = (tiles * (1 + groups) * 4 + 255) / 256 * 256;
    w.split_bytes = tiles * (g.splits + groups) * Cfg::BM * Cfg::BN * 4;
  }
  return w;
}

// batch index of a tensor argument: batches that agree modulo l_mod, or l_div
// consecutive ones, share elements
__host__ __device__ inline int batch_index(int batch, int l_mod, int l_div) {
  return (l_mod > 0 ? batch % l_mod : batch) / l_div;
}
// element offset of a batch: two levels, batch = outer * l_div + inner (stride_l2 = 0: the l_div inner ones share)
__host__ __device__ inline int64_t batch_offset(int batch, int l_mod, int l_div, int64_t stride_l, int64_t stride_l2) {
  const int lb = l_mod > 0 ? batch % l_mod : batch;
  return (int64_t)(lb / l_div) * stride_l + (int64_t)(lb % l_div) * stride_l2;
}
// folded per-row reductions: the result a batch contributes to, and the j-th batch that contributes to a result
__host__ __device__ inline int fold_key(const GemmArgs& g, int batch) {
  return g.row_fold_count == 1 ? batch : (g.row_fold_mod ? batch % g.row_fold_step : batch / g.row_fold_count);
}
__host__ __device__ inline int fold_member(const GemmArgs& g, int key, int j) {
  return g.row_fold_count == 1 ? key : (g.row_fold_mod ? key + j * g.row_fold_step : key * g.row_fold_count + j);
}
// folded per-column reductions (batches that agree modulo col_fold_step share a result)
__host__ __device__ inline bool col_uses_workspace(const GemmArgs& g) { return g.tiles_m > 1 || g.col_fold_count > 1; }
__host__ __device__ inline int col_fold_key(const GemmArgs& g, int batch) {
  return g.col_fold_count == 1 ? batch : batch % g.col_fold_step;
}
__host__ __device__ inline int col_fold_member(const GemmArgs& g, int key, int j) {
  return g.col_fold_count == 1 ? key : key + j * g.col_fold_step;
}

// Device-scope accesses for data exchanged between workgroups inside one
// kernel.  The eight XCDs have separate L2 caches; a relaxed agent-scope atomic
// store is written through and a relaxed agent-scope atomic load is served
// from the coherence point, so neither needs the L2 write-back / invalidate a
// release / acquire fence would cost.
EVT_DEV void st_device(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// N consecutive floats at byte offset `voff` of `rs` with the same cache policy (sc1: written through to, read
// from the point where the XCDs' L2s meet), in accesses of up to 16 bytes.  A state of three floats moved word by
// word costs three transactions per cache line, and the reading side, which bypasses its caches, fetches every
// line three times.
constexpr int kAuxDevice = 16;   // sc1
// (a __builtin_bit_cast applied directly to an element of a vector reads the vector's first element with this
// compiler: the element goes through a scalar first)
EVT_DEV float word_as_float(uint32_t w) { return __builtin_bit_cast(float, w); }
template <int N>
EVT_DEV void st_device_n(__amdgpu_buffer_rsrc_t rs, uint32_t voff, const float* v) {
  if constexpr (N >= 4) {
    __builtin_amdgcn_raw_buffer_store_b128(u32x4{__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
                                                 __builtin_bit_cast(uint32_t, v[2]), __builtin_bit_cast(uint32_t, v[3])},
                                           rs, voff, 0, kAuxDevice);
    if constexpr (N > 4) st_device_n<N - 4>(rs, voff + 16, v + 4);
  } else if constexpr (N == 3) {
    typedef uint32_t u32x3_t __attribute__((ext_vector_type(3)));
    __builtin_amdgcn_raw_buffer_store_b96(u32x3_t{__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
                                                  __builtin_bit_cast(uint32_t, v[2])}, rs, voff, 0, kAuxDevice);
  } else if constexpr (N == 2) {
    __builtin_amdgcn_raw_buffer_store_b64(u32x2{__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1])},
                                          rs, voff, 0, kAuxDevice);
  } else if constexpr (N == 1) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v[0]), rs, voff, 0, kAuxDevice);
  }
}
template <int N>
EVT_DEV void ld_device_n(__amdgpu_buffer_rsrc_t rs, uint32_t voff, float* out) {
  if constexpr (N >= 4) {
    const u32x4 r = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, 0, kAuxDevice);
#pragma unroll
    for (int c = 0; c < 4; ++c) out[c] = word_as_float(r[c]);
    if constexpr (N > 4) ld_device_n<N - 4>(rs, voff + 16, out + 4);
  } else if constexpr (N == 3) {
    typedef uint32_t u32x3_t __attribute__((ext_vector_type(3)));
    const u32x3_t r = __builtin_amdgcn_raw_buffer_load_b96(rs, voff, 0, kAuxDevice);
#pragma unroll
    for (int c = 0; c < 3; ++c) out[c] = word_as_float(r[c]);
  } else if constexpr (N == 2) {
    const u32x2 r = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs, voff, 0, kAuxDevice));
    out[0] = word_as_float(r[0]); out[1] = word_as_float(r[1]);
  } else if constexpr (N == 1) {
    out[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, voff, 0, kAuxDevice));
  }
}
EVT_DEV float ld_device(const float* p) {
  return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Count this workgroup in at `counter`.  Every thread's partials were stored
// with st_device before the call; the wait below lets them complete before
// the ticket is taken, so the workgroup that draws the last ticket reads all
// of them.  In two halves, so that the caller can issue independent stores
// while the ticket travels: arrive_begin returns the ticket (meaningful in
// thread 0, -1 when the caller passed no counter), arrive_end tells every
// thread whether this workgroup arrived last of `expected`.
EVT_DEV int arrive_begin(int* counter) {
  __builtin_amdgcn_s_waitcnt(0);   // vmcnt(0): my device-scope stores have been acknowledged
  __syncthreads();
  int ticket = -1;
  if (threadIdx.x == 0) ticket = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return ticket;
}
EVT_DEV bool arrive_end(int ticket, int expected, int* smem_flag) {
  if (threadIdx.x == 0) *smem_flag = ticket;
  __syncthreads();
  return *smem_flag == expected - 1;
}
EVT_DEV bool arrive_last(int* counter, int expected, int* smem_flag) {
  return arrive_end(arrive_begin(counter), expected, smem_flag);
}

// Per-row reductions.  The tile visitor leaves one state per (wave column,
// row) in LDS: state[wn][local_row][ROW_STATE] floats at smem, then one flag.
// Phase 1 (row_reduce_publish): combine the WN waves' states; with one tile
// along N the result is final, otherwise it is this tile's partial, written to
// the workspace.  When phase 2 runs inside this kernel the workgroup also
// draws its arrival ticket here.  The caller then issues its output-tile
// stores (the ticket had to wait for this wave's earlier stores to be
// acknowledged, and 64 KB of tile stores in front of it cost microseconds;
// behind it they travel together with the ticket), asks row_reduce_arrived
// whether it was the last workgroup of its row block and, if so, runs
// row_reduce_complete.
template <class Epi>
EVT_DEV bool row_phase2_here(const GemmArgs& g) {
  return Epi::ROW_STATE > 0 && row_uses_workspace(g) && g.row_inkernel;
}
template <class Cfg, class Epi, class Tile>
EVT_DEV int row_reduce_publish(const typename Epi::Params& p, const Tile& t, const GemmArgs& g) {
  constexpr int RS = Epi::ROW_STATE;
  if constexpr (RS > 0) {
    const float* lds = (const float*)t.smem;
    const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(g);
    float* part = (float*)(t.workspace + wl.counter_bytes);
    __syncthreads();
    for (int lr = t.tid; lr < Cfg::BM; lr += Cfg::THREADS) {
      const int row = t.m0 + lr;
      if (row >= t.M) continue;
      float st[RS];
#pragma unroll
      for (int c = 0; c < RS; ++c) st[c] = lds[lr * RS + c];
#pragma unroll
      for (int w = 1; w < Cfg::WN; ++w) Epi::row_combine(st, lds + (w * Cfg::BM + lr) * RS);
      if constexpr (Cfg::WALK) {
        // fold this tile into the walk's running state, earlier tiles on the left
        float* run = t.walk_state + lr * RS;
        if (!t.walk_first) {
          float sofar[RS];
#pragma unroll
          for (int c = 0; c < RS; ++c) sofar[c] = run[c];
          Epi::row_combine(sofar, st);
#pragma unroll
          for (int c = 0; c < RS; ++c) st[c] = sofar[c];
        }
        if (!t.walk_last) {
#pragma unroll
          for (int c = 0; c < RS; ++c) run[c] = st[c];
          continue;
        }
      }
      if (!row_uses_workspace(g)) {
        Epi::row_finalize(p, t.batch, row, st);
      } else {
        st_device_n<RS>(make_rsrc((const char*)(part + ((int64_t)t.batch * t.parts_n + t.part_n) * t.M * RS)),
                        (uint32_t)row * (RS * 4), st);
      }
    }
    if constexpr (Cfg::WALK) {
      if (!t.walk_last) return -1;
    }
    if (!row_phase2_here<Epi>(g)) return -1;
    return arrive_begin((int*)t.workspace + fold_key(g, t.batch) * t.tiles_m + t.tile_m);
  } else {
    return -1;
  }
}
template <class Cfg, class Epi, class Tile>
EVT_DEV bool row_reduce_arrived(const Tile& t, const GemmArgs& g, int ticket) {
  if constexpr (Epi::ROW_STATE > 0) {
    if (!row_phase2_here<Epi>(g)) return false;
    if constexpr (Cfg::WALK) {
      if (!t.walk_last) return false;
    }
    return arrive_end(ticket, t.parts_n * g.row_fold_count, (int*)(t.smem + Cfg::WN * Cfg::BM * Epi::ROW_STATE * 4));
  } else {
    return false;
  }
}

// Phase 2 in the last workgroup of a row block.  SHARES threads per row each
// fold every SHARES-th partial (batches in fold order, tiles in tile order;
// their loads are in flight together), then LDS combines the shares in order:
// the combination tree depends on the problem and the tile only, so the result
// is the same whichever workgroup arrives last.
template <class Cfg, class Epi, class Tile>
EVT_DEV void row_reduce_complete(const typename Epi::Params& p, const Tile& t, const GemmArgs& g) {
  constexpr int RS = Epi::ROW_STATE;
  if constexpr (RS > 0) {
    constexpr int SHARES = Cfg::THREADS >= Cfg::BM ? Cfg::THREADS / Cfg::BM : 1;
    constexpr int ROWS_PER_PASS = Cfg::THREADS >= Cfg::BM ? Cfg::BM : Cfg::THREADS;
    static_assert(SHARES * ROWS_PER_PASS * RS * 4 <= Cfg::LDS_BYTES, "share exchange area exceeds the operand LDS");
    float* lds = (float*)t.smem;
    const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(g);
    const float* part = (const float*)(t.workspace + wl.counter_bytes);
    const int key = fold_key(g, t.batch);
    int* counter = (int*)t.workspace + key * t.tiles_m + t.tile_m;
    const int share = t.tid / ROWS_PER_PASS, lr0 = t.tid % ROWS_PER_PASS;
    for (int base = 0; base < Cfg::BM; base += ROWS_PER_PASS) {
      const int lr = base + lr0;
      const int row = t.m0 + lr;
      const bool live = share < SHARES && lr < Cfg::BM && row < t.M;
      float st[RS];
      Epi::row_identity(st);
      if (live) {
        // Share s folds partials s, s + SHARES, ... of every batch of the fold, batches in fold order.  GROUP
        // loads are in flight together (a device-scope load takes microseconds), and the addresses advance by a
        // constant: no division per partial.
        constexpr int GROUP = RS <= 3 ? 32 : 16;
        const uint32_t step = (uint32_t)t.M * RS;        // floats from one partial of a row to the next (the host
                                                         // keeps parts_n * M * RS * 4 below 2 GiB for this path)
        for (int f = 0; f < g.row_fold_count; ++f) {
          const __amdgpu_buffer_rsrc_t pf = make_rsrc((const char*)(part + (int64_t)fold_member(g, key, f) * t.parts_n * t.M * RS));
          for (int j0 = share; j0 < t.parts_n; j0 += SHARES * GROUP) {
            float o[GROUP][RS];
#pragma unroll
            for (int u = 0; u < GROUP; ++u) {
              const int j = j0 + u * SHARES;
              if (j < t.parts_n) ld_device_n<RS>(pf, (uint32_t)(j * step + row * RS) * 4u, o[u]);
            }
#pragma unroll
            for (int u = 0; u < GROUP; ++u) {
              if (j0 + u * SHARES < t.parts_n) Epi::row_combine(st, o[u]);
            }
          }
        }
      }
      if constexpr (SHARES > 1) {
        __syncthreads();   // the exchange area is free (phase-1 states / the previous pass have been consumed)
        if (share < SHARES) {
#pragma unroll
          for (int c = 0; c < RS; ++c) lds[(share * ROWS_PER_PASS + lr0) * RS + c] = st[c];
        }
        __syncthreads();
        if (live && share == 0) {
          for (int s2 = 1; s2 < SHARES; ++s2) Epi::row_combine(st, lds + (s2 * ROWS_PER_PASS + lr0) * RS);
        }
      }
      if (live && share == 0) Epi::row_finalize(p, fold_member(g, key, 0), row, st);
    }
    if (t.tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  (void)g;
}

// Per-column reductions.  `cs[ni][c]` holds this lane's state for column
// col(ni) over all its rows.  LDS layout: state[wm][local_col][COL_STATE]
// floats placed after the row-reduction area, then one flag.  Same three steps
// as for rows: publish (+ ticket), arrived, complete.
template <class Epi>
EVT_DEV bool col_phase2_here(const GemmArgs& g) {
  return Epi::COL_STATE > 0 && col_uses_workspace(g) && g.col_inkernel;
}
template <class Cfg, class Epi>
struct ColArea {
  static constexpr int ROW_AREA = Epi::ROW_STATE > 0 ? (Cfg::WN * Cfg::BM * Epi::ROW_STATE * 4 + 16) : 0;
  static constexpr int SHARES = Cfg::THREADS / Cfg::BN > 0 ? Cfg::THREADS / Cfg::BN : 1;
  static constexpr int FLAG = ROW_AREA + (Cfg::WM > SHARES ? Cfg::WM : SHARES) * Cfg::BN * (Epi::COL_STATE > 0 ? Epi::COL_STATE : 1) * 4;
};
template <class Cfg, class Epi, class Tile>
EVT_DEV int col_reduce_publish(const typename Epi::Params& p, const Tile& t, const GemmArgs& g,
                               float (&cs)[Tile::NI][Epi::COL_STATE > 0 ? Epi::COL_STATE : 1]) {
  constexpr int CS = Epi::COL_STATE;
  if constexpr (CS > 0) {
    float* lds = (float*)(t.smem + ColArea<Cfg, Epi>::ROW_AREA);
    // the two halves of a wave hold different rows of the same columns
#pragma unroll
    for (int ni = 0; ni < Tile::NI; ++ni) {
      float o[CS];
#pragma unroll
      for (int c = 0; c < CS; ++c) o[c] = __shfl_xor(cs[ni][c], 32);
      Epi::col_combine(cs[ni], o);
    }
    if (t.lane < 32) {
#pragma unroll
      for (int ni = 0; ni < Tile::NI; ++ni)
#pragma unroll
        for (int c = 0; c < CS; ++c) lds[(t.wm * Cfg::BN + t.lcol(ni)) * CS + c] = cs[ni][c];
    }
    __syncthreads();
    const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(g);
    float* part = (float*)(t.workspace + wl.counter_bytes + wl.row_bytes);
    for (int lc = t.tid; lc < Cfg::BN; lc += Cfg::THREADS) {
      const int col = t.n0 + lc;
      if (col >= t.N) continue;
      float st[CS];
#pragma unroll
      for (int c = 0; c < CS; ++c) st[c] = lds[lc * CS + c];
#pragma unroll
      for (int w = 1; w < Cfg::WM; ++w) Epi::col_combine(st, lds + (w * Cfg::BN + lc) * CS);
      if (!col_uses_workspace(g)) {
        Epi::col_finalize(p, t.batch, col, st);
      } else {
        float* dst = part + (((int64_t)t.batch * t.tiles_m + t.tile_m) * t.N + col) * CS;
#pragma unroll
        for (int c = 0; c < CS; ++c) st_device(dst + c, st[c]);
      }
    }
    if (!col_phase2_here<Epi>(g)) return -1;
    const int row_counters = (Epi::ROW_STATE > 0 && row_uses_workspace(g)) ? t.L * t.tiles_m : 0;
    return arrive_begin((int*)t.workspace + row_counters + col_fold_key(g, t.batch) * t.tiles_n + t.tile_n);
  } else {
    return -1;
  }
}
template <class Cfg, class Epi, class Tile>
EVT_DEV bool col_reduce_arrived(const Tile& t, const GemmArgs& g, int ticket) {
  if constexpr (Epi::COL_STATE > 0) {
    if (!col_phase2_here<Epi>(g)) return false;
    return arrive_end(ticket, t.tiles_m * g.col_fold_count, (int*)(t.smem + ColArea<Cfg, Epi>::FLAG));
  } else {
    return false;
  }
}

// Phase 2 in the last workgroup of a column block.
template <class Cfg, class Epi, class Tile>
EVT_DEV void col_reduce_complete(const typename Epi::Params& p, const Tile& t, const GemmArgs& g) {
  constexpr int CS = Epi::COL_STATE;
  if constexpr (CS > 0) {
    constexpr int SHARES = ColArea<Cfg, Epi>::SHARES;
    float* lds = (float*)(t.smem + ColArea<Cfg, Epi>::ROW_AREA);
    const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(g);
    const float* part = (const float*)(t.workspace + wl.counter_bytes + wl.row_bytes);
    const int row_counters = (Epi::ROW_STATE > 0 && row_uses_workspace(g)) ? t.L * t.tiles_m : 0;
    const int key = col_fold_key(g, t.batch);
    int* counter = (int*)t.workspace + row_counters + key * t.tiles_n + t.tile_n;
    // SHARES threads per column each fold every SHARES-th partial in (batch, tile) order
    // (independent loads in flight together), LDS then combines the shares in order
    const int lc = t.tid % Cfg::BN, share = t.tid / Cfg::BN;
    const int col = t.n0 + lc;
    const bool live = share < SHARES && col < t.N;
    float st[CS];
    Epi::col_identity(st);
    if (live) {
#pragma unroll 8
      for (int q = share; q < t.tiles_m * g.col_fold_count; q += SHARES) {
        const int f = q / t.tiles_m, j = q - f * t.tiles_m;
        const float* src = part + (((int64_t)col_fold_member(g, key, f) * t.tiles_m + j) * t.N + col) * CS;
        float o[CS];
#pragma unroll
        for (int c = 0; c < CS; ++c) o[c] = ld_device(src + c);
        Epi::col_combine(st, o);
      }
    }
    __syncthreads();   // phase-1 LDS values are no longer needed
    if (share < SHARES) {
#pragma unroll
      for (int c = 0; c < CS; ++c) lds[(share * Cfg::BN + lc) * CS + c] = st[c];
    }
    __syncthreads();
    if (live && share == 0) {
      for (int s2 = 1; s2 < SHARES; ++s2) Epi::col_combine(st, lds + (s2 * Cfg::BN + lc) * CS);
      Epi::col_finalize(p, key, col, st);
    }
    if (t.tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  (void)g;
}

// Phase 2 of per-row reductions: 2^LG lanes share one row; each folds every
// 2^LG-th tile partial (in tile order), then the lanes combine pairwise.  The
// combination tree is fixed by (tiles_n, LG), so results are reproducible.
template <class Epi, int LG>
__global__ void __launch_bounds__(256) evt_row_finalize_kernel(typename Epi::Params p, const float* part, GemmArgs g) {
  constexpr int RS = Epi::ROW_STATE > 0 ? Epi::ROW_STATE : 1;
  constexpr int G = 1 << LG;
  const int M = g.M, tiles_n = g.parts_n;   // partials per row and batch
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t rowid = gid >> LG;
  const int sub = (int)(gid & (G - 1));
  const bool live = rowid < (int64_t)(g.L / g.row_fold_count) * M;
  const int key = live ? (int)(rowid / M) : 0;
  const int row = live ? (int)(rowid % M) : 0;
  const int batch = fold_member(g, key, 0);
  float st[RS];
  Epi::row_identity(st);
  if (live) {
    // partial q = (batch f of the fold, tile j); lane `sub` folds every G-th one
    for (int q = sub; q < tiles_n * g.row_fold_count; q += G) {
      const int f = q / tiles_n, j = q - f * tiles_n;
      Epi::row_combine(st, part + (((int64_t)fold_member(g, key, f) * tiles_n + j) * M + row) * RS);
    }
  }
#pragma unroll
  for (int o = G >> 1; o > 0; o >>= 1) {
    float other[RS];
#pragma unroll
    for (int c = 0; c < RS; ++c) other[c] = __shfl_xor(st[c], o);
    Epi::row_combine(st, other);
  }
  if (live && sub == 0) Epi::row_finalize(p, batch, row, st);
}

// Phase 2 of per-column reductions: a block of 256 threads covers 256 / G
// columns; G threads per column each fold every G-th partial (batches of a
// fold in fold order, tiles in tile order), LDS combines the G results in
// order.  Threads of equal share index read adjacent columns, i.e. adjacent
// addresses.  One result per (fold key, column): without a fold the key is
// the batch.
template <class Epi>
__global__ void __launch_bounds__(256) evt_col_finalize_kernel(typename Epi::Params p, const float* part, GemmArgs g, int G) {
  constexpr int CS = Epi::COL_STATE > 0 ? Epi::COL_STATE : 1;
  __shared__ float lds[256 * CS];
  const int N = g.N, tiles_m = g.tiles_m;
  const int keys = g.L / g.col_fold_count;
  const int per = 256 / G;
  const int sub = threadIdx.x / per, c = threadIdx.x % per;
  const int64_t colid = (int64_t)blockIdx.x * per + c;
  const bool live = colid < (int64_t)keys * N;
  const int key = live ? (int)(colid / N) : 0, col = live ? (int)(colid % N) : 0;
  float st[CS];
  Epi::col_identity(st);
  if (live) {
    const int nq = tiles_m * g.col_fold_count;
#pragma unroll 4
    for (int q = sub; q < nq; q += G) {
      const int f = q / tiles_m, j = q - f * tiles_m;
      Epi::col_combine(st, part + (((int64_t)col_fold_member(g, key, f) * tiles_m + j) * N + col) * CS);
    }
  }
#pragma unroll
  for (int k = 0; k < CS; ++k) lds[threadIdx.x * CS + k] = st[k];
  __syncthreads();
  if (live && sub == 0) {
    for (int s2 = 1; s2 < G; ++s2) Epi::col_combine(st, lds + (s2 * per + c) * CS);
    Epi::col_finalize(p, col_fold_member(g, key, 0), col, st);
  }
}

// Host side: enqueue the phase-2 kernels a launch needs (none when a single
// tile spans the reduced axis).
template <class Epi>
inline int launch_finalize(const typename Epi::Params& p, const GemmArgs& g, hipStream_t stream) {
  const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(g);
  if (Epi::ROW_STATE > 0 && row_uses_workspace(g) && !g.row_inkernel) {
    const float* part = (const float*)(g.workspace + wl.counter_bytes);
    int lg = 0;
    while ((1 << lg) < g.parts_n * g.row_fold_count && lg < 6) ++lg;
    const int64_t threads = ((int64_t)(g.L / g.row_fold_count) * g.M) << lg;
    const unsigned grid = (unsigned)((threads + 255) / 256);
    switch (lg) {
      case 1: hipLaunchKernelGGL((evt_row_finalize_kernel<Epi, 1>), dim3(grid), dim3(256), 0, stream, p, part, g); break;
      case 2: hipLaunchKernelGGL((evt_row_finalize_kernel<Epi, 2>), dim3(grid), dim3(256), 0, stream, p, part, g); break;
      case 3: hipLaunchKernelGGL((evt_row_finalize_kernel<Epi, 3>), dim3(grid), dim3(256), 0, stream, p, part, g); break;
      case 4: hipLaunchKernelGGL((evt_row_finalize_kernel<Epi, 4>), dim3(grid), dim3(256), 0, stream, p, part, g); break;
      case 5: hipLaunchKernelGGL((evt_row_finalize_kernel<Epi, 5>), dim3(grid), dim3(256), 0, stream, p, part, g); break;
      default: hipLaunchKernelGGL((evt_row_finalize_kernel<Epi, 6>), dim3(grid), dim3(256), 0, stream, p, part, g); break;
    }
  }
  if (Epi::COL_STATE > 0 && col_uses_workspace(g) && !g.col_inkernel) {
    const float* part = (const float*)(g.workspace + wl.counter_bytes + wl.row_bytes);
    int G = 1;
    while (G < 16 && G * 4 <= g.tiles_m * g.col_fold_count) G *= 2;      // >= 4 partials per thread
    const int per = 256 / G;
    const int64_t cols = (int64_t)(g.L / g.col_fold_count) * g.N;
    hipLaunchKernelGGL((evt_col_finalize_kernel<Epi>), dim3((unsigned)((cols + per - 1) / per)), dim3(256), 0, stream,
                       p, part, g, G);
  }
  return (int)hipGetLastError();
}

// Write one per-wave row state into the LDS exchange area (lane 0 of each half): for wave tiles of one 32-row
// block, whose rows are reduced one by one with half_wave_sum / half_wave_max.
template <class Cfg, int RS, class Tile>
EVT_DEV void row_state_to_lds(const Tile& t, int mi, int v, const float (&st)[RS]) {
  if ((t.lane & 31) == 0) {
    float* lds = (float*)t.smem + (t.wn * Cfg::BM + t.lrow(mi, v)) * RS;
#pragma unroll
    for (int c = 0; c < RS; ++c) lds[c] = st[c];
  }
}

// ---------------------------------------------------------------------------
// Per-row reductions of a wave tile, all rows at once.
//
// A lane holds one partial per accumulator row it owns (R = 16 MI rows, index r = 16 mi + v); each row is spread
// over the 32 lanes of a half wave.  Instead of one 5-step butterfly per row (160 cross-lane operations per 32
// rows, every lane ending up with every total) the rows are reduced together: at each step a lane hands the
// partner half of its registers and keeps the other half, so the work halves with the lanes involved -- 31
// exchanges for 32 rows -- and lane j ends up with the total of row j alone.  Steps, by the lane bit that tells the
// partners apart: bit 4 v_permlane16_swap, bit 3 row_mirror, bit 2 row_half_mirror, bit 1 / bit 0 quad_perm.
// After the steps x[e], e < R / 32, holds the total of row (lane & 31) * R / 32 + e.  (Wave tiles of a single
// 32-row block reduce row by row instead, see row_state_to_lds.)
// ---------------------------------------------------------------------------
template <bool MAX>
EVT_DEV float red_op(float a, float b) { return MAX ? fmaxf(a, b) : a + b; }

template <int N, bool MAX>
EVT_DEV void rows_step_swap16(float* x) {   // even rows of 16 lanes keep x[i], odd ones x[i + N/2]
#pragma unroll
  for (int i = 0; i < N / 2; ++i) {
    float a = x[i], b = x[i + N / 2];
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    x[i] = red_op<MAX>(a, b);
  }
}
template <int N, int CTRL, int BIT, bool MAX>
EVT_DEV void rows_step_dpp(float* x, int lane) {
  const bool up = (lane >> BIT) & 1;
#pragma unroll
  for (int i = 0; i < N / 2; ++i) {
    const float keep = up ? x[i + N / 2] : x[i];
    const float send = up ? x[i] : x[i + N / 2];
    const float got = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, send), CTRL, 0xf, 0xf, true));
    x[i] = red_op<MAX>(keep, got);
  }
}
template <int R, bool MAX>
EVT_DEV void rows_reduce(float (&x)[R], int lane) {
  static_assert(R == 32 || R == 64 || R == 128, "two or more 32-row blocks per wave tile");
  rows_step_swap16<R, MAX>(x);
  rows_step_dpp<R / 2, 0x140, 3, MAX>(x, lane);    // row_mirror
  rows_step_dpp<R / 4, 0x141, 2, MAX>(x, lane);    // row_half_mirror
  rows_step_dpp<R / 8, 0x4E, 1, MAX>(x, lane);     // quad_perm [2,3,0,1]
  rows_step_dpp<R / 16, 0xB1, 0, MAX>(x, lane);    // quad_perm [1,0,3,2]
}
// rows (of this lane's half) whose totals the lane holds after rows_reduce, and which
template <int R>
constexpr int rows_owned() { return R / 32; }
template <int R>
EVT_DEV int row_owned(int lane, int e) { return (lane & 31) * (R / 32) + e; }

// LDS areas of the epilogue's reductions inside the operand stages: row states [wn][bm][RS] + flag, column states
// [max(wm, shares)][bn][CS] + flag, then per wave and half R floats through which a row's first-pass result (its
// maximum, its mean) goes back to all the lanes that hold the row.
template <class Cfg, int RS, int CS>
struct RedAreas {
  static constexpr int ROW_AREA = RS > 0 ? (Cfg::WN * Cfg::BM * RS * 4 + 16) : 0;
  static constexpr int SHARES = Cfg::THREADS / Cfg::BN > 0 ? Cfg::THREADS / Cfg::BN : 1;
  static constexpr int COL_AREA = CS > 0 ? ((Cfg::WM > SHARES ? Cfg::WM : SHARES) * Cfg::BN * CS * 4 + 16) : 0;
  static constexpr int BACK = (ROW_AREA + COL_AREA + 15) / 16 * 16;
  static constexpr int BACK_BYTES = Cfg::WAVES * 2 * 16 * Cfg::MI * 4;
};

// Hand the first-pass result of every row back to all lanes of its half: owners write, everybody reads.
template <class Cfg, int R>
EVT_DEV void rows_broadcast(char* area, int lane, int wave, const float (&own)[rows_owned<R>()], float (&all)[R]) {
  float* slot = (float*)area + (wave * 2 + (lane >> 5)) * R;
#pragma unroll
  for (int e = 0; e < rows_owned<R>(); ++e) slot[row_owned<R>(lane, e)] = own[e];
  // same wave: LDS operations complete in order, no barrier needed
#pragma unroll
  for (int r = 0; r < R; r += 4) {
    const float4 q = *(const float4*)(slot + r);
    all[r] = q.x; all[r + 1] = q.y; all[r + 2] = q.z; all[r + 3] = q.w;
  }
}

// Store component c of the row state of every row this lane owns: state[wn][local row][RS] at smem.
template <class Cfg, int RS, class Tile>
EVT_DEV void rows_state_store(const Tile& t, int c, const float (&own)[rows_owned<16 * Cfg::MI>()]) {
  constexpr int R = 16 * Cfg::MI;
#pragma unroll
  for (int e = 0; e < rows_owned<R>(); ++e) {
    const int r = row_owned<R>(t.lane, e);
    const int lrow = t.row0 - t.m0 + (r >> 4) * 32 + 8 * ((r & 15) >> 2) + (r & 3);
    ((float*)t.smem)[(t.wn * Cfg::BM + lrow) * RS + c] = own[e];
  }
}

// The four kinds of per-row reduction over this wave's columns; results go to components [o ...] of the rows'
// states in LDS.  The two-pass kinds take the values `x[r][ni]` (r = 16 mi + v) and mask them by column validity.
template <class Cfg, int RS, bool MAX, class Tile>
EVT_DEV void rows_simple(const Tile& t, float (&part)[16 * Cfg::MI], int o) {   // part[r]: this lane's columns of row r
  constexpr int R = 16 * Cfg::MI;
  rows_reduce<R, MAX>(part, t.lane);
  float own[rows_owned<R>()];
#pragma unroll
  for (int e = 0; e < rows_owned<R>(); ++e) own[e] = part[e];
  rows_state_store<Cfg, RS>(t, o, own);
}
// component o of the rows' states when every term of a sum is known to be zero (a gather whose labels all lie
// outside this wave's columns): the same stores as rows_simple, without the reduction
template <class Cfg, int RS, class Tile>
EVT_DEV void rows_fill(const Tile& t, int o, float value) {
  float own[rows_owned<16 * Cfg::MI>()];
#pragma unroll
  for (int e = 0; e < rows_owned<16 * Cfg::MI>(); ++e) own[e] = value;
  rows_state_store<Cfg, RS>(t, o, own);
}
template <class Cfg, int RS, int CS, class Tile>
EVT_DEV void rows_maxsumexp(const Tile& t, const float (&x)[16 * Cfg::MI][Cfg::NI], int o) {
  constexpr int R = 16 * Cfg::MI;
  float part[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float a = -INFINITY;
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni) a = t.col_ok(ni) ? fmaxf(a, x[r][ni]) : a;
    part[r] = a;
  }
  rows_reduce<R, true>(part, t.lane);
  float mx[rows_owned<R>()];
#pragma unroll
  for (int e = 0; e < rows_owned<R>(); ++e) mx[e] = part[e];
  float m[R];
  rows_broadcast<Cfg, R>(t.smem + RedAreas<Cfg, RS, CS>::BACK, t.lane, t.wm * Cfg::WN + t.wn, mx, m);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float ms = m[r] * kLog2e;
    float a = t.col_ok(0) ? op_exp_minus(x[r][0], ms) : 0.f;
#pragma unroll
    for (int ni = 1; ni < Cfg::NI; ++ni) a += t.col_ok(ni) ? op_exp_minus(x[r][ni], ms) : 0.f;
    part[r] = a;
  }
  rows_reduce<R, false>(part, t.lane);
  float se[rows_owned<R>()];
#pragma unroll
  for (int e = 0; e < rows_owned<R>(); ++e) se[e] = part[e];
  rows_state_store<Cfg, RS>(t, o, mx);
  rows_state_store<Cfg, RS>(t, o + 1, se);
}
template <class Cfg, int RS, int CS, class Tile>
EVT_DEV void rows_welford(const Tile& t, const float (&x)[16 * Cfg::MI][Cfg::NI], int o) {
  constexpr int R = 16 * Cfg::MI;
  const float cnt = (float)t.wave_cols();
  const float rcnt = cnt > 0.f ? 1.f / cnt : 0.f;
  float part[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float a = 0.f;
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni) a += t.col_ok(ni) ? x[r][ni] : 0.f;
    part[r] = a;
  }
  rows_reduce<R, false>(part, t.lane);
  float mean[rows_owned<R>()], n[rows_owned<R>()];
#pragma unroll
  for (int e = 0; e < rows_owned<R>(); ++e) { mean[e] = part[e] * rcnt; n[e] = cnt; }
  float m[R];
  rows_broadcast<Cfg, R>(t.smem + RedAreas<Cfg, RS, CS>::BACK, t.lane, t.wm * Cfg::WN + t.wn, mean, m);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float a = 0.f;
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni) { const float d = x[r][ni] - m[r]; a += t.col_ok(ni) ? d * d : 0.f; }
    part[r] = a;
  }
  rows_reduce<R, false>(part, t.lane);
  float m2[rows_owned<R>()];
#pragma unroll
  for (int e = 0; e < rows_owned<R>(); ++e) m2[e] = part[e];
  rows_state_store<Cfg, RS>(t, o, n);
  rows_state_store<Cfg, RS>(t, o + 1, mean);
  rows_state_store<Cfg, RS>(t, o + 2, m2);
}

// ---------------------------------------------------------------------------
// reduction state algebra used by generated combine functions
// ---------------------------------------------------------------------------
// (m, l): running max and sum of exp(x - m)
EVT_DEV void combine_maxsumexp(float& m, float& l, float m2, float l2) {
  const float mm = fmaxf(m, m2);
  // exp(-inf - -inf) would be NaN: an empty side contributes nothing
  const float a = (m == -INFINITY) ? 0.f : l * __expf(m - mm);
  const float b = (m2 == -INFINITY) ? 0.f : l2 * __expf(m2 - mm);
  m = mm;
  l = a + b;
}
// (n, mean, M2): Chan et al. parallel mean / sum of squared deviations
EVT_DEV void combine_welford(float& n, float& mean, float& m2, float nb, float meanb, float m2b) {
  const float nt = n + nb;
  if (nt > 0.f) {
    const float d = meanb - mean;
    const float f = nb / nt;
    mean = mean + d * f;
    m2 = m2 + m2b + d * d * n * f;
  }
  n = nt;
}

// The fused kernel.
#ifdef EVT_CLOCK_PROBE
// Diagnostic build only: {main-loop shader cycles, main-loop 100 MHz ticks,
// epilogue shader cycles, epilogue 100 MHz ticks} of workgroup 0.  The ratio
// cycles / ticks is the shader clock the kernel actually ran at.
__device__ uint64_t evt_clock_probe[4];
#endif

// Split-K exchange.  Every workgroup of the tile leaves its accumulators in the workspace in register order
// (consecutive lanes write consecutive words); the one whose ticket is the last reads all of them back in split
// order -- its own included, so the sum does not depend on who arrived last -- and returns true: it goes on to
// the epilogue; the others are done.
template <class Cfg>
EVT_DEV void split_k_store(float* dst, const f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) st_device(dst + ((mi * Cfg::NI + ni) * 16 + v) * Cfg::THREADS, acc[mi][ni][v]);
}
// acc = tiles[first] + ... + tiles[first + count - 1], added in that order
template <class Cfg>
EVT_DEV void split_k_sum(const float* tiles, int first, int count, f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
  constexpr int REGS = Cfg::MI * Cfg::NI * 16;
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;
  for (int sp = first; sp < first + count; ++sp) {
    const float* src = tiles + (int64_t)sp * REGS * Cfg::THREADS + threadIdx.x;
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[mi][ni][v] += ld_device(src + ((mi * Cfg::NI + ni) * 16 + v) * Cfg::THREADS);
  }
}
// With groups (split_groups(g) > 0) the exchange has two levels: the last workgroup of a group of consecutive splits
// adds the group's tiles up in split order and leaves the sum as the group's tile, the last group to finish adds the
// groups' tiles up in group order.  Which workgroup does either is a matter of timing; what is added, and in which
// order, is not.
template <class Cfg, class Epi>
EVT_DEV bool split_k_exchange(const GemmArgs& g, unsigned tile_id, int split, char* smem, f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
  const WsLayout wl = ws_layout_split<Cfg, Epi::ROW_STATE, Epi::COL_STATE>(g);
  char* region = g.workspace + wl.counter_bytes + wl.row_bytes + wl.col_bytes;
  const int groups = split_groups(g);
  const int64_t tiles_total = (int64_t)g.L * g.tiles_m * g.tiles_n;
  int* counter = (int*)region + tile_id;
  constexpr int REGS = Cfg::MI * Cfg::NI * 16;
  float* part = (float*)(region + wl.split_counter_bytes) + (int64_t)tile_id * (g.splits + groups) * REGS * Cfg::THREADS;
  split_k_store<Cfg>(part + (int64_t)split * REGS * Cfg::THREADS + threadIdx.x, acc);
  __syncthreads();                 // nobody still reads operand tiles from the LDS the flag lives in
  if (groups == 0) {
    if (!arrive_last(counter, g.splits, (int*)smem)) return false;
    split_k_sum<Cfg>(part, 0, g.splits, acc);
  } else {
    const int grp = split / g.split_group, first = grp * g.split_group;
    const int count = g.splits - first < g.split_group ? g.splits - first : g.split_group;
    int* group_counter = (int*)region + tiles_total + (int64_t)tile_id * groups + grp;
    if (!arrive_last(group_counter, count, (int*)smem)) return false;
    split_k_sum<Cfg>(part, first, count, acc);
    __syncthreads();               // everybody has read the flag
    if (threadIdx.x == 0) __hip_atomic_store(group_counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    split_k_store<Cfg>(part + (int64_t)(g.splits + grp) * REGS * Cfg::THREADS + threadIdx.x, acc);
    if (!arrive_last(counter, groups, (int*)smem)) return false;
    split_k_sum<Cfg>(part, g.splits, groups, acc);
  }
  __syncthreads();
  if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // clean for the next launch
  return true;
}

// One tile's epilogue: interior tiles of an all-unit-stride epilogue (p.fast, decided on the host) take the
// check-free instantiation.  `part`, `first`, `last`, `state`: TileCtx::set_walk (WALK kernels only).
template <class Cfg, class Epi>
EVT_DEV void run_epilogue(const GemmArgs& g, const typename Epi::Params& p, int batch, int tm, int tn, char* smem,
                          const f32x16 (&acc)[Cfg::MI][Cfg::NI], int part, bool first, bool last, float* state) {
  if (p.fast && (tm + 1) * Cfg::BM <= g.M && (tn + 1) * Cfg::BN <= g.N) {
    TileCtx<Cfg, true> t;
    t.init(g, batch, tm, tn, smem);
    if constexpr (Cfg::WALK) t.set_walk(part, g.parts_n, first, last, state);
    Epi::template tile<Cfg, TileCtx<Cfg, true>, true>(p, t, g, acc);
  } else if (Epi::EDGE_TILES && p.fast && (!Cfg::ADJACENT || g.N % Cfg::NI == 0)) {
    // a tile on the matrix's edge: the same buffer accesses, lanes outside the matrix masked by their offsets
    TileCtx<Cfg, false> t;
    t.init(g, batch, tm, tn, smem);
    if constexpr (Cfg::WALK) t.set_walk(part, g.parts_n, first, last, state);
    Epi::template tile<Cfg, TileCtx<Cfg, false>, true>(p, t, g, acc);
  } else {
    TileCtx<Cfg, false> t;
    t.init(g, batch, tm, tn, smem);
    if constexpr (Cfg::WALK) t.set_walk(part, g.parts_n, first, last, state);
    Epi::template tile<Cfg, TileCtx<Cfg, false>, false>(p, t, g, acc);
  }
}

// Behind a main loop with split k-tiles (GemmCfg::KSPLIT): wave 4 g + p holds, for the loop's wave tile p, the sums
// over its half of every k-tile -- 2 MI x NI blocks of accumulators.  It keeps blocks [g MI, (g + 1) MI), hands the
// others to its partner 4 (1 - g) + p through LDS (64 lanes x 16 bytes per store: no bank conflicts), and adds what
// the partner hands over: own half + other half, the same sum on whichever side it is formed.
template <class Cfg, int KEEP>
EVT_DEV void ksplit_exchange(float4* mine, const float4* theirs, f32x16 (&lacc)[Cfg::LMI][Cfg::LNI],
                             f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
  constexpr int SEND = Cfg::MI - KEEP;     // first block handed over: MI when the first MI are kept, else 0
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x16& x = lacc[SEND + mi][ni];
        mine[((mi * Cfg::NI + ni) * 4 + q) * 64] = make_float4(x[4 * q], x[4 * q + 1], x[4 * q + 2], x[4 * q + 3]);
      }
  __syncthreads();
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 y = theirs[((mi * Cfg::NI + ni) * 4 + q) * 64];
        const f32x16& x = lacc[KEEP + mi][ni];
        acc[mi][ni][4 * q] = x[4 * q] + y.x;
        acc[mi][ni][4 * q + 1] = x[4 * q + 1] + y.y;
        acc[mi][ni][4 * q + 2] = x[4 * q + 2] + y.z;
        acc[mi][ni][4 * q + 3] = x[4 * q + 3] + y.w;
      }
}
template <class Cfg>
EVT_DEV void ksplit_reduce(char* smem, f32x16 (&lacc)[Cfg::LMI][Cfg::LNI], f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
  constexpr int BYTES = Cfg::MI * Cfg::NI * 4096;      // what one wave hands over
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float4* mine = (float4*)(smem + wave * BYTES) + lane;
  const float4* theirs = (const float4*)(smem + (wave ^ 4) * BYTES) + lane;
  __syncthreads();   // every wave has left the operand ring (its transfers were waited for inside the loop)
  if ((wave >> 2) == 0) ksplit_exchange<Cfg, 0>(mine, theirs, lacc, acc);
  else ksplit_exchange<Cfg, Cfg::MI>(mine, theirs, lacc, acc);
  __syncthreads();   // the area is the epilogue's from here on
}

template <class Cfg, class Epi>
__global__ void __launch_bounds__(Cfg::THREADS, Cfg::MIN_WAVES_PER_SIMD) evt_gemm_kernel(GemmArgs g, typename Epi::Params p) {
  // a walking workgroup keeps one running state per row behind the operand stages
  constexpr int WALK_BYTES = Cfg::WALK ? Cfg::BM * (Epi::ROW_STATE > 0 ? Epi::ROW_STATE : 1) * 4 : 0;
  __shared__ __attribute__((aligned(1024))) char smem[Cfg::LDS_BYTES + WALK_BYTES];
  int batch, tm, tn;
  f32x16 acc[Cfg::MI][Cfg::NI];
#ifdef EVT_CLOCK_PROBE
  uint64_t probe_main[2] = {0, 0}, probe_epi[2] = {0, 0};
#endif
  if constexpr (Cfg::WALK) {
    // one workgroup per (row block, run of g.walk tiles): main loop and epilogue alternate, the operand ring
    // running on from tile to tile (Mainloop::Walk)
    int pn;
    tile_coords<Cfg::GROUP_M>(blockIdx.x, gridDim.x, g.tiles_m, g.parts_n, batch, tm, pn);
    const int tn_first = pn * g.walk;
    const int tn_end = tn_first + g.walk < g.tiles_n ? tn_first + g.walk : g.tiles_n;
    typename Mainloop<Cfg>::Walk wk;
    for (tn = tn_first; tn < tn_end; ++tn) {
      const bool more = tn + 1 < tn_end;
#ifdef EVT_CLOCK_PROBE
      const uint64_t c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
#endif
      Mainloop<Cfg>::run(g, batch, tm * Cfg::BM, tn * Cfg::BN, 0, smem, acc, wk, more);
      regroup_columns<Cfg>(acc);
#ifdef EVT_CLOCK_PROBE
      const uint64_t c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
#endif
      run_epilogue<Cfg, Epi>(g, p, batch, tm, tn, Mainloop<Cfg>::epilogue_lds(wk, smem), acc, pn, tn == tn_first, !more,
                             (float*)(smem + Cfg::LDS_BYTES));
#ifdef EVT_CLOCK_PROBE
      const uint64_t c2 = __builtin_amdgcn_s_memtime(), r2 = __builtin_amdgcn_s_memrealtime();
      probe_main[0] += c1 - c0; probe_main[1] += r1 - r0; probe_epi[0] += c2 - c1; probe_epi[1] += r2 - r1;
#endif
    }
  } else {
    const int split = g.splits > 1 ? (int)(blockIdx.x % (unsigned)g.splits) : 0;
    const unsigned tile_id = g.splits > 1 ? blockIdx.x / (unsigned)g.splits : blockIdx.x;
    tile_coords<Cfg::GROUP_M>(tile_id, g.splits > 1 ? gridDim.x / (unsigned)g.splits : gridDim.x, g.tiles_m, g.tiles_n, batch, tm, tn);
#ifdef EVT_CLOCK_PROBE
    const uint64_t c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
#endif
    if constexpr (Cfg::KSPLIT) {
      f32x16 loop_acc[Cfg::LMI][Cfg::LNI];
      Mainloop<Cfg>::run(g, batch, tm * Cfg::BM, tn * Cfg::BN, split, smem, loop_acc);
      ksplit_reduce<Cfg>(smem, loop_acc, acc);
    } else {
      Mainloop<Cfg>::run(g, batch, tm * Cfg::BM, tn * Cfg::BN, split, smem, acc);
    }
    if (g.splits > 1) {
      if (!split_k_exchange<Cfg, Epi>(g, tile_id, split, smem, acc)) return;
    }
    regroup_columns<Cfg>(acc);
#ifdef EVT_CLOCK_PROBE
    const uint64_t c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
#endif
    run_epilogue<Cfg, Epi>(g, p, batch, tm, tn, smem, acc, tn, true, true, nullptr);
#ifdef EVT_CLOCK_PROBE
    __builtin_amdgcn_s_waitcnt(0);   // the epilogue's stores have been issued and acknowledged
    const uint64_t c2 = __builtin_amdgcn_s_memtime(), r2 = __builtin_amdgcn_s_memrealtime();
    probe_main[0] = c1 - c0; probe_main[1] = r1 - r0; probe_epi[0] = c2 - c1; probe_epi[1] = r2 - r1;
#endif
  }
#ifdef EVT_CLOCK_PROBE
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    evt_clock_probe[0] = probe_main[0];
    evt_clock_probe[1] = probe_main[1];
    evt_clock_probe[2] = probe_epi[0];
    evt_clock_probe[3] = probe_epi[1];
  }
#endif
}

__global__ void evt_fill_zero_kernel(uint32_t* p, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0u;
}

}  // namespace evt
