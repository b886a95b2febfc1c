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
// outputs (visitor_store.hpp:293-301, :544-553).  Each workgroup reduces its
// tile with wave64 cross-lane operations and LDS, writes one partial per
// (tile, row) or (tile, column) to a workspace, and the last workgroup to
// arrive for a row block / column block combines the partials in tile order
// and finalises the outputs, so results are deterministic.
#pragma once

#include "evt_gemm.hpp"

namespace evt {

// ---------------------------------------------------------------------------
// elementwise functions (fp32)
// ---------------------------------------------------------------------------
EVT_DEV float op_exp(float x) { return __expf(x); }
EVT_DEV float op_log(float x) { return __logf(x); }
EVT_DEV float op_rcp(float x) { return __frcp_rn(x); }
EVT_DEV float op_tanh(float x) {
  // tanh(x) = 1 - 2 / (1 + exp(2x)); saturates correctly for |x| large
  const float e = __expf(2.f * x);
  return 1.f - 2.f * __frcp_rn(1.f + e);
}
EVT_DEV float op_sigmoid(float x) { return __frcp_rn(1.f + __expf(-x)); }
EVT_DEV float op_relu(float x) { return x > 0.f ? x : 0.f; }
EVT_DEV float op_gelu_tanh(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  const float u = k0 * (x + k1 * x * x * x);
  return 0.5f * x * (1.f + op_tanh(u));
}
EVT_DEV float op_gelu_erf(float x) { return 0.5f * x * (1.f + erff(x * 0.7071067811865476f)); }
EVT_DEV float op_tanh_backward(float gy, float y) { return gy * (1.f - y * y); }
EVT_DEV float op_gelu_backward_tanh(float gy, float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  const float x2 = x * x;
  const float t = op_tanh(k0 * (x + k1 * x * x2));
  const float dt = (1.f - t * t) * k0 * (1.f + 3.f * k1 * x2);
  return gy * (0.5f * (1.f + t) + 0.5f * x * dt);
}
EVT_DEV float op_gelu_backward_erf(float gy, float x) {
  const float cdf = 0.5f * (1.f + erff(x * 0.7071067811865476f));
  const float pdf = 0.3989422804014327f * __expf(-0.5f * x * x);
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

// ---------------------------------------------------------------------------
// Where this lane's accumulator elements live in the output.
// acc[mi][ni][v] is element (row(mi, v), col(ni)).
// ---------------------------------------------------------------------------
template <class Cfg>
struct TileCtx {
  static constexpr int MI = Cfg::MI, NI = Cfg::NI;
  static constexpr bool INTERLEAVE = Cfg::INTERLEAVE;
  static constexpr int COL_STEP = INTERLEAVE ? 1 : 32;
  int M, N, L;
  int batch, tile_m, tile_n, tiles_m, tiles_n;
  int m0, n0;          // tile origin
  int row0, col0;      // this lane's first row / column
  int tid, lane, wm, wn;
  char* smem;
  char* workspace;

  EVT_DEV void init(const GemmArgs& g, int batch_, int tm, int tn, char* smem_) {
    M = g.M; N = g.N; L = g.L;
    batch = batch_; tile_m = tm; tile_n = tn; tiles_m = g.tiles_m; tiles_n = g.tiles_n;
    m0 = tm * Cfg::BM; n0 = tn * Cfg::BN;
    tid = threadIdx.x; lane = tid & 63;
    const int wave = tid >> 6;
    wm = wave / Cfg::WN; wn = wave % Cfg::WN;
    row0 = m0 + wm * Cfg::TM + 4 * (lane >> 5);
    col0 = n0 + wn * Cfg::TN + (INTERLEAVE ? (lane & 31) * NI : (lane & 31));
    smem = smem_; workspace = g.workspace;
  }
  EVT_DEV int row(int mi, int v) const { return row0 + mi * 32 + 8 * (v >> 2) + (v & 3); }
  EVT_DEV int col(int ni) const { return col0 + ni * COL_STEP; }
  EVT_DEV bool col_ok(int ni) const { return col(ni) < N; }
  // row / column index local to the workgroup tile
  EVT_DEV int lrow(int mi, int v) const { return row(mi, v) - m0; }
  EVT_DEV int lcol(int ni) const { return col(ni) - n0; }
  // number of valid columns in this wave's slice of the row
  EVT_DEV int wave_cols() const {
    const int left = N - (n0 + wn * Cfg::TN);
    return left < 0 ? 0 : (left > Cfg::TN ? Cfg::TN : left);
  }
};

// Load NI values of one accumulator row from an (l, m, n)-strided tensor.
// `off` is the element offset of (batch, row, col(0)); `vec` says the tensor
// is unit-stride along n and aligned so NI adjacent elements can move at once.
template <class T, class Tile>
EVT_DEV void aux_load(const Tile& t, const T* p, int64_t off, int64_t sn, bool vec, bool rok,
                      float (&out)[Tile::NI]) {
  constexpr int NI = Tile::NI;
  if constexpr (Tile::INTERLEAVE && sizeof(T) == 2 && (NI == 2 || NI == 4)) {
    if (vec && rok && t.col0 + NI <= t.N) {
      if constexpr (NI == 4) {
        const u32x2 raw = *(const u32x2*)(p + off);
        const T* e = (const T*)&raw;
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) out[ni] = (float)e[ni];
      } else {
        const uint32_t raw = *(const uint32_t*)(p + off);
        const T* e = (const T*)&raw;
        out[0] = (float)e[0]; out[1] = (float)e[1];
      }
      return;
    }
  }
#pragma unroll
  for (int ni = 0; ni < NI; ++ni)
    out[ni] = (rok && t.col_ok(ni)) ? ld_f32<T>(p, off + (int64_t)ni * Tile::COL_STEP * sn) : 0.f;
}

template <class T, class Tile>
EVT_DEV void aux_store(const Tile& t, T* p, int64_t off, int64_t sn, bool vec, bool rok,
                       const float (&val)[Tile::NI]) {
  constexpr int NI = Tile::NI;
  if constexpr (Tile::INTERLEAVE && sizeof(T) == 2 && (NI == 2 || NI == 4)) {
    if (vec && rok && t.col0 + NI <= t.N) {
      T e[NI];
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) e[ni] = (T)val[ni];
      if constexpr (NI == 4) {
        *(u32x2*)(p + off) = *(const u32x2*)e;
      } else {
        *(uint32_t*)(p + off) = *(const uint32_t*)e;
      }
      return;
    }
  }
#pragma unroll
  for (int ni = 0; ni < NI; ++ni)
    if (rok && t.col_ok(ni)) st_f32<T>(p, off + (int64_t)ni * Tile::COL_STEP * sn, val[ni]);
}

// ---------------------------------------------------------------------------
// cross-lane exchange inside one 32-lane half of a wave (the 32 lanes that hold
// the 32 columns of one accumulator row).  After the 5 steps every lane of the
// half holds the combined value.
// ---------------------------------------------------------------------------
template <int STEP>
EVT_DEV float half_wave_xchg(float x) {
  const int xi = __builtin_bit_cast(int, x);
  int r;
  if constexpr (STEP == 0) r = __builtin_amdgcn_mov_dpp(xi, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
  else if constexpr (STEP == 1) r = __builtin_amdgcn_mov_dpp(xi, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
  else if constexpr (STEP == 2) r = __builtin_amdgcn_mov_dpp(xi, 0x141, 0xf, 0xf, true);  // row_half_mirror
  else if constexpr (STEP == 3) r = __builtin_amdgcn_mov_dpp(xi, 0x140, 0xf, 0xf, true);  // row_mirror
  else r = __builtin_amdgcn_ds_swizzle(xi, 0x401F);                                       // lane ^ 16
  return __builtin_bit_cast(float, r);
}

EVT_DEV float half_wave_sum(float x) {
  x += half_wave_xchg<0>(x);
  x += half_wave_xchg<1>(x);
  x += half_wave_xchg<2>(x);
  x += half_wave_xchg<3>(x);
  x += half_wave_xchg<4>(x);
  return x;
}
EVT_DEV float half_wave_max(float x) {
  x = fmaxf(x, half_wave_xchg<0>(x));
  x = fmaxf(x, half_wave_xchg<1>(x));
  x = fmaxf(x, half_wave_xchg<2>(x));
  x = fmaxf(x, half_wave_xchg<3>(x));
  x = fmaxf(x, half_wave_xchg<4>(x));
  return x;
}

// ---------------------------------------------------------------------------
// workspace layout (bytes): [counters | row partials | column partials]
// ---------------------------------------------------------------------------
struct WsLayout {
  int64_t counters_bytes, row_bytes, col_bytes;
  EVT_DEV __host__ int64_t total() const { return counters_bytes + row_bytes + col_bytes; }
};

template <int ROW_STATE, int COL_STATE>
__host__ __device__ inline WsLayout ws_layout(int M, int N, int L, int tiles_m, int tiles_n) {
  WsLayout w;
  const bool row = ROW_STATE > 0 && tiles_n > 1;
  const bool col = COL_STATE > 0 && tiles_m > 1;
  int64_t ncnt = 0;
  if (row) ncnt += (int64_t)L * tiles_m;
  if (col) ncnt += (int64_t)L * tiles_n;
  w.counters_bytes = (ncnt * 4 + 255) / 256 * 256;
  w.row_bytes = row ? ((int64_t)L * tiles_n * M * ROW_STATE * 4 + 255) / 256 * 256 : 0;
  w.col_bytes = col ? ((int64_t)L * tiles_m * N * COL_STATE * 4 + 255) / 256 * 256 : 0;
  return w;
}

// Arrive at `counter`; returns true in every thread of the workgroup that
// arrives last of `expected`.  Partials written before the call are visible
// to the last arriver after it.
EVT_DEV bool arrive_last(int* counter, int expected, int* smem_flag) {
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    const int ticket = __hip_atomic_fetch_add(counter, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    *smem_flag = ticket;
  }
  __syncthreads();
  const bool last = (*smem_flag == expected - 1);
  if (last) __threadfence();
  return last;
}

// Per-row reductions: combine the per-wave states left in LDS by the tile
// visitor across the WN waves, then across workgroups.
//   LDS layout: state[wn][local_row][ROW_STATE] floats at smem.
template <class Cfg, class Epi, class Tile>
EVT_DEV void row_reduce_finish(const typename Epi::Params& p, const Tile& t) {
  constexpr int RS = Epi::ROW_STATE;
  if constexpr (RS > 0) {
    float* lds = (float*)t.smem;
    int* flag = (int*)(t.smem + Cfg::WN * Cfg::BM * RS * 4);
    __syncthreads();
    const int row = t.m0 + t.tid;
    const bool mine = t.tid < Cfg::BM && row < t.M;
    float st[RS];
    if (mine) {
#pragma unroll
      for (int c = 0; c < RS; ++c) st[c] = lds[t.tid * RS + c];
#pragma unroll
      for (int w = 1; w < Cfg::WN; ++w) Epi::row_combine(st, lds + (w * Cfg::BM + t.tid) * RS);
    }
    if (t.tiles_n == 1) {
      if (mine) Epi::row_finalize(p, t.batch, row, st);
      return;
    }
    const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(t.M, t.N, t.L, t.tiles_m, t.tiles_n);
    float* part = (float*)(t.workspace + wl.counters_bytes);
    int* counters = (int*)t.workspace;
    const int64_t brow = (int64_t)t.batch * t.tiles_n;
    if (mine) {
      float* dst = part + ((brow + t.tile_n) * t.M + row) * RS;
#pragma unroll
      for (int c = 0; c < RS; ++c) dst[c] = st[c];
    }
    int* counter = counters + t.batch * t.tiles_m + t.tile_m;
    if (arrive_last(counter, t.tiles_n, flag)) {
      if (mine) {
        const float* src = part + (brow * t.M + row) * RS;
#pragma unroll
        for (int c = 0; c < RS; ++c) st[c] = src[c];
        for (int j = 1; j < t.tiles_n; ++j) Epi::row_combine(st, src + (int64_t)j * t.M * RS);
        Epi::row_finalize(p, t.batch, row, st);
      }
      if (t.tid == 0) *counter = 0;
    }
  }
}

// Per-column reductions.  `cs[ni][c]` holds this lane's state for column
// col(ni) over all its rows.  LDS layout: state[wm][local_col][COL_STATE] floats
// placed after the row-reduction area.
template <class Cfg, class Epi, class Tile>
EVT_DEV void col_reduce_finish(const typename Epi::Params& p, const Tile& t,
                               float (&cs)[Tile::NI][Epi::COL_STATE > 0 ? Epi::COL_STATE : 1]) {
  constexpr int CS = Epi::COL_STATE;
  if constexpr (CS > 0) {
    constexpr int ROW_AREA = Epi::ROW_STATE > 0 ? (Cfg::WN * Cfg::BM * Epi::ROW_STATE * 4 + 16) : 0;
    float* lds = (float*)(t.smem + ROW_AREA);
    int* flag = (int*)(t.smem + ROW_AREA + Cfg::WM * Cfg::BN * CS * 4);
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
    for (int lc = t.tid; lc < Cfg::BN; lc += Cfg::THREADS) {
      const int col = t.n0 + lc;
      if (col >= t.N) continue;
      float st[CS];
#pragma unroll
      for (int c = 0; c < CS; ++c) st[c] = lds[lc * CS + c];
#pragma unroll
      for (int w = 1; w < Cfg::WM; ++w) Epi::col_combine(st, lds + (w * Cfg::BN + lc) * CS);
      if (t.tiles_m == 1) {
        Epi::col_finalize(p, t.batch, col, st);
      } else {
        const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(t.M, t.N, t.L, t.tiles_m, t.tiles_n);
        float* part = (float*)(t.workspace + wl.counters_bytes + wl.row_bytes);
        float* dst = part + (((int64_t)t.batch * t.tiles_m + t.tile_m) * t.N + col) * CS;
#pragma unroll
        for (int c = 0; c < CS; ++c) dst[c] = st[c];
      }
    }
    if (t.tiles_m == 1) return;
    const WsLayout wl = ws_layout<Epi::ROW_STATE, Epi::COL_STATE>(t.M, t.N, t.L, t.tiles_m, t.tiles_n);
    float* part = (float*)(t.workspace + wl.counters_bytes + wl.row_bytes);
    int* counters = (int*)t.workspace;
    const int row_counters = (Epi::ROW_STATE > 0 && t.tiles_n > 1) ? t.L * t.tiles_m : 0;
    int* counter = counters + row_counters + t.batch * t.tiles_n + t.tile_n;
    if (arrive_last(counter, t.tiles_m, flag)) {
      for (int lc = t.tid; lc < Cfg::BN; lc += Cfg::THREADS) {
        const int col = t.n0 + lc;
        if (col >= t.N) continue;
        const float* src = part + ((int64_t)t.batch * t.tiles_m * t.N + col) * CS;
        float st[CS];
#pragma unroll
        for (int c = 0; c < CS; ++c) st[c] = src[c];
        for (int j = 1; j < t.tiles_m; ++j) Epi::col_combine(st, src + (int64_t)j * t.N * CS);
        Epi::col_finalize(p, t.batch, col, st);
      }
      if (t.tid == 0) *counter = 0;
    }
  }
}

// Write one per-wave row state into the LDS exchange area (lane 0 of each half).
template <class Cfg, int RS, class Tile>
EVT_DEV void row_state_to_lds(const Tile& t, int mi, int v, const float (&st)[RS]) {
  if ((t.lane & 31) == 0) {
    float* lds = (float*)t.smem + (t.wn * Cfg::BM + t.lrow(mi, v)) * RS;
#pragma unroll
    for (int c = 0; c < RS; ++c) lds[c] = st[c];
  }
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
template <class Cfg, class Epi>
__global__ void __launch_bounds__(Cfg::THREADS) evt_gemm_kernel(GemmArgs g, typename Epi::Params p) {
  __shared__ __attribute__((aligned(1024))) char smem[Cfg::LDS_BYTES];
  int batch, tm, tn;
  tile_coords<Cfg::GROUP_M>(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, batch, tm, tn);
  f32x16 acc[Cfg::MI][Cfg::NI];
  Mainloop<Cfg>::run(g, batch, tm * Cfg::BM, tn * Cfg::BN, smem, acc);
  TileCtx<Cfg> t;
  t.init(g, batch, tm, tn, smem);
  Epi::template tile<Cfg>(p, t, acc);
}

__global__ void evt_fill_zero_kernel(uint32_t* p, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0u;
}

}  // namespace evt
