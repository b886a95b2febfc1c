// Row-wise reduce-apply anchors: softmax, softmax backward, layer norm and
// layer norm backward over the last axis, with the same epilogue visitor tree
// behind them as the GEMM kernels have.
//
// Role in the reference (apuaaChen/EVT_AE): src/cuda/softmax, src/cuda/layernorm
// and src/cuda/reduce_apply (warp-per-row kernels instantiated by
// SoftmaxOperation / LayerNormOperation with an epilogue visitor,
// python/gtl/compiler/passes/evt_fuser.py:700-970).
//
// MI355X design: HBM-bound, so the only goals are one read of every input,
// one write of every output, 16-byte accesses and enough rows in flight.  A
// row lives in the registers of LPR lanes of one wave64 (LPR = 8 .. 64, a
// power of two; 64 / LPR rows per wave), 8 consecutive columns per lane and
// chunk, CH chunks (row length <= CH * LPR * 8).  Reductions run over DPP
// operands and scalar lane reads inside the LPR-lane group; nothing goes
// through LDS and no workgroup barrier is needed, so a workgroup is just 4
// independent waves.  The normalised
// values stay in registers and are handed to the generated epilogue as the
// "accumulator".  Rows longer than 8192 elements (vocabulary-sized softmax)
// are spread over the WPR = 2 .. 16 waves of one workgroup, still register
// cached and read once; the only addition is that each row reduction ends
// with an exchange of one value per wave through LDS and a barrier.
#pragma once

#include "evt_epilogue.hpp"

namespace evt {

enum RowOp : int { ROW_SOFTMAX = 0, ROW_SOFTMAX_BWD = 1, ROW_LAYERNORM = 2, ROW_LAYERNORM_BWD = 3 };

struct RowArgs {
  int M, N, L;               // rows per batch, row length, batches (rows are r = l * M + m)
  const char* A;             // softmax / layer norm: input; backward kernels: incoming gradient
  int64_t lda, bsA;          // row and batch stride of A in elements
  const char* B;             // softmax backward: softmax output; layer norm backward: forward input
  int64_t ldb, bsB;
  const float* mean;         // layer norm backward: per-row statistics of the forward pass
  const float* rstd;
  const char* gamma;         // layer norm backward: weight [N] in the operands' element type, or null
  int vecG;
  float eps;                 // layer norm
  int vecA, vecB;            // rows of A / B may be read with 16-byte loads
  float* colws;              // per-column reductions of the epilogue: [workgroups][COL_STATE][N] partials
  int fast;                  // every anchor operand is dword aligned and 2: N % 8 == 0, whole 8-column groups only;
                             // 1: N >= 8, whole groups move as 16 bytes without checks, the group that straddles the
                             // row end on its own; 0: neither
};

// ELT: 0 = f16, 1 = bf16, 2 = f32 element type of the anchor operands
// AV: per-element values besides the result that the anchor hands to the epilogue (layer norm backward with
// weight / bias gradients: the incoming gradient and the normalised input)
// WPR: waves per row; above 1 the whole workgroup (WAVES == WPR full waves) holds one row
template <int OP_, int CH_, int LPR_, int ELT_, int AV_ = 0, int WAVES_ = 4, int WPR_ = 1>
struct RowCfg {
  static constexpr int OP = OP_, CH = CH_, LPR = LPR_, ELT = ELT_, AV = AV_, WAVES = WAVES_, WPR = WPR_;
  static constexpr int THREADS = WAVES * 64;
  static constexpr int RPW = 64 / LPR;              // rows per wave
  static constexpr int ROWS = WAVES * RPW / WPR;    // rows per workgroup
  static constexpr int GROUP = LPR * WPR;           // lanes per row
  static constexpr int SPAN = GROUP * 8;            // columns per chunk
  // a wave fetches its next row before it reduces the present one; 16 waves leave 128 registers per lane, not
  // enough for two rows' worth
  static constexpr bool LOOKAHEAD = WPR < 16;
  static_assert(LPR >= 1 && LPR <= 64 && (LPR & (LPR - 1)) == 0, "lanes per row: a power of two up to 64");
  static_assert(CH >= 1 && CH <= 16, "a row is cached in at most 128 registers per lane");
  static_assert(WPR == 1 || (LPR == 64 && WAVES == WPR && WPR <= 16 && (WPR & (WPR - 1)) == 0),
                "a row over several waves takes whole waves and the whole workgroup");
};

template <int ELT> struct RowElt;
template <> struct RowElt<0> { using type = f16; };
template <> struct RowElt<1> { using type = bf16; };
template <> struct RowElt<2> { using type = float; };

template <class Cfg>
struct RowCtx {
  int M, N, L;
  int64_t r;       // global row (clamped to a valid row for lanes past the end; `ok` says which)
  int l, m;        // batch and row inside the batch
  int sub;         // lane inside the row's lane group
  bool ok;
  EVT_DEV int col0(int c) const { return c * Cfg::SPAN + sub * 8; }
  EVT_DEV int valid(int c) const {             // how many of this lane's 8 columns of chunk c exist
    const int v = N - col0(c);
    return v < 0 ? 0 : (v > 8 ? 8 : v);
  }
};

// All-reduce over the LPR lanes of a row.  Inside a row of 16 lanes the partner
// values come through DPP operands (quad permutes for lane ^ 1 and lane ^ 2,
// then the mirrored half row and the mirrored row: by then all lanes of a quad
// / of 8 hold the same value, so a mirror reaches the other half just as an
// xor would); the four rows of 16 are combined from scalar lane reads.  No
// LDS-crossbar shuffle is involved: a reduction costs a few dozen cycles.
template <int CTRL>
EVT_DEV float dpp_move(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
EVT_DEV float lane_read(float x, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}
struct OpSum { static EVT_DEV float f(float a, float b) { return a + b; } };
struct OpMax { static EVT_DEV float f(float a, float b) { return fmaxf(a, b); } };

template <int LPR, class Op>
EVT_DEV float group_reduce(float x) {
  if constexpr (LPR >= 2) x = Op::f(x, dpp_move<0xB1>(x));     // quad_perm [1,0,3,2]
  if constexpr (LPR >= 4) x = Op::f(x, dpp_move<0x4E>(x));     // quad_perm [2,3,0,1]
  if constexpr (LPR >= 8) x = Op::f(x, dpp_move<0x141>(x));    // row_half_mirror
  if constexpr (LPR >= 16) x = Op::f(x, dpp_move<0x140>(x));   // row_mirror
  if constexpr (LPR == 32) {
    const float lo = Op::f(lane_read(x, 0), lane_read(x, 16));
    const float hi = Op::f(lane_read(x, 32), lane_read(x, 48));
    x = (threadIdx.x & 32) ? hi : lo;
  }
  if constexpr (LPR == 64) {
    x = Op::f(Op::f(lane_read(x, 0), lane_read(x, 16)), Op::f(lane_read(x, 32), lane_read(x, 48)));
  }
  return x;
}
// All-reduce over a row: the lane group of a wave, then (rows spread over several waves) one value per wave
// through LDS.  Successive reductions alternate between two sets of slots, so one barrier each is enough: a wave
// can only overwrite a set after the barrier of the reduction in between, which every wave reaches after it
// has read that set.  Every wave of the workgroup must take part in every reduction.
template <class Cfg>
struct RowReduce {
  float* slots;      // [2][16] floats of LDS (unused when a row lives in one wave)
  int phase;
  template <class Op>
  EVT_DEV float all(float x) {
    x = group_reduce<Cfg::LPR, Op>(x);
    if constexpr (Cfg::WPR > 1) {
      float* s = slots + phase * 16;
      if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = x;
      __syncthreads();
      float y = s[0];
#pragma unroll
      for (int w = 1; w < Cfg::WPR; ++w) y = Op::f(y, s[w]);
      x = y;
      phase ^= 1;
    }
    return x;
  }
  EVT_DEV float sum(float x) { return all<OpSum>(x); }
  EVT_DEV float max(float x) { return all<OpMax>(x); }
};

// 16 / 8 bytes moved by one instruction.  Multi-dword global accesses need dword alignment only, so the types
// promise no more than that: rows whose length is no multiple of 8 elements (a 30522-entry vocabulary) still
// move 16 bytes per lane wherever 8 whole columns are left.
typedef uint32_t q16 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t q8 __attribute__((ext_vector_type(2), aligned(4)));

// 8 consecutive elements starting at p[0] (unit stride), `valid` of them inside the row
template <class T>
EVT_DEV void load8(const T* p, bool vec, int valid, float fill, float (&out)[8]) {
  if (vec && valid == 8) {
    if constexpr (sizeof(T) == 2) {
      union { q16 q; T e[8]; } u;
      u.q = *reinterpret_cast<const q16*>(p);
#pragma unroll
      for (int j = 0; j < 8; ++j) out[j] = (float)u.e[j];
    } else if constexpr (sizeof(T) == 4 && !std::is_same<T, bool>::value) {
      union { q16 q[2]; T e[8]; } u;
      u.q[0] = reinterpret_cast<const q16*>(p)[0];
      u.q[1] = reinterpret_cast<const q16*>(p)[1];
#pragma unroll
      for (int j = 0; j < 8; ++j) out[j] = (float)u.e[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) out[j] = ld_f32<T>(p, j);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = j < valid ? ld_f32<T>(p, j) : fill;
  }
}

// generic strided variant for epilogue tensors (element stride sn)
template <class T>
EVT_DEV void load8s(const T* p, int64_t sn, bool vec, int valid, float (&out)[8]) {
  if (sn == 1) {
    load8<T>(p, vec, valid, 0.f, out);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = j < valid ? ld_f32<T>(p, (int64_t)j * sn) : 0.f;
  }
}

template <class T>
EVT_DEV void store8s(T* p, int64_t sn, bool vec, int valid, const float (&val)[8]) {
  if (sn == 1 && vec && valid == 8) {
    if constexpr (sizeof(T) == 2) {
      union { q16 q; T e[8]; } u;
#pragma unroll
      for (int j = 0; j < 8; ++j) u.e[j] = (T)val[j];
      *reinterpret_cast<q16*>(p) = u.q;
      return;
    } else if constexpr (sizeof(T) == 4 && !std::is_same<T, bool>::value) {
      union { q16 q[2]; T e[8]; } u;
#pragma unroll
      for (int j = 0; j < 8; ++j) u.e[j] = (T)val[j];
      reinterpret_cast<q16*>(p)[0] = u.q[0];
      reinterpret_cast<q16*>(p)[1] = u.q[1];
      return;
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (j < valid) st_f32<T>(p, (int64_t)j * sn, val[j]);
}

// whole, aligned 8-column groups (the check-free epilogue path)
template <class T>
EVT_DEV void load8v(const T* p, float (&out)[8]) {
  constexpr int Q = (sizeof(T) * 8 + 15) / 16;
  union { q16 q[Q]; T e[8]; } u;
  if constexpr (sizeof(T) * 8 >= 16) {
#pragma unroll
    for (int i = 0; i < Q; ++i) u.q[i] = reinterpret_cast<const q16*>(p)[i];
  } else {   // 1-byte elements: one 8-byte load
    *reinterpret_cast<q8*>(&u) = *reinterpret_cast<const q8*>(p);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if constexpr (std::is_same<T, bool>::value) out[j] = u.e[j] ? 1.f : 0.f;
    else out[j] = (float)u.e[j];
  }
}
template <class T>
EVT_DEV void store8v(T* p, const float (&val)[8]) {
  constexpr int Q = (sizeof(T) * 8 + 15) / 16;
  union { q16 q[Q]; T e[8]; } u;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if constexpr (std::is_same<T, bool>::value) u.e[j] = val[j] != 0.f;
    else u.e[j] = (T)val[j];
  }
  if constexpr (sizeof(T) * 8 >= 16) {
#pragma unroll
    for (int i = 0; i < Q; ++i) reinterpret_cast<q16*>(p)[i] = u.q[i];
  } else {
    *reinterpret_cast<q8*>(p) = *reinterpret_cast<const q8*>(&u);
  }
}

// The same through buffer instructions, for kernels whose lanes all work on one row (RowCfg::RPW == 1): `rs`
// starts at the row, a lane without columns passes kOobOffset and the hardware drops its access (loads give 0).
// No lane is masked off and no branch surrounds the access, so the compiler knows how many memory operations
// an iteration issues and can wait for the row fetched ahead without also waiting for the stores behind it.
// a pointer that has the same value in every lane, moved to scalar registers
EVT_DEV const char* wave_uniform(const void* p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
template <class T>
EVT_DEV void load8v_b(__amdgpu_buffer_rsrc_t rs, uint32_t voff, float (&out)[8]) {
  constexpr int Q = (sizeof(T) * 8 + 15) / 16;
  union { q16 q[Q]; q8 h; T e[8]; } u;
  if constexpr (sizeof(T) * 8 >= 16) {
#pragma unroll
    for (int i = 0; i < Q; ++i) u.q[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff + 16 * i, 0, 0);
  } else {
    u.h = __builtin_bit_cast(q8, __builtin_amdgcn_raw_buffer_load_b64(rs, voff, 0, 0));
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if constexpr (std::is_same<T, bool>::value) out[j] = u.e[j] ? 1.f : 0.f;
    else out[j] = (float)u.e[j];
  }
}
template <class T>
EVT_DEV void store8v_b(__amdgpu_buffer_rsrc_t rs, uint32_t voff, const float (&val)[8]) {
  constexpr int Q = (sizeof(T) * 8 + 15) / 16;
  union { q16 q[Q]; q8 h; T e[8]; } u;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if constexpr (std::is_same<T, bool>::value) u.e[j] = val[j] != 0.f;
    else u.e[j] = (T)val[j];
  }
  if constexpr (sizeof(T) * 8 >= 16) {
#pragma unroll
    for (int i = 0; i < Q; ++i) __builtin_amdgcn_raw_buffer_store_b128(u.q[i], rs, voff + 16 * i, 0, 0);
  } else {
    __builtin_amdgcn_raw_buffer_store_b64(u.h, rs, voff, 0, 0);
  }
}

// ---------------------------------------------------------------------------
// the four anchors: fill acc[CH][8] (and rv[0..1] = per-row values) for row t
// ---------------------------------------------------------------------------
// A row as it comes from memory, still in the operands' element type: fetched one
// row ahead of the arithmetic, so the conversion (which would wait for the
// load) happens only when the row is consumed.
template <class Cfg>
struct RowRaw {
  using T = typename RowElt<Cfg::ELT>::type;
  static constexpr bool TWO = Cfg::OP == ROW_SOFTMAX_BWD || Cfg::OP == ROW_LAYERNORM_BWD;
  T a[Cfg::CH][8];
  T b[TWO ? Cfg::CH : 1][8];
  float mean, rstd;
};

template <class T>
EVT_DEV void load8_raw(const T* p, bool vec, int valid, T fill, T (&out)[8]) {
  if (vec && valid == 8) {
    constexpr int Q = sizeof(T) * 8 / 16;
    union { q16 q[Q]; T e[8]; } u;
#pragma unroll
    for (int i = 0; i < Q; ++i) u.q[i] = reinterpret_cast<const q16*>(p)[i];
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = u.e[j];
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = j < valid ? p[j] : fill;
  }
}

template <class Cfg, int FAST>
EVT_DEV void row_fetch_one(const char* base, int64_t ld, int64_t bs, int vec, const RowCtx<Cfg>& t, float fill,
                           typename RowElt<Cfg::ELT>::type (&x)[Cfg::CH][8]) {
  using T = typename RowElt<Cfg::ELT>::type;
  const T* row = reinterpret_cast<const T*>(base) + (t.L == 1 ? (int64_t)0 : (int64_t)t.l * bs) + (int64_t)t.m * ld;
  // FAST 2: N is a multiple of 8 and the rows are dword aligned; FAST 1: the rows are dword aligned and N >= 8.
  if constexpr (FAST != 0) {
    // Every lane loads 16-byte groups; a lane whose group is not (wholly) inside the row reads the row's first
    // group instead (always there) and the value is replaced afterwards: no branch in the body.  FAST 1: one
    // lane per row holds a group that straddles the row end; it fetches its few elements one by one in a tail
    // of its own, so all whole groups keep the straight-line body.
    constexpr int Q = sizeof(T) * 8 / 16;
#pragma unroll
    for (int c = 0; c < Cfg::CH; ++c) {
      const bool full = FAST == 2 ? t.col0(c) < t.N : t.valid(c) == 8;
      union { q16 q[Q]; T e[8]; } u;
      const q16* src = reinterpret_cast<const q16*>(row + (full ? t.col0(c) : 0));
#pragma unroll
      for (int i = 0; i < Q; ++i) u.q[i] = src[i];
      // FAST 2: the registers are taken as they come; groups past the row end are replaced by `fill` when the
      // row is consumed (row_widen), so that nothing here waits for the loads and a row fetched ahead stays in
      // flight under the arithmetic of the row before it
#pragma unroll
      for (int j = 0; j < 8; ++j) x[c][j] = (FAST == 2 || full) ? u.e[j] : (T)fill;
    }
    if constexpr (FAST == 1) {
#pragma unroll
      for (int c = 0; c < Cfg::CH; ++c) {
        const int v = t.valid(c);
        if (v > 0 && v < 8) {
#pragma unroll
          for (int j = 0; j < 7; ++j)
            if (j < v) x[c][j] = row[t.col0(c) + j];
        }
      }
    }
    return;
  }
#pragma unroll
  for (int c = 0; c < Cfg::CH; ++c) {
    const int v = t.valid(c);
    if (v > 0) {
      load8_raw<T>(row + t.col0(c), vec != 0, v, (T)fill, x[c]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[c][j] = (T)fill;
    }
  }
}

template <class Cfg, int FAST>
EVT_DEV void row_fetch(const RowArgs& g, const RowCtx<Cfg>& t, RowRaw<Cfg>& raw) {
  row_fetch_one<Cfg, FAST>(g.A, g.lda, g.bsA, g.vecA, t, Cfg::OP == ROW_SOFTMAX ? -INFINITY : 0.f, raw.a);
  if constexpr (RowRaw<Cfg>::TWO) row_fetch_one<Cfg, FAST>(g.B, g.ldb, g.bsB, g.vecB, t, 0.f, raw.b);
  if constexpr (Cfg::OP == ROW_LAYERNORM_BWD) { raw.mean = g.mean[t.r]; raw.rstd = g.rstd[t.r]; }
}

// FAST 2: lanes whose group lies past the row end hold some other group's values (row_fetch_one): `fill` there
template <class Cfg, int FAST>
EVT_DEV void row_widen(const RowCtx<Cfg>& t, float fill, const typename RowElt<Cfg::ELT>::type (&x)[Cfg::CH][8],
                       float (&y)[Cfg::CH][8]) {
#pragma unroll
  for (int c = 0; c < Cfg::CH; ++c) {
    const bool in = FAST != 2 || t.col0(c) < t.N;
#pragma unroll
    for (int j = 0; j < 8; ++j) y[c][j] = in ? (float)x[c][j] : fill;
  }
}

template <class Cfg, int FAST>
EVT_DEV void row_main(const RowArgs& g, const RowCtx<Cfg>& t, const RowRaw<Cfg>& raw, const float (&gz)[Cfg::CH][8],
                      float (&acc)[Cfg::CH][8], float (&rv)[2], float (&av)[Cfg::AV > 0 ? Cfg::AV : 1][Cfg::CH][8],
                      RowReduce<Cfg>& red) {
  constexpr int CH = Cfg::CH;
  const float rn = 1.f / (float)g.N;
  if constexpr (Cfg::OP == ROW_SOFTMAX) {
    // aten._softmax over the last axis: exp(x - max) / sum, all in fp32
    row_widen<Cfg, FAST>(t, -INFINITY, raw.a, acc);
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) mx = fmaxf(mx, acc[c][j]);
    mx = red.max(mx);
    const float off = (mx == -INFINITY) ? 0.f : mx * kLog2e;    // a row of -inf gives NaN below, as torch does
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        acc[c][j] = __builtin_amdgcn_exp2f(acc[c][j] * kLog2e - off);
        s += acc[c][j];
      }
    s = red.sum(s);
    const float inv = 1.f / s;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[c][j] *= inv;
    rv[0] = mx; rv[1] = s;
  } else if constexpr (Cfg::OP == ROW_SOFTMAX_BWD) {
    // aten._softmax_backward_data: (g - sum(g * y)) * y
    float y[CH][8];
    row_widen<Cfg, FAST>(t, 0.f, raw.a, acc);
    row_widen<Cfg, FAST>(t, 0.f, raw.b, y);
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) s += acc[c][j] * y[c][j];
    s = red.sum(s);
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[c][j] = (acc[c][j] - s) * y[c][j];
    rv[0] = s; rv[1] = 0.f;
  } else if constexpr (Cfg::OP == ROW_LAYERNORM) {
    // aten.native_layer_norm without weight and bias: (x - mean) * rstd, mean, rstd;
    // two passes over the registers (mean first, then centred squares)
    row_widen<Cfg, FAST>(t, 0.f, raw.a, acc);
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) s += acc[c][j];
    const float mean = red.sum(s) * rn;
    float q = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int v = t.valid(c);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float d = acc[c][j] - mean;
        acc[c][j] = d;
        q += j < v ? d * d : 0.f;
      }
    }
    const float rstd = rsqrtf(red.sum(q) * rn + g.eps);
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[c][j] *= rstd;
    rv[0] = mean; rv[1] = rstd;
  } else {
    // aten.native_layer_norm_backward, input gradient, without weight:
    //   xh = (x - mean) rstd ;  dx = rstd (g - mean_n(g) - xh mean_n(g xh))
    //   (g already multiplied by the weight when there is one)
    float xh[CH][8];
    row_widen<Cfg, FAST>(t, 0.f, raw.a, acc);
    if constexpr (Cfg::AV >= 1) {      // the weight / bias gradients are column sums of g * xhat and of g
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) av[0][c][j] = acc[c][j];
    }
    if (g.gamma) {
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[c][j] *= gz[c][j];
    }
    row_widen<Cfg, FAST>(t, 0.f, raw.b, xh);
    const float mean = raw.mean, rstd = raw.rstd;
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int v = t.valid(c);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        xh[c][j] = j < v ? (xh[c][j] - mean) * rstd : 0.f;
        s1 += acc[c][j];
        s2 += acc[c][j] * xh[c][j];
      }
    }
    s1 = red.sum(s1) * rn;
    s2 = red.sum(s2) * rn;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[c][j] = rstd * (acc[c][j] - s1 - xh[c][j] * s2);
    if constexpr (Cfg::AV >= 2) {
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) av[1][c][j] = xh[c][j];
    }
    rv[0] = mean; rv[1] = rstd;
  }
  (void)av;
}

// Rows are dealt in runs: walker w (a wave, or the workgroup when it shares a
// row) visits rows [w * run, (w + 1) * run), RPW at a time, and fetches the
// next visit's rows before it reduces the present ones, so it always has a
// row's worth of loads in flight; the grid is sized to fill the chip once
// instead of one workgroup per handful of rows.  A run of consecutive rows lets
// the per-row outputs of the epilogue (a layer norm's mean and rstd) leave
// together: lane j keeps the values of the j-th row since the last flush, and
// up to 64 rows are written by one store instruction per output.  One 4-byte
// store per row and output costs a fifth of the kernel's time on 131072 x 1024.
template <class Cfg, class Epi, int FAST>
__global__ __launch_bounds__(Cfg::THREADS) void evt_row_kernel(RowArgs g, typename Epi::Params p) {
  constexpr int CS = Epi::COL_STATE;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t rows = (int64_t)g.L * g.M;
  constexpr int STEP = Cfg::WPR > 1 ? 1 : Cfg::RPW;        // rows per visit
  const int64_t walkers = Cfg::WPR > 1 ? (int64_t)gridDim.x : (int64_t)gridDim.x * Cfg::WAVES;
  const int64_t me = Cfg::WPR > 1 ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * Cfg::WAVES + wave;
  // With per-row outputs in the epilogue a walker takes a run of consecutive rows (RUNS), so that their outputs
  // can leave together; otherwise the walkers' rows interleave (visit k of walker w is row block w + k * walkers),
  // which keeps the whole chip inside one window of the tensor at any time and measures a few percent faster.
  constexpr bool RUNS = Epi::NRS > 0;
  const int64_t run = RUNS ? (rows + walkers * STEP - 1) / (walkers * STEP) * STEP : rows;
  const int64_t first = RUNS ? me * run : me * STEP;
  const int64_t end = (RUNS && first + run < rows) ? first + run : rows;
  const int64_t stride = RUNS ? (int64_t)STEP : walkers * STEP;      // from one visit to the next
  RowCtx<Cfg> t;
  t.M = g.M; t.N = g.N; t.L = g.L;
  t.sub = Cfg::WPR > 1 ? (int)threadIdx.x : lane % Cfg::LPR;
  __shared__ float xch[2 * 16];
  RowReduce<Cfg> red{xch, 0};
  // (batch, row in the batch) of the walker's present row: kept up to date by addition, since the rows of a run
  // follow each other (a 64-bit division per visit costs more instructions than the rest of a short row's work).
  // Batches shorter than 64 rows take the division.
  const bool stepwise = RUNS && g.M >= 64;                                  // uniform
  int cur_l = 0, cur_m = 0;                                                 // of row `base`
  if (first < rows) { cur_l = (int)(first / g.M); cur_m = (int)(first % g.M); }
  auto locate = [&](int64_t base) {
    const int sub_row = Cfg::WPR > 1 ? 0 : lane / Cfg::LPR;
    const int64_t r = base + sub_row;
    t.ok = r < end;                 // rows from `end` on belong to the next walker (or do not exist)
    t.r = t.ok ? r : rows - 1;      // lanes past the end recompute the last row and store nothing
    if (stepwise) {
      int m = cur_m + sub_row, l = cur_l;
      if (m >= g.M) { m -= g.M; l += 1; }
      t.l = t.ok ? l : g.L - 1;
      t.m = t.ok ? m : g.M - 1;
    } else if (g.L == 1) {          // uniform: a single batch needs no division
      t.l = 0;
      t.m = (int)t.r;
    } else {
      t.l = (int)(t.r / g.M);
      t.m = (int)(t.r % g.M);
    }
  };
  auto advance = [&]() {            // `base` moves on by one visit
    cur_m += STEP;
    if (cur_m >= g.M) { cur_m -= g.M; cur_l += 1; }
  };
  // this lane's share of the epilogue's per-column reductions, carried over all rows the wave visits
  float cst[CS > 0 ? CS : 1][Cfg::CH][8];
  if constexpr (CS > 0) {
#pragma unroll
    for (int c = 0; c < Cfg::CH; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float id[CS];
        Epi::col_identity(id);
#pragma unroll
        for (int k = 0; k < CS; ++k) cst[k][c][j] = id[k];
      }
  }
  // wave-uniform; the same for every wave of the workgroup when they share a row (so all of them reach the barriers
  // of the reductions the same number of times)
  int64_t base = first;
  // per-row outputs on their way out: lane j holds those of row flush_first + j
  constexpr int NRS = Epi::NRS;
  float hold[NRS > 0 ? NRS : 1];
  int64_t flush_first = first;
  int flush_l = cur_l, flush_m = cur_m;      // (batch, row) of flush_first
  int held = 0;
  if (base < end) {
    locate(base);
    float hz[Epi::NH > 0 ? Epi::NH : 1][Cfg::CH][8];
    Epi::template hoist<Cfg, FAST>(p, t, hz);
    float gz[Cfg::CH][8];          // layer norm backward: this lane's columns of the weight, read once
    if constexpr (Cfg::OP == ROW_LAYERNORM_BWD) {
      using T = typename RowElt<Cfg::ELT>::type;
      if (g.gamma) {
#pragma unroll
        for (int c = 0; c < Cfg::CH; ++c) {
          const int v = t.valid(c);
          if (v > 0) {
            load8<T>(reinterpret_cast<const T*>(g.gamma) + t.col0(c), g.vecG != 0, v, 0.f, gz[c]);
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) gz[c][j] = 0.f;
          }
        }
      }
    }
    // everything that happens to one fetched row; `more`: the walker has further rows
    auto consume = [&](const RowCtx<Cfg>& here, const RowRaw<Cfg>& raw, bool more) {
      float acc[Cfg::CH][8];
      float rv[2];
      float av[Cfg::AV > 0 ? Cfg::AV : 1][Cfg::CH][8];
      row_main<Cfg, FAST>(g, here, raw, gz, acc, rv, av, red);
      float rsv[NRS > 0 ? NRS : 1];
      if (here.ok) Epi::template row<Cfg, FAST>(p, here, acc, rv, av, hz, cst, rsv);
      if constexpr (NRS > 0) {
        // the rows of this visit take slots held .. held + STEP - 1 (STEP divides 64, so a visit never wraps)
#pragma unroll
        for (int i = 0; i < NRS; ++i) {
          float v = rsv[i];
          if constexpr (STEP > 1) v = __shfl(v, ((lane - held) & (STEP - 1)) * Cfg::LPR, 64);   // row group -> slot lane
          if (lane >= held && lane < held + STEP) hold[i] = v;
        }
        held += STEP;
        if (held == 64 || !more) {
          const int64_t r = flush_first + lane;
          if (lane < held && r < end && (Cfg::WPR == 1 || wave == 0)) {
            int l, m;
            if (stepwise) {
              l = flush_l; m = flush_m + lane;
              if (m >= g.M) { m -= g.M; l += 1; }
            } else {
              l = (int)(r / g.M); m = (int)(r % g.M);
            }
#pragma unroll
            for (int i = 0; i < NRS; ++i) Epi::row_store_one(p, g.L, l, m, i, hold[i]);
          }
          flush_first += held;
          flush_m += held;
          if (stepwise && flush_m >= g.M) { flush_m -= g.M; flush_l += 1; }
          held = 0;
        }
      }
    };
    {
      RowRaw<Cfg> cur;
      row_fetch<Cfg, FAST>(g, t, cur);
      // The first row is waited for here, once.  Left to the compiler, the wait sits at the top of the loop body
      // (where the first row's registers may still be on their way), behind the fetch of the next row, and
      // because the counter runs in issue order it would then wait for that fetch in every iteration.
      if constexpr (Cfg::LOOKAHEAD) __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
      while (true) {
        const RowCtx<Cfg> here = t;
        const int64_t next = base + stride;
        const bool more = next < end;                                          // wave-uniform
        RowRaw<Cfg> ahead;
        if constexpr (Cfg::LOOKAHEAD) {
          if (more) {
            advance();
            locate(next);
            row_fetch<Cfg, FAST>(g, t, ahead);
          }
        }
        consume(here, cur, more);
        if (!more) break;
        if constexpr (Cfg::LOOKAHEAD) {
          cur = ahead;
        } else {
          advance();
          locate(next);
          row_fetch<Cfg, FAST>(g, t, cur);
        }
        base = next;
      }
    }
  }
  if constexpr (CS > 0 && Cfg::WPR > 1) {
    // A row over the whole workgroup: every thread has carried the partials of its own columns over all the rows
    // the workgroup visited, so there is nothing to combine inside the workgroup.  One partial per (workgroup,
    // column) goes to the workspace, as below.
#pragma unroll
    for (int k = 0; k < CS; ++k)
#pragma unroll
      for (int c = 0; c < Cfg::CH; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int n = c * Cfg::SPAN + t.sub * 8 + j;
          if (n < g.N) g.colws[((int64_t)blockIdx.x * CS + k) * g.N + n] = cst[k][c][j];
        }
  } else if constexpr (CS > 0) {
    // Column partials of the workgroup: first across the row groups of a wave (lanes that hold the same
    // columns of different rows), then across the waves, which add their share into one LDS copy one after
    // the other in wave order; one partial per (workgroup, column) goes to the workspace and a second kernel
    // adds the workgroups up in a fixed order.
    __shared__ float red[CS][Cfg::CH * Cfg::SPAN];
#pragma unroll
    for (int k = 0; k < CS; ++k)
#pragma unroll
      for (int c = 0; c < Cfg::CH; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float x = cst[k][c][j];
#pragma unroll
          for (int m = Cfg::LPR; m < 64; m <<= 1) {
            float a[CS], b[CS];
            Epi::col_identity(a); Epi::col_identity(b);
            a[k] = x; b[k] = __shfl_xor(x, m, 64);
            Epi::col_combine(a, b);
            x = a[k];
          }
          cst[k][c][j] = x;
        }
    for (int w = 0; w < Cfg::WAVES; ++w) {
      if (wave == w && lane < Cfg::LPR) {
#pragma unroll
        for (int c = 0; c < Cfg::CH; ++c)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int n = c * Cfg::SPAN + t.sub * 8 + j;
            float a[CS], b[CS];
#pragma unroll
            for (int k = 0; k < CS; ++k) { a[k] = red[k][n]; b[k] = cst[k][c][j]; }
            if (w == 0) {
#pragma unroll
              for (int k = 0; k < CS; ++k) a[k] = b[k];
            } else {
              Epi::col_combine(a, b);
            }
#pragma unroll
            for (int k = 0; k < CS; ++k) red[k][n] = a[k];
          }
      }
      __syncthreads();
    }
    for (int n = threadIdx.x; n < g.N; n += Cfg::THREADS) {
#pragma unroll
      for (int k = 0; k < CS; ++k) g.colws[((int64_t)blockIdx.x * CS + k) * g.N + n] = red[k][n];
    }
  }
}

// Second phase of the per-column reductions.  A workgroup owns 16 columns (kColFinalizeCols); a wave reads them
// from four workgroup partials at once (lane = 16 * partial + column: four 64-byte segments), its 16 waves
// stride over the partials, so with P partials a lane adds P / 64 of them, with independent loads, and N / 16
// workgroups share the work (64 columns per workgroup left all but 16 CUs idle on a 1024-column layer norm:
// 12.6 us for 1024 partials, against 5.8 us this way; 8 columns per workgroup: 6.9 us).  Then the four lanes of a column combine, one wave adds
// the 16 waves' sub-sums in wave order and evaluates the per-column output expressions.  The order of the
// additions is fixed by (partial index mod 64, lane pairs, then wave), so results do not depend on timing.
constexpr int kColFinalizeCols = 16;
template <class Epi>
__global__ __launch_bounds__(1024) void evt_row_col_finalize_kernel(RowArgs g, typename Epi::Params p, int blocks) {
  constexpr int CS = Epi::COL_STATE > 0 ? Epi::COL_STATE : 1;
  constexpr int COLS = kColFinalizeCols, AT_ONCE = 64 / COLS;
  __shared__ float part[16][CS][COLS];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & (COLS - 1), sub = lane / COLS;
  const int n = blockIdx.x * COLS + c;
  float a[CS];
  Epi::col_identity(a);
  if (n < g.N) {
#pragma unroll 4
    for (int b = wave * AT_ONCE + sub; b < blocks; b += 16 * AT_ONCE) {
      float x[CS];
#pragma unroll
      for (int k = 0; k < CS; ++k) x[k] = g.colws[((int64_t)b * CS + k) * g.N + n];
      Epi::col_combine(a, x);
    }
  }
#pragma unroll
  for (int m = COLS; m < 64; m <<= 1) {     // the lanes that hold the same column
    float x[CS];
#pragma unroll
    for (int k = 0; k < CS; ++k) x[k] = __shfl_xor(a[k], m, 64);
    Epi::col_combine(a, x);
  }
  if (sub == 0) {
#pragma unroll
    for (int k = 0; k < CS; ++k) part[wave][k][c] = a[k];
  }
  __syncthreads();
  if (wave == 0 && sub == 0 && n < g.N) {
#pragma unroll
    for (int w = 1; w < 16; ++w) {
      float x[CS];
#pragma unroll
      for (int k = 0; k < CS; ++k) x[k] = part[w][k][c];
      Epi::col_combine(a, x);
    }
    Epi::col_finalize(p, 0, n, a);
  }
}

}  // namespace evt
