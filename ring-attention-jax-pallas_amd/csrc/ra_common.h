// Shared device-side helpers for the gfx950 ring-attention kernels: vector types, the
// bank-conflict-free LDS tile layout, global->LDS tile staging, MFMA operand fetches and
// the per-tile bias functor.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ring_attention_hip.h"

namespace ra {

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define RA_DEV __device__ __forceinline__

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
#define RA_NEG_INF (-__builtin_inff())

// Device-side view of ra_bias for one (batch, head): pointers already moved to the batch
// row, the ALiBi slope already multiplied by log2(e).
struct BiasArgs {
  int flags;
  int window;
  int q_off;   // position of local query 0
  int kv_off;  // position of local key 0
  const int* q_seg;
  const int* kv_seg;
  long long q_seg_sb, kv_seg_sb;
  const int* q_pre;
  const int* kv_pre;
  long long q_pre_sb, kv_pre_sb;
  const float* slopes;
  const float* dense;  // additive bias block [B|1, H|1, Lq, Lk], keys contiguous
  long long dense_sb, dense_sh, dense_sq;
  // optional summary of the block, one byte per cell of 32 queries x 32 keys (dense_map_kernel):
  // bit 0 = the cell holds a value other than -inf, bit 1 = it holds a value other than 0;
  // [B|1, H|1, ceil(Lq / 32), ceil(Lk / 32)], broadcast like the block itself
  const unsigned char* dense_map;
};

constexpr int kMapCell = 32;  // queries and keys per cell of a dense block's summary
constexpr int kMapLive = 1, kMapNonZero = 2;

// The summary's rows of one (batch, head) and the OR over a rectangle of its cells: what a
// workgroup needs to know about the part of the block that its rows and one tile span.
RA_DEV const unsigned char* dense_map_of(const BiasArgs& bs, int b, int h, int H, int Lq, int Lk) {
  const long long cells = (long long)((Lq + kMapCell - 1) / kMapCell) * ((Lk + kMapCell - 1) / kMapCell);
  const long long hm = bs.dense_sh ? H : 1;
  return bs.dense_map + ((bs.dense_sb ? b : 0) * hm + (bs.dense_sh ? h : 0)) * cells;
}
RA_DEV int dense_map_or(const unsigned char* mp, int Lk, int q_lo, int q_hi, int k_lo, int k_hi) {
  // queries [q_lo, q_hi] x keys [k_lo, k_hi], inclusive and in range
  const int ncols = (Lk + kMapCell - 1) / kMapCell;
  int bits = 0;
  for (int r = q_lo / kMapCell; r <= q_hi / kMapCell; ++r)
    for (int c = k_lo / kMapCell; c <= k_hi / kMapCell; ++c) bits |= mp[(long long)r * ncols + c];
  return bits;
}

struct TensorArg {
  const bf16_t* ptr;
  long long sb, sh, sl;
};

// ---------------------------------------------------------------------------------------
// wave-level helpers (wave64)
// ---------------------------------------------------------------------------------------
// Value held by the partner lane (lane ^ 32) combined with the own one.
RA_DEV float half_max(float x) {
  unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
RA_DEV float half_sum(float x) {
  unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
RA_DEV int wave_min(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}
RA_DEV int wave_max(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}
RA_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---------------------------------------------------------------------------------------
// LDS tile layout.  A tile is [rows][D] bf16, row-major, and the 16-byte chunks of a row
// are permuted by an XOR with a function of the row so that BOTH access patterns the
// kernels use hit 64 distinct banks:
//   * "natural" MFMA operand fetch: 16 consecutive rows, the same chunk, one b128 per lane;
//   * transposing fetch (ds_read_b64_tr_b16): 4 consecutive rows x 64 contiguous bytes.
// ---------------------------------------------------------------------------------------
template <int D>
RA_DEV int tile_off(int row, int chunk) {
  if (D == 128) {
    int f = ((row & 3) << 2) | ((row >> 2) & 3);
    return row * 256 + ((chunk ^ f) << 4);
  } else {
    int f = (row >> 1) & 7;
    return row * 128 + ((chunk ^ f) << 4);
  }
}

typedef __attribute__((address_space(3))) char lds_char;

// A/B operand of v_mfma_f32_32x32x16_bf16 taken along the contiguous (head-dim) axis:
// lane holds row (row0 + lane%32), elements [16*ks + 8*(lane/32), +8).
template <int D>
RA_DEV bf16x8 frag_nat(const char* tile, int row, int ks, int g) {
  return *(const bf16x8*)(tile + tile_off<D>(row, 2 * ks + g));
}

// Operand taken ACROSS rows (the contraction index is the tile's row index): lane gets,
// for column (col0 + lane%32), the 8 rows  rbase + {0..3}  and  rbase + 8 + {0..3}  where
// rbase = row16 + 4*(lane/32).  That is the row set an accumulator lane of the 32x32
// MFMA holds in registers 8*ks .. 8*ks+7, so the two operands pair up element by element.
template <int D>
RA_DEV bf16x8 frag_tr(const char* tile, int row16, int col0, int lane) {
  const int j = lane & 15;
  const int row = row16 + 4 * (lane >> 5) + (j >> 2);
  const int col = col0 + 16 * ((lane >> 4) & 1) + 4 * (j & 3);  // element index
  const int chunk = col >> 3;
  const int sub = (col & 4) << 1;  // byte offset inside the chunk (0 or 8)
  const lds_char* p0 = (const lds_char*)(tile + tile_off<D>(row, chunk) + sub);
  const lds_char* p1 = (const lds_char*)(tile + tile_off<D>(row + 8, chunk) + sub);
  bf16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p0);
  bf16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p1);
  return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Global -> registers -> LDS staging of a [ROWS][D] bf16 tile by NT threads.
template <int D, int ROWS, int NT>
struct TileStage {
  static constexpr int CPR = D / 8;  // 16-byte chunks per row
  static constexpr int TOTAL = ROWS * CPR;
  static constexpr int N = (TOTAL + NT - 1) / NT;
  u32x4 r[N];
  // rows row0 .. row0+ROWS-1 of a [L][D] matrix with row stride sl; rows >= L are clamped
  RA_DEV void load(const bf16_t* base, long long sl, int row0, int L, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int idx = tid + i * NT;
      if (TOTAL % NT == 0 || idx < TOTAL) {
        int row = idx / CPR, c = idx % CPR;
        int gr = min(row0 + row, L - 1);
        r[i] = *(const u32x4*)(base + (long long)gr * sl + c * 8);
      }
    }
  }
  RA_DEV void store(char* tile, int tid) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int idx = tid + i * NT;
      if (TOTAL % NT == 0 || idx < TOTAL) {
        int row = idx / CPR, c = idx % CPR;
        *(u32x4*)(tile + tile_off<D>(row, c)) = r[i];
      }
    }
  }
};

// 16 bytes per lane from global memory straight into LDS: lane l lands at lds_addr + 16*l.
// lds_addr is a wave-uniform LDS byte address (it travels through M0).  The global address is
// a wave-uniform 64-bit base (scalar registers) plus a per-lane unsigned 32-bit byte offset.
// Issued as inline assembly so that the compiler does not guard later, unrelated LDS reads
// with a full vmcnt wait; completion is the caller's business (s_waitcnt vmcnt(0) before the
// barrier that publishes the tile).  The "x2" form moves two pieces that are 1 KiB apart in
// LDS with one M0 write: the instruction offset applies to the LDS address AND to the global
// address, so the second base must already have 1024 bytes subtracted.
// The compiler inserts no wait states around the instructions of an assembly statement, so the
// statements carry their own: the LDS address reaches M0 one wait state before the load uses it,
// and a scalar base address that the compiler may have just restored from a vector register
// lane (v_readlane: a vector instruction writing a scalar register) is five wait states old
// before the memory instruction reads it.
RA_DEV void global_to_lds16(const void* gptr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gptr), "s"(lds_addr) : "memory", "m0");
}
RA_DEV void global_to_lds16_s(const void* sbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %0" : : "s"(sbase), "v"(voff), "s"(lds_addr) : "memory", "m0");
}
// Both pieces go through ONE scalar base: the second piece's distance from the first, minus the
// 1 KiB of the instruction offset, travels in its per-lane offset (an unsigned 32-bit byte count,
// which bounds the row stride at the ABI).  A second base would cost two scalar additions per call,
// and the loops that call this are bound by instruction issue.
RA_DEV void global_to_lds16_s_x2(const void* sbase, unsigned voff0, unsigned voff1_minus_1k, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %0\n\tglobal_load_lds_dwordx4 %2, %0 offset:1024"
               : : "s"(sbase), "v"(voff0), "v"(voff1_minus_1k), "s"(lds_addr) : "memory", "m0");
}
// Workgroup barrier of the straight-line loops, whose only LDS writes are tile loads that the caller
// counts with vmcnt: nothing is awaited, and LDS reads of this wave may stay in flight across it
// (__syncthreads() puts a workgroup fence on either side of s_barrier, which orders nothing there).
RA_DEV void barrier_bare() { asm volatile("s_barrier" ::: "memory"); }
// one dword per lane: lane l's word lands at lds_addr + 4 l
RA_DEV void global_to_lds4(const void* gptr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(gptr), "s"(lds_addr) : "memory", "m0");
}
// LDS byte address of an object declared __shared__
#define RA_LDS_ADDR(obj) ((unsigned)(uintptr_t)(lds_char*)(obj))

RA_DEV bf16x8 pack8(const f32x16& p, int base) {
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = (bf16_t)p[base + i];
  return r;
}

// ---------------------------------------------------------------------------------------
// Bias functor on one 32x32 accumulator block.
// The accumulator lane owns ONE index on the "fixed" side (lane%32) and 16 indices on the
// "varying" side: var0 + 8*(r/4) + (r%4), r = 0..15 (var0 already includes 4*(lane/32)).
// QFIXED = true : fixed side is the query, varying side the keys (S^T blocks);
// QFIXED = false: fixed side is the key, varying side the queries (S blocks).
// `rel0` = q_pos - kv_pos for r = 0.  fixed_seg / fixed_pre are the lane's own id values,
// var_seg / var_pre point at the LDS copies of the varying side's ids for var0.
// ---------------------------------------------------------------------------------------
struct TileBias {
  int flags;     // terms that must be evaluated for this block
  int window;
  float slope2;  // ALiBi slope * log2(e), in the units of the score tile it is added to
  float dense_mul;  // factor that takes a dense bias value (natural-log units) to those units
  int var_limit; // varying-side indices >= var_limit (relative to var0) are out of range
  const float* dense;   // dense bias element of (fixed index, var0); natural-log units
  long long dense_vs;   // its stride along the varying side (1 when the keys vary)
  int dense_vec;        // keys vary, the whole block is in range and rows are 16-byte aligned: vector loads
};

// Branch-free per element: the uniform `flags` only shape a handful of per-lane constants up
// front (evaluated per element they cost ~25 instructions per score, three times the softmax
// itself).  Range limit, causal and window terms are ONE interval [lo, hi] of the element's offset
// `off` on the varying side (rel = rel0 -+ off is monotonic in it); the prefix term is a second
// bound that only counts where not both sides carry the prefix flag; a segment test against the
// lane's own id when there is no segment term compares equal; ALiBi with slope 0 adds nothing.
// TERMS = false: a kernel variant that knows causal / window terms only (the rest compiles away).
template <bool QFIXED, bool DENSE, bool TERMS>
RA_DEV void apply_bias(f32x16& t, const TileBias& tb, int rel0, int fixed_seg, int fixed_pre,
                       const int* var_seg, const int* var_pre) {
  constexpr int kFar = 1 << 30;
  // one value per wave (a block belongs to one wave's rows and one tile): say so, or the compiler
  // carries every flag test as a lane mask
  int flags = __builtin_amdgcn_readfirstlane(tb.flags);
  if (!TERMS) flags &= RA_BIAS_CAUSAL | RA_BIAS_WINDOW;
  const bool causal = flags & RA_BIAS_CAUSAL, window = flags & RA_BIAS_WINDOW;
  const bool segment = flags & RA_BIAS_SEGMENT, prefix = flags & RA_BIAS_PREFIX;
  const bool dense_vec = DENSE && __builtin_amdgcn_readfirstlane(tb.dense_vec) != 0;
  // the block is read for this tile (always, unless its summary says that the tile holds zeros)
  const bool dense_on = DENSE && (flags & RA_BIAS_DENSE);
  int lo = 0, hi = tb.var_limit - 1;  // off >= var_limit: out of range
  int pre_lo = -kFar, pre_hi = kFar;  // outside [pre_lo, pre_hi]: rel < 0, masked unless both sides are prefix
  // |rel0| < 2^30 and window <= 2^30 (the host checks positions and clamps the window), so the sums
  // below stay inside 32 bits, and the prefix interval - open to 2^30 on one side - holds every
  // rel0 without a clamp (an instruction more per block costs the 256-register kernels a spill)
  if (QFIXED) {  // rel = rel0 - off: rel < 0 <=> off > rel0, rel >= w <=> off <= rel0 - w, -rel >= w <=> off >= rel0 + w
    if (causal) hi = min(hi, rel0);
    if (window) lo = max(lo, rel0 - tb.window + 1);
    if (window && !causal) hi = min(hi, rel0 + tb.window - 1);
    if (prefix) pre_hi = rel0;
  } else {  // rel = rel0 + off: rel < 0 <=> off < -rel0, rel >= w <=> off >= w - rel0, -rel >= w <=> off <= -rel0 - w
    if (causal) lo = max(lo, -rel0);
    if (window) hi = min(hi, tb.window - 1 - rel0);
    if (window && !causal) lo = max(lo, 1 - rel0 - tb.window);
    if (prefix) pre_lo = -rel0;
  }
  // off in [lo, hi] <=> (unsigned)(off - lo) <= (unsigned)(hi - lo); an empty interval (hi < lo)
  // becomes lo = 1 << 30, span = 0: no off in 0..63 passes
  const bool none = hi < lo;
  const unsigned nlo = (unsigned)(none ? -(1 << 30) : -lo), span = (unsigned)(none ? 0 : hi - lo);
  const unsigned pnlo = (unsigned)(-pre_lo), pspan = (unsigned)pre_hi - (unsigned)pre_lo;  // < 2^31 under a prefix term
  const int seg_ref = fixed_seg;
  const int pre_on = (prefix && fixed_pre != 0) ? -1 : 0;  // all ones where this lane's side carries the flag
  const float slope = -tb.slope2;
  const float relf0 = (float)rel0;
  // The two terms that cost the most per element, ALiBi (two instructions) and prefix (six), get
  // code of their own, chosen once per block by a uniform branch.
  auto body = [&](auto with_alibi, auto with_prefix) {
    constexpr bool ALI = decltype(with_alibi)::value, PRE = decltype(with_prefix)::value;
#pragma unroll
    for (int bb = 0; bb < 4; ++bb) {
      i32x4 vs = {seg_ref, seg_ref, seg_ref, seg_ref}, vp = {0, 0, 0, 0};
      if (segment) vs = *(const i32x4*)(var_seg + 8 * bb);
      if (PRE) vp = *(const i32x4*)(var_pre + 8 * bb);
      float dn[4] = {0.f, 0.f, 0.f, 0.f};
      if (DENSE && dense_on) {
        if (QFIXED && dense_vec) {
          // a lane's four keys are 16 contiguous bytes of its row: one load instead of four
          const f32x4 v4 = *(const f32x4*)(tb.dense + 8 * bb);
#pragma unroll
          for (int c = 0; c < 4; ++c) dn[c] = v4[c];
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (8 * bb + c < tb.var_limit) dn[c] = QFIXED ? tb.dense[8 * bb + c] : tb.dense[(8 * bb + c) * tb.dense_vs];
        }
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int r = 4 * bb + c;
        const int off = 8 * bb + c;
        float x = t[r];
        if (ALI) {
          // moving along the varying side: keys advance -> rel decreases; queries advance -> rel increases
          const float relf = QFIXED ? relf0 - (float)off : relf0 + (float)off;
          x = fmaf(fabsf(relf), slope, x);
        }
        if (DENSE) x = fmaf(dn[c], tb.dense_mul, x);
        bool msk = ((unsigned)off + nlo > span) | (vs[c] != seg_ref);
        if (PRE) msk |= ((unsigned)off + pnlo > pspan) & ((vp[c] & pre_on) == 0);
        t[r] = msk ? RA_NEG_INF : x;
      }
    }
  };
  using Yes = std::true_type;
  using No = std::false_type;
  const bool alibi = flags & RA_BIAS_ALIBI;
  if (!TERMS) body(No{}, No{});
  else if (alibi && prefix) body(Yes{}, Yes{});
  else if (alibi) body(Yes{}, No{});
  else if (prefix) body(No{}, Yes{});
  else body(No{}, No{});
}

// Positional classification of a rectangle of scores: queries [qlo, qhi], keys [klo, khi]
// (global positions, inclusive).  Returns bit 0 = every score masked, bit 1 = some score may
// be masked (the elementwise test is needed).
RA_DEV int classify_pos(int flags, int window, int qlo, int qhi, int klo, int khi) {
  bool all = false, some = false;
  if (flags & RA_BIAS_CAUSAL) {
    all |= klo > qhi;
    some |= khi > qlo;
  }
  if (flags & RA_BIAS_WINDOW) {
    all |= (qlo - khi) >= window;
    some |= (qhi - klo) >= window;
    if (!(flags & RA_BIAS_CAUSAL)) {
      all |= (klo - qhi) >= window;
      some |= (khi - qlo) >= window;
    }
  }
  return (all ? 1 : 0) | (some ? 2 : 0);
}

RA_DEV int floor_div(int a, int b) { return (a >= 0) ? a / b : -((-a + b - 1) / b); }
RA_DEV int ceil_div(int a, int b) { return -floor_div(-a, b); }

// Range [lo, hi) of T-sized tiles on the key side that can hold an unmasked score for
// queries at positions [qlo, qhi]; keys of tile j are at positions kv_off + T*j + [0, T).
RA_DEV void key_tile_range(int flags, int window, int qlo, int qhi, int kv_off, int ntiles, int T,
                           int& lo, int& hi) {
  lo = 0;
  hi = ntiles;
  if (flags & RA_BIAS_PREFIX) return;
  if (flags & RA_BIAS_CAUSAL) hi = min(hi, floor_div(qhi - kv_off, T) + 1);
  if (flags & RA_BIAS_WINDOW) {
    lo = max(lo, ceil_div(qlo - window + 1 - (T - 1) - kv_off, T));
    if (!(flags & RA_BIAS_CAUSAL)) hi = min(hi, floor_div(qhi + window - 1 - kv_off, T) + 1);
  }
  hi = max(hi, 0);
  lo = min(max(lo, 0), hi);
}

// Range [lo, hi) of T-sized key tiles in which EVERY score of queries [qlo, qhi] is unmasked by
// the positional terms (so no elementwise test is needed), tile j = positions kv_off + T*j + [0, T).
RA_DEV void key_tile_plain_range(int flags, int window, int qlo, int qhi, int kv_off, int ntiles, int T,
                                 int& lo, int& hi) {
  lo = 0;
  hi = ntiles;
  if (flags & RA_BIAS_CAUSAL) hi = min(hi, floor_div(qlo - kv_off - (T - 1), T) + 1);
  if (flags & RA_BIAS_WINDOW) {
    lo = max(lo, floor_div(qhi - window - kv_off, T) + 1);
    if (!(flags & RA_BIAS_CAUSAL)) hi = min(hi, ceil_div(qlo + window - kv_off - (T - 1), T));
  }
  hi = max(hi, 0);
  lo = min(max(lo, 0), hi);
}
// Mirror image: T-sized query tiles all of whose scores against keys [klo, khi] are unmasked.
RA_DEV void query_tile_plain_range(int flags, int window, int klo, int khi, int q_off, int ntiles, int T,
                                   int& lo, int& hi) {
  lo = 0;
  hi = ntiles;
  if (flags & RA_BIAS_CAUSAL) lo = max(lo, ceil_div(khi - q_off, T));
  if (flags & RA_BIAS_WINDOW) {
    hi = min(hi, ceil_div(klo + window - q_off - (T - 1), T));
    if (!(flags & RA_BIAS_CAUSAL)) lo = max(lo, floor_div(khi - window - q_off, T) + 1);
  }
  hi = max(hi, 0);
  lo = min(max(lo, 0), hi);
}

// Same for the query side: tiles of queries that can see keys at positions [klo, khi].
RA_DEV void query_tile_range(int flags, int window, int klo, int khi, int q_off, int ntiles, int T,
                             int& lo, int& hi) {
  lo = 0;
  hi = ntiles;
  if (flags & RA_BIAS_PREFIX) return;
  if (flags & RA_BIAS_CAUSAL) lo = max(lo, ceil_div(klo - (T - 1) - q_off, T));
  if (flags & RA_BIAS_WINDOW) {
    hi = min(hi, floor_div(khi + window - 1 - q_off, T) + 1);
    if (!(flags & RA_BIAS_CAUSAL)) lo = max(lo, ceil_div(klo - window + 1 - (T - 1) - q_off, T));
  }
  hi = max(hi, 0);
  lo = min(max(lo, 0), hi);
}

// Smallest and largest id of tile t (T tokens) of an id array of length L.  The loads are
// independent of each other and issued together (a loop with a data-dependent bound would wait
// for each load in turn: tens of microseconds per tile).
template <int T>
RA_DEV void tile_id_range(const int* ids, int t, int L, int& mn, int& mx) {
  mn = 0x7fffffff;
  mx = (int)0x80000000;
  const int base = t * T;
  if (base + T <= L && (((unsigned long long)(ids + base)) & 15ull) == 0) {
#pragma unroll 4
    for (int c = 0; c < T / 4; ++c) {
      const i32x4 v = *(const i32x4*)(ids + base + 4 * c);
      mn = min(min(mn, v[0]), min(v[1], min(v[2], v[3])));
      mx = max(max(mx, v[0]), max(v[1], max(v[2], v[3])));
    }
  } else {
#pragma unroll 8
    for (int e = 0; e < T; ++e) {
      const int sid = ids[min(base + e, L - 1)];  // repeats of the last id change nothing
      mn = min(mn, sid);
      mx = max(mx, sid);
    }
  }
}

// Executed by ONE wave.  `list` holds `cnt` entries (tile index in bits 0..14, bit 15 set when
// the tile needs the elementwise segment test).  Finds the first run, at or after ordinal `from`,
// of entries that need no test and whose tile indices are consecutive: ordinals [start, end), and
// `tile_base` such that entry i of the run is tile `tile_base + i`.  Such a run can be walked with
// running addresses.  No run: start = end = cnt.
RA_DEV void uniform_run(const unsigned short* list, int cnt, int lane, int from, int& start, int& end, int& tile_base) {
  start = -1;
  for (int base = from; base < cnt && start < 0; base += 64) {
    const int i = base + lane;
    const bool ok = i < cnt && !(list[i] >> 15);
    const unsigned long long mask = __ballot(ok);
    if (mask) start = base + __ffsll((long long)mask) - 1;
  }
  if (start < 0) {
    start = end = cnt;
    tile_base = 0;
    return;
  }
  end = cnt;
  for (int base = start; base < cnt; base += 64) {
    const int i = base + lane;
    const bool brk = i < cnt && i > start && ((list[i] >> 15) || (list[i] & 0x7fff) != (list[i - 1] & 0x7fff) + 1);
    const unsigned long long mask = __ballot(brk);
    if (mask) {
      end = base + __ffsll((long long)mask) - 1;
      break;
    }
  }
  tile_base = (list[start] & 0x7fff) - start;
}

// Executed by ONE wave.  First ordinal behind `from` whose tile index does not follow its
// predecessor's (`cnt` if the list counts up to its end): up to there, loads that advance by one
// tile per iteration fetch exactly the listed tiles.
RA_DEV int consecutive_end(const unsigned short* list, int cnt, int lane, int from) {
  for (int base = from; base < cnt; base += 64) {
    const int i = base + lane;
    const bool brk = i < cnt && i > from && (list[i] & 0x7fff) != (list[i - 1] & 0x7fff) + 1;
    const unsigned long long mask = __ballot(brk);
    if (mask) return base + __ffsll((long long)mask) - 1;
  }
  return cnt;
}

// Decode the flat workgroup id into (batch*head index, tile index).  Workgroups are handed
// to the 8 XCDs round-robin, each XCD has its own L2: keep all tiles of one head on one
// XCD so they share the head's K/V (or Q/dO) stream, and start with the last tile, which
// has the most work under a causal mask.
RA_DEV void decode_block(int bid, int BH, int ntile, int& hh, int& tile) {
  if ((BH & 7) == 0) {
    int xcd = bid & 7, slot = bid >> 3;
    hh = (slot / ntile) * 8 + xcd;
    tile = ntile - 1 - (slot % ntile);
  } else {
    hh = bid / ntile;
    tile = ntile - 1 - (bid % ntile);
  }
}

}  // namespace ra
