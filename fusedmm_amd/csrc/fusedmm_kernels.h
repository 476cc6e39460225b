// Device code for the fused SDDMM+SpMM path on gfx950 (wave64).
//
// One wavefront walks one CSR row (or one fixed-length edge segment of a heavy
// row).  A wavefront is cut into S = 64/L sub-waves of L lanes; a sub-wave owns
// one neighbour row Y[c] at a time, each lane holding R four-element slices of
// it, so a gather is L coalesced 16-byte loads (two per lane in double
// precision).  The X[i] slice and the Z accumulator live in VGPRs for the whole
// row.  The per-edge reduction (ROP) is a DPP / swizzle XOR butterfly over the L
// lanes, the scalar op (SOP) and the scaled accumulate (MOP, AOP) happen in
// registers.
//
// Element e of a K-vector sits in lane (e/4) % L, register (e/4) / L,
// component e % 4.  A lane reduces its own elements with a fused multiply-add
// chain (register ascending, component ascending) and lanes are combined by XOR
// offsets 1, 2, 4 ... L/2.  That order is part of the numerical contract: the
// table sigmoid is discontinuous in the dot product, and the CPU oracle's
// "wavefront order" mode reproduces exactly this sum.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fmm {

// The library is compiled once per value type, as the reference is (-DDREAL).
#ifdef FMM_DOUBLE
typedef double real_t;
#else
typedef float real_t;
#endif
struct alignas(16) real4 {
   real_t x, y, z, w;
};

// ---- op-tuple nibbles (values of the public header) -------------------------
enum : int {
   kVopCopyLhs = 0x1, kVopCopyRhs = 0x2, kVopAdd = 0x3, kVopSubl = 0x4, kVopSubr = 0x5,
   kVopMax = 0x6, kVopMin = 0x7,
   kRopNoop = 0x00, kRopDot = 0x10, kRopAddLhs = 0x20, kRopAddRhs = 0x30, kRopNormL = 0x40,
   kRopNormR = 0x50,
   kSopNoop = 0x000, kSopCopy = 0x100, kSopUdef = 0xF00,
   kVscNoop = 0x0000, kVscMul = 0x1000, kVscAdd = 0x2000,
   kAopNoop = 0x00000, kAopAdd = 0x10000, kAopMax = 0x20000, kAopMin = 0x30000
};

// Pattern-matched kernels and the runtime-switched general one.
enum : int { OP_GCN = 0, OP_SPMM = 1, OP_DOT = 2, OP_DIST = 3, OP_GENERIC = 4 };

// Device-native bodies for SOP_UDEF (numbering shared with the public header).
enum : int { SOP_IDENTITY = 0, SOP_SIGMOID = 1, SOP_TDIST = 2, SOP_FR = 3, SOP_LL = 4, SOP_FA = 5, SOP_TDIST_PLAIN = 6 };

constexpr int kSigmoidTableSize = 2048;
constexpr int kBlockThreads = 256;
constexpr int kWavesPerBlock = kBlockThreads / 64;

// Queue and claim counters of one call.  The queue counters, the row and retire
// counters are zero between calls: the last workgroup of the fused kernel to
// finish puts them back (and clears the queued-row bits), so a call needs no
// reset pass of its own.
struct Counters {
   unsigned int n_heavy;    // heavy rows queued by the classify kernel   } advanced together, as one
   unsigned int n_seg;      // edge segments queued                       } 64-bit word (n_heavy low)
   unsigned int overflow;   // heavy rows that did not fit the queue (processed whole in phase B)
   unsigned int done_groups; // groups of workgroups of the fused kernel that have finished (see retire[])
   unsigned int invalid;    // set by the optional operand check
   unsigned int last_heavy, last_seg, last_overflow;   // n_heavy, n_seg, overflow of the call that finished last
   unsigned int merge_heavy;      // heavy rows the merge kernel of this call has to fold (n_heavy, capped)
   unsigned int pad1;
   // Edges of rows that are not split, in the lower (low word) and upper half of the row space, over a sample
   // of the rows and scaled down, left by the classify kernel: tells the fused kernel whether the row phase's
   // work is spread evenly along the rows.
   unsigned long long skew;
   unsigned long long last_skew;  // skew of the call that finished last
   unsigned int last_scattered;   // 1: that call's row phase took the stretches of the row space in scattered order
   unsigned int pad2[17];         // keep the row counters on their own 128-byte lines
   // Row claim counters.  Read-modify-writes on ONE address retire one per
   // ~12 ns on this GPU however many CUs issue them; on distinct 128-byte
   // lines they proceed in parallel.  So the row space is dealt to
   // kRowCounters counters and a wave works its home counter first.
   struct alignas(128) RowCounter { unsigned long long next; } rows[64];
   // Workgroups of the fused kernel that have finished, counted per group of
   // workgroups (blockIdx % 64) for the same reason: one shared counter would
   // make the kernel's end wait ~12 ns per workgroup.
   struct alignas(128) RetireCounter { unsigned int done; } retire[64];
};
constexpr int kRowCounters = 64;

struct HeavyRow {
   int64_t row;
   unsigned int seg_base;
   unsigned int n_seg;
};

struct SegDesc {
   int64_t row;            // -1: slot of a row that did not fit the queue
   int64_t first;          // first edge slot of the segment
   unsigned int count;     // edges in the segment
   unsigned int pad;
};

constexpr int kRowsPerClaim = 8;        // rows a wave claims at a time
constexpr unsigned int kMaxSegsPerRow = 512;   // longer rows get longer segments

template <typename IdxT>
struct Params {
   const IdxT *pntrb, *pntre, *indx;
   const real_t *val;
   const real_t *x, *y;
   real_t *z;
   int64_t m;
   int64_t ldx, ldy, ldz;
   int k;
   int beta_zero;          // 1: overwrite Z, 0: accumulate into Z
   int sop_kind;           // device SOP body for SOP_UDEF
   int imessage;           // op tuple (read by OP_GENERIC only)
   const real_t *sigmoid_table;
   // heavy-row queue
   int64_t heavy_deg;      // rows with more edges than this are split
   int seg_len;            // edges per segment
   Counters *ctr;
   HeavyRow *heavy;
   SegDesc *segs;
   real_t *partial;        // [cap_seg][kpad]
   unsigned int *queued;   // one bit per row: set by the classify kernel for rows it put on the heavy-row queue
   unsigned int cap_heavy, cap_seg;
   int kpad;
   int row_counters;       // claim counters in use: kRowCounters; 1 when the grid has fewer waves; 0: wave w takes chunk w
   int row_order;          // 0: decided from the classify kernel's sample; 1: first to last; 2: scattered stretches
   int pack_rows;          // 1: groups of short rows are walked one row per sub-wave (sub-waves of 8 or 16 lanes)
   int store_shift;        // finished Z rows leave LDS when the 100 MHz clock >> store_shift changes; 0: stored as they finish
   int stage_vecs;         // LDS each wavefront has for such rows, in 4-element registers (the launch's dynamic LDS / waves)
};

// ---- wave primitives --------------------------------------------------------
// Cross-lane moves work on 32-bit registers; a double is moved as two halves.
__device__ __forceinline__ float as_f(int v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ int as_i(float v) { return __builtin_bit_cast(int, v); }

template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false); }
__device__ __forceinline__ int xor16_i(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x401F); }

#define FMM_SPLIT64(v, lo, hi)                                    \
   const long long bits_ = __builtin_bit_cast(long long, v);      \
   const int lo = (int)(bits_ & 0xFFFFFFFFll), hi = (int)(bits_ >> 32)
__device__ __forceinline__ double join64(int lo, int hi)
{
   return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)(unsigned int)lo);
}

template <int CTRL>
__device__ __forceinline__ float dpp(float v) { return as_f(dpp_i<CTRL>(as_i(v))); }
template <int CTRL>
__device__ __forceinline__ double dpp(double v)
{
   FMM_SPLIT64(v, lo, hi);
   return join64(dpp_i<CTRL>(lo), dpp_i<CTRL>(hi));
}
// value held by lane ^ 16
__device__ __forceinline__ float lane_xor16(float v) { return as_f(xor16_i(as_i(v))); }
__device__ __forceinline__ double lane_xor16(double v)
{
   FMM_SPLIT64(v, lo, hi);
   return join64(xor16_i(lo), xor16_i(hi));
}

// v[lane] + v[lane ^ 32]: one v_permlane32_swap gives both halves to every lane.
__device__ __forceinline__ float add_xor32(float v)
{
   auto r = __builtin_amdgcn_permlane32_swap(as_i(v), as_i(v), false, false);
   return as_f(r[0]) + as_f(r[1]);
}
__device__ __forceinline__ double add_xor32(double v)
{
   FMM_SPLIT64(v, lo, hi);
   auto a = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
   auto b = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
   return join64(a[0], b[0]) + join64(a[1], b[1]);
}

__device__ __forceinline__ float fma_r(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_r(double a, double b, double c) { return __builtin_fma(a, b, c); }
__device__ __forceinline__ real_t max_r(real_t a, real_t b) { return a > b ? a : b; }
__device__ __forceinline__ real_t min_r(real_t a, real_t b) { return a < b ? a : b; }

// Sum over the L lanes of a sub-wave; every lane ends with the same bits.
// After the quad steps all lanes of a quad agree, so the half-row and row
// mirrors deliver exactly the value lane^4 / lane^8 holds.
template <int L>
__device__ __forceinline__ real_t subwave_sum(real_t v)
{
   if (L >= 2) v = v + dpp<0xB1>(v);   // quad_perm [1,0,3,2]  : lane ^ 1
   if (L >= 4) v = v + dpp<0x4E>(v);   // quad_perm [2,3,0,1]  : lane ^ 2
   if (L >= 8) v = v + dpp<0x141>(v);  // row_half_mirror      : lane ^ 4 (by value)
   if (L >= 16) v = v + dpp<0x140>(v); // row_mirror           : lane ^ 8 (by value)
   if (L >= 32) v = v + lane_xor16(v);
   if (L >= 64) v = add_xor32(v);
   return v;
}

// Combine the S = 64/L sub-wave accumulators (same element slice, different
// edges).  Offsets L, 2L .. 32 are true lane XORs (row_ror:8 == lane ^ 8).
template <int L>
__device__ __forceinline__ real_t cross_subwave_sum(real_t v)
{
   static_assert(L >= 8, "sub-waves narrower than 8 lanes are not used");
   if (L <= 8) v = v + dpp<0x128>(v);  // row_ror:8
   if (L <= 16) v = v + lane_xor16(v);
   if (L <= 32) v = add_xor32(v);
   return v;
}
// MAX and MIN of the accumulate stage across sub-waves.  The reference's fmax / fmin are the ternaries
// (x) > (y) ? (x) : (y) and (x) < (y) ? (x) : (y) (fusedMM.c:18-19): a NaN on the left loses, a NaN on the
// right wins, so what a row with a NaN term comes to depends on the order of its edges.  Here a sub-wave
// folds its own edges with that very ternary, in edge order; where accumulators are combined a NaN is kept
// (both lanes of a pair then agree, and a row with a single edge gives exactly the reference's result).
__device__ __forceinline__ real_t merge_max(real_t v, real_t o) { const real_t r = max_r(v, o); return v != v ? v : r; }
__device__ __forceinline__ real_t merge_min(real_t v, real_t o) { const real_t r = min_r(v, o); return v != v ? v : r; }
template <int L>
__device__ __forceinline__ real_t cross_subwave_max(real_t v)
{
   if (L <= 8) v = merge_max(v, dpp<0x128>(v));
   if (L <= 16) v = merge_max(v, lane_xor16(v));
   if (L <= 32) v = merge_max(v, (real_t)__shfl_xor(v, 32, 64));
   return v;
}
template <int L>
__device__ __forceinline__ real_t cross_subwave_min(real_t v)
{
   if (L <= 8) v = merge_min(v, dpp<0x128>(v));
   if (L <= 16) v = merge_min(v, lane_xor16(v));
   if (L <= 32) v = merge_min(v, (real_t)__shfl_xor(v, 32, 64));
   return v;
}

template <typename T>
__device__ __forceinline__ T wave_uniform(T v);
template <>
__device__ __forceinline__ int32_t wave_uniform<int32_t>(int32_t v) { return __builtin_amdgcn_readfirstlane(v); }
template <>
__device__ __forceinline__ int64_t wave_uniform<int64_t>(int64_t v)
{
   int lo = __builtin_amdgcn_readfirstlane((int)(v & 0xFFFFFFFFll));
   int hi = __builtin_amdgcn_readfirstlane((int)(v >> 32));
   return ((int64_t)hi << 32) | (uint32_t)lo;
}

// value held by lane `t` (wave-uniform t), delivered to every lane
template <typename T>
__device__ __forceinline__ T lane_value(T v, int t);
template <>
__device__ __forceinline__ int32_t lane_value<int32_t>(int32_t v, int t) { return __builtin_amdgcn_readlane(v, t); }
template <>
__device__ __forceinline__ int64_t lane_value<int64_t>(int64_t v, int t)
{
   int lo = __builtin_amdgcn_readlane((int)(v & 0xFFFFFFFFll), t);
   int hi = __builtin_amdgcn_readlane((int)(v >> 32), t);
   return ((int64_t)hi << 32) | (uint32_t)lo;
}

// The sigmoid table as the fused kernel reads it: always the workgroup's copy in LDS.
// The pointer carries the address space in its type, so that a look-up is an LDS read
// (its own counter) also where the SOP body is picked at run time; through a plain
// pointer it would be a flat load, which waits behind every gather in flight.
typedef const __attribute__((address_space(3))) real_t *lds_table_t;

// ---- SOP bodies ---------------------------------------------------------------
// Same expressions, in the same precision, as the SOP_UDEF_FUNC bodies of the
// reference's tester (test/fusedMMtime.cpp:606-660): constants there are double
// literals, so the arithmetic is done in double and (single-precision build)
// rounded once to float.
template <typename TabPtr>
__device__ __forceinline__ real_t sop_eval(int kind, real_t s, TabPtr tab)
{
   switch (kind)
   {
      case SOP_SIGMOID:
      {
         // floor-indexed 2048-entry table on [-5,5] (test/fusedMMtime.cpp:128-130, 606-611);
         // s == 5 exactly would index one past the end there: clamp to the last entry.
         // Written without branches (the look-up is made for every lane, from a clamped
         // argument, and the saturated ends are selected afterwards): lanes of a wave
         // take different sides, and straight-line code lets the look-ups of the edges
         // in flight overlap.
         const real_t sc = s > (real_t)5.0 ? (real_t)5.0 : (s < (real_t)-5.0 ? (real_t)-5.0 : s);
#ifdef FMM_DOUBLE
         int idx = (int)((sc + 5.0) * 2048.0 / 10.0);
#else
         // The reference evaluates ((double)s + 5.0) * 2048 / 10.0.  One multiply by
         // 204.8 truncates to the same integer for every float in [-5, 5]
         // (checked exhaustively over all 2 168 455 170 of them on the CPU), and
         // spares a double-precision division per edge.
         int idx = (int)(((double)sc + 5.0) * 204.8);
#endif
         idx = idx > kSigmoidTableSize - 1 ? kSigmoidTableSize - 1 : idx;
         idx = idx < 0 ? 0 : idx;   // only a NaN gets here (no comparison holds for it)
         real_t t = tab[idx];
         t = s > (real_t)5.0 ? (real_t)1.0 : t;
         t = s < (real_t)-5.0 ? (real_t)0.0 : t;
         return (real_t)1.0 - t;   // single precision: exact in double for table values, one rounding either way
      }
      case SOP_TDIST:
      {
         real_t t = (real_t)(-2.0 / (1.0 + (double)s));
         t = t > (real_t)5.0 ? (real_t)5.0 : t;
         t = t < (real_t)-5.0 ? (real_t)-5.0 : t;
         return t;
      }
      case SOP_FR:
         return (real_t)(1.0 + 1.0 / (double)s);
#ifdef FMM_DOUBLE
      case SOP_LL:
         return log2(1 + sqrt(s));
      case SOP_FA:
         return sqrt(s) + 1.0 / s;
#else
      case SOP_LL:
         return log2f(1.0f + sqrtf(s));
      case SOP_FA:
         return (float)((double)sqrtf(s) + 1.0 / (double)s);
#endif
      case SOP_TDIST_PLAIN:
         return (real_t)(1.0 / (1.0 + (double)s));   // the t-dist body without its constant -2 and its clamp
      default:
         return s;
   }
}

// Four consecutive elements: 16 bytes in single precision (one 16-byte access),
// 32 bytes in double precision (two 16-byte accesses; rows need 16-byte alignment only).
__device__ __forceinline__ real4 ld4(const real_t *p) { return *reinterpret_cast<const real4 *>(p); }
__device__ __forceinline__ void st4(real_t *p, real4 v) { *reinterpret_cast<real4 *>(p) = v; }
// Streaming variants for data touched once per call (X rows, Z rows): the
// non-temporal hint keeps them from displacing gathered Y rows in the caches.
#ifdef FMM_DOUBLE
typedef double vec16_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ real4 ld4_stream(const real_t *p)
{
   const vec16_t a = __builtin_nontemporal_load(reinterpret_cast<const vec16_t *>(p));
   const vec16_t b = __builtin_nontemporal_load(reinterpret_cast<const vec16_t *>(p) + 1);
   return real4{a.x, a.y, b.x, b.y};
}
__device__ __forceinline__ void st4_stream(real_t *p, real4 v)
{
   vec16_t a = {v.x, v.y}, b = {v.z, v.w};
   __builtin_nontemporal_store(a, reinterpret_cast<vec16_t *>(p));
   __builtin_nontemporal_store(b, reinterpret_cast<vec16_t *>(p) + 1);
}
#else
typedef float vec16_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ real4 ld4_stream(const real_t *p)
{
   const vec16_t v = __builtin_nontemporal_load(reinterpret_cast<const vec16_t *>(p));
   return real4{v.x, v.y, v.z, v.w};
}
__device__ __forceinline__ void st4_stream(real_t *p, real4 v)
{
   vec16_t t = {v.x, v.y, v.z, v.w};
   __builtin_nontemporal_store(t, reinterpret_cast<vec16_t *>(p));
}
#endif
__device__ __forceinline__ real4 zero4() { return real4{(real_t)0, (real_t)0, (real_t)0, (real_t)0}; }

// One row slice per lane: R real4 registers.
template <int R>
struct Slice {
   real4 v[R];
};

// V == 4: lane sl holds elements 4*(r*L+sl) .. +3 in register r (16-byte accesses).
// V == 1: rows that are not 16-byte aligned (K or a leading dimension not a
// multiple of 4, or an unaligned base): component c of register r holds
// element (4r+c)*L + sl, loaded and stored 4 bytes at a time.
template <int V, int L, int R, bool EXACT, bool STREAM = false>
__device__ __forceinline__ void load_slice(Slice<R> &s, const real_t *row, int sl, int k)
{
#pragma unroll
   for (int r = 0; r < R; r++)
   {
      if (V == 4)
      {
         const int e0 = 4 * (r * L + sl);
         if (EXACT || e0 < k) s.v[r] = STREAM ? ld4_stream(row + e0) : ld4(row + e0);
         else s.v[r] = zero4();
      }
      else
      {
         const int e0 = (4 * r) * L + sl;
         s.v[r].x = (e0 < k) ? row[e0] : (real_t)0;
         s.v[r].y = (e0 + L < k) ? row[e0 + L] : (real_t)0;
         s.v[r].z = (e0 + 2 * L < k) ? row[e0 + 2 * L] : (real_t)0;
         s.v[r].w = (e0 + 3 * L < k) ? row[e0 + 3 * L] : (real_t)0;
      }
   }
}

template <int V, int L, int R, bool EXACT, bool STREAM = false>
__device__ __forceinline__ void store_slice(real_t *row, const Slice<R> &s, int sl, int k)
{
#pragma unroll
   for (int r = 0; r < R; r++)
   {
      if (V == 4)
      {
         const int e0 = 4 * (r * L + sl);
         if (EXACT || e0 < k)
         {
            if (STREAM) st4_stream(row + e0, s.v[r]);
            else st4(row + e0, s.v[r]);
         }
      }
      else
      {
         const int e0 = (4 * r) * L + sl;
         if (e0 < k) row[e0] = s.v[r].x;
         if (e0 + L < k) row[e0 + L] = s.v[r].y;
         if (e0 + 2 * L < k) row[e0 + 2 * L] = s.v[r].z;
         if (e0 + 3 * L < k) row[e0 + 3 * L] = s.v[r].w;
      }
   }
}

template <int L, int R>
__device__ __forceinline__ real_t dot_slices(const Slice<R> &a, const Slice<R> &b)
{
   real_t p = (real_t)0;
#pragma unroll
   for (int r = 0; r < R; r++)
   {
      p = fma_r(a.v[r].x, b.v[r].x, p);
      p = fma_r(a.v[r].y, b.v[r].y, p);
      p = fma_r(a.v[r].z, b.v[r].z, p);
      p = fma_r(a.v[r].w, b.v[r].w, p);
   }
   return subwave_sum<L>(p);
}

template <int L, int R>
__device__ __forceinline__ real_t sum_slice(const Slice<R> &a)
{
   real_t p = (real_t)0;
#pragma unroll
   for (int r = 0; r < R; r++) p = ((((p + a.v[r].x) + a.v[r].y) + a.v[r].z) + a.v[r].w);
   return subwave_sum<L>(p);
}

// acc = fma(d, t, acc) over a slice
template <int R>
__device__ __forceinline__ void axpy_slice(Slice<R> &acc, real_t d, const Slice<R> &t)
{
#pragma unroll
   for (int r = 0; r < R; r++)
   {
      acc.v[r].x = fma_r(d, t.v[r].x, acc.v[r].x);
      acc.v[r].y = fma_r(d, t.v[r].y, acc.v[r].y);
      acc.v[r].z = fma_r(d, t.v[r].z, acc.v[r].z);
      acc.v[r].w = fma_r(d, t.v[r].w, acc.v[r].w);
   }
}

template <int R>
__device__ __forceinline__ void sub_slices(Slice<R> &t, const Slice<R> &a, const Slice<R> &b)
{
#pragma unroll
   for (int r = 0; r < R; r++)
   {
      t.v[r].x = a.v[r].x - b.v[r].x;
      t.v[r].y = a.v[r].y - b.v[r].y;
      t.v[r].z = a.v[r].z - b.v[r].z;
      t.v[r].w = a.v[r].w - b.v[r].w;
   }
}

template <class F, int R>
__device__ __forceinline__ void map2(Slice<R> &o, const Slice<R> &a, const Slice<R> &b, F f)
{
#pragma unroll
   for (int r = 0; r < R; r++)
   {
      o.v[r].x = f(a.v[r].x, b.v[r].x);
      o.v[r].y = f(a.v[r].y, b.v[r].y);
      o.v[r].z = f(a.v[r].z, b.v[r].z);
      o.v[r].w = f(a.v[r].w, b.v[r].w);
   }
}

// Identity element of the accumulate stage (what a sub-wave that did not load
// Z starts from).
__device__ __forceinline__ real_t aop_identity(int aop)
{
   if (aop == kAopMax) return -(real_t)__builtin_inf();
   if (aop == kAopMin) return (real_t)__builtin_inf();
   return (real_t)0;
}

// T = VOP(x, y) and s = ROP(x, T) of the general pipeline (reference
// fusedMM.c:28-202, 721-725); s starts as the edge value (:717).
template <int L, int R>
__device__ __forceinline__ real_t vop_rop(Slice<R> &t, const Slice<R> &xs, const Slice<R> &ys, real_t edge_val, int vop,
                                         int rop)
{
   switch (vop)
   {
      case kVopCopyLhs: t = xs; break;
      case kVopCopyRhs: t = ys; break;
      case kVopAdd: map2(t, xs, ys, [](real_t a, real_t b) { return a + b; }); break;
      case kVopSubl: map2(t, xs, ys, [](real_t a, real_t b) { return -a + b; }); break;
      case kVopSubr: map2(t, xs, ys, [](real_t a, real_t b) { return a - b; }); break;
      case kVopMax: map2(t, xs, ys, [](real_t a, real_t b) { return a > b ? a : b; }); break;
      default: map2(t, xs, ys, [](real_t a, real_t b) { return a < b ? a : b; }); break;
   }
   real_t scal = edge_val;
   switch (rop)
   {
      case kRopDot: scal = dot_slices<L, R>(xs, t); break;
      case kRopAddLhs: scal = sum_slice<L, R>(xs); break;
      case kRopAddRhs: scal = sum_slice<L, R>(t); break;
      case kRopNormL: scal = dot_slices<L, R>(xs, xs); break;
      case kRopNormR: scal = dot_slices<L, R>(t, t); break;
      default: break;
   }
   return scal;
}

// One edge of the four optimised tuples: T = VOP(x, y); s = ROP(x, T); d = SOP(s);
// acc += d * T, fused.  `xs` is the X[i] slice, `ys` the gathered Y[c] slice.  (The
// general pipeline is general_steps below.)
template <int L, int R, int OP>
__device__ __forceinline__ void edge_step(Slice<R> &acc, const Slice<R> &xs, const Slice<R> &ys,
                                          real_t edge_val, int sop_kind, lds_table_t tab)
{
   static_assert(OP != OP_GENERIC, "the general pipeline goes through general_steps");
   if (OP == OP_GCN)
   {
#pragma unroll
      for (int r = 0; r < R; r++)
      {
         acc.v[r].x += ys.v[r].x;
         acc.v[r].y += ys.v[r].y;
         acc.v[r].z += ys.v[r].z;
         acc.v[r].w += ys.v[r].w;
      }
   }
   else if (OP == OP_SPMM)
   {
      axpy_slice<R>(acc, edge_val, ys);
   }
   else if (OP == OP_DOT)
   {
      const real_t s = dot_slices<L, R>(xs, ys);
      const real_t d = sop_eval(sop_kind, s, tab);
      axpy_slice<R>(acc, d, ys);
   }
   else if (OP == OP_DIST)
   {
      Slice<R> t;
      sub_slices<R>(t, xs, ys);
      const real_t s = dot_slices<L, R>(t, t);
      const real_t d = sop_eval(sop_kind, s, tab);
      axpy_slice<R>(acc, d, t);
   }
}

// The general pipeline over the U edges a sub-wave has in flight, stage by stage:
// each stage's switch on the op tuple is taken once for the batch, and inside a case
// the U edges are straight-line code (their reductions and table look-ups overlap).
// Arithmetic and order of accumulation are those of edge_step, edge 0 first; edges
// with ok[u] false change nothing.  ys[u] is overwritten with T.
template <int L, int R, int U>
__device__ __forceinline__ void general_steps(Slice<R> &acc, const Slice<R> &xs, Slice<R> *ys, const real_t *ev,
                                              const bool *ok, int sop_kind, int imsg, lds_table_t tab)
{
   const int vop = imsg & 0xF, rop = imsg & 0xF0, sop = imsg & 0xF00, vsc = imsg & 0xF000, aop = imsg & 0xF0000;
#define FMM_EACH_EDGE for (int u = 0; u < U; u++)
   switch (vop)
   {
      case kVopCopyLhs:
#pragma unroll
         FMM_EACH_EDGE ys[u] = xs;
         break;
      case kVopCopyRhs: break;
      case kVopAdd:
#pragma unroll
         FMM_EACH_EDGE map2(ys[u], xs, ys[u], [](real_t a, real_t b) { return a + b; });
         break;
      case kVopSubl:
#pragma unroll
         FMM_EACH_EDGE map2(ys[u], xs, ys[u], [](real_t a, real_t b) { return -a + b; });
         break;
      case kVopSubr:
#pragma unroll
         FMM_EACH_EDGE map2(ys[u], xs, ys[u], [](real_t a, real_t b) { return a - b; });
         break;
      case kVopMax:
#pragma unroll
         FMM_EACH_EDGE map2(ys[u], xs, ys[u], [](real_t a, real_t b) { return a > b ? a : b; });
         break;
      default:
#pragma unroll
         FMM_EACH_EDGE map2(ys[u], xs, ys[u], [](real_t a, real_t b) { return a < b ? a : b; });
         break;
   }
   real_t d[U];
#pragma unroll
   FMM_EACH_EDGE d[u] = ev[u];
   switch (rop)
   {
      case kRopDot:
#pragma unroll
         FMM_EACH_EDGE d[u] = dot_slices<L, R>(xs, ys[u]);
         break;
      case kRopAddLhs:
      {
         const real_t sx = sum_slice<L, R>(xs);
#pragma unroll
         FMM_EACH_EDGE d[u] = sx;
         break;
      }
      case kRopAddRhs:
#pragma unroll
         FMM_EACH_EDGE d[u] = sum_slice<L, R>(ys[u]);
         break;
      case kRopNormL:
      {
         const real_t nx = dot_slices<L, R>(xs, xs);
#pragma unroll
         FMM_EACH_EDGE d[u] = nx;
         break;
      }
      case kRopNormR:
#pragma unroll
         FMM_EACH_EDGE d[u] = dot_slices<L, R>(ys[u], ys[u]);
         break;
      default: break;
   }
   if (sop == kSopUdef)
   {
      switch (sop_kind)
      {
#define FMM_SOP_CASE(K_)                                 \
   case K_:                                              \
      _Pragma("unroll") FMM_EACH_EDGE d[u] = sop_eval(K_, d[u], tab); \
      break;
         FMM_SOP_CASE(SOP_SIGMOID)
         FMM_SOP_CASE(SOP_TDIST)
         FMM_SOP_CASE(SOP_FR)
         FMM_SOP_CASE(SOP_LL)
         FMM_SOP_CASE(SOP_FA)
         FMM_SOP_CASE(SOP_TDIST_PLAIN)
#undef FMM_SOP_CASE
         default: break;
      }
   }
   if (vsc == kVscMul)
   {
#pragma unroll
      FMM_EACH_EDGE
      {
#pragma unroll
         for (int r = 0; r < R; r++)
         {
            ys[u].v[r].x = d[u] * ys[u].v[r].x; ys[u].v[r].y = d[u] * ys[u].v[r].y;
            ys[u].v[r].z = d[u] * ys[u].v[r].z; ys[u].v[r].w = d[u] * ys[u].v[r].w;
         }
      }
   }
   else if (vsc == kVscAdd)
   {
#pragma unroll
      FMM_EACH_EDGE
      {
#pragma unroll
         for (int r = 0; r < R; r++)
         {
            ys[u].v[r].x = d[u] + ys[u].v[r].x; ys[u].v[r].y = d[u] + ys[u].v[r].y;
            ys[u].v[r].z = d[u] + ys[u].v[r].z; ys[u].v[r].w = d[u] + ys[u].v[r].w;
         }
      }
   }
   if (aop == kAopAdd)
   {
#pragma unroll
      FMM_EACH_EDGE map2(acc, acc, ys[u], [&](real_t a, real_t b) { return ok[u] ? a + b : a; });
   }
   else if (aop == kAopMax)
   {
#pragma unroll
      FMM_EACH_EDGE map2(acc, acc, ys[u], [&](real_t a, real_t b) { return ok[u] ? (a > b ? a : b) : a; });
   }
   else if (aop == kAopMin)
   {
#pragma unroll
      FMM_EACH_EDGE map2(acc, acc, ys[u], [&](real_t a, real_t b) { return ok[u] ? (a < b ? a : b) : a; });
   }
#undef FMM_EACH_EDGE
}

// A batch in which only the first `nu` (wave-uniform) of the U edges per sub-wave
// exist, the short last batch of a row, goes through the pipeline at half, a
// quarter, ... of the width instead of carrying empty edges through every stage.
template <int L, int R, int U>
__device__ __forceinline__ void general_group(Slice<R> &acc, const Slice<R> &xs, Slice<R> *ys, const real_t *ev,
                                              const bool *ok, int nu, int sop_kind, int imsg, lds_table_t tab)
{
   if constexpr (U >= 2)
   {
      if (nu <= U / 2)
      {
         general_group<L, R, U / 2>(acc, xs, ys, ev, ok, nu, sop_kind, imsg, tab);
         return;
      }
   }
   general_steps<L, R, U>(acc, xs, ys, ev, ok, sop_kind, imsg, tab);
}

// Whole-wave rows take the U edges in flight through the pipeline together.  Sub-waves
// take them two at a time: all at once would hold every stage's temporaries for all of
// them in registers and cost a resident workgroup per CU (measured on the K=128 sigmoid
// and K=64 t-dist benchmarks: 1.69 against 1.86 ms and 24.5 against 25.5 ms; K=256 and
// K=512 are 3 % and 1 % slower in pairs).
template <int L, int R, int U>
__device__ __forceinline__ void general_batch(Slice<R> &acc, const Slice<R> &xs, Slice<R> *ys, const real_t *ev,
                                              const bool *ok, int nu, int sop_kind, int imsg, lds_table_t tab)
{
   constexpr int G = ((L == 64 && R <= 2) || U < 2) ? U : 2;   // rows wider than 512 columns: pairs as well
#pragma unroll
   for (int g0 = 0; g0 < U; g0 += G)
      if (g0 < nu) general_group<L, R, G>(acc, xs, ys + g0, ev + g0, ok + g0, nu - g0, sop_kind, imsg, tab);
}

// 64 consecutive edge slots of a row, one per lane: column id and edge value.
template <typename IdxT>
struct EdgeChunk {
   IdxT col;
   real_t val;
};

template <int OP, typename IdxT>
__device__ __forceinline__ void load_chunk(EdgeChunk<IdxT> &c, const Params<IdxT> &p, IdxT j0, IdxT je, int lane)
{
   c.col = 0;
   c.val = (real_t)0;
   if (j0 < je && (IdxT)lane < je - j0)   // written so that an int32 slot number next to 2^31 cannot wrap
   {
      c.col = p.indx[j0 + lane];
      if ((OP == OP_SPMM || OP == OP_GENERIC) && p.val) c.val = p.val[j0 + lane];
   }
}

// Entry `e` of a chunk.  Whole-wave rows (L == 64): e is wave-uniform and the
// value lands in a scalar register (v_readlane), so the gather address is
// scalar too.  Narrower sub-waves each want a different entry: ds_bpermute.
template <int L>
__device__ __forceinline__ int32_t chunk_entry(int32_t v, int e)
{
   if (L == 64) return __builtin_amdgcn_readlane(v, e);
   return __builtin_amdgcn_ds_bpermute(e << 2, v);
}
template <int L>
__device__ __forceinline__ int64_t chunk_entry(int64_t v, int e)
{
   const int lo = chunk_entry<L>((int32_t)(v & 0xFFFFFFFFll), e);
   const int hi = chunk_entry<L>((int32_t)(v >> 32), e);
   return ((int64_t)hi << 32) | (uint32_t)lo;
}
template <int L>
__device__ __forceinline__ float chunk_entry(float v, int e)
{
   return as_f(chunk_entry<L>(as_i(v), e));
}
template <int L>
__device__ __forceinline__ double chunk_entry(double v, int e)
{
   FMM_SPLIT64(v, lo, hi);
   return join64(chunk_entry<L>(lo, e), chunk_entry<L>(hi, e));
}

// Edges [jb, je) of one row, dealt round-robin to the sub-waves.  Column ids
// (and edge values) are fetched 64 at a time with one coalesced load per
// array, the next 64 while the current ones are being used; U gathers are in
// flight per sub-wave.  All lanes of the wave call this with the same arguments.
template <int V, int L, int R, bool EXACT, int OP, int SOPK, int U, typename IdxT>
__device__ __forceinline__ void walk_edges(Slice<R> &acc, const Slice<R> &xs, const Params<IdxT> &p,
                                           IdxT jb, IdxT je, EdgeChunk<IdxT> &cur, IdxT next_b, IdxT next_e, int lane,
                                           lds_table_t tab)
{
   constexpr int S = 64 / L;
   const int sub = (L == 64) ? 0 : lane / L, sl = (L == 64) ? lane : lane % L;
   const int sop_kind = SOPK >= 0 ? SOPK : p.sop_kind;
   // On entry `cur` holds slots [jb, jb+64) (requested by the caller); on exit it
   // holds slots [next_b, next_b+64) of whatever the caller walks next, requested
   // while the last chunk of this row was being gathered.
   if (jb >= je)
   {
      load_chunk<OP, IdxT>(cur, p, next_b, next_e, lane);
      return;
   }
   for (IdxT j0 = jb; j0 < je;)
   {
      EdgeChunk<IdxT> nxt;
      const IdxT left = je - j0;          // > 0; comparisons on differences: no wrap next to 2^31
      if (left > 64) load_chunk<OP, IdxT>(nxt, p, j0 + 64, je, lane);
      else load_chunk<OP, IdxT>(nxt, p, next_b, next_e, lane);
      const int n = left < 64 ? (int)left : 64;
      for (int b0 = 0; b0 < n; b0 += S * U)
      {
         IdxT col[U];
         real_t ev[U];
         bool ok[U];
         Slice<R> ys[U];
#pragma unroll
         for (int u = 0; u < U; u++)
         {
            const int e = b0 + u * S + sub;     // L == 64: sub == 0, e is uniform
            ok[u] = e < n;
            col[u] = chunk_entry<L>(cur.col, e & 63);
            ev[u] = (OP == OP_SPMM || OP == OP_GENERIC) ? chunk_entry<L>(cur.val, e & 63) : (real_t)0;
         }
#pragma unroll
         for (int u = 0; u < U; u++)
         {
            if (ok[u]) load_slice<V, L, R, EXACT>(ys[u], p.y + (int64_t)col[u] * p.ldy, sl, p.k);
            else if (OP == OP_GENERIC)
            {
#pragma unroll
               for (int r = 0; r < R; r++) ys[u].v[r] = zero4();
            }
         }
         if constexpr (OP == OP_GENERIC)
         {
            const int in_batch = n - b0;      // > 0; edges e = b0 + u*S + sub of this batch exist for e < n
            const int nu = in_batch >= S * U ? U : (in_batch + S - 1) / S;
            general_batch<L, R, U>(acc, xs, ys, ev, ok, nu, sop_kind, p.imessage, tab);
         }
         else
         {
#pragma unroll
            for (int u = 0; u < U; u++)
               if (ok[u]) edge_step<L, R, OP>(acc, xs, ys[u], ev[u], sop_kind, tab);
         }
      }
      cur = nxt;
      if (left <= 64) break;
      j0 += 64;
   }
}

template <int L, int R, int OP>
__device__ __forceinline__ void merge_subwaves(Slice<R> &acc, int imsg)
{
   if (L == 64) return;
   const int aop = imsg & 0xF0000;
#pragma unroll
   for (int r = 0; r < R; r++)
   {
      if (OP == OP_GENERIC && aop == kAopMax)
      {
         acc.v[r].x = cross_subwave_max<L>(acc.v[r].x); acc.v[r].y = cross_subwave_max<L>(acc.v[r].y);
         acc.v[r].z = cross_subwave_max<L>(acc.v[r].z); acc.v[r].w = cross_subwave_max<L>(acc.v[r].w);
      }
      else if (OP == OP_GENERIC && aop == kAopMin)
      {
         acc.v[r].x = cross_subwave_min<L>(acc.v[r].x); acc.v[r].y = cross_subwave_min<L>(acc.v[r].y);
         acc.v[r].z = cross_subwave_min<L>(acc.v[r].z); acc.v[r].w = cross_subwave_min<L>(acc.v[r].w);
      }
      else
      {
         acc.v[r].x = cross_subwave_sum<L>(acc.v[r].x); acc.v[r].y = cross_subwave_sum<L>(acc.v[r].y);
         acc.v[r].z = cross_subwave_sum<L>(acc.v[r].z); acc.v[r].w = cross_subwave_sum<L>(acc.v[r].w);
      }
   }
}

template <int OP>
__device__ __forceinline__ bool op_reads_x(int imsg)
{
   if (OP == OP_DOT || OP == OP_DIST) return true;
   if (OP == OP_GENERIC)
   {
      const int vop = imsg & 0xF, rop = imsg & 0xF0;
      return vop != kVopCopyRhs || rop == kRopDot || rop == kRopAddLhs || rop == kRopNormL;
   }
   return false;
}

__device__ __forceinline__ lds_table_t stage_table(const real_t *gtab, real_t *lds, bool need)
{
   if (need)
   {
      for (int i = threadIdx.x; i < kSigmoidTableSize; i += kBlockThreads) lds[i] = gtab[i];
      __syncthreads();
   }
   return (lds_table_t)lds;      // read only when `need` held
}

// ---- finished Z rows leave together -----------------------------------------------
// A finished row of Z is one store of 128 bytes to a few KiB, and on rows of a few dozen
// edges such stores are a twentieth of the bytes a call moves.  Sent out one by one as
// rows finish they reach the memory system as a thin, steady trickle between random
// reads, and cost it several times their share (a 16-edge graph at K=512: 4 GB of Z took
// as long as 23 GB of gathers).  So finished rows wait in LDS, and every wavefront of
// the grid sends its waiting rows when the same clock tick passes: the device's constant
// 100 MHz counter (s_memrealtime, one counter for all compute dies) shifted right by
// store_shift.  The stores of the whole grid then arrive in bursts a few microseconds
// long, once per period, with nothing but reads in between; what is summed, and in which
// order, does not change.  A wavefront whose LDS share fills up before the tick sends
// early.  Each wavefront has its share of the workgroup's dynamic LDS, in slots of one sub-wave row (L lanes x
// R registers) followed by the slots' destinations.  Rows to be cleared (empty rows under the
// overwrite rule) need no slot, only their address.
constexpr int kClearList = 32;          // rows waiting to be cleared, per wavefront

// What a wavefront carries from row to row is four scalars; where its slots and lists lie is worked out from the
// kernel's arguments when a row is put down or the rows go out (scalar registers are the scarce kind in this kernel).
struct RowStage {
   int cap;             // slots this wavefront has; 0: rows are stored as they finish
   int n, nclear;       // slots in use, rows to clear
   unsigned int tick;   // clock >> store_shift at the last look
};                      // (every member is wave-uniform)

extern __shared__ __attribute__((aligned(32))) unsigned char fmm_dynamic_lds[];

// Registers (real4) per slot: L*R, or only those that hold elements of the row when K is not a multiple of 4*L
// (16-byte layout: register r of lane sl is element-vector r*L + sl; vectors past the row's end hold nothing).
template <int V, int L, int R, bool EXACT, typename IdxT>
__device__ __forceinline__ int stage_width(const Params<IdxT> &p)
{
   return (V == 4 && !EXACT) ? (p.k + 3) / 4 : L * R;
}
// This wavefront's share of the staging area: cap slots, then where each slot goes (nullptr: nowhere), then the
// rows waiting to be cleared.
template <typename IdxT>
__device__ __forceinline__ real4 *stage_slots(const Params<IdxT> &p)
{
   const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
   return reinterpret_cast<real4 *>(fmm_dynamic_lds) + wave * p.stage_vecs;
}
template <int V, int L, int R, bool EXACT, typename IdxT>
__device__ __forceinline__ real_t **stage_to(const Params<IdxT> &p, const RowStage &st)
{
   return reinterpret_cast<real_t **>(stage_slots<IdxT>(p) + st.cap * stage_width<V, L, R, EXACT, IdxT>(p));
}

// The staging area is the workgroup's dynamic LDS: stage_vecs registers' worth (real4) per wavefront, sized by
// the host to what the CU's LDS leaves each resident workgroup.
template <int V, int L, int R, bool EXACT, bool STAGED, typename IdxT>
__device__ __forceinline__ void stage_begin(RowStage &st, const Params<IdxT> &p)
{
   constexpr int S = 64 / L;
   if constexpr (!STAGED)
   {
      st.cap = 0;
      st.n = 0;
      st.nclear = 0;
      st.tick = 0u;
      return;
   }
   const int share = p.stage_vecs * (int)sizeof(real4);
   int cap = (share - kClearList * (int)sizeof(real_t *)) /
             (stage_width<V, L, R, EXACT, IdxT>(p) * (int)sizeof(real4) + (int)sizeof(real_t *));
   cap = cap > 64 ? 64 : cap;
   st.cap = (p.store_shift > 0 && cap >= 2 * S) ? cap : 0;     // room for two rows, or two packed groups, at least
   st.n = 0;
   st.nclear = 0;
   st.tick = st.cap ? (unsigned int)(__builtin_amdgcn_s_memrealtime() >> p.store_shift) : 0u;
}

template <int V, int L, int R, bool EXACT, typename IdxT>
__device__ __forceinline__ void stage_flush(RowStage &st, const Params<IdxT> &p, int lane)
{
   constexpr int S = 64 / L;
   const int sub = (L == 64) ? 0 : lane / L, sl = (L == 64) ? lane : lane % L;
   const int width = stage_width<V, L, R, EXACT, IdxT>(p);
   const real4 *slots = stage_slots<IdxT>(p);
   real_t *const *to_list = stage_to<V, L, R, EXACT, IdxT>(p, st);
   real_t *const *clear_list = to_list + st.cap;
   __builtin_amdgcn_wave_barrier();
   for (int i = 0; i < st.n; i += S)
   {
      const int slot = i + sub;
      if (slot < st.n)
      {
         real_t *to = to_list[slot];
         if (to)
         {
            Slice<R> row;
#pragma unroll
            for (int r = 0; r < R; r++)
               row.v[r] = (V != 4 || EXACT || r * L + sl < width) ? slots[slot * width + r * L + sl] : zero4();
            store_slice<V, L, R, EXACT, true>(to, row, sl, p.k);
         }
      }
   }
   for (int i = 0; i < st.nclear; i += S)
   {
      const int at = i + sub;
      if (at < st.nclear)
      {
         Slice<R> zero;
#pragma unroll
         for (int r = 0; r < R; r++) zero.v[r] = zero4();
         store_slice<V, L, R, EXACT, true>(clear_list[at], zero, sl, p.k);
      }
   }
   __builtin_amdgcn_wave_barrier();
   st.n = 0;
   st.nclear = 0;
}

// Has the tick passed?  Then everything waiting goes out.  `clock` is a reading of the 100 MHz counter.
template <int V, int L, int R, bool EXACT, typename IdxT>
__device__ __forceinline__ void stage_tick(RowStage &st, const Params<IdxT> &p, unsigned long long clock, int lane)
{
   if (st.cap == 0) return;
   const unsigned int now = (unsigned int)(clock >> p.store_shift);
   if (now != st.tick)
   {
      if (st.n | st.nclear) stage_flush<V, L, R, EXACT, IdxT>(st, p, lane);
      st.tick = now;
   }
}

// One finished row, held by the wavefront's first sub-wave; zrow is wave-uniform.
template <int V, int L, int R, bool EXACT, typename IdxT>
__device__ __forceinline__ void stage_row(RowStage &st, const Params<IdxT> &p, real_t *zrow, const Slice<R> &acc, int lane)
{
   const int sub = (L == 64) ? 0 : lane / L, sl = (L == 64) ? lane : lane % L;
   if (st.cap == 0)
   {
      if (sub == 0) store_slice<V, L, R, EXACT, true>(zrow, acc, sl, p.k);
      return;
   }
   if (st.n >= st.cap) stage_flush<V, L, R, EXACT, IdxT>(st, p, lane);   // (a packed group may have filled the last slot)
   const int width = stage_width<V, L, R, EXACT, IdxT>(p);
   real4 *slots = stage_slots<IdxT>(p);
   if (sub == 0)
   {
#pragma unroll
      for (int r = 0; r < R; r++)
         if (V != 4 || EXACT || r * L + sl < width) slots[st.n * width + r * L + sl] = acc.v[r];
   }
   if (lane == 0) stage_to<V, L, R, EXACT, IdxT>(p, st)[st.n] = zrow;
   st.n++;
}

// One row per sub-wave (a packed group): sub-wave s holds a row for `zrow` (its own; nullptr: nothing to store).
template <int V, int L, int R, bool EXACT, typename IdxT>
__device__ __forceinline__ void stage_group(RowStage &st, const Params<IdxT> &p, real_t *zrow, const Slice<R> &acc, int lane)
{
   constexpr int S = 64 / L;
   const int sub = lane / L, sl = lane % L;
   if (st.cap == 0)
   {
      if (zrow) store_slice<V, L, R, EXACT, true>(zrow, acc, sl, p.k);
      return;
   }
   if (st.n + S > st.cap) stage_flush<V, L, R, EXACT, IdxT>(st, p, lane);
   const int width = stage_width<V, L, R, EXACT, IdxT>(p);
   real4 *slots = stage_slots<IdxT>(p);
   const int slot = st.n + sub;
#pragma unroll
   for (int r = 0; r < R; r++)
      if (V != 4 || EXACT || r * L + sl < width) slots[slot * width + r * L + sl] = acc.v[r];
   if (sl == 0) stage_to<V, L, R, EXACT, IdxT>(p, st)[slot] = zrow;
   st.n += S;
}

// An empty row under the overwrite rule: to be cleared; zrow is wave-uniform.
template <int V, int L, int R, bool EXACT, typename IdxT>
__device__ __forceinline__ void stage_clear(RowStage &st, const Params<IdxT> &p, real_t *zrow, int lane)
{
   const int sub = (L == 64) ? 0 : lane / L, sl = (L == 64) ? lane : lane % L;
   if (st.cap == 0)
   {
      if (sub == 0)
      {
         Slice<R> zero;
#pragma unroll
         for (int r = 0; r < R; r++) zero.v[r] = zero4();
         store_slice<V, L, R, EXACT, true>(zrow, zero, sl, p.k);
      }
      return;
   }
   if (st.nclear >= kClearList) stage_flush<V, L, R, EXACT, IdxT>(st, p, lane);
   if (lane == 0) (stage_to<V, L, R, EXACT, IdxT>(p, st) + st.cap)[st.nclear] = zrow;
   st.nclear++;
}

// ---- short rows, one per sub-wave --------------------------------------------------
// A wavefront walks a row with all its S = 64/L sub-waves: S*U edges are gathered at a
// time.  Rows much shorter than that leave most of those gathers unused (a 16-edge row
// at K=32 fills 16 of 64), and every row pays its own round of pointer, column-id and
// store latency.  So a group of S consecutive rows (row ids g*S .. g*S+S-1, inside one
// claim) whose longest row has  md <= S*U  edges and  ceil(md / U) <= (rows of the group
// that have edges)  is walked with one row per sub-wave instead: the sub-wave gathers its
// own row's edges U at a time, in edge order, into its own accumulator; nothing is merged
// across sub-waves, and the S rows of X and Z are read and written as one contiguous
// piece.  The rule compares the batches each way costs (ceil(md/U) against one per
// non-empty row) and depends on the row pointers only, so the CPU oracle applies the same
// rule; for such a row the sum runs over its edges in order in ONE accumulator (the
// oracle's wavefront order with S = 1).
template <int L, int U>
__device__ __forceinline__ bool packs(int64_t md, int nz, int64_t heavy_deg)
{
   constexpr int S = 64 / L;
   return nz > 0 && md <= (int64_t)(S * U) && md <= heavy_deg && (md + U - 1) / U <= (int64_t)nz;
}

// The group of S rows starting at `row_first` (wave-uniform), sub-wave s taking row
// row_first + s with edge slots [jb, je) (per sub-wave; empty for rows past m), md the
// longest row of the group.  All lanes of the wave call this together.
template <int V, int L, int R, bool EXACT, int OP, int SOPK, int U, typename IdxT>
__device__ __forceinline__ void packed_group(const Params<IdxT> &p, int64_t row_first, IdxT jb, IdxT je, int md, int lane,
                                             lds_table_t tab, RowStage &st)
{
   static_assert(L == 8 || L == 16, "sub-waves of 8 or 16 lanes");
   constexpr int P = 16 / L;                 // column ids a lane holds per fetch: 16 ids per sub-wave and fetch
   constexpr bool generic = (OP == OP_GENERIC);
   constexpr bool uses_val = (OP == OP_SPMM || OP == OP_GENERIC);
   const int sl = lane % L, base = lane - sl;
   const int64_t row = row_first + lane / L;
   const int deg = (int)(je - jb);           // <= S*U; 0 for empty rows and rows past m
   const int sop_kind = SOPK >= 0 ? SOPK : p.sop_kind;
   const bool reads_x = op_reads_x<OP>(p.imessage);
   const int aop = p.imessage & 0xF0000;
   real_t *zrow = p.z + row * p.ldz;

   // ids [c0, c0 + 16) of the sub-wave's row: lane sl holds id c0 + sl (and c0 + 8 + sl when L == 8)
   IdxT ids[P];
   real_t vals[P];
   auto fetch = [&](int c0, IdxT *id_out, real_t *val_out) {
#pragma unroll
      for (int q = 0; q < P; q++)
      {
         const int e = c0 + q * L + sl;
         id_out[q] = 0;
         val_out[q] = (real_t)0;
         if (e < deg)
         {
            id_out[q] = p.indx[jb + (IdxT)e];
            if (uses_val && p.val) val_out[q] = p.val[jb + (IdxT)e];
         }
      }
   };
   fetch(0, ids, vals);

   Slice<R> xs, acc;
   if (reads_x && deg > 0) load_slice<V, L, R, EXACT, true>(xs, p.x + row * p.ldx, sl, p.k);
   else
   {
#pragma unroll
      for (int r = 0; r < R; r++) xs.v[r] = zero4();
   }
   if (generic && deg > 0) load_slice<V, L, R, EXACT>(acc, zrow, sl, p.k);   // general rule: fold into the caller's Z
   else
   {
#pragma unroll
      for (int r = 0; r < R; r++) acc.v[r] = zero4();
   }

   for (int c0 = 0; c0 < md; c0 += 16)
   {
      IdxT nids[P];
      real_t nvals[P];
      if (c0 + 16 < md) fetch(c0 + 16, nids, nvals);     // wave-uniform: the next 16 ids while these are used
      auto batch = [&](int b) {
         if (c0 + b < md)                                 // wave-uniform
         {
         IdxT col[U];
         real_t ev[U];
         bool ok[U];
         Slice<R> ys[U];
#pragma unroll
         for (int u = 0; u < U; u++)
         {
            const int i = b + u;                          // id i of the 16 fetched: register i / L, lane i % L
            ok[u] = c0 + i < deg;
            // (a select, not an indexed array: where the general pipeline keeps this loop rolled, b is not a constant)
            const IdxT id_reg = (P == 1 || i < L) ? ids[0] : ids[P - 1];
            const real_t val_reg = (P == 1 || i < L) ? vals[0] : vals[P - 1];
            col[u] = chunk_entry<L>(id_reg, base + i % L);
            ev[u] = uses_val ? chunk_entry<L>(val_reg, base + i % L) : (real_t)0;
         }
#pragma unroll
         for (int u = 0; u < U; u++)
         {
            if (ok[u]) load_slice<V, L, R, EXACT>(ys[u], p.y + (int64_t)col[u] * p.ldy, sl, p.k);
            else if (generic)
            {
#pragma unroll
               for (int r = 0; r < R; r++) ys[u].v[r] = zero4();
            }
         }
         if constexpr (generic)
         {
            const int left = md - (c0 + b);               // wave-uniform: the longest row's edges from here on
            general_batch<L, R, U>(acc, xs, ys, ev, ok, left >= U ? U : left, sop_kind, p.imessage, tab);
         }
         else
         {
#pragma unroll
            for (int u = 0; u < U; u++)
               if (ok[u]) edge_step<L, R, OP>(acc, xs, ys[u], ev[u], sop_kind, tab);
         }
         }
      };
      if constexpr (generic)
      {
         for (int b = 0; b < 16; b += U) batch(b);        // the general pipeline's stages are large: kept as a loop
      }
      else
      {
#pragma unroll
         for (int b = 0; b < 16; b += U) batch(b);
      }
      if (c0 + 16 < md)
      {
#pragma unroll
         for (int q = 0; q < P; q++) { ids[q] = nids[q]; vals[q] = nvals[q]; }
      }
   }

   bool stores;
   if (deg > 0)
   {
      stores = !(generic && aop == kAopNoop);             // no accumulate stage: Z is left alone
      if (!generic && !p.beta_zero)
      {
         Slice<R> zin;
         load_slice<V, L, R, EXACT>(zin, zrow, sl, p.k);
         map2(acc, zin, acc, [](real_t a, real_t b) { return a + b; });
      }
   }
   else stores = !generic && p.beta_zero && row < p.m;    // empty row under the overwrite rule: zeros
   stage_group<V, L, R, EXACT, IdxT>(st, p, stores ? zrow : nullptr, acc, lane);
}

// Does the row phase take the stretches of 64 chunks in scattered order?  When rows are claimed dynamically,
// there are stretches to permute, and one half of the row space holds more than 1.25 times the other's
// edges (the classify kernel's sample; 1.0 +- a few per cent where degrees do not follow the row id).
template <typename IdxT>
__device__ __forceinline__ bool scattered_order(const Params<IdxT> &p)
{
   const int64_t nchunks = (p.m + kRowsPerClaim - 1) / kRowsPerClaim;
   const unsigned long long skew = p.ctr->skew;
   const unsigned long long e_lo = skew & 0xFFFFFFFFull, e_hi = skew >> 32;
   if (p.row_counters <= 0 || (nchunks >> 6) <= 1 || p.row_order == 1) return false;
   return p.row_order == 2 || 4 * e_lo > 5 * e_hi || 4 * e_hi > 5 * e_lo;
}

// Turn the value an atomicAdd on counter `cur` returned (in lane 0) into a
// chunk id, moving to another counter when this one is used up.  Returns -1
// when every counter is used up; counters only grow, so every wave gets there.
template <typename IdxT>
__device__ __forceinline__ int64_t resolve_claim(const Params<IdxT> &p, unsigned long long claimed, int &cur, int nc,
                                                 int64_t nchunks, int lane)
{
   for (;;)
   {
      const int64_t t = wave_uniform<int64_t>((int64_t)claimed);
      const unsigned int mix = ((unsigned int)t * 2654435761u) >> 26;
      const int64_t id = t * nc + (int64_t)((cur ^ mix) & (unsigned)(nc - 1));
      if (id < nchunks) return id;
      if (nc == 1) return -1;
      // counter `cur` is spent (an id past the end can only occur in its last round)
      unsigned long long seen = ~0ull;
      if (lane < nc) seen = __hip_atomic_load(&p.ctr->rows[lane].next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool has = lane < nc && (int64_t)seen * nc < nchunks;
      const unsigned long long mask = __ballot(has);
      if (mask == 0) return -1;
      const int sh = (cur + 1) & 63;
      const unsigned long long rot = sh ? ((mask >> sh) | (mask << (64 - sh))) : mask;
      cur = (sh + __builtin_ctzll(rot)) & 63;
      claimed = 0;
      if (lane == 0) claimed = atomicAdd(&p.ctr->rows[cur].next, 1ull);
   }
}

// ---- kernel 1: put heavy rows on the queue -----------------------------------------
// One thread per row; reads the row pointers only.  A row with more than
// heavy_deg edges gets a HeavyRow entry and one SegDesc per segment (at most
// kMaxSegsPerRow: hub rows get longer segments) and its bit in `queued` is set.
// When the queue is full the row is left for phase B to process whole.
//
// Queue entries are handed out by a 64-bit read-modify-write on n_heavy (low word)
// and n_seg (high word), which advance together.  Read-modify-writes on that one
// cache line retire one per ~12 ns however many CUs issue them (13 000 heavy rows of
// an R-MAT graph taking it one by one: 0.2 ms; one per wavefront and 64 rows: 0.15 ms),
// so a workgroup first collects the heavy rows among all the rows it looks at in LDS
// and then takes the counters once for all of them.
constexpr int kClassifyList = 512;   // heavy rows a workgroup collects; more are queued one by one

template <typename IdxT>
__device__ __forceinline__ unsigned int segments_of(const Params<IdxT> &p, int64_t deg, int64_t *seg_len_out)
{
   int64_t seg_len = p.seg_len;
   if (deg > seg_len * (int64_t)kMaxSegsPerRow) seg_len = (deg + kMaxSegsPerRow - 1) / kMaxSegsPerRow;
   *seg_len_out = seg_len;
   return (unsigned int)((deg + seg_len - 1) / seg_len);
}

// Entry `slot` of the heavy-row queue and its segment descriptors [base, base + nseg), written by the
// threads tid, tid + nthreads, ... of the caller's group; or, when the queue is full, the entry
// poisoned (the merge kernel skips n_seg == 0; every queue entry below the cap has exactly one writer).
template <typename IdxT>
__device__ __forceinline__ void write_queue_entry(const Params<IdxT> &p, unsigned int slot, unsigned int base, unsigned int nseg,
                                                  int64_t row, int64_t jb, int64_t deg, int64_t seg_len, int tid, int nthreads)
{
   if (slot < p.cap_heavy && (uint64_t)base + nseg <= (uint64_t)p.cap_seg)
   {
      if (tid == 0)
      {
         p.heavy[slot] = HeavyRow{row, base, nseg};
         atomicOr(&p.queued[row >> 5], 1u << (row & 31));
      }
      for (unsigned int s = (unsigned int)tid; s < nseg; s += (unsigned int)nthreads)
      {
         const int64_t off = (int64_t)s * seg_len;
         const int64_t cnt = deg - off < seg_len ? deg - off : seg_len;
         p.segs[base + s] = SegDesc{row, jb + off, (unsigned int)cnt, 0u};
      }
   }
   else
   {
      if (tid == 0)
      {
         if (slot < p.cap_heavy) p.heavy[slot] = HeavyRow{row, 0u, 0u};
         atomicAdd(&p.ctr->overflow, 1u);
      }
      for (uint64_t s = (uint64_t)base + (unsigned int)tid; s < (uint64_t)base + nseg && s < (uint64_t)p.cap_seg; s += (unsigned int)nthreads)
         p.segs[s] = SegDesc{-1, 0, 0u, 0u};
   }
}

template <typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void classify_kernel(const Params<IdxT> p)
{
   __shared__ int64_t l_row[kClassifyList], l_jb[kClassifyList], l_deg[kClassifyList];
   __shared__ unsigned int l_base[kClassifyList];
   __shared__ unsigned int l_scan[kBlockThreads];
   __shared__ unsigned int l_count;
   __shared__ unsigned long long l_before;
   const int tid = threadIdx.x, lane = threadIdx.x & 63;
   const int64_t stride = (int64_t)gridDim.x * kBlockThreads;
   unsigned long long *both = reinterpret_cast<unsigned long long *>(&p.ctr->n_heavy);
   __shared__ unsigned long long l_edges[2];   // edges of this workgroup's rows in the lower / upper half of the row space
   if (tid == 0) { l_count = 0u; l_edges[0] = 0ull; l_edges[1] = 0ull; }
   __syncthreads();
   // 32 workgroups spread evenly over the grid (all of a small grid) report where the edges of their rows lie
   const unsigned int sample_step = gridDim.x >= 64u ? gridDim.x / 32u : 1u;
   const bool sampled = blockIdx.x % sample_step == 0u;
   unsigned long long edges_lo = 0ull, edges_hi = 0ull;

   // A wavefront that finds many heavy rows among its 64 (R-MAT degrees follow the bits
   // of the row id, so they come in runs) takes the counters for all of them at once;
   // a few here and there go on the workgroup's list.  All lanes call this together.
   auto wave_takes_counters = [&](int64_t row, int64_t jb, int64_t deg, bool heavy, unsigned long long mask) {
      int64_t seg_len = p.seg_len;
      const unsigned int nseg = heavy ? segments_of(p, deg, &seg_len) : 0u;
      unsigned int incl = nseg;                                    // inclusive prefix sum of nseg over the lanes
#pragma unroll
      for (int d = 1; d < 64; d <<= 1)
      {
         const unsigned int up = __shfl_up(incl, d, 64);
         if (lane >= d) incl += up;
      }
      const unsigned int total = __shfl(incl, 63, 64);
      const int leader = __builtin_ctzll(mask);
      unsigned long long before = 0ull;
      if (lane == leader)
         before = atomicAdd(both, (unsigned long long)__builtin_popcountll(mask) | ((unsigned long long)total << 32));
      before = __shfl(before, leader, 64);
      if (!heavy) return;
      const unsigned int slot = (unsigned int)(before & 0xFFFFFFFFull) + (unsigned int)__builtin_popcountll(mask & ((1ull << lane) - 1ull));
      write_queue_entry(p, slot, (unsigned int)(before >> 32) + (incl - nseg), nseg, row, jb, deg, seg_len, 0, 1);
   };
   constexpr int kManyInAWave = 8;

   // four rows per thread and turn, their pointers requested together; the turn's
   // bounds are the wave's (its first lane's row), so that every lane takes part in
   // the wave-wide steps
   constexpr int kRowsPerTurn = 4;
   for (int64_t row0 = (int64_t)blockIdx.x * kBlockThreads + tid; row0 - lane < p.m; row0 += kRowsPerTurn * stride)
   {
      IdxT jb[kRowsPerTurn], je[kRowsPerTurn];
#pragma unroll
      for (int i = 0; i < kRowsPerTurn; i++)
      {
         const int64_t row = row0 + i * stride;
         jb[i] = row < p.m ? p.pntrb[row] : (IdxT)0;
         je[i] = row < p.m ? p.pntre[row] : (IdxT)0;
      }
#pragma unroll
      for (int i = 0; i < kRowsPerTurn; i++)
      {
         const int64_t row = row0 + i * stride;
         const int64_t deg = (int64_t)je[i] - (int64_t)jb[i];
         if (sampled && deg > 0 && deg <= p.heavy_deg)              // rows the row phase will walk
         {
            const bool upper = 2 * row >= p.m;
            edges_lo += upper ? 0ull : (unsigned long long)deg;
            edges_hi += upper ? (unsigned long long)deg : 0ull;
         }
         const bool heavy = deg > p.heavy_deg;
         const unsigned long long mask = __ballot(heavy);
         if (mask == 0ull) continue;                               // wave-uniform
         const int found = __builtin_popcountll(mask);
         bool listed = false;
         if (found < kManyInAWave)
         {
            const int leader = __builtin_ctzll(mask);
            unsigned int at0 = 0xFFFFFFFFu;
            if (lane == leader)
            {
               unsigned int seen = l_count;
               while (seen + (unsigned int)found <= (unsigned int)kClassifyList)
               {
                  const unsigned int was = atomicCAS(&l_count, seen, seen + (unsigned int)found);
                  if (was == seen) { at0 = seen; break; }
                  seen = was;
               }
            }
            at0 = (unsigned int)__shfl((int)at0, leader, 64);
            if (at0 != 0xFFFFFFFFu)                                // room on the list
            {
               if (heavy)
               {
                  const unsigned int at = at0 + (unsigned int)__builtin_popcountll(mask & ((1ull << lane) - 1ull));
                  l_row[at] = row; l_jb[at] = (int64_t)jb[i]; l_deg[at] = deg;
               }
               listed = true;
            }
         }
         if (!listed) wave_takes_counters(row, (int64_t)jb[i], deg, heavy, mask);
      }
   }
   if (sampled)
   {
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1)                            // wave sums, then one LDS update per wave
      {
         edges_lo += (unsigned long long)__shfl_xor((long long)edges_lo, d, 64);
         edges_hi += (unsigned long long)__shfl_xor((long long)edges_hi, d, 64);
      }
      if (lane == 0 && edges_lo) atomicAdd(&l_edges[0], edges_lo);
      if (lane == 0 && edges_hi) atomicAdd(&l_edges[1], edges_hi);
   }
   __syncthreads();
   if (sampled && tid == 0)
   {
      // both halves in one word, scaled down so that neither can wrap
      const unsigned long long lo = l_edges[0] >> 6, hi = l_edges[1] >> 6;
      if (lo | hi) atomicAdd(&p.ctr->skew, (lo & 0xFFFFFFFFull) | (hi << 32));
   }
   const unsigned int n = l_count;                                 // <= kClassifyList
   if (n == 0u) return;                                            // uniform over the workgroup

   // thread tid owns entries kPerThread * tid + i; exclusive prefix of their segment counts over the list
   constexpr int kPerThread = kClassifyList / kBlockThreads;
   unsigned int mine[kPerThread], sum = 0u;
#pragma unroll
   for (int i = 0; i < kPerThread; i++)
   {
      const unsigned int e = (unsigned int)(tid * kPerThread + i);
      int64_t seg_len;
      mine[i] = e < n ? segments_of(p, l_deg[e], &seg_len) : 0u;
      sum += mine[i];
   }
   l_scan[tid] = sum;
   __syncthreads();
   for (int d = 1; d < kBlockThreads; d <<= 1)                     // inclusive scan of the threads' sums
   {
      const unsigned int add = tid >= d ? l_scan[tid - d] : 0u;
      __syncthreads();
      l_scan[tid] += add;
      __syncthreads();
   }
   if (tid == kBlockThreads - 1) l_before = atomicAdd(both, (unsigned long long)n | ((unsigned long long)l_scan[tid] << 32));
   __syncthreads();
   const unsigned int slot0 = (unsigned int)(l_before & 0xFFFFFFFFull), base0 = (unsigned int)(l_before >> 32);
   {
      unsigned int b = base0 + l_scan[tid] - sum;                  // first segment slot of this thread's first entry
#pragma unroll
      for (int i = 0; i < kPerThread; i++)
      {
         const unsigned int e = (unsigned int)(tid * kPerThread + i);
         if (e < n) l_base[e] = b;
         b += mine[i];
      }
   }
   __syncthreads();
   // an entry per wavefront at a time, its segment descriptors dealt to the lanes
   for (unsigned int e = (unsigned int)(tid >> 6); e < n; e += (unsigned int)kWavesPerBlock)
   {
      int64_t seg_len;
      const unsigned int nseg = segments_of(p, l_deg[e], &seg_len);
      write_queue_entry(p, slot0 + e, l_base[e], nseg, l_row[e], l_jb[e], l_deg[e], seg_len, lane, 64);
   }
}

// ---- phase A of the fused kernel: one wavefront per queued edge segment -> partial Z ----
template <int V, int L, int R, bool EXACT, int OP, int SOPK, int U, typename IdxT>
__device__ __forceinline__ void segments_phase(const Params<IdxT> &p, lds_table_t tab)
{
   unsigned int nseg = p.ctr->n_seg;
   if (nseg > p.cap_seg) nseg = p.cap_seg;   // rows beyond the cap are done whole in phase B
   if (nseg == 0) return;

   const int lane = threadIdx.x & 63;
   const int sub = lane / L, sl = lane % L;
   const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
   const bool reads_x = op_reads_x<OP>(p.imessage);
   const int aop = p.imessage & 0xF0000;

   // Segments are dealt round-robin to the waves, so the next one is known: its
   // descriptor is fetched while the current segment is walked, and its first 64
   // column ids while the current segment's last chunk is gathered.
   auto fetch_desc = [&](int64_t q) -> SegDesc {
      if (q < (int64_t)nseg) return p.segs[q];
      return SegDesc{-1, 0, 0u, 0u};
   };
   SegDesc sd = fetch_desc(wave0);
   EdgeChunk<IdxT> chunk;
   {
      const IdxT b0 = (IdxT)wave_uniform<int64_t>(sd.first);
      const IdxT n0 = (IdxT)__builtin_amdgcn_readfirstlane((int)sd.count);
      load_chunk<OP, IdxT>(chunk, p, b0, b0 + n0, lane);
   }
   for (int64_t q = wave0; q < (int64_t)nseg; q += nwaves)
   {
      const int64_t row = wave_uniform<int64_t>(sd.row);
      const IdxT jb = (IdxT)wave_uniform<int64_t>(sd.first);
      const IdxT je = jb + (IdxT)__builtin_amdgcn_readfirstlane((int)sd.count);
      const SegDesc sdn = fetch_desc(q + nwaves);
      if (row < 0)
      {
         // slot of a row that was handled inline: nothing to do but keep the pipeline fed
         const IdxT nb = (IdxT)wave_uniform<int64_t>(sdn.first);
         load_chunk<OP, IdxT>(chunk, p, nb, nb + (IdxT)__builtin_amdgcn_readfirstlane((int)sdn.count), lane);
         sd = sdn;
         continue;
      }

      Slice<R> xs, acc;
      if (reads_x) load_slice<V, L, R, EXACT, true>(xs, p.x + row * p.ldx, sl, p.k);
      else
      {
#pragma unroll
         for (int r = 0; r < R; r++) xs.v[r] = zero4();
      }
      const real_t id = (OP == OP_GENERIC) ? aop_identity(aop) : (real_t)0;
#pragma unroll
      for (int r = 0; r < R; r++) acc.v[r] = real4{id, id, id, id};

      // the descriptor of the next segment was requested before this walk's first
      // gather, so it has arrived by the time the walk asks for the next chunk
      // (kept per-lane, not made wave-uniform here: that would wait for it now)
      const IdxT nb = (IdxT)sdn.first;
      const IdxT ne = nb + (IdxT)sdn.count;
      walk_edges<V, L, R, EXACT, OP, SOPK, U, IdxT>(acc, xs, p, jb, je, chunk, nb, ne, lane, tab);
      merge_subwaves<L, R, OP>(acc, p.imessage);

      if (sub == 0) store_slice<V, L, R, EXACT>(p.partial + (int64_t)q * p.kpad, acc, sl, p.k);
      sd = sdn;
   }
}


// ---- phase B of the fused kernel: one wavefront per row ---------------------------
template <int V, int L, int R, bool EXACT, int OP, int SOPK, int U, typename IdxT>
__device__ __forceinline__ void rows_phase(const Params<IdxT> &p, lds_table_t tab)
{
   // (the general pipeline's instances write rows as they finish: their large bodies lost 10 % to the added state and
   // code -- general sigmoid K=128: 1.52 -> 1.68 ms -- and they are not the instances anyone runs at scale)
   RowStage st;
   stage_begin<V, L, R, EXACT, OP != OP_GENERIC, IdxT>(st, p);
   const int lane = threadIdx.x & 63;
   const int sub = lane / L, sl = lane % L;
   const bool reads_x = op_reads_x<OP>(p.imessage);
   const int aop = p.imessage & 0xF0000;
   const bool generic = (OP == OP_GENERIC);

   // Rows are claimed dynamically in chunks of kRowsPerClaim: degree-skewed
   // graphs (R-MAT, power law) leave any static row -> wave map unbalanced.
   // Counter c hands out, in round t, chunk  t * nc + ((c ^ mix(t)) & (nc-1)):
   // every chunk has one owner, and a counter's chunks do not share row-id
   // bits (R-MAT degrees depend on them).  A wave drains its home counter,
   // then looks at all counters with one vector load and moves to the next one
   // that still has chunks.  The next claim is issued before the current rows
   // are walked, so its latency is hidden.
   // Small inputs (no more chunks than waves in the grid): row_counters == 0 and
   // wave w simply takes chunk w -- nothing to balance, no counter traffic.
   const int nc = p.row_counters;                        // 64, 1 for tiny grids, 0: static
   const int64_t nchunks = (p.m + kRowsPerClaim - 1) / kRowsPerClaim;
   // one half of the row space holds more than 1.5 times the edges of the other (classify kernel's sample)
   const int64_t stretches = nchunks >> 6;
   const bool scatter = scattered_order(p);
   const int64_t wave_id = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   int cur = nc > 0 ? (int)(wave_id & (unsigned)(nc - 1)) : 0;
   unsigned long long claimed = 0;
   int64_t chunk;
   if (nc == 0) chunk = wave_id < nchunks ? wave_id : -1;
   else
   {
      if (lane == 0) claimed = atomicAdd(&p.ctr->rows[cur].next, 1ull);
      chunk = resolve_claim<IdxT>(p, claimed, cur, nc, nchunks, lane);
   }
   while (chunk >= 0)
   {
   // Where the rows' work follows their position (R-MAT degrees follow the bits of the row id; vertices
   // sorted by degree), stretches of 64 chunks are taken in a scattered order, so that what the GPU works
   // on at any time is a mix of the whole row space rather than one stretch of it, all dense or all
   // nearly empty.  The map is one-to-one: the multiplier is a prime larger than any number of stretches.
   int64_t at = chunk;
   if (scatter && (chunk >> 6) < stretches)
      at = (int64_t)(((unsigned long long)(chunk >> 6) * 2654435761ull) % (unsigned long long)stretches) * 64 + (chunk & 63);
   const int64_t row0 = at * kRowsPerClaim;
   IdxT my_b = 0, my_e = 0;   // lane t holds the pointers of row0 + t
   if (lane < kRowsPerClaim && row0 + lane < p.m)
   {
      my_b = p.pntrb[row0 + lane];
      my_e = p.pntre[row0 + lane];
   }
   if (nc > 0 && lane == 0) claimed = atomicAdd(&p.ctr->rows[cur].next, 1ull);
   // rows of this claim that have edges, one bit per row: while a row is walked, the
   // first column ids and the X slice of the next such row are already on their way
   unsigned int has_edges = (unsigned int)__ballot(lane < kRowsPerClaim && my_e > my_b);
   unsigned int packed_rows = 0u;   // rows of this claim that were walked one per sub-wave
   if constexpr (V == 4 && L <= 16)
   {
      if (p.pack_rows && !(generic && aop == kAopNoop))
      {
         constexpr int S = 64 / L;
         for (int g0 = 0; g0 < kRowsPerClaim; g0 += S)
         {
            const unsigned int gmask = ((1u << S) - 1u) << g0;
            const int nz = __builtin_popcount(has_edges & gmask);
            int64_t md = 0;
#pragma unroll
            for (int t = g0; t < g0 + S; t++)
            {
               const int64_t d = (int64_t)lane_value<IdxT>(my_e, t) - (int64_t)lane_value<IdxT>(my_b, t);
               md = d > md ? d : md;
            }
            if (packs<L, U>(md, nz, p.heavy_deg))
            {
               // sub-wave s takes row row0 + g0 + s: its pointers are in lane g0 + s
               const IdxT gb = chunk_entry<L>(my_b, g0 + lane / L), ge = chunk_entry<L>(my_e, g0 + lane / L);
               packed_group<V, L, R, EXACT, OP, SOPK, U, IdxT>(p, row0 + g0, gb, ge > gb ? ge : gb, (int)md, lane, tab, st);
               stage_tick<V, L, R, EXACT, IdxT>(st, p, __builtin_amdgcn_s_memrealtime(), lane);
               packed_rows |= gmask;
            }
         }
         has_edges &= ~packed_rows;
      }
   }
   EdgeChunk<IdxT> first;
   Slice<R> xs_next;
   int fetched_t = -1;        // row of this claim whose first chunk `first` (and X slice `xs_next`) hold
   for (int t = 0; t < kRowsPerClaim && row0 + t < p.m; t++)
   {
      if ((packed_rows >> t) & 1u) continue;
      const int64_t row = row0 + t;
      const IdxT jb = lane_value<IdxT>(my_b, t);
      const IdxT je = lane_value<IdxT>(my_e, t);
      const int64_t deg = (int64_t)je - (int64_t)jb;

      if (deg > p.heavy_deg)
      {
         // queued by the classify kernel and already walked, segment by segment, in
         // phase A -- unless the queue was full, in which case the row is done here
         const unsigned int word = p.queued[row >> 5];
         if ((word >> (row & 31)) & 1u) continue;
      }

      real_t *zrow = p.z + row * p.ldz;
      if (deg <= 0)
      {
         // empty row (about half the rows of an R-MAT graph): nothing to gather; the
         // overwrite rule still clears Z, every other rule leaves it alone
         if (!generic && p.beta_zero) stage_clear<V, L, R, EXACT, IdxT>(st, p, zrow, lane);
         continue;
      }
      if (generic && aop == kAopNoop) continue;   // general semantics with no accumulate stage: Z is left alone

      Slice<R> xs, acc;
      if (fetched_t == t) xs = xs_next;
      else
      {
         if (reads_x) load_slice<V, L, R, EXACT, true>(xs, p.x + row * p.ldx, sl, p.k);
         else
         {
#pragma unroll
            for (int r = 0; r < R; r++) xs.v[r] = zero4();
         }
         load_chunk<OP, IdxT>(first, p, jb, je, lane);
      }
      if (generic)
      {
         // general semantics: fold the edges into the caller's Z with AOP
         if (sub == 0) load_slice<V, L, R, EXACT>(acc, zrow, sl, p.k);
         else
         {
            const real_t id = aop_identity(aop);
#pragma unroll
            for (int r = 0; r < R; r++) acc.v[r] = real4{id, id, id, id};
         }
      }
      else
      {
#pragma unroll
         for (int r = 0; r < R; r++) acc.v[r] = zero4();
      }

      // next row of the claim with edges: its X slice is requested now, its first 64
      // column ids by the walk below while this row's last chunk is gathered
      const unsigned int later = (t + 1 < kRowsPerClaim) ? (has_edges >> (t + 1)) : 0u;
      IdxT nb = 0, ne = 0;
      fetched_t = -1;
      if (later)
      {
         fetched_t = t + 1 + __builtin_ctz(later);
         nb = lane_value<IdxT>(my_b, fetched_t);
         ne = lane_value<IdxT>(my_e, fetched_t);
         if (reads_x) load_slice<V, L, R, EXACT, true>(xs_next, p.x + (row0 + fetched_t) * p.ldx, sl, p.k);
         else
         {
#pragma unroll
            for (int r = 0; r < R; r++) xs_next.v[r] = zero4();
         }
      }
      walk_edges<V, L, R, EXACT, OP, SOPK, U, IdxT>(acc, xs, p, jb, je, first, nb, ne, lane, tab);
      // (the clock is read here, not before the walk, so that it is not one more value to keep through it; the read
      // is under way while the sub-waves' sums are merged)
      const unsigned long long clock = st.cap ? __builtin_amdgcn_s_memrealtime() : 0ull;
      merge_subwaves<L, R, OP>(acc, p.imessage);

      if (sub == 0 && !generic && !p.beta_zero)
      {
         Slice<R> zin;
         load_slice<V, L, R, EXACT>(zin, zrow, sl, p.k);
         map2(acc, zin, acc, [](real_t a, real_t b) { return a + b; });
      }
      stage_row<V, L, R, EXACT, IdxT>(st, p, zrow, acc, lane);
      stage_tick<V, L, R, EXACT, IdxT>(st, p, clock, lane);
   }
   if (st.nclear) stage_tick<V, L, R, EXACT, IdxT>(st, p, __builtin_amdgcn_s_memrealtime(), lane);   // a claim of empty rows
   chunk = nc > 0 ? resolve_claim<IdxT>(p, claimed, cur, nc, nchunks, lane) : -1;
   }
   if (st.n | st.nclear) stage_flush<V, L, R, EXACT, IdxT>(st, p, lane);
}

// Every wavefront ends here.  The last workgroup to finish, when nobody reads the
// queues any more, puts them back to their resting state for the next call: the
// bits of the queued rows cleared, the counters zero (their values kept in
// last_*, and the number of rows to fold handed to the merge kernel in
// merge_heavy).  "Last" is found in two steps, workgroups counting into one of 64
// group counters and complete groups into one more, so that no counter sees more
// than a few dozen read-modify-writes.
template <typename IdxT>
__device__ __forceinline__ void retire_wave(const Params<IdxT> &p)
{
   const int lane = threadIdx.x & 63;
   __syncthreads();                       // the whole workgroup is done with the queues
   if (threadIdx.x >= 64) return;
   Counters *c = p.ctr;
   const unsigned int groups = gridDim.x < 64u ? gridDim.x : 64u;
   const unsigned int grp = blockIdx.x & 63u;
   const unsigned int in_group = (gridDim.x - grp + 63u) / 64u;   // workgroups b with b % 64 == grp
   unsigned int before = 0u;
   if (lane == 0) before = __hip_atomic_fetch_add(&c->retire[grp].done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
   before = (unsigned int)__builtin_amdgcn_readfirstlane((int)before);
   if (before + 1u != in_group) return;
   if (lane == 0) before = __hip_atomic_fetch_add(&c->done_groups, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
   before = (unsigned int)__builtin_amdgcn_readfirstlane((int)before);
   if (before + 1u != groups) return;
   __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
   const unsigned int queued_heavy = c->n_heavy < p.cap_heavy ? c->n_heavy : p.cap_heavy;
   for (unsigned int h = lane; h < queued_heavy; h += 64)
   {
      const HeavyRow hr = p.heavy[h];
      if (hr.n_seg) p.queued[hr.row >> 5] = 0u;   // every bit of the word belongs to a row on this list
   }
   c->rows[lane].next = 0ull;
   c->retire[lane].done = 0u;
   if (lane == 0)
   {
      c->last_heavy = c->n_heavy;
      c->last_seg = c->n_seg;
      c->last_overflow = c->overflow;
      c->merge_heavy = queued_heavy;
      c->n_heavy = 0u;
      c->n_seg = 0u;
      c->overflow = 0u;
      c->done_groups = 0u;
      c->last_skew = c->skew;
      c->last_scattered = scattered_order(p) ? 1u : 0u;
      c->skew = 0ull;
   }
}

// ---- kernel 2: the fused SDDMM+SpMM kernel ------------------------------------------
// Long work first: every wave takes its share of the queued segments of heavy
// rows (phase A), then claims ordinary rows until none are left (phase B).  One
// kernel, so the short rows fill in behind the long segments instead of waiting
// for them at a kernel boundary.
// The float / int32 instances whose rows take one register per lane on sub-waves of 32 lanes or fewer are held to
// the residency they had before rows could wait in LDS -- 128 vector registers, four wavefronts per SIMD -- at the
// price of a few spilled values (0-24 bytes per lane): measured faster that way than with the 130-145 registers the
// compiler takes when left alone (K=32 on 2^23 nodes: 3.18 against 3.42 ms; K=64 on R-MAT 24: 23.1 against 23.7).
// The wider instances, the general pipeline and the other libraries keep the compiler's own allocation: held to
// 128 registers, K=256 lost 2.5 %, and the int64 and double instances 4-6 % at K=64.
#define FMM_MIN_WAVES ((sizeof(IdxT) == 4 && sizeof(real_t) == 4 && R == 1 && L <= 32 && OP != OP_GENERIC) ? 4 : 1)
template <int V, int L, int R, bool EXACT, int OP, int SOPK, int U, typename IdxT>
__global__ __launch_bounds__(kBlockThreads, FMM_MIN_WAVES) void fused_kernel(const Params<IdxT> p)
{
   __shared__ real_t lds_tab[(OP >= OP_DOT) ? kSigmoidTableSize : 1];
   const bool uses_sop = (OP == OP_DOT || OP == OP_DIST || (OP == OP_GENERIC && (p.imessage & 0xF00) == kSopUdef));
   const lds_table_t tab = stage_table(p.sigmoid_table, lds_tab, (OP >= OP_DOT) && uses_sop && (SOPK >= 0 ? SOPK : p.sop_kind) == SOP_SIGMOID);
   segments_phase<V, L, R, EXACT, OP, SOPK, U, IdxT>(p, tab);
   // finished Z rows wait in the dynamic LDS for the grid's common store tick
   rows_phase<V, L, R, EXACT, OP, SOPK, U, IdxT>(p, tab);
   retire_wave<IdxT>(p);
}

// ---- kernel 3: fold the partials of each heavy row -------------------------------------
// One block per heavy row.  The block's 256 threads form G groups; group g folds
// segments g, g+G, g+2G ... in ascending order starting from zero, then the G
// group sums are added in ascending g.  G depends only on K, so the order of
// every addition is fixed and results are the same on every run.
template <typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void merge_kernel(const Params<IdxT> p, int generic)
{
   __shared__ real_t red[kBlockThreads];
   const unsigned int nheavy = p.ctr->merge_heavy;   // left by the fused kernel's last workgroup
   const int aop = p.imessage & 0xF0000;
   const int cols = p.k < kBlockThreads ? p.k : kBlockThreads;   // elements handled per pass
   int G = kBlockThreads / cols;                                  // groups (power of two not required)
   if (G < 1) G = 1;
   const int grp = threadIdx.x / cols, col = threadIdx.x % cols;
   const bool active = grp < G;
   for (unsigned int h = blockIdx.x; h < nheavy; h += gridDim.x)
   {
      const HeavyRow hr = p.heavy[h];
      if (hr.n_seg == 0) continue;
      real_t *zrow = p.z + hr.row * p.ldz;
      // columns in passes of `cols`, the passes dealt to the grid's second dimension
      for (int e0 = (int)blockIdx.y * cols; e0 < p.k; e0 += (int)gridDim.y * cols)
      {
         const int e = e0 + col;
         const bool live = active && e < p.k;
         const real_t *pp = p.partial + (int64_t)hr.seg_base * p.kpad + e;
         const bool is_max = generic && aop == kAopMax, is_min = generic && aop == kAopMin;
         real_t a = is_max ? -(real_t)__builtin_inf() : (is_min ? (real_t)__builtin_inf() : (real_t)0);
         if (live)
         {
            unsigned int s = grp;
            if (!is_max && !is_min)
            {
               // 16 partials requested at a time, added in ascending order as before
               for (; s + 15u * G < hr.n_seg; s += 16u * G)
               {
                  real_t v[16];
#pragma unroll
                  for (unsigned int i = 0; i < 16u; i++) v[i] = pp[(int64_t)(s + i * G) * p.kpad];
#pragma unroll
                  for (unsigned int i = 0; i < 16u; i++) a += v[i];
               }
               for (; s + 3u * G < hr.n_seg; s += 4u * G)
               {
                  const real_t v0 = pp[(int64_t)s * p.kpad], v1 = pp[(int64_t)(s + G) * p.kpad],
                              v2 = pp[(int64_t)(s + 2u * G) * p.kpad], v3 = pp[(int64_t)(s + 3u * G) * p.kpad];
                  a += v0; a += v1; a += v2; a += v3;
               }
            }
            for (; s < hr.n_seg; s += G)
            {
               const real_t v = pp[(int64_t)s * p.kpad];
               a = is_max ? max_r(a, v) : (is_min ? min_r(a, v) : a + v);
            }
         }
         __syncthreads();
         red[threadIdx.x] = a;
         __syncthreads();
         if (live && grp == 0)
         {
            real_t t = red[col];
            for (int g2 = 1; g2 < G; g2++)
            {
               const real_t v = red[g2 * cols + col];
               t = is_max ? max_r(t, v) : (is_min ? min_r(t, v) : t + v);
            }
            if (generic)
            {
               const real_t zi = zrow[e];
               t = is_max ? max_r(zi, t) : (is_min ? min_r(zi, t) : zi + t);
            }
            else if (!p.beta_zero) t = zrow[e] + t;
            zrow[e] = t;
         }
      }
   }
}

}  // namespace fmm
