// C-ABI layer of libfusedmm_amd_i{32,64}.so: decodes the op tuple, picks the
// kernel instance for (K, alignment, op), keeps the per-device work queues and
// staging buffers, and launches the gfx950 kernels of fusedmm_kernels.h.
//
// Replaces the dispatch of the reference's fusedMM.c:487-744 and
// kernels/src/kernels.c:456-631.  Built once per index width (-DINDEXTYPE=...).
#include <hip/hip_runtime.h>
#include <dlfcn.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <condition_variable>
#include <mutex>
#include <thread>
#include <vector>

#ifndef INDEXTYPE
#error "compile with -DINDEXTYPE=int32_t or -DINDEXTYPE=int64_t"
#endif
#ifdef DREAL          /* the reference's switch for double precision (fusedMM.c:9-13) */
#define FMM_DOUBLE 1
#define VALUETYPE double
#else
#define VALUETYPE float
#endif
#include "../../include/fusedMM.h"
#include "../../include/fusedmm_amd.h"
#include "fusedmm_kernels.h"

// Device memory of the entry point that allocates nothing (fusedMM_csr_stream_noalloc):
// the sigmoid table, the queue and claim counters, the queued-row bitmap, the
// heavy-row queue, the segment descriptors and the partial results of split rows,
// carved out of this array call by call.  Every GPU the library runs on holds its
// own copy until the process ends.  In host code the name is only a handle: the
// address kernels and copies use comes from hipGetSymbolAddress, once per device.
#define FUSEDMM_AMD_SCRATCH_BYTES (32u << 20)
static __device__ __align__(256) unsigned char fmm_scratch[FUSEDMM_AMD_SCRATCH_BYTES];

namespace {

using namespace fmm;
typedef INDEXTYPE idx_t;
typedef VALUETYPE val_t;
constexpr size_t kValBytes = sizeof(val_t);

#define FMM_LOG(...)                                   \
   do {                                                \
      fprintf(stderr, "fusedmm_amd: " __VA_ARGS__);    \
      fprintf(stderr, "\n");                           \
   } while (0)

// hipError -> reference status code (fusedMM.h:103-112)
inline int hip_status(hipError_t e, const char *what)
{
   if (e == hipSuccess) return FUSEDMM_SUCCESS_RETURN;
   FMM_LOG("%s failed: %s", what, hipGetErrorString(e));
   (void)hipGetLastError();
   return e == hipErrorOutOfMemory ? FUSEDMM_NOT_ENOUGH_MEM : FUSEDMM_FAIL_RETURN;
}
#define FMM_HIP(call)                                  \
   do {                                                \
      int st_ = hip_status((call), #call);             \
      if (st_ != FUSEDMM_SUCCESS_RETURN) return st_;   \
   } while (0)

constexpr int kMaxDevices = 16;
constexpr int kTimingSlots = 512;
constexpr int kMaxK = 2048;

struct Buffer {
   void *ptr = nullptr;
   size_t bytes = 0;
};

// The two sets of work queues a GPU can hold: buffers that grow with the
// largest call seen (every ordinary entry point), and the fixed static array.
enum : int { kQueuesGrown = 0, kQueuesStatic = 1 };

struct DeviceState {
   bool basics = false;       // num_cu and the ordering events
   bool ready = false;        // allocated table and counters of the ordinary entry points
   int num_cu = 0;
   val_t *sigmoid_table = nullptr;
   Counters *ctr = nullptr;
   Buffer heavy, segs, partial, queued;
   Buffer stage[8];           // host-pointer mode: pntrb, pntre, indx, val, x, y, z, spare
   Buffer edge_t;             // per-edge vectors T[j][0..k) of the stage-by-stage path (host-function stages)
   // host-pointer mode: two pinned buffers each way, copies are pipelined through them
   void *pin[4] = {nullptr, nullptr, nullptr, nullptr};
   hipEvent_t pin_ev[4];
   bool pin_busy[4] = {false, false, false, false};
   // opt-in device mirrors of read-only host operands, keyed by host address and size
   struct Mirror { const void *host; size_t bytes; void *dev; unsigned long long last_use; };
   std::vector<Mirror> mirrors;
   // the static array of this device (address from hipGetSymbolAddress), once set up
   unsigned char *scratch = nullptr;
   // Calls that share a set of queues must not overlap: a call on another stream than
   // the previous one first waits for order_ev, recorded on that earlier stream.
   hipEvent_t order_ev[2];
   hipStream_t last_stream[2] = {nullptr, nullptr};
   bool pending[2] = {false, false};
   // A call whose kernels could not all be launched may leave counters or queued-row
   // bits set; the next call on these queues then clears them before it starts.
   bool dirty[2] = {false, false};
   Counters *last_ctr = nullptr;   // counters of the most recent call (fusedMM_amd_last_split)
   // timing
   hipEvent_t ev[kTimingSlots][4];   // around the three kernels of a call
   bool ev_made = false;
};

struct Globals {
   std::mutex mu;
   int sop_kind = FUSEDMM_SOP_KIND_HOST;
   bool sop_kind_from_env_done = false;
   int opt = 1;
   int64_t heavy_deg = 0;
   int seg_len = 0;
   int blocks_per_cu = 0;
   int validate = 0;
   int row_order = 0;         // 0 auto, 1 first to last, 2 scattered stretches (FUSEDMM_ROW_ORDER)
   int cache = 0;             // 1: keep device mirrors of read-only host operands between calls
   unsigned long long cache_clock = 0;
   double phase_ms[3] = {0, 0, 0};   // upload, kernels, download of the last host-pointer call
   bool phase_valid = false;
   fusedMM_amd_sop_fn sop_fn = nullptr;
   fusedMM_amd_vop_fn vop_fn = nullptr;
   fusedMM_amd_rop_fn rop_fn = nullptr;
   fusedMM_amd_vsc_fn vsc_fn = nullptr;
   fusedMM_amd_aop_fn aop_fn = nullptr;
   int timing = 0;            // 0: off; n: HIP events around the kernels of every n-th call
   int timing_seen = 0;       // calls since timing was switched on
   int timing_calls = 0;      // calls recorded
   int timing_dev = 0;
   DeviceState dev[kMaxDevices];
};
Globals g;

int sop_kind_from_name(const char *s)
{
   if (!s) return FUSEDMM_SOP_KIND_HOST;
   if (!strcmp(s, "host")) return FUSEDMM_SOP_KIND_HOST;
   if (!strcmp(s, "identity")) return FUSEDMM_SOP_KIND_IDENTITY;
   if (!strcmp(s, "sigmoid")) return FUSEDMM_SOP_KIND_SIGMOID;
   if (!strcmp(s, "tdist")) return FUSEDMM_SOP_KIND_TDIST;
   if (!strcmp(s, "fr")) return FUSEDMM_SOP_KIND_FR;
   if (!strcmp(s, "ll")) return FUSEDMM_SOP_KIND_LL;
   if (!strcmp(s, "fa")) return FUSEDMM_SOP_KIND_FA;
   FMM_LOG("FUSEDMM_SOP_KIND=%s is not a known kind; using host", s);
   return FUSEDMM_SOP_KIND_HOST;
}

void read_env_once()
{
   if (g.sop_kind_from_env_done) return;
   g.sop_kind_from_env_done = true;
   if (const char *e = getenv("FUSEDMM_SOP_KIND")) g.sop_kind = sop_kind_from_name(e);
   if (const char *e = getenv("FUSEDMM_BLOCKS_PER_CU")) g.blocks_per_cu = atoi(e);
   if (const char *e = getenv("FUSEDMM_VALIDATE")) g.validate = atoi(e);
   if (const char *e = getenv("FUSEDMM_CACHE")) g.cache = atoi(e) ? 1 : 0;
   if (const char *e = getenv("FUSEDMM_ROW_ORDER"))   // "auto", "plain" (first to last) or "scattered"
      g.row_order = !strcmp(e, "plain") ? 1 : (!strcmp(e, "scattered") ? 2 : 0);
   if (const char *e = getenv("FUSEDMM_SPLIT"))   // "heavy_deg,seg_len", as fusedMM_amd_set_split
   {
      long long h = 0;
      int sl = 0;
      if (sscanf(e, "%lld,%d", &h, &sl) == 2 && h > 0 && sl > 0) { g.heavy_deg = h; g.seg_len = sl; }
   }
}

// The 2048-entry sigmoid table, built with the expressions of the reference's
// tester (test/fusedMMtime.cpp:594-604, a C++ file: exp() resolves to the
// overload of VALUETYPE).  Single precision: x is a float, exp is expf, 1 + e is
// a float sum, the quotient is formed in double and rounded.  Double precision:
// everything is double.
void build_sigmoid_table(val_t *t)
{
   for (int i = 0; i < kSigmoidTableSize; i++)
   {
#ifdef FMM_DOUBLE
      double x = 2.0 * 5.0 * i / kSigmoidTableSize - 5.0;
      t[i] = 1.0 / (1 + exp(-x));
#else
      float x = (float)(2.0 * 5.0 * i / kSigmoidTableSize - 5.0);
      float e = expf(-x);
      float denom = 1 + e;
      t[i] = (float)(1.0 / (double)denom);
#endif
   }
}

// `capturing`: the call is being recorded into a HIP graph.  Replacing a buffer
// then would leave the graph (and any graph captured earlier) with the address
// of freed memory, so the call is refused instead.
int grow(Buffer &b, size_t bytes, bool capturing = false)
{
   if (bytes <= b.bytes) return FUSEDMM_SUCCESS_RETURN;
   if (capturing)
   {
      FMM_LOG("a work buffer would have to grow (%zu -> %zu bytes) while the stream is being captured; "
              "run one call of this size outside the capture first, or use fusedMM_csr_stream_noalloc",
              b.bytes, bytes);
      return FUSEDMM_NOT_ENOUGH_MEM;
   }
   if (b.ptr) FMM_HIP(hipFree(b.ptr));
   b.ptr = nullptr;
   b.bytes = 0;
   FMM_HIP(hipMalloc(&b.ptr, bytes));
   b.bytes = bytes;
   return FUSEDMM_SUCCESS_RETURN;
}

// What every entry point needs of the current device; allocates no device memory.
int device_basics(DeviceState **out)
{
   int dev = 0;
   FMM_HIP(hipGetDevice(&dev));
   if (dev < 0 || dev >= kMaxDevices) return FUSEDMM_FAIL_RETURN;
   DeviceState &d = g.dev[dev];
   if (!d.basics)
   {
      int cus = 0;
      FMM_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
      d.num_cu = cus > 0 ? cus : 256;
      for (int q = 0; q < 2; q++) FMM_HIP(hipEventCreateWithFlags(&d.order_ev[q], hipEventDisableTiming));
      d.basics = true;
   }
   *out = &d;
   return FUSEDMM_SUCCESS_RETURN;
}

int device_state(DeviceState **out)
{
   DeviceState *dp = nullptr;
   int st0 = device_basics(&dp);
   if (st0) return st0;
   DeviceState &d = *dp;
   if (!d.ready)
   {
      val_t host_tab[kSigmoidTableSize];
      build_sigmoid_table(host_tab);
      FMM_HIP(hipMalloc((void **)&d.sigmoid_table, sizeof(host_tab)));
      FMM_HIP(hipMemcpy(d.sigmoid_table, host_tab, sizeof(host_tab), hipMemcpyHostToDevice));
      FMM_HIP(hipMalloc((void **)&d.ctr, sizeof(Counters)));
      FMM_HIP(hipMemset(d.ctr, 0, sizeof(Counters)));
      d.ready = true;
   }
   *out = &d;
   return FUSEDMM_SUCCESS_RETURN;
}

// ---- the static array: fixed head, then the queues of the call in progress ----------
constexpr size_t align256(size_t v) { return (v + 255u) & ~(size_t)255u; }
constexpr size_t kScratchTableOff = 0;
constexpr size_t kScratchCtrOff = align256(kSigmoidTableSize * sizeof(val_t));
constexpr size_t kScratchBitmapOff = kScratchCtrOff + align256(sizeof(Counters));
// The queued-row bits stay zero between calls only if nothing else is ever written
// where they live: a fixed region, one bit per row for the largest m accepted.
constexpr int64_t kScratchMaxRows = (int64_t)1 << 25;
constexpr size_t kScratchQueuesOff = kScratchBitmapOff + (size_t)(kScratchMaxRows / 8);

// Once per device, with that device current: find this device's copy of the
// array, put the sigmoid table at its head and zero the counters.
int scratch_setup(DeviceState &d)
{
   if (d.scratch) return FUSEDMM_SUCCESS_RETURN;
   unsigned char *base = nullptr;
   FMM_HIP(hipGetSymbolAddress((void **)&base, HIP_SYMBOL(fmm_scratch)));
   if (!base) return FUSEDMM_FAIL_RETURN;
   val_t host_tab[kSigmoidTableSize];
   build_sigmoid_table(host_tab);
   FMM_HIP(hipMemcpy(base + kScratchTableOff, host_tab, sizeof(host_tab), hipMemcpyHostToDevice));
   FMM_HIP(hipMemset(base + kScratchCtrOff, 0, kScratchQueuesOff - kScratchCtrOff));   // counters and queued-row bits
   d.scratch = base;
   return FUSEDMM_SUCCESS_RETURN;
}

// ---- kernel instance selection ---------------------------------------------------
struct Shape {
   int V, L, R, exact, U;
};

bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

int pick_shape(int k, bool vec_ok, Shape *s)
{
   if (k < 1 || k > kMaxK) return FUSEDMM_FAIL_RETURN;
   if (vec_ok)
   {
      if (k == 32) *s = {4, 8, 1, 1, 8};
      else if (k == 64) *s = {4, 16, 1, 1, 8};
      else if (k == 128) *s = {4, 32, 1, 1, 8};
      else if (k == 256) *s = {4, 64, 1, 1, 16};
      else if (k == 512) *s = {4, 64, 2, 1, 8};
      else if (k <= 32) *s = {4, 8, 1, 0, 8};
      else if (k <= 64) *s = {4, 16, 1, 0, 8};
      else if (k <= 128) *s = {4, 32, 1, 0, 8};
      else if (k <= 256) *s = {4, 64, 1, 0, 16};
      else if (k <= 512) *s = {4, 64, 2, 0, 8};
      else if (k <= 1024) *s = {4, 64, 4, 0, 4};
      else *s = {4, 64, 8, 0, 2};
   }
   else
   {
      if (k <= 256) *s = {1, 64, 1, 0, 16};
      else if (k <= 512) *s = {1, 64, 2, 0, 8};
      else if (k <= 1024) *s = {1, 64, 4, 0, 4};
      else *s = {1, 64, 8, 0, 2};
   }
   return FUSEDMM_SUCCESS_RETURN;
}

// (V, L, R, exact, U) of every kernel instance; pick_shape() returns one of these.
// U (gathers in flight per sub-wave) is halved in double precision: same bytes in flight.
#ifdef FMM_DOUBLE
#define FMM_U(u) ((u) / 2)
#else
#define FMM_U(u) (u)
#endif
#define FMM_SHAPES(X) \
   X(4, 8, 1, 1, FMM_U(8)) X(4, 16, 1, 1, FMM_U(8)) X(4, 32, 1, 1, FMM_U(8)) X(4, 64, 1, 1, FMM_U(16)) \
   X(4, 64, 2, 1, FMM_U(8)) \
   X(4, 8, 1, 0, FMM_U(8)) X(4, 16, 1, 0, FMM_U(8)) X(4, 32, 1, 0, FMM_U(8)) X(4, 64, 1, 0, FMM_U(16)) \
   X(4, 64, 2, 0, FMM_U(8)) X(4, 64, 4, 0, FMM_U(4)) X(4, 64, 8, 0, FMM_U(2)) \
   X(1, 64, 1, 0, FMM_U(16)) X(1, 64, 2, 0, FMM_U(8)) X(1, 64, 4, 0, FMM_U(4)) X(1, 64, 8, 0, FMM_U(2))

struct Launch {
   int num_cu, blocks_per_cu;
   int64_t nnz_hint;
   hipStream_t stream;
   hipEvent_t *ev;   // 4 events or nullptr
};

template <int V, int L, int R, bool EXACT, int OP, int SOPK, int U>
int launch_instance(const Params<idx_t> &p, const Launch &l)
{
   // persistent grid: as many blocks as stay resident; waves share out the
   // queued segments, then claim rows
   static int occ = 0;
   if (occ == 0)
   {
      FMM_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fused_kernel<V, L, R, EXACT, OP, SOPK, U, idx_t>, kBlockThreads, 0));
      if (occ < 1) occ = 1;
   }
   // enough blocks for the rows, or for the segments the caller's nnz could give rise to
   int64_t need = (p.m + kWavesPerBlock - 1) / kWavesPerBlock;
   const int64_t need_segs = (l.nnz_hint / p.seg_len + kWavesPerBlock - 1) / kWavesPerBlock;
   if (need < need_segs) need = need_segs;
   // Four workgroups (16 waves) per CU at most: with 8-16 gathers in flight per wave
   // that saturates the memory system, and more waves only evict each other's lines
   // (measured on the sigmoid K=128 benchmark: 1.307 ms at 4 per CU, 1.314 at 5, 1.335 at 6).
   const int resident = occ < 4 ? occ : 4;
   int64_t gr = (int64_t)l.num_cu * (l.blocks_per_cu > 0 ? l.blocks_per_cu : resident);
   if (gr > need) gr = need;
   if (gr < 1) gr = 1;
   Params<idx_t> pr = p;
   const int64_t nchunks = (p.m + kRowsPerClaim - 1) / kRowsPerClaim;
   if (nchunks <= gr * kWavesPerBlock) pr.row_counters = 0;   // one chunk per wave at most: static
   else pr.row_counters = (gr * kWavesPerBlock >= kRowCounters) ? kRowCounters : 1;
   int64_t gc = (p.m + kBlockThreads - 1) / kBlockThreads;
   if (gc > (int64_t)l.num_cu * 8) gc = (int64_t)l.num_cu * 8;
   if (l.ev) FMM_HIP(hipEventRecord(l.ev[0], l.stream));
   hipLaunchKernelGGL((classify_kernel<idx_t>), dim3((unsigned int)gc), dim3(kBlockThreads), 0, l.stream, p);
   if (l.ev) FMM_HIP(hipEventRecord(l.ev[1], l.stream));
   hipLaunchKernelGGL((fused_kernel<V, L, R, EXACT, OP, SOPK, U, idx_t>), dim3((unsigned int)gr), dim3(kBlockThreads), 0, l.stream, pr);
   if (l.ev) FMM_HIP(hipEventRecord(l.ev[2], l.stream));
   // one workgroup per heavy row and pass of 256 columns
   const unsigned int col_passes = (unsigned int)((p.k + kBlockThreads - 1) / kBlockThreads);
   hipLaunchKernelGGL((merge_kernel<idx_t>), dim3((unsigned int)(l.num_cu * 2), col_passes), dim3(kBlockThreads), 0, l.stream,
                      p, (int)(OP == OP_GENERIC));
   if (l.ev) FMM_HIP(hipEventRecord(l.ev[3], l.stream));
   return hip_status(hipGetLastError(), "kernel launch");
}

// SOPK >= 0: the SOP body is fixed at compile time (the three the reference's
// benchmarks use: sigmoid on the dot tuple, t-dist and FR on the distance
// tuple); SOPK == -1: switched at run time on Params::sop_kind.
template <int OP, int SOPK>
int launch_op(const Params<idx_t> &p, const Shape &s, const Launch &l)
{
#define FMM_CASE(V_, L_, R_, X_, U_) \
   if (s.V == V_ && s.L == L_ && s.R == R_ && s.exact == X_) return launch_instance<V_, L_, R_, (X_ != 0), OP, SOPK, U_>(p, l);
   FMM_SHAPES(FMM_CASE)
#undef FMM_CASE
   return FUSEDMM_FAIL_RETURN;
}

// ---- op tuple --------------------------------------------------------------------
struct Plan {
   int op;            // OP_*
   bool opt_rule;     // optimised write-back rule (beta == 0 overwrites)
   bool needs_sop;    // tuple uses SOP_UDEF
   bool reads_x, reads_val;
   int udef_stages;   // stages that are the caller's host functions: kUdefVop | kUdefRop | kUdefVsc | kUdefAop
};
enum : int { kUdefVop = 1, kUdefRop = 2, kUdefVsc = 4, kUdefAop = 8 };

// Stage validation in the order of reference fusedMM.c:610-628, then the
// pattern match of :523-583.
int make_plan(int32_t imsg, int opt_enabled, Plan *pl)
{
   const int vop = GET_VOP_FLAG(imsg), rop = GET_ROP_FLAG(imsg), sop = GET_SOP_FLAG(imsg),
             vsc = GET_VSC_FLAG(imsg), aop = GET_AOP_FLAG(imsg);
   if (imsg & ~0xFFFFF) { FMM_LOG("Unknown bits in imessage 0x%x", imsg); return FUSEDMM_FAIL_RETURN; }
   // A *_UDEF stage is the caller's host function (the entry point checks that there is one).
   pl->udef_stages = 0;
   if (vop == VOP_UDEF) pl->udef_stages |= kUdefVop;
   else if (vop < VOP_COPY_LHS || vop > VOP_MIN) { FMM_LOG("Unknown VOP Message"); return FUSEDMM_VOP_FAIL_RETURN; }
   if (rop == ROP_UDEF) pl->udef_stages |= kUdefRop;
   else if (rop > ROP_NORMR) { FMM_LOG("Unknown ROP Message"); return FUSEDMM_ROP_FAIL_RETURN; }
   if (!(sop == SOP_NOOP || sop == SOP_COPY || sop == SOP_UDEF)) { FMM_LOG("Unknown SOP Message"); return FUSEDMM_SOP_FAIL_RETURN; }
   if (vsc == VSC_UDEF) pl->udef_stages |= kUdefVsc;
   else if (vsc > VSC_ADD) { FMM_LOG("Unknown VSC Message"); return FUSEDMM_VSC_FAIL_RETURN; }
   if (aop == AOP_UDEF) pl->udef_stages |= kUdefAop;
   else if (aop > AOP_MIN) { FMM_LOG("Unknown AOP Message"); return FUSEDMM_AOP_FAIL_RETURN; }

   pl->needs_sop = (sop == SOP_UDEF);
   pl->opt_rule = false;
   pl->op = OP_GENERIC;
   if (opt_enabled && vop == VOP_COPY_RHS && vsc != VSC_ADD && aop == AOP_ADD)
   {
      if (rop == ROP_NOOP && sop == SOP_NOOP && vsc == VSC_NOOP) pl->op = OP_GCN;
      else if (rop == ROP_NOOP && sop == SOP_COPY && vsc == VSC_MUL) pl->op = OP_SPMM;
      else if (rop == ROP_DOT && sop == SOP_UDEF && vsc == VSC_MUL) pl->op = OP_DOT;
   }
   if (opt_enabled && vop == VOP_SUBR && rop == ROP_NORMR && sop == SOP_UDEF && vsc == VSC_MUL && aop == AOP_ADD)
      pl->op = OP_DIST;
   pl->opt_rule = (pl->op != OP_GENERIC);
   if (opt_enabled == 2 && pl->op == OP_GENERIC)
   {
      // the reference built with MUST_OPT_FUSEDMM (fusedMM.c:599-604)
      FMM_LOG("NO opt implementation for this message! Run the general FusedMM by not requiring the optimised kernels");
      return FUSEDMM_NO_OPT_IMPL;
   }
   pl->reads_x = (pl->op == OP_DOT || pl->op == OP_DIST) ||
                 (pl->op == OP_GENERIC && (vop != VOP_COPY_RHS || rop == ROP_DOT || rop == ROP_ADD_LHS || rop == ROP_NORML));
   // the general pipeline seeds the scalar with val[j]; it matters only when no ROP overwrites it
   pl->reads_val = (pl->op == OP_SPMM) || (pl->op == OP_GENERIC && rop == ROP_NOOP && vsc != VSC_NOOP);
   if (pl->udef_stages)
   {
      // a host VOP or ROP is handed X[i]; a host ROP is handed the edge value as the scalar's start
      if (pl->udef_stages & (kUdefVop | kUdefRop)) pl->reads_x = true;
      pl->reads_val = (rop == ROP_NOOP && vsc != VSC_NOOP) || rop == ROP_UDEF;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

struct Args {
   int32_t imessage;
   int64_t m, n, k, nnz;
   const val_t *val;
   const idx_t *indx, *pntrb, *pntre;
   const val_t *x, *y;
   val_t *z;
   int64_t ldx, ldy, ldz;
   val_t beta;
};

int run_on_device(const Args &a, const Plan &pl, int sop_kind, hipStream_t stream, int queues = kQueuesGrown);
int validate_host_pointers(const Args &h);
int validate_operands(const Args &a, hipStream_t stream, int queues = kQueuesGrown);

// Make `stream` wait for the work of the previous call that used this set of
// queues, when that call went to another stream.  The event is recorded only now,
// on that earlier stream (it then covers the earlier call and whatever the caller
// enqueued there since): a record after every call would sit between consecutive
// calls of the common one-stream case and keep them from running back to back.
int order_after_previous(DeviceState &d, int queues, hipStream_t stream)
{
   if (!d.pending[queues] || d.last_stream[queues] == stream) return FUSEDMM_SUCCESS_RETURN;
   hipError_t e = hipEventRecord(d.order_ev[queues], d.last_stream[queues]);
   if (e == hipSuccess) e = hipStreamWaitEvent(stream, d.order_ev[queues], 0);
   if (e != hipSuccess)
   {
      // the earlier stream is gone (destroyed by the caller; its work still completes)
      (void)hipGetLastError();
      FMM_HIP(hipDeviceSynchronize());
   }
   d.pending[queues] = false;
   return FUSEDMM_SUCCESS_RETURN;
}

// Is `stream` being recorded into a HIP graph?  The legacy default stream cannot be.
int stream_capturing(hipStream_t stream, bool *capturing)
{
   *capturing = false;
   if (!stream) return FUSEDMM_SUCCESS_RETURN;
   hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
   FMM_HIP(hipStreamIsCapturing(stream, &cs));
   *capturing = (cs != hipStreamCaptureStatusNone);
   return FUSEDMM_SUCCESS_RETURN;
}

// One call of the kernels, k <= kMaxK.  Everything here is device memory.
// Enqueues on `stream`, does not wait.  `queues` says where the call's work
// queues live: kQueuesGrown (allocated, grown to the largest call seen) or
// kQueuesStatic (carved out of the static array; the call is refused when they
// do not fit, and nothing is allocated).
int run_slab(const Args &a, const Plan &pl, int sop_kind, hipStream_t stream, int queues)
{
   if (a.m <= 0) return FUSEDMM_SUCCESS_RETURN;
   if (a.k < 1) return FUSEDMM_SUCCESS_RETURN;
   if (a.k > kMaxK)
   {
      FMM_LOG("feature dimension k=%lld is beyond the supported maximum %d", (long long)a.k, kMaxK);
      return FUSEDMM_FAIL_RETURN;
   }
   if (a.ldy < a.k || a.ldz < a.k || (pl.reads_x && a.ldx < a.k))
   {
      FMM_LOG("leading dimension smaller than k");
      return FUSEDMM_FAIL_RETURN;
   }
   if (!a.indx || !a.pntrb || !a.pntre || !a.y || !a.z || (pl.reads_x && !a.x) || (pl.op == OP_SPMM && !a.val))
   {
      FMM_LOG("NULL operand");
      return FUSEDMM_FAIL_RETURN;
   }
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   bool capturing = false;
   st = stream_capturing(stream, &capturing);
   if (st) return st;
   // First use on a device copies the sigmoid table and clears the counters with
   // blocking calls (and, for the grown queues, allocates): not while a capture is open.
   if (capturing && (queues == kQueuesStatic ? d->scratch == nullptr : !d->ready))
   {
      FMM_LOG("first use on this device while the stream is being captured; call fusedMM_amd_init() before the capture");
      return FUSEDMM_FAIL_RETURN;
   }
   if (queues == kQueuesStatic) st = scratch_setup(*d);
   else st = device_state(&d);
   if (st) return st;

   // 16-byte accesses need 16-byte aligned rows: leading dimensions a multiple of 4 floats / 2 doubles
   constexpr int64_t ld_mult = 16 / (int64_t)kValBytes;
   const bool vec_ok = (a.k % 4 == 0) && (a.ldy % ld_mult == 0) && (a.ldz % ld_mult == 0) && aligned16(a.y) &&
                       aligned16(a.z) && (!pl.reads_x || ((a.ldx % ld_mult == 0) && aligned16(a.x)));
   Shape sh;
   st = pick_shape((int)a.k, vec_ok, &sh);
   if (st) return st;

   Params<idx_t> p;
   memset(&p, 0, sizeof(p));
   p.pntrb = a.pntrb; p.pntre = a.pntre; p.indx = a.indx;
   p.val = pl.reads_val ? a.val : nullptr;
   p.x = a.x; p.y = a.y; p.z = a.z;
   p.m = a.m; p.ldx = a.ldx; p.ldy = a.ldy; p.ldz = a.ldz;
   p.k = (int)a.k;
   p.beta_zero = (pl.opt_rule && a.beta == 0.0f) ? 1 : 0;
   p.sop_kind = sop_kind;
   p.imessage = a.imessage;
   p.row_order = g.row_order;

   // heavy-row split: segments of about 1 MiB of gathered rows but at most 2048 edges
   // (measured best on the R-MAT and power-law benchmark graphs: shorter segments pay
   // their start-up and partial-result cost more often, longer ones leave long rows
   // to single waves)
   int seg_len = g.seg_len > 0 ? g.seg_len : (int)(1048576 / ((int64_t)kValBytes * a.k));
   if (g.seg_len <= 0 && seg_len > 2048) seg_len = 2048;
   if (seg_len < 64 && g.seg_len <= 0) seg_len = 64;
   int64_t heavy_deg = g.heavy_deg > 0 ? g.heavy_deg : 2 * (int64_t)seg_len;
   if (heavy_deg < seg_len) heavy_deg = seg_len;
   p.seg_len = seg_len;
   p.heavy_deg = heavy_deg;
   p.kpad = (int)((a.k + 3) / 4 * 4);

   // queue capacities from the caller's nnz when it is plausible; rows that do
   // not fit are processed whole in the row phase, so this is never a
   // correctness question
   int64_t nnz_hint = (a.nnz > 0 && a.nnz < ((int64_t)1 << 40)) ? a.nnz : (int64_t)1 << 26;
   int64_t cap_seg = nnz_hint / seg_len * 3 / 2 + 1024;   // a row of d edges has at most d/seg_len + 1 segments
   int64_t cap_heavy = nnz_hint / heavy_deg + 1024;
   const int64_t max_partial_bytes = (int64_t)8 << 30;
   if (cap_seg * p.kpad * (int64_t)kValBytes > max_partial_bytes) cap_seg = max_partial_bytes / (p.kpad * (int64_t)kValBytes);
   if (cap_seg > 0x7FFFFFFF) cap_seg = 0x7FFFFFFF;
   if (cap_heavy > 0x7FFFFFFF) cap_heavy = 0x7FFFFFFF;
   const int64_t queued_words = (a.m + 31) / 32;
   const size_t b_heavy = (size_t)cap_heavy * sizeof(HeavyRow), b_segs = (size_t)cap_seg * sizeof(SegDesc),
                b_partial = (size_t)cap_seg * p.kpad * kValBytes, b_queued = (size_t)queued_words * sizeof(unsigned int);
   if (queues == kQueuesStatic)
   {
      // same capacities as the allocating entry points (so the same rows are split and
      // the results are the same bits), laid out behind the fixed head of the array
      const size_t o_queued = kScratchBitmapOff, o_heavy = kScratchQueuesOff,
                   o_segs = o_heavy + align256(b_heavy), o_partial = o_segs + align256(b_segs),
                   end = o_partial + align256(b_partial);
      if (a.m > kScratchMaxRows || end > (size_t)FUSEDMM_AMD_SCRATCH_BYTES)
      {
         FMM_LOG("fusedMM_csr_stream_noalloc: m=%lld, nnz=%lld, k=%lld need %zu bytes of work queues; the static "
                 "array holds %zu (use fusedMM_csr_stream for this size)",
                 (long long)a.m, (long long)nnz_hint, (long long)a.k, end, (size_t)FUSEDMM_AMD_SCRATCH_BYTES);
         return FUSEDMM_NOT_ENOUGH_MEM;
      }
      unsigned char *base = d->scratch;   // this device's address, never the array's name
      p.sigmoid_table = (const val_t *)(base + kScratchTableOff);
      p.ctr = (Counters *)(base + kScratchCtrOff);
      p.queued = (unsigned int *)(base + o_queued);
      p.heavy = (HeavyRow *)(base + o_heavy);
      p.segs = (SegDesc *)(base + o_segs);
      p.partial = (val_t *)(base + o_partial);
   }
   else
   {
      st = grow(d->heavy, b_heavy, capturing); if (st) return st;
      st = grow(d->segs, b_segs, capturing); if (st) return st;
      st = grow(d->partial, b_partial, capturing); if (st) return st;
      {
         // the queued-row bits are zero between calls (the fused kernel's last wavefront
         // clears what the call set), so a new buffer starts out zero and stays that way
         const void *before = d->queued.ptr;
         st = grow(d->queued, b_queued, capturing); if (st) return st;
         if (d->queued.ptr != before) FMM_HIP(hipMemsetAsync(d->queued.ptr, 0, d->queued.bytes, stream));
      }
      p.sigmoid_table = d->sigmoid_table;
      p.ctr = d->ctr;
      p.heavy = (HeavyRow *)d->heavy.ptr;
      p.segs = (SegDesc *)d->segs.ptr;
      p.partial = (val_t *)d->partial.ptr;
      p.queued = (unsigned int *)d->queued.ptr;
   }
   p.cap_heavy = (unsigned int)cap_heavy;
   p.cap_seg = (unsigned int)cap_seg;
   d->last_ctr = p.ctr;
   if (d->dirty[queues])
   {
      if (capturing)
      {
         FMM_LOG("an earlier call failed part-way; call once outside the capture (or fusedMM_amd_finalize()) first");
         return FUSEDMM_FAIL_RETURN;
      }
      FMM_HIP(hipDeviceSynchronize());
      FMM_HIP(hipMemset(p.ctr, 0, sizeof(Counters)));
      FMM_HIP(hipMemset(p.queued, 0, queues == kQueuesStatic ? (size_t)(kScratchMaxRows / 8) : d->queued.bytes));
      d->dirty[queues] = false;
   }

   // Calls that share these queues must run one after the other.  On one stream
   // they do; a call on another stream first waits for what the previous call's
   // stream holds.  (Not while capturing: an event recorded into a graph cannot be
   // waited on from outside it; the graph's launches are ordered by their stream.)
   if (!capturing)
   {
      st = order_after_previous(*d, queues, stream);
      if (st) return st;
   }

   Launch l;
   l.num_cu = d->num_cu;
   l.blocks_per_cu = g.blocks_per_cu;
   l.nnz_hint = nnz_hint;
   l.stream = stream;
   l.ev = nullptr;
   if (g.timing > 0 && queues == kQueuesGrown && !capturing && (g.timing_seen++ % g.timing) == 0 &&
       g.timing_calls < kTimingSlots)
   {
      if (!d->ev_made)
      {
         for (int i = 0; i < kTimingSlots; i++)
            for (int e = 0; e < 4; e++) FMM_HIP(hipEventCreate(&d->ev[i][e]));
         d->ev_made = true;
      }
      l.ev = d->ev[g.timing_calls++];
      FMM_HIP(hipGetDevice(&g.timing_dev));
   }

   switch (pl.op)
   {
      case OP_GCN: st = launch_op<OP_GCN, -1>(p, sh, l); break;
      case OP_SPMM: st = launch_op<OP_SPMM, -1>(p, sh, l); break;
      case OP_DOT:
         if (sop_kind == SOP_SIGMOID) st = launch_op<OP_DOT, SOP_SIGMOID>(p, sh, l);
         else st = launch_op<OP_DOT, -1>(p, sh, l);
         break;
      case OP_DIST:
         if (sop_kind == SOP_TDIST) st = launch_op<OP_DIST, SOP_TDIST>(p, sh, l);
         else if (sop_kind == SOP_FR) st = launch_op<OP_DIST, SOP_FR>(p, sh, l);
         else st = launch_op<OP_DIST, -1>(p, sh, l);
         break;
      default: st = launch_op<OP_GENERIC, -1>(p, sh, l); break;
   }
   if (st)
   {
      d->dirty[queues] = true;
      return st;
   }
   if (!capturing)
   {
      d->pending[queues] = true;
      d->last_stream[queues] = stream;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

bool is_device_pointer(const void *p)
{
   if (!p) return false;
   hipPointerAttribute_t attr;
   hipError_t e = hipPointerGetAttributes(&attr, p);
   if (e != hipSuccess)
   {
      (void)hipGetLastError();   // plain host memory: not an error for us
      return false;
   }
   return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

// The synchronous entry point takes operands that are all host memory or all
// device memory.  Returns 1 (device), 0 (host) or -1 (mixed: refused, a kernel
// dereferencing a host address would fault the GPU).
int operand_residence(const Args &a)
{
   const void *ops[] = {a.z, a.y, a.x, a.val, a.indx, a.pntrb, a.pntre};
   int dev = 0, host = 0;
   for (const void *o : ops)
   {
      if (!o) continue;
      if (is_device_pointer(o)) dev++;
      else host++;
   }
   if (dev && host)
   {
      FMM_LOG("operands mix host and device memory; pass all of one kind");
      return -1;
   }
   return dev ? 1 : 0;
}

// ---- host-pointer mode: pinned staging ------------------------------------------------
// The caller's arrays are ordinary pageable memory.  They move through two pinned
// buffers each way, 16 MiB at a time: a few threads copy chunk i+1 between the
// caller's array and a pinned buffer while the DMA engine moves chunk i.
constexpr size_t kPinChunk = (size_t)16 << 20;
constexpr size_t kPinMinBytes = (size_t)1 << 20;   // smaller copies go straight through hipMemcpyAsync

class CopyPool {
 public:
   void copy(void *dst, const void *src, size_t bytes)
   {
      if (bytes < ((size_t)1 << 20) || !start()) { memcpy(dst, src, bytes); return; }
      std::unique_lock<std::mutex> lk(m_);
      dst_ = (char *)dst; src_ = (const char *)src; bytes_ = bytes;
      remaining_ = (int)th_.size();
      generation_++;
      cv_.notify_all();
      done_.wait(lk, [&] { return remaining_ == 0; });
   }
   ~CopyPool()
   {
      {
         std::lock_guard<std::mutex> lk(m_);
         stop_ = true;
         generation_++;
      }
      cv_.notify_all();
      for (auto &t : th_) t.join();
   }

 private:
   bool start()
   {
      if (!th_.empty()) return true;
      unsigned int n = std::thread::hardware_concurrency();
      n = n < 2 ? 0 : (n > 8 ? 8 : n);
      for (unsigned int i = 0; i < n; i++) th_.emplace_back([this, i, n] { work(i, n); });
      return n > 0;
   }
   void work(unsigned int i, unsigned int n)
   {
      int seen = 0;
      for (;;)
      {
         std::unique_lock<std::mutex> lk(m_);
         cv_.wait(lk, [&] { return generation_ != seen; });
         seen = generation_;
         if (stop_) return;
         char *d = dst_; const char *s = src_; const size_t b = bytes_;
         lk.unlock();
         const size_t lo = b / n * i, hi = (i + 1 == n) ? b : b / n * (i + 1);
         memcpy(d + lo, s + lo, hi - lo);
         lk.lock();
         if (--remaining_ == 0) done_.notify_one();
      }
   }
   std::vector<std::thread> th_;
   std::mutex m_;
   std::condition_variable cv_, done_;
   char *dst_ = nullptr; const char *src_ = nullptr; size_t bytes_ = 0;
   int generation_ = 0, remaining_ = 0;
   bool stop_ = false;
};
CopyPool copy_pool;

int pinned_buffers(DeviceState &d)
{
   if (d.pin[0]) return FUSEDMM_SUCCESS_RETURN;
   for (int i = 0; i < 4; i++)
   {
      FMM_HIP(hipHostMalloc(&d.pin[i], kPinChunk, hipHostMallocDefault));
      FMM_HIP(hipEventCreateWithFlags(&d.pin_ev[i], hipEventDisableTiming));
      d.pin_busy[i] = false;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

// host -> device, enqueued on `s`; returns when the host array has been read
int upload(DeviceState &d, void *dev, const void *host, size_t bytes, hipStream_t s)
{
   if (bytes == 0) return FUSEDMM_SUCCESS_RETURN;
   if (bytes < kPinMinBytes) { FMM_HIP(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, s)); return FUSEDMM_SUCCESS_RETURN; }
   int st = pinned_buffers(d);
   if (st) return st;
   int b = 0;
   for (size_t off = 0; off < bytes; off += kPinChunk, b ^= 1)
   {
      const size_t n = bytes - off < kPinChunk ? bytes - off : kPinChunk;
      if (d.pin_busy[b]) FMM_HIP(hipEventSynchronize(d.pin_ev[b]));   // its previous DMA has drained
      copy_pool.copy(d.pin[b], (const char *)host + off, n);
      FMM_HIP(hipMemcpyAsync((char *)dev + off, d.pin[b], n, hipMemcpyHostToDevice, s));
      FMM_HIP(hipEventRecord(d.pin_ev[b], s));
      d.pin_busy[b] = true;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

// device -> host through the other two pinned buffers; returns when `host` holds the data
int download(DeviceState &d, void *host, const void *dev, size_t bytes, hipStream_t s)
{
   if (bytes == 0) return FUSEDMM_SUCCESS_RETURN;
   if (bytes < kPinMinBytes)
   {
      FMM_HIP(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, s));
      return hip_status(hipStreamSynchronize(s), "hipStreamSynchronize");
   }
   int st = pinned_buffers(d);
   if (st) return st;
   size_t prev_off = 0, prev_n = 0;
   int b = 2, prev_b = -1;
   for (size_t off = 0; off < bytes; off += kPinChunk)
   {
      const size_t n = bytes - off < kPinChunk ? bytes - off : kPinChunk;
      FMM_HIP(hipMemcpyAsync(d.pin[b], (const char *)dev + off, n, hipMemcpyDeviceToHost, s));
      FMM_HIP(hipEventRecord(d.pin_ev[b], s));
      if (prev_b >= 0)
      {
         FMM_HIP(hipEventSynchronize(d.pin_ev[prev_b]));
         copy_pool.copy((char *)host + prev_off, d.pin[prev_b], prev_n);
      }
      prev_b = b; prev_off = off; prev_n = n;
      b = (b == 2) ? 3 : 2;
   }
   FMM_HIP(hipEventSynchronize(d.pin_ev[prev_b]));
   copy_pool.copy((char *)host + prev_off, d.pin[prev_b], prev_n);
   d.pin_busy[2] = d.pin_busy[3] = false;
   return FUSEDMM_SUCCESS_RETURN;
}

// Device copy of a read-only host operand.  With the mirror cache off (the
// default) it is uploaded into the staging buffer `stage` on every call, as
// the caller may have changed it.  With the cache on, a mirror keyed by host
// address and size is kept and reused until fusedMM_amd_invalidate().
int device_copy(DeviceState &d, Buffer &stage, const void *host, size_t bytes, size_t copy_bytes, hipStream_t s, const void **out)
{
   if (!g.cache)
   {
      int st = grow(stage, bytes);
      if (st) return st;
      *out = stage.ptr;
      return upload(d, stage.ptr, host, copy_bytes, s);
   }
   for (auto &mi : d.mirrors)
      if (mi.host == host && mi.bytes == copy_bytes)
      {
         mi.last_use = ++g.cache_clock;
         *out = mi.dev;
         return FUSEDMM_SUCCESS_RETURN;
      }
   if (d.mirrors.size() >= 32)   // drop the mirror used longest ago
   {
      size_t victim = 0;
      for (size_t i = 1; i < d.mirrors.size(); i++)
         if (d.mirrors[i].last_use < d.mirrors[victim].last_use) victim = i;
      (void)hipFree(d.mirrors[victim].dev);
      d.mirrors.erase(d.mirrors.begin() + (long)victim);
   }
   void *dev = nullptr;
   FMM_HIP(hipMalloc(&dev, bytes > 0 ? bytes : 16));
   d.mirrors.push_back(DeviceState::Mirror{host, copy_bytes, dev, ++g.cache_clock});
   *out = dev;
   return upload(d, dev, host, copy_bytes, s);
}

// Host-pointer mode: copy the operands to the GPU.  On return `a` holds device
// addresses and `slots` is one past the last edge slot any processed row uses.
int stage_up(const Args &h, const Plan &pl, Args *a, int64_t *slots_out)
{
   if (h.n <= 0) { FMM_LOG("n (rows of Y) must be positive for host operands"); return FUSEDMM_FAIL_RETURN; }
   if (h.ldy < h.k || h.ldz < h.k || (pl.reads_x && h.ldx < h.k))
   {
      FMM_LOG("leading dimension smaller than k");
      return FUSEDMM_FAIL_RETURN;
   }
   if (!h.indx || !h.pntrb || !h.pntre || !h.y || !h.z || (pl.reads_x && !h.x))
   {
      FMM_LOG("NULL operand");
      return FUSEDMM_FAIL_RETURN;
   }
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   if (g.validate)
   {
      st = validate_host_pointers(h);
      if (st) return st;
   }
   int64_t slots = 0;
   for (int64_t i = 0; i < h.m; i++)
      if ((int64_t)h.pntre[i] > slots) slots = (int64_t)h.pntre[i];
   const bool need_val = pl.reads_val;
   if (need_val && !h.val) { FMM_LOG("NULL operand"); return FUSEDMM_FAIL_RETURN; }
   const size_t b_ptr = (size_t)h.m * sizeof(idx_t);
   const size_t b_idx = (size_t)(slots > 0 ? slots : 1) * sizeof(idx_t);
   const size_t b_val = (size_t)(slots > 0 ? slots : 1) * kValBytes;
   const size_t b_x = (size_t)h.m * (size_t)h.ldx * kValBytes;
   const size_t b_y = (size_t)h.n * (size_t)h.ldy * kValBytes;
   const size_t b_z = (size_t)h.m * (size_t)h.ldz * kValBytes;
   // the caller's arrays need not extend past the last element the reference reads:
   // (rows - 1) * ld + k elements, not rows * ld
   hipStream_t s = 0;
   const void *dp[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
   st = device_copy(*d, d->stage[0], h.pntrb, b_ptr, b_ptr, s, &dp[0]); if (st) return st;
   st = device_copy(*d, d->stage[1], h.pntre, b_ptr, b_ptr, s, &dp[1]); if (st) return st;
   st = device_copy(*d, d->stage[2], h.indx, b_idx, (size_t)slots * sizeof(idx_t), s, &dp[2]); if (st) return st;
   if (need_val) { st = device_copy(*d, d->stage[3], h.val, b_val, (size_t)slots * kValBytes, s, &dp[3]); if (st) return st; }
   st = device_copy(*d, d->stage[5], h.y, b_y, b_y - (size_t)(h.ldy - h.k) * kValBytes, s, &dp[5]); if (st) return st;
   if (pl.reads_x)
   {
      if ((const void *)h.x == (const void *)h.y && h.ldx == h.ldy && b_x <= b_y) dp[4] = dp[5];   // A = B: one copy serves both
      else { st = device_copy(*d, d->stage[4], h.x, b_x, b_x - (size_t)(h.ldx - h.k) * kValBytes, s, &dp[4]); if (st) return st; }
   }
   st = grow(d->stage[6], b_z); if (st) return st;
   const bool overwrite = pl.opt_rule && h.beta == 0.0f;
   if (!overwrite)   // one contiguous copy, padding columns included (they are never written back)
   {
      st = upload(*d, d->stage[6].ptr, h.z, b_z - (size_t)(h.ldz - h.k) * kValBytes, s);
      if (st) return st;
   }
   *a = h;
   a->pntrb = (const idx_t *)dp[0];
   a->pntre = (const idx_t *)dp[1];
   a->indx = (const idx_t *)dp[2];
   a->val = need_val ? (const val_t *)dp[3] : nullptr;
   a->x = pl.reads_x ? (const val_t *)dp[4] : nullptr;
   a->y = (const val_t *)dp[5];
   a->z = (val_t *)d->stage[6].ptr;
   if (a->nnz <= 0 || a->nnz > slots) a->nnz = slots;
   *slots_out = slots;
   return FUSEDMM_SUCCESS_RETURN;
}

// Only the first k columns of each Z row are written back, as the reference
// touches nothing else.  With ldz == k that is one contiguous copy; otherwise
// the block is fetched contiguously and the k columns of every row are copied
// out on the host (a strided device copy of millions of short rows is far
// slower than either).
int stage_down(const Args &h, const Args &a)
{
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   const size_t span = ((size_t)h.m * (size_t)h.ldz - (size_t)(h.ldz - h.k)) * kValBytes;
   if (h.ldz == h.k) return download(*d, h.z, a.z, span, 0);
   std::vector<val_t> tmp(span / kValBytes);
   st = download(*d, tmp.data(), a.z, span, 0);
   if (st) return st;
   for (int64_t i = 0; i < h.m; i++)
      memcpy(h.z + i * h.ldz, tmp.data() + i * h.ldz, (size_t)h.k * kValBytes);
   return FUSEDMM_SUCCESS_RETURN;
}

int run_staged(const Args &h, const Plan &pl, int sop_kind)
{
   if (h.m <= 0 || h.k < 1) return FUSEDMM_SUCCESS_RETURN;
   typedef std::chrono::steady_clock clk;
   auto ms = [](clk::time_point a, clk::time_point b) { return std::chrono::duration<double, std::milli>(b - a).count(); };
   g.phase_valid = false;
   const clk::time_point t0 = clk::now();
   Args a;
   int64_t slots = 0;
   int st = stage_up(h, pl, &a, &slots);
   if (st) return st;
   FMM_HIP(hipStreamSynchronize(0));
   const clk::time_point t1 = clk::now();
   if (g.validate)
   {
      st = validate_operands(a, 0);
      if (st) return st;
   }
   st = run_on_device(a, pl, sop_kind, 0);
   if (st) return st;
   FMM_HIP(hipStreamSynchronize(0));
   const clk::time_point t2 = clk::now();
   st = stage_down(h, a);
   if (st) return st;
   const clk::time_point t3 = clk::now();
   g.phase_ms[0] = ms(t0, t1); g.phase_ms[1] = ms(t1, t2); g.phase_ms[2] = ms(t2, t3);
   g.phase_valid = true;
   return FUSEDMM_SUCCESS_RETURN;
}

// ---- SOP_UDEF evaluated by the caller's host function ---------------------------------------
// The reference calls SOP_UDEF_FUNC once per edge from inside its kernels
// (genkern.base:487, 554; fusedMM.c:729).  Here: pass 1 on the GPU writes the
// ROP result of every edge, the host applies the function to each of them,
// pass 2 on the GPU runs the rest of the pipeline (MOP, AOP) with those
// scalars as edge values.  Synchronous; device operands `a`, host copies of
// the row pointers in h_pb / h_pe.
template <int V, int L, int R, bool EXACT, int U>
int launch_edge_scalar(const Params<idx_t> &p, val_t *s_out, int accumulate, int num_cu, hipStream_t stream)
{
   int64_t blocks = (p.m + kWavesPerBlock - 1) / kWavesPerBlock;
   if (blocks > (int64_t)num_cu * 8) blocks = (int64_t)num_cu * 8;
   hipLaunchKernelGGL((edge_scalar_kernel<V, L, R, EXACT, U, idx_t>), dim3((unsigned int)blocks), dim3(kBlockThreads), 0,
                      stream, p, s_out, accumulate);
   return hip_status(hipGetLastError(), "edge scalar launch");
}

// d_s[j] = ROP(X[i], VOP(X[i], Y[c])) for every edge slot of the processed rows,
// column slab by column slab when k exceeds what one kernel instance holds.
int edge_scalars(const Args &a, val_t *d_s, DeviceState *d, hipStream_t stream)
{
   constexpr int64_t ld_mult = 16 / (int64_t)kValBytes;
   for (int64_t off = 0; off < a.k; off += kMaxK)
   {
      const int64_t ks = a.k - off < kMaxK ? a.k - off : kMaxK;
      const val_t *xs = a.x ? a.x + off : nullptr, *ys = a.y + off;
      const bool vec_ok = (ks % 4 == 0) && (a.ldy % ld_mult == 0) && aligned16(ys) && (!xs || ((a.ldx % ld_mult == 0) && aligned16(xs)));
      Shape sh;
      int st = pick_shape((int)ks, vec_ok, &sh);
      if (st) return st;
      Params<idx_t> p;
      memset(&p, 0, sizeof(p));
      p.pntrb = a.pntrb; p.pntre = a.pntre; p.indx = a.indx; p.val = a.val;
      p.x = xs ? xs : ys;   // tuples that never read X still index it; any valid row will do
      p.y = ys; p.m = a.m; p.ldx = xs ? a.ldx : 0; p.ldy = a.ldy; p.k = (int)ks; p.imessage = a.imessage;
      st = FUSEDMM_FAIL_RETURN;
#define FMM_CASE(V_, L_, R_, X_, U_) \
   if (sh.V == V_ && sh.L == L_ && sh.R == R_ && sh.exact == X_) \
      st = launch_edge_scalar<V_, L_, R_, (X_ != 0), U_>(p, d_s, off > 0 ? 1 : 0, d->num_cu, stream);
      FMM_SHAPES(FMM_CASE)
#undef FMM_CASE
      if (st) return st;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

// FUSEDMM_VALIDATE=1 / fusedMM_amd_set_validate(1): check row pointers and
// column ids on the device before any kernel dereferences them.  Costs a pass
// over the CSR arrays and a synchronisation per call.
int validate_operands(const Args &a, hipStream_t stream, int queues)
{
   if (a.n <= 0 || !a.indx || !a.pntrb || !a.pntre)
   {
      FMM_LOG("operand check: n must be positive and the CSR arrays non-NULL");
      return FUSEDMM_FAIL_RETURN;
   }
   DeviceState *d = nullptr;
   int st = (queues == kQueuesStatic) ? device_basics(&d) : device_state(&d);
   if (st) return st;
   if (queues == kQueuesStatic) { st = scratch_setup(*d); if (st) return st; }
   Counters *ctr = (queues == kQueuesStatic) ? (Counters *)(d->scratch + kScratchCtrOff) : d->ctr;
   Params<idx_t> p;
   memset(&p, 0, sizeof(p));
   p.pntrb = a.pntrb; p.pntre = a.pntre; p.indx = a.indx; p.m = a.m;
   // the flag is one of the shared counters: wait for a call still using them on another stream
   st = order_after_previous(*d, queues, stream);
   if (st) return st;
   d->pending[queues] = true;
   d->last_stream[queues] = stream;
   unsigned int *flag = &ctr->invalid;
   FMM_HIP(hipMemsetAsync(flag, 0, sizeof(unsigned int), stream));
   int64_t blocks = (a.m + kWavesPerBlock - 1) / kWavesPerBlock;
   if (blocks > (int64_t)d->num_cu * 8) blocks = (int64_t)d->num_cu * 8;
   hipLaunchKernelGGL(validate_kernel<idx_t>, dim3((unsigned int)blocks), dim3(kBlockThreads), 0, stream, p, a.n, flag);
   unsigned int h = 0;
   FMM_HIP(hipMemcpyAsync(&h, flag, sizeof(h), hipMemcpyDeviceToHost, stream));
   FMM_HIP(hipStreamSynchronize(stream));
   if (h)
   {
      FMM_LOG("operand check failed: a column id outside [0, n) or a row with pntre < pntrb");
      return FUSEDMM_FAIL_RETURN;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

// The same check for row pointers that are host memory, before anything is sized from them.
int validate_host_pointers_of(const Args &h, const idx_t *pb, const idx_t *pe)
{
   if (!pb || !pe)
   {
      FMM_LOG("operand check: NULL row pointers");
      return FUSEDMM_FAIL_RETURN;
   }
   for (int64_t i = 0; i < h.m; i++)
      if (pb[i] < 0 || pe[i] < pb[i])
      {
         FMM_LOG("operand check failed: row %lld has pntrb=%lld, pntre=%lld", (long long)i, (long long)pb[i],
                 (long long)pe[i]);
         return FUSEDMM_FAIL_RETURN;
      }
   return FUSEDMM_SUCCESS_RETURN;
}
int validate_host_pointers(const Args &h) { return validate_host_pointers_of(h, h.pntrb, h.pntre); }

int64_t max_slot(const idx_t *h_pe, int64_t m)
{
   int64_t slots = 0;
   for (int64_t i = 0; i < m; i++)
      if ((int64_t)h_pe[i] > slots) slots = (int64_t)h_pe[i];
   return slots;
}

bool column_separable(const Plan &pl, int32_t imsg)
{
   return pl.op == OP_GCN || pl.op == OP_SPMM || (pl.op == OP_GENERIC && GET_ROP_FLAG(imsg) == ROP_NOOP);
}

// Rest of the pipeline (VOP, MOP, AOP) with per-edge scalars already in d_s.
int accumulate_with_scalars(const Args &a, val_t *d_s, hipStream_t stream)
{
   Args a2 = a;
   a2.val = d_s;
   a2.imessage = GET_VOP_FLAG(a.imessage) | ROP_NOOP | SOP_COPY | GET_VSC_FLAG(a.imessage) | GET_AOP_FLAG(a.imessage);
   Plan p2;
   int st = make_plan(a2.imessage, 0, &p2);   // general rule: accumulate (Z is cleared first when it must be overwritten)
   if (st) return st;
   return run_on_device(a2, p2, FUSEDMM_SOP_KIND_IDENTITY, stream);
}

// k > kMaxK with a reduction over the whole row (dot / distance tuples): the
// per-edge scalar is assembled from column slabs, the device SOP applied to it,
// then the accumulate stage runs slab by slab.  Synchronous (needs the largest
// edge slot, read back from the row pointers).
int run_wide_reduction(const Args &a, const Plan &pl, int sop_kind)
{
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   std::vector<idx_t> he((size_t)a.m);
   FMM_HIP(hipMemcpy(he.data(), a.pntre, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
   const int64_t slots = max_slot(he.data(), a.m);
   if (pl.opt_rule && a.beta == 0.0f)
      hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned int)(d->num_cu * 8)), dim3(kBlockThreads), 0, 0, a.z, a.m, a.k, a.ldz);
   if (slots <= 0) return FUSEDMM_SUCCESS_RETURN;
   st = grow(d->stage[7], (size_t)slots * kValBytes);
   if (st) return st;
   val_t *d_s = (val_t *)d->stage[7].ptr;
   st = edge_scalars(a, d_s, d, 0);
   if (st) return st;
   if (pl.needs_sop)
   {
      hipLaunchKernelGGL(apply_sop_kernel, dim3((unsigned int)(d->num_cu * 4)), dim3(kBlockThreads), 0, 0, d_s, slots,
                         sop_kind, (const val_t *)d->sigmoid_table);
      st = hip_status(hipGetLastError(), "apply sop launch");
      if (st) return st;
   }
   return accumulate_with_scalars(a, d_s, 0);
}

// Everything here is device memory.  Enqueues on `stream`, does not wait
// (except for wide rows with a whole-row reduction, see run_wide_reduction).
int run_on_device(const Args &a, const Plan &pl, int sop_kind, hipStream_t stream, int queues)
{
   if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
   if (a.k <= kMaxK) return run_slab(a, pl, sop_kind, stream, queues);
   if (queues == kQueuesStatic)
   {
      FMM_LOG("fusedMM_csr_stream_noalloc: k=%lld is beyond the %d columns one kernel instance holds "
              "(use fusedMM_csr_stream)", (long long)a.k, kMaxK);
      return FUSEDMM_NOT_ENOUGH_MEM;
   }
   if (a.ldy < a.k || a.ldz < a.k || (pl.reads_x && a.ldx < a.k))
   {
      FMM_LOG("leading dimension smaller than k");
      return FUSEDMM_FAIL_RETURN;
   }
   if (column_separable(pl, a.imessage))
   {
      // no stage looks across columns: every slab of kMaxK columns is a call of its own
      for (int64_t off = 0; off < a.k; off += kMaxK)
      {
         Args s = a;
         s.k = a.k - off < kMaxK ? a.k - off : kMaxK;
         s.x = a.x ? a.x + off : nullptr;
         s.y = a.y + off;
         s.z = a.z + off;
         int st = run_slab(s, pl, sop_kind, stream, queues);
         if (st) return st;
      }
      return FUSEDMM_SUCCESS_RETURN;
   }
   if (stream != 0)
   {
      FMM_LOG("k=%lld with a whole-row reduction needs the synchronous entry point", (long long)a.k);
      return FUSEDMM_FAIL_RETURN;
   }
   return run_wide_reduction(a, pl, sop_kind);
}

int run_host_sop(const Args &a, const idx_t *h_pb, const idx_t *h_pe, int64_t slots, const Plan &pl,
                 fusedMM_amd_sop_fn fn)
{
   if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   if (g.validate)   // before pass 1 dereferences a column id, and before the host indexes by the row pointers
   {
      st = validate_host_pointers_of(a, h_pb, h_pe);
      if (st) return st;
      st = validate_operands(a, 0);
      if (st) return st;
   }
   const bool overwrite = pl.opt_rule && a.beta == 0.0f;
   if (overwrite)
      hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned int)(d->num_cu * 8)), dim3(kBlockThreads), 0, 0, a.z, a.m, a.k, a.ldz);
   if (slots <= 0) return hip_status(hipStreamSynchronize(0), "hipStreamSynchronize");
   st = grow(d->stage[7], (size_t)slots * kValBytes);
   if (st) return st;
   val_t *d_s = (val_t *)d->stage[7].ptr;

   // pass 1
   st = edge_scalars(a, d_s, d, 0);
   if (st) return st;
   std::vector<val_t> hs((size_t)slots);
   FMM_HIP(hipMemcpyAsync(hs.data(), d_s, (size_t)slots * kValBytes, hipMemcpyDeviceToHost, 0));
   FMM_HIP(hipStreamSynchronize(0));

   // host SOP, rows dealt to a few threads (the function must be thread-safe, reference fusedMM.h:125-126)
   unsigned int nthreads = std::thread::hardware_concurrency();
   if (nthreads < 1) nthreads = 1;
   if (nthreads > 16) nthreads = 16;
   if ((int64_t)nthreads > a.m) nthreads = (unsigned int)a.m;
   std::vector<std::thread> pool;
   for (unsigned int t = 0; t < nthreads; t++)
      pool.emplace_back([&, t]() {
         const int64_t lo = a.m * t / nthreads, hi = a.m * (t + 1) / nthreads;
         for (int64_t i = lo; i < hi; i++)
            for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
            {
               val_t out = hs[(size_t)j];
               (void)fn(hs[(size_t)j], &out);
               hs[(size_t)j] = out;
            }
      });
   for (auto &th : pool) th.join();
   FMM_HIP(hipMemcpyAsync(d_s, hs.data(), (size_t)slots * kValBytes, hipMemcpyHostToDevice, 0));

   // pass 2: same VOP / MOP / AOP, the scalar comes in as the edge value
   st = accumulate_with_scalars(a, d_s, 0);
   if (st) return st;
   return hip_status(hipStreamSynchronize(0), "hipStreamSynchronize");
}

// ---- VOP / ROP / VSC / AOP evaluated by the caller's host functions ---------------------------
// The reference calls the five stage functions once per edge (fusedMM.c:696-740):
//    VOP(k, X[i], k, Y[c], k, T); ROP(k, X[i], k, T, &scal); SOP(scal, &out); VSC(k, T, out, k, T); AOP(k, T, k, Z[i])
// with scal starting as the edge value.  Here T and the scalar of every edge slot live
// in device buffers; a built-in stage is a kernel over them, a *_UDEF stage is a host
// pass (the buffers are copied to the host, the caller's function is applied edge by
// edge -- rows dealt to a few threads, the accumulate stage in edge order within a row
// -- and copied back), so any mix of built-in and user stages is served and only the
// user's functions run on the CPU.  Synchronous; device operands `a`, host copies of
// the row pointers in h_pb / h_pe.
struct StageFns {
   fusedMM_amd_vop_fn vop;
   fusedMM_amd_rop_fn rop;
   fusedMM_amd_sop_fn sop;
   fusedMM_amd_vsc_fn vsc;
   fusedMM_amd_aop_fn aop;
};

template <class F>
void for_row_ranges(int64_t m, F body)
{
   unsigned int nthreads = std::thread::hardware_concurrency();
   if (nthreads < 1) nthreads = 1;
   if (nthreads > 16) nthreads = 16;
   if ((int64_t)nthreads > m) nthreads = (unsigned int)(m > 0 ? m : 1);
   std::vector<std::thread> pool;
   for (unsigned int t = 0; t < nthreads; t++)
      pool.emplace_back([&, t]() { body(m * t / nthreads, m * (t + 1) / nthreads); });
   for (auto &th : pool) th.join();
}

int run_host_stages(const Args &a, const idx_t *h_pb, const idx_t *h_pe, int64_t slots, const Plan &pl, const StageFns &f,
                    int sop_kind)
{
   if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   if (a.ldy < a.k || a.ldz < a.k || (pl.reads_x && a.ldx < a.k))
   {
      FMM_LOG("leading dimension smaller than k");
      return FUSEDMM_FAIL_RETURN;
   }
   if (!a.indx || !a.pntrb || !a.pntre || !a.y || !a.z || (pl.reads_x && !a.x))
   {
      FMM_LOG("NULL operand");
      return FUSEDMM_FAIL_RETURN;
   }
   if (g.validate)
   {
      st = validate_host_pointers_of(a, h_pb, h_pe);
      if (st) return st;
      st = validate_operands(a, 0);
      if (st) return st;
   }
   if (slots <= 0) return FUSEDMM_SUCCESS_RETURN;   // no processed row has an edge: Z is left alone (general rule)
   const int vop = GET_VOP_FLAG(a.imessage), rop = GET_ROP_FLAG(a.imessage), sop = GET_SOP_FLAG(a.imessage),
             vsc = GET_VSC_FLAG(a.imessage), aop = GET_AOP_FLAG(a.imessage);
   const int64_t m = a.m, k = a.k;
   const size_t nT = (size_t)slots * (size_t)k;
   st = grow(d->edge_t, nT * kValBytes); if (st) return st;
   st = grow(d->stage[7], (size_t)slots * kValBytes); if (st) return st;
   val_t *d_T = (val_t *)d->edge_t.ptr, *d_s = (val_t *)d->stage[7].ptr;

   Params<idx_t> p;
   memset(&p, 0, sizeof(p));
   p.pntrb = a.pntrb; p.pntre = a.pntre; p.indx = a.indx; p.val = a.val;
   p.x = a.x ? a.x : a.y;   // built-in stages that never read X still index it; any valid row will do
   p.y = a.y; p.z = a.z; p.m = m; p.ldx = a.x ? a.ldx : 0; p.ldy = a.ldy; p.ldz = a.ldz; p.k = (int)k;
   p.imessage = a.imessage;
   int64_t blocks = (m + kWavesPerBlock - 1) / kWavesPerBlock;
   if (blocks > (int64_t)d->num_cu * 8) blocks = (int64_t)d->num_cu * 8;
   const dim3 grid((unsigned int)blocks), block(kBlockThreads);

   // host copies, made when a host stage first needs them
   std::vector<val_t> hT, hs, hX, hY, hZ;
   std::vector<idx_t> hidx;
   bool T_dev = false, T_host = false, s_dev = false, s_host = false;
   auto need_T_host = [&]() -> int {
      if (T_host) return FUSEDMM_SUCCESS_RETURN;
      hT.resize(nT);
      if (T_dev) FMM_HIP(hipMemcpy(hT.data(), d_T, nT * kValBytes, hipMemcpyDeviceToHost));
      T_host = true;
      return FUSEDMM_SUCCESS_RETURN;
   };
   auto need_T_dev = [&]() -> int {
      if (T_dev) return FUSEDMM_SUCCESS_RETURN;
      if (T_host) FMM_HIP(hipMemcpy(d_T, hT.data(), nT * kValBytes, hipMemcpyHostToDevice));
      T_dev = true;
      return FUSEDMM_SUCCESS_RETURN;
   };
   auto need_s_host = [&]() -> int {
      if (s_host) return FUSEDMM_SUCCESS_RETURN;
      hs.resize((size_t)slots);
      if (s_dev) FMM_HIP(hipMemcpy(hs.data(), d_s, (size_t)slots * kValBytes, hipMemcpyDeviceToHost));
      s_host = true;
      return FUSEDMM_SUCCESS_RETURN;
   };
   auto need_s_dev = [&]() -> int {
      if (s_dev) return FUSEDMM_SUCCESS_RETURN;
      if (s_host) FMM_HIP(hipMemcpy(d_s, hs.data(), (size_t)slots * kValBytes, hipMemcpyHostToDevice));
      s_dev = true;
      return FUSEDMM_SUCCESS_RETURN;
   };
   auto need_X_host = [&]() -> int {
      if (!hX.empty()) return FUSEDMM_SUCCESS_RETURN;
      hX.resize((size_t)(m - 1) * (size_t)a.ldx + (size_t)k);
      FMM_HIP(hipMemcpy(hX.data(), a.x, hX.size() * kValBytes, hipMemcpyDeviceToHost));
      return FUSEDMM_SUCCESS_RETURN;
   };

   // ---- VOP
   if (pl.udef_stages & kUdefVop)
   {
      st = need_X_host(); if (st) return st;
      hidx.resize((size_t)slots);
      FMM_HIP(hipMemcpy(hidx.data(), a.indx, (size_t)slots * sizeof(idx_t), hipMemcpyDeviceToHost));
      // the host function is handed rows of a host copy of Y: as many rows as the processed edges reach
      // (n is not trusted: the reference never reads it)
      int64_t y_rows = 0;
      for (int64_t i = 0; i < m; i++)
         for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
         {
            const int64_t c = (int64_t)hidx[(size_t)j];
            if (c < 0)
            {
               FMM_LOG("negative column id %lld in row %lld", (long long)c, (long long)i);
               return FUSEDMM_FAIL_RETURN;
            }
            if (c >= y_rows) y_rows = c + 1;
         }
      if (y_rows > 0)
      {
         hY.resize((size_t)(y_rows - 1) * (size_t)a.ldy + (size_t)k);
         FMM_HIP(hipMemcpy(hY.data(), a.y, hY.size() * kValBytes, hipMemcpyDeviceToHost));
      }
      hT.assign(nT, (val_t)0);
      for_row_ranges(m, [&](int64_t lo, int64_t hi) {
         for (int64_t i = lo; i < hi; i++)
            for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
               (void)f.vop((idx_t)k, hX.data() + i * a.ldx, (idx_t)k, hY.data() + (int64_t)hidx[(size_t)j] * a.ldy, (idx_t)k,
                           hT.data() + (size_t)j * (size_t)k);
      });
      T_host = true;
   }
   else
   {
      hipLaunchKernelGGL(stage_vop_kernel<idx_t>, grid, block, 0, 0, p, d_T);
      st = hip_status(hipGetLastError(), "stage kernel launch"); if (st) return st;
      T_dev = true;
   }

   // ---- ROP: the scalar starts as the edge value (fusedMM.c:717)
   if (a.val) FMM_HIP(hipMemcpyAsync(d_s, a.val, (size_t)slots * kValBytes, hipMemcpyDeviceToDevice, 0));
   else FMM_HIP(hipMemsetAsync(d_s, 0, (size_t)slots * kValBytes, 0));
   s_dev = true;
   if (pl.udef_stages & kUdefRop)
   {
      st = need_X_host(); if (st) return st;
      st = need_T_host(); if (st) return st;
      st = need_s_host(); if (st) return st;
      for_row_ranges(m, [&](int64_t lo, int64_t hi) {
         for (int64_t i = lo; i < hi; i++)
            for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
               (void)f.rop((idx_t)k, hX.data() + i * a.ldx, (idx_t)k, hT.data() + (size_t)j * (size_t)k, &hs[(size_t)j]);
      });
      s_dev = false;
   }
   else if (rop != ROP_NOOP)
   {
      st = need_T_dev(); if (st) return st;
      hipLaunchKernelGGL(stage_rop_kernel<idx_t>, grid, block, 0, 0, p, (const val_t *)d_T, d_s);
      st = hip_status(hipGetLastError(), "stage kernel launch"); if (st) return st;
   }

   // ---- SOP
   if (sop == SOP_UDEF && vsc != VSC_NOOP)
   {
      if (sop_kind == FUSEDMM_SOP_KIND_HOST)
      {
         st = need_s_host(); if (st) return st;
         for_row_ranges(m, [&](int64_t lo, int64_t hi) {
            for (int64_t i = lo; i < hi; i++)
               for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
               {
                  val_t out = hs[(size_t)j];
                  (void)f.sop(hs[(size_t)j], &out);
                  hs[(size_t)j] = out;
               }
         });
         s_dev = false;
      }
      else
      {
         st = need_s_dev(); if (st) return st;
         hipLaunchKernelGGL(apply_sop_kernel, dim3((unsigned int)(d->num_cu * 4)), block, 0, 0, d_s, slots, sop_kind,
                            (const val_t *)d->sigmoid_table);
         st = hip_status(hipGetLastError(), "apply sop launch"); if (st) return st;
         s_host = false;
      }
   }

   // ---- VSC
   if (pl.udef_stages & kUdefVsc)
   {
      st = need_T_host(); if (st) return st;
      st = need_s_host(); if (st) return st;
      for_row_ranges(m, [&](int64_t lo, int64_t hi) {
         for (int64_t i = lo; i < hi; i++)
            for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
            {
               val_t *t = hT.data() + (size_t)j * (size_t)k;
               (void)f.vsc((idx_t)k, t, hs[(size_t)j], (idx_t)k, t);
            }
      });
      T_dev = false;
   }
   else if (vsc != VSC_NOOP)
   {
      st = need_T_dev(); if (st) return st;
      st = need_s_dev(); if (st) return st;
      hipLaunchKernelGGL(stage_vsc_kernel<idx_t>, grid, block, 0, 0, p, d_T, (const val_t *)d_s);
      st = hip_status(hipGetLastError(), "stage kernel launch"); if (st) return st;
      T_host = false;
   }

   // ---- AOP
   if (pl.udef_stages & kUdefAop)
   {
      st = need_T_host(); if (st) return st;
      hZ.resize((size_t)(m - 1) * (size_t)a.ldz + (size_t)k);
      FMM_HIP(hipMemcpy(hZ.data(), a.z, hZ.size() * kValBytes, hipMemcpyDeviceToHost));
      for_row_ranges(m, [&](int64_t lo, int64_t hi) {
         for (int64_t i = lo; i < hi; i++)
            for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)   // in edge order: the function folds into Z[i]
               (void)f.aop((idx_t)k, hT.data() + (size_t)j * (size_t)k, (idx_t)k, hZ.data() + i * a.ldz);
      });
      FMM_HIP(hipMemcpy(a.z, hZ.data(), hZ.size() * kValBytes, hipMemcpyHostToDevice));
   }
   else if (aop != AOP_NOOP)
   {
      st = need_T_dev(); if (st) return st;
      hipLaunchKernelGGL(stage_aop_kernel<idx_t>, grid, block, 0, 0, p, (const val_t *)d_T);
      st = hip_status(hipGetLastError(), "stage kernel launch"); if (st) return st;
   }
   return hip_status(hipStreamSynchronize(0), "hipStreamSynchronize");
}

fusedMM_amd_sop_fn host_sop_function()
{
   if (g.sop_fn) return g.sop_fn;
   return (fusedMM_amd_sop_fn)dlsym(RTLD_DEFAULT, "SOP_UDEF_FUNC");
}

int entry(const Args &a, bool async, hipStream_t stream, int queues = kQueuesGrown)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   Plan pl;
   int st = make_plan(a.imessage, g.opt, &pl);
   if (st) return st;
   int sop_kind = g.sop_kind;
   if (pl.udef_stages)
   {
      // stages that are the caller's host functions: registered, or found by the names the reference binds
      StageFns f;
      f.vop = g.vop_fn ? g.vop_fn : (fusedMM_amd_vop_fn)dlsym(RTLD_DEFAULT, "VOP_UDEF_FUNC");
      f.rop = g.rop_fn ? g.rop_fn : (fusedMM_amd_rop_fn)dlsym(RTLD_DEFAULT, "ROP_UDEF_FUNC");
      f.vsc = g.vsc_fn ? g.vsc_fn : (fusedMM_amd_vsc_fn)dlsym(RTLD_DEFAULT, "VSC_UDEF_FUNC");
      f.aop = g.aop_fn ? g.aop_fn : (fusedMM_amd_aop_fn)dlsym(RTLD_DEFAULT, "AOP_UDEF_FUNC");
      f.sop = nullptr;
      if (((pl.udef_stages & kUdefVop) && !f.vop) || ((pl.udef_stages & kUdefRop) && !f.rop) ||
          ((pl.udef_stages & kUdefVsc) && !f.vsc) || ((pl.udef_stages & kUdefAop) && !f.aop))
      {
         // what the reference's default build does with such a tuple: its stubs return this code (fusedMM_internal.h:50-84)
         FMM_LOG("the op tuple 0x%x names a *_UDEF stage for which the process defines no <STAGE>_UDEF_FUNC "
                 "(and none was registered with fusedMM_amd_set_stage_callbacks)", a.imessage);
         return FUSEDMM_UNDEFINED_USER_FUNCTION;
      }
      if (pl.needs_sop && sop_kind == FUSEDMM_SOP_KIND_HOST && GET_VSC_FLAG(a.imessage) != VSC_NOOP)
      {
         f.sop = host_sop_function();
         if (!f.sop)
         {
            FMM_LOG("SOP_UDEF: no host SOP_UDEF_FUNC found and no device body selected "
                    "(fusedMM_amd_set_sop_kind / FUSEDMM_SOP_KIND)");
            return FUSEDMM_UNDEFINED_USER_FUNCTION;
         }
      }
      if (async)
      {
         FMM_LOG("a stage evaluated by a host function needs the synchronous entry point");
         return FUSEDMM_UNDEFINED_USER_FUNCTION;
      }
      if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
      if (!a.val) pl.reads_val = false;
      const int where = operand_residence(a);
      if (where < 0) return FUSEDMM_FAIL_RETURN;
      if (where == 1)
      {
         std::vector<idx_t> hb((size_t)a.m), he((size_t)a.m);
         FMM_HIP(hipMemcpy(hb.data(), a.pntrb, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
         FMM_HIP(hipMemcpy(he.data(), a.pntre, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
         return run_host_stages(a, hb.data(), he.data(), max_slot(he.data(), a.m), pl, f, sop_kind);
      }
      Args dv;
      int64_t slots = 0;
      st = stage_up(a, pl, &dv, &slots);
      if (st) return st;
      st = run_host_stages(dv, a.pntrb, a.pntre, slots, pl, f, sop_kind);
      if (st) return st;
      return stage_down(a, dv);
   }
   if (pl.needs_sop && sop_kind == FUSEDMM_SOP_KIND_HOST)
   {
      if (GET_VSC_FLAG(a.imessage) == VSC_NOOP)
         sop_kind = FUSEDMM_SOP_KIND_IDENTITY;   // the SOP result is never used
      else
      {
         fusedMM_amd_sop_fn fn = host_sop_function();
         if (!fn)
         {
            FMM_LOG("SOP_UDEF: no host SOP_UDEF_FUNC found and no device body selected "
                    "(fusedMM_amd_set_sop_kind / FUSEDMM_SOP_KIND)");
            return FUSEDMM_UNDEFINED_USER_FUNCTION;
         }
         if (async)
         {
            FMM_LOG("SOP_UDEF through a host function needs the synchronous entry point");
            return FUSEDMM_UNDEFINED_USER_FUNCTION;
         }
         if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
         const int where = operand_residence(a);
         if (where < 0) return FUSEDMM_FAIL_RETURN;
         if (where == 1)
         {
            std::vector<idx_t> hb((size_t)a.m), he((size_t)a.m);
            FMM_HIP(hipMemcpy(hb.data(), a.pntrb, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
            FMM_HIP(hipMemcpy(he.data(), a.pntre, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
            int64_t slots = 0;
            for (int64_t i = 0; i < a.m; i++) if ((int64_t)he[(size_t)i] > slots) slots = (int64_t)he[(size_t)i];
            return run_host_sop(a, hb.data(), he.data(), slots, pl, fn);
         }
         Args dv;
         int64_t slots = 0;
         st = stage_up(a, pl, &dv, &slots);
         if (st) return st;
         st = run_host_sop(dv, a.pntrb, a.pntre, slots, pl, fn);
         if (st) return st;
         return stage_down(a, dv);
      }
   }
   if (async)
   {
      if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
      if (g.validate)
      {
         // the check reads a flag back and waits for it: impossible inside a capture
         bool capturing = false;
         st = stream_capturing(stream, &capturing);
         if (st) return st;
         if (capturing)
         {
            FMM_LOG("operand validation is switched on and the stream is being captured; "
                    "validate once outside the capture, then switch it off (fusedMM_amd_set_validate(0))");
            return FUSEDMM_FAIL_RETURN;
         }
         st = validate_operands(a, stream, queues);
         if (st) return st;
      }
      return run_on_device(a, pl, sop_kind, stream, queues);
   }
   if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
   const int where = operand_residence(a);
   if (where < 0) return FUSEDMM_FAIL_RETURN;
   if (where == 1)
   {
      if (g.validate)
      {
         st = validate_operands(a, 0);
         if (st) return st;
      }
      st = run_on_device(a, pl, sop_kind, 0);
      if (st) return st;
      return hip_status(hipStreamSynchronize(0), "hipStreamSynchronize");
   }
   return run_staged(a, pl, sop_kind);
}

}  // namespace

// ---- exported C ABI -------------------------------------------------------------------
extern "C" {

int fusedMM_csr(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
                const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
                const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
                const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz)
{
   (void)alpha; (void)rows; (void)cols;
   Args a = {imessage, (int64_t)m, (int64_t)n, (int64_t)k, (int64_t)nnz, val, indx, pntrb, pntre, x, y, z,
             (int64_t)ldx, (int64_t)ldy, (int64_t)ldz, beta};
   return entry(a, false, 0);
}

int fusedMM_csr_stream(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
                       const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
                       const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                       const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
                       const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz, void *stream)
{
   (void)alpha; (void)rows; (void)cols;
   Args a = {imessage, (int64_t)m, (int64_t)n, (int64_t)k, (int64_t)nnz, val, indx, pntrb, pntre, x, y, z,
             (int64_t)ldx, (int64_t)ldy, (int64_t)ldz, beta};
   return entry(a, true, (hipStream_t)stream);
}

int fusedMM_csr_stream_noalloc(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
                               const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
                               const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                               const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
                               const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz, void *stream)
{
   (void)alpha; (void)rows; (void)cols;
   Args a = {imessage, (int64_t)m, (int64_t)n, (int64_t)k, (int64_t)nnz, val, indx, pntrb, pntre, x, y, z,
             (int64_t)ldx, (int64_t)ldy, (int64_t)ldz, beta};
   return entry(a, true, (hipStream_t)stream, kQueuesStatic);
}

int fusedMM_amd_init(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   return scratch_setup(*d);
}

int64_t fusedMM_amd_noalloc_capacity(void) { return (int64_t)FUSEDMM_AMD_SCRATCH_BYTES; }

#ifdef FMM_DOUBLE
#define FMM_GFUSEDMM dgfusedMM_csr
#else
#define FMM_GFUSEDMM sgfusedMM_csr
#endif
void FMM_GFUSEDMM(const char tkern, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k, const VALUETYPE alpha,
                  const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols, const VALUETYPE *val,
                  const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre, const VALUETYPE *a,
                  const INDEXTYPE lda, const VALUETYPE *b, const INDEXTYPE ldb, const VALUETYPE beta, VALUETYPE *c,
                  const INDEXTYPE ldc)
{
   int32_t imsg;
   switch (tkern)
   {
      case 'g': imsg = VOP_COPY_RHS | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_ADD; break;
      case 'm': imsg = VOP_COPY_RHS | ROP_NOOP | SOP_COPY | VSC_MUL | AOP_ADD; break;
      case 's': imsg = VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD; break;
      case 't': imsg = VOP_SUBR | ROP_NORMR | SOP_UDEF | VSC_MUL | AOP_ADD; break;
      default:
         fprintf(stderr, "unknown kernel type!\n");   // reference kernels.c:627-629 only prints
         return;
   }
   (void)fusedMM_csr(imsg, m, n, k, alpha, nnz, rows, cols, val, indx, pntrb, pntre, a, lda, b, ldb, beta, c, ldc);
}

int fusedMM_amd_index_bytes(void) { return (int)sizeof(INDEXTYPE); }

int fusedMM_amd_value_bytes(void) { return (int)sizeof(VALUETYPE); }

int fusedMM_amd_set_sop_kind(int kind)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   if (kind < FUSEDMM_SOP_KIND_HOST || kind > FUSEDMM_SOP_KIND_FA) return -2;
   int prev = g.sop_kind;
   g.sop_kind = kind;
   return prev;
}

int fusedMM_amd_get_sop_kind(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   return g.sop_kind;
}

void fusedMM_amd_set_sop_callback(fusedMM_amd_sop_fn fn)
{
   std::lock_guard<std::mutex> lock(g.mu);
   g.sop_fn = fn;
}

void fusedMM_amd_set_stage_callbacks(fusedMM_amd_vop_fn vop, fusedMM_amd_rop_fn rop, fusedMM_amd_vsc_fn vsc,
                                     fusedMM_amd_aop_fn aop)
{
   std::lock_guard<std::mutex> lock(g.mu);
   g.vop_fn = vop;
   g.rop_fn = rop;
   g.vsc_fn = vsc;
   g.aop_fn = aop;
}

int fusedMM_amd_set_opt(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   int prev = g.opt;
   g.opt = enable < 0 ? 0 : (enable > 2 ? 2 : enable);
   return prev;
}

int fusedMM_amd_set_cache(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   int prev = g.cache;
   g.cache = enable ? 1 : 0;
   return prev;
}

void fusedMM_amd_invalidate(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   int cur = 0;
   if (hipGetDevice(&cur) != hipSuccess) return;
   for (int dev = 0; dev < kMaxDevices; dev++)
   {
      DeviceState &d = g.dev[dev];
      if (d.mirrors.empty()) continue;
      if (hipSetDevice(dev) != hipSuccess) continue;
      (void)hipDeviceSynchronize();
      for (auto &mi : d.mirrors) (void)hipFree(mi.dev);
      d.mirrors.clear();
   }
   (void)hipSetDevice(cur);
}

int fusedMM_amd_last_host_phases(double *upload_ms, double *kernels_ms, double *download_ms)
{
   std::lock_guard<std::mutex> lock(g.mu);
   if (!g.phase_valid) return FUSEDMM_FAIL_RETURN;
   if (upload_ms) *upload_ms = g.phase_ms[0];
   if (kernels_ms) *kernels_ms = g.phase_ms[1];
   if (download_ms) *download_ms = g.phase_ms[2];
   return FUSEDMM_SUCCESS_RETURN;
}

int fusedMM_amd_set_validate(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   int prev = g.validate;
   g.validate = enable ? 1 : 0;
   return prev;
}

void fusedMM_amd_set_split(int64_t heavy_deg, int seg_len)
{
   std::lock_guard<std::mutex> lock(g.mu);
   g.heavy_deg = heavy_deg > 0 ? heavy_deg : 0;
   g.seg_len = seg_len > 0 ? seg_len : 0;
}

void fusedMM_amd_timing(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   g.timing = enable > 0 ? enable : 0;
   g.timing_seen = 0;
   g.timing_calls = 0;
   if (g.timing > 0)
   {
      // the events are made here, on the current device, not inside the first timed call
      DeviceState *d = nullptr;
      if (device_basics(&d) == FUSEDMM_SUCCESS_RETURN && !d->ev_made)
      {
         bool ok = true;
         for (int i = 0; i < kTimingSlots && ok; i++)
            for (int e = 0; e < 4 && ok; e++) ok = (hipEventCreate(&d->ev[i][e]) == hipSuccess);
         d->ev_made = ok;
      }
   }
}

int fusedMM_amd_timing_summary(double *classify_ms, double *fused_ms, double *merge_ms)
{
   std::lock_guard<std::mutex> lock(g.mu);
   double t[3] = {0, 0, 0};
   int n = g.timing_calls;
   if (n > 0)
   {
      DeviceState &d = g.dev[g.timing_dev];
      if (hipEventSynchronize(d.ev[n - 1][3]) != hipSuccess) return -1;
      for (int i = 0; i < n; i++)
         for (int e = 0; e < 3; e++)
         {
            float ms = 0.f;
            if (hipEventElapsedTime(&ms, d.ev[i][e], d.ev[i][e + 1]) != hipSuccess) return -1;
            t[e] += ms;
         }
   }
   if (classify_ms) *classify_ms = t[0];
   if (fused_ms) *fused_ms = t[1];
   if (merge_ms) *merge_ms = t[2];
   return n;
}

int fusedMM_amd_timing_call(int i, double *classify_ms, double *fused_ms, double *merge_ms)
{
   std::lock_guard<std::mutex> lock(g.mu);
   if (i < 0 || i >= g.timing_calls) return FUSEDMM_FAIL_RETURN;
   DeviceState &d = g.dev[g.timing_dev];
   if (hipEventSynchronize(d.ev[i][3]) != hipSuccess) return FUSEDMM_FAIL_RETURN;
   double *out[3] = {classify_ms, fused_ms, merge_ms};
   for (int e = 0; e < 3; e++)
   {
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, d.ev[i][e], d.ev[i][e + 1]) != hipSuccess) return FUSEDMM_FAIL_RETURN;
      if (out[e]) *out[e] = ms;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

int fusedMM_amd_last_split(unsigned int *heavy_rows, unsigned int *segments, unsigned int *overflow)
{
   std::lock_guard<std::mutex> lock(g.mu);
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   Counters c;
   memset(&c, 0, sizeof(c));
   FMM_HIP(hipDeviceSynchronize());
   if (d->last_ctr) FMM_HIP(hipMemcpy(&c, d->last_ctr, sizeof(c), hipMemcpyDeviceToHost));
   if (heavy_rows) *heavy_rows = c.last_heavy;
   if (segments) *segments = c.last_seg;
   if (overflow) *overflow = c.last_overflow;
   return FUSEDMM_SUCCESS_RETURN;
}

int fusedMM_amd_last_row_order(int *scattered, unsigned int *edges_lower_half, unsigned int *edges_upper_half)
{
   std::lock_guard<std::mutex> lock(g.mu);
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   Counters c;
   memset(&c, 0, sizeof(c));
   FMM_HIP(hipDeviceSynchronize());
   if (d->last_ctr) FMM_HIP(hipMemcpy(&c, d->last_ctr, sizeof(c), hipMemcpyDeviceToHost));
   if (scattered) *scattered = (int)c.last_scattered;
   if (edges_lower_half) *edges_lower_half = (unsigned int)(c.last_skew & 0xFFFFFFFFull);
   if (edges_upper_half) *edges_upper_half = (unsigned int)(c.last_skew >> 32);
   return FUSEDMM_SUCCESS_RETURN;
}

int fusedMM_amd_copy_probe(void *dst, const void *src, int64_t bytes, void *stream)
{
   if (!dst || !src || bytes < 16 || (bytes & 15) || !aligned16(dst) || !aligned16(src)) return FUSEDMM_FAIL_RETURN;
   std::lock_guard<std::mutex> lock(g.mu);
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   hipLaunchKernelGGL(copy_probe_kernel, dim3((unsigned int)(d->num_cu * 8)), dim3(kBlockThreads), 0, (hipStream_t)stream,
                      (float4 *)dst, (const float4 *)src, bytes / 16);
   return hip_status(hipGetLastError(), "copy probe launch");
}

int fusedMM_amd_read_probe(const void *src, int64_t bytes, int blocks_per_cu, int in_flight, int nontemporal,
                           void *sink, void *stream)
{
   if (!src || !sink || bytes < 16 || (bytes & 15) || !aligned16(src)) return FUSEDMM_FAIL_RETURN;
   std::lock_guard<std::mutex> lock(g.mu);
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   if (blocks_per_cu < 1) blocks_per_cu = 8;
   const dim3 grid((unsigned int)(d->num_cu * blocks_per_cu)), block(kBlockThreads);
   const probe16_t *s4 = (const probe16_t *)src;
   unsigned int *out = (unsigned int *)sink;
   const int64_t n16 = bytes / 16;
   hipStream_t hs = (hipStream_t)stream;
#define FMM_PROBE(U_)                                                                                     \
   if (nontemporal) hipLaunchKernelGGL((read_probe_kernel<U_, true>), grid, block, 0, hs, s4, n16, out);  \
   else hipLaunchKernelGGL((read_probe_kernel<U_, false>), grid, block, 0, hs, s4, n16, out)
   if (in_flight >= 16) { FMM_PROBE(16); }
   else if (in_flight >= 8) { FMM_PROBE(8); }
   else if (in_flight >= 4) { FMM_PROBE(4); }
   else { FMM_PROBE(2); }
#undef FMM_PROBE
   return hip_status(hipGetLastError(), "read probe launch");
}

int fusedMM_amd_gather_probe(const void *src, int row_bytes, const unsigned int *ids, int64_t n_ids, int blocks_per_cu,
                             int in_flight, int nontemporal, void *sink, void *stream)
{
   if (!src || !ids || !sink || n_ids < 1 || !aligned16(src)) return FUSEDMM_FAIL_RETURN;
   if (row_bytes < 16 || row_bytes > 2048 || (row_bytes & (row_bytes - 1))) return FUSEDMM_FAIL_RETURN;
   std::lock_guard<std::mutex> lock(g.mu);
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   if (blocks_per_cu < 1) blocks_per_cu = 4;
   const dim3 grid((unsigned int)(d->num_cu * blocks_per_cu)), block(kBlockThreads);
   const probe16_t *s4 = (const probe16_t *)src;
   unsigned int *out = (unsigned int *)sink;
   const int row16 = row_bytes / 16;
   hipStream_t hs = (hipStream_t)stream;
#define FMM_GPROBE(U_, R_)                                                                                              \
   if (nontemporal) hipLaunchKernelGGL((gather_probe_kernel<U_, R_, true>), grid, block, 0, hs, s4, row16, ids, n_ids, out); \
   else hipLaunchKernelGGL((gather_probe_kernel<U_, R_, false>), grid, block, 0, hs, s4, row16, ids, n_ids, out)
   if (row16 > 64)   // 2 KiB rows: two pieces per lane
   {
      if (in_flight >= 8) { FMM_GPROBE(8, 2); }
      else { FMM_GPROBE(4, 2); }
   }
   else if (in_flight >= 16) { FMM_GPROBE(16, 1); }
   else if (in_flight >= 8) { FMM_GPROBE(8, 1); }
   else { FMM_GPROBE(4, 1); }
#undef FMM_GPROBE
   return hip_status(hipGetLastError(), "gather probe launch");
}

void fusedMM_amd_finalize(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   int cur = 0;
   if (hipGetDevice(&cur) != hipSuccess) return;
   for (int dev = 0; dev < kMaxDevices; dev++)
   {
      DeviceState &d = g.dev[dev];
      if (!d.basics) continue;
      if (hipSetDevice(dev) != hipSuccess) continue;
      (void)hipDeviceSynchronize();
      for (int q = 0; q < 2; q++) (void)hipEventDestroy(d.order_ev[q]);
      if (d.sigmoid_table) (void)hipFree(d.sigmoid_table);
      if (d.ctr) (void)hipFree(d.ctr);
      Buffer *bufs[] = {&d.heavy, &d.segs, &d.partial, &d.queued};
      for (Buffer *b : bufs) { if (b->ptr) (void)hipFree(b->ptr); *b = Buffer(); }
      for (Buffer &b : d.stage) { if (b.ptr) (void)hipFree(b.ptr); b = Buffer(); }
      if (d.edge_t.ptr) (void)hipFree(d.edge_t.ptr);
      for (auto &mi : d.mirrors) (void)hipFree(mi.dev);
      d.mirrors.clear();
      if (d.pin[0])
         for (int i = 0; i < 4; i++) { (void)hipHostFree(d.pin[i]); (void)hipEventDestroy(d.pin_ev[i]); }
      if (d.ev_made)
         for (int i = 0; i < kTimingSlots; i++)
            for (int e = 0; e < 4; e++) (void)hipEventDestroy(d.ev[i][e]);
      d = DeviceState();   // also forgets the static array's address: its head is cleared again on next use
   }
   (void)hipSetDevice(cur);
}

}  // extern "C"
