// Host side of libfusedmm_amd_*.so, shared by its translation units:
//
//   fusedmm_state.hip        per-device state, environment, work queues, the static array
//   fusedmm_dispatch.hip     op tuple -> plan, kernel shape, one call of the kernels, column slabs
//   fusedmm_launch.hip       the fused kernel's instances, one object per op (-DFMM_LAUNCH_UNIT=n)
//   fusedmm_staging.hip      host-pointer mode: pinned staging, mirrors of read-only operands
//   fusedmm_host_stages.hip  SOP/VOP/ROP/VSC/AOP_UDEF through the caller's host functions
//   fusedmm_exports.hip      the entry points (extern "C")
//
// Replaces the dispatch of the reference's fusedMM.c:487-744 and
// kernels/src/kernels.c:456-631.  Built once per (INDEXTYPE, VALUETYPE).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
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
// the library is compiled with hidden visibility: only what the public headers declare is exported
#pragma GCC visibility push(default)
#include "../../include/fusedMM.h"
#include "../../include/fusedmm_amd.h"
#pragma GCC visibility pop
#include "fusedmm_kernels.h"

namespace fmm_host {

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
   bool env_read = false;
   int opt = 1;
   int64_t heavy_deg = 0;
   int seg_len = 0;
   int blocks_per_cu = 0;
   int validate = 0;
   int row_order = 0;         // 0 auto, 1 first to last, 2 scattered stretches (FUSEDMM_ROW_ORDER)
   int pack = 0;              // short rows one per sub-wave: 0 auto, 1 never, 2 always where the shape allows (FUSEDMM_PACK_ROWS)
   int store_shift = -1;      // finished Z rows leave together when the 100 MHz clock >> this changes: -1 auto, 0 never (FUSEDMM_STORE_TICK)
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
extern Globals g;

// ---- fusedmm_state.hip ------------------------------------------------------------
void read_env_once();
void build_sigmoid_table(val_t *t);
int grow(Buffer &b, size_t bytes, bool capturing = false);
int device_basics(DeviceState **out);   // allocates no device memory
int device_state(DeviceState **out);    // table and counters of the ordinary entry points
int scratch_setup(DeviceState &d);      // the static array of the entry point that allocates nothing
int order_after_previous(DeviceState &d, int queues, hipStream_t stream);
int stream_capturing(hipStream_t stream, bool *capturing);
void release_device(DeviceState &d);    // everything the library holds on the current device

// the static array: fixed head, then the queues of the call in progress
constexpr size_t align256(size_t v) { return (v + 255u) & ~(size_t)255u; }
#define FUSEDMM_AMD_SCRATCH_BYTES (32u << 20)
constexpr size_t kScratchTableOff = 0;
constexpr size_t kScratchCtrOff = align256(kSigmoidTableSize * sizeof(val_t));
constexpr size_t kScratchBitmapOff = kScratchCtrOff + align256(sizeof(Counters));
// The queued-row bits stay zero between calls only if nothing else is ever written
// where they live: a fixed region, one bit per row for the largest m accepted.
constexpr int64_t kScratchMaxRows = (int64_t)1 << 25;
constexpr size_t kScratchQueuesOff = kScratchBitmapOff + (size_t)(kScratchMaxRows / 8);

// ---- fusedmm_dispatch.hip ---------------------------------------------------------
struct Shape {
   int V, L, R, exact, U;
};

struct Launch {
   int num_cu, blocks_per_cu;
   int64_t nnz_hint;
   hipStream_t stream;
   hipEvent_t *ev;   // 4 events or nullptr
};

struct Plan {
   int op;            // OP_*
   bool opt_rule;     // optimised write-back rule (beta == 0 overwrites)
   bool needs_sop;    // tuple uses SOP_UDEF
   bool reads_x, reads_val;
   int udef_stages;   // stages that are the caller's host functions: kUdefVop | kUdefRop | kUdefVsc | kUdefAop
};
enum : int { kUdefVop = 1, kUdefRop = 2, kUdefVsc = 4, kUdefAop = 8 };

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

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }
int pick_shape(int k, bool vec_ok, Shape *s);
int make_plan(int32_t imsg, int opt_enabled, Plan *pl);
int run_on_device(const Args &a, const Plan &pl, int sop_kind, hipStream_t stream, int queues = kQueuesGrown);
int validate_operands(const Args &a, hipStream_t stream, int queues = kQueuesGrown);
int validate_host_pointers_of(const Args &h, const idx_t *pb, const idx_t *pe);
int validate_host_pointers(const Args &h);
int operand_residence(const Args &a);   // 1 device, 0 host, -1 mixed (refused)
// [first, last) edge slots the processed rows use (0, 0 when none has an edge)
void slot_range(const idx_t *h_pb, const idx_t *h_pe, int64_t m, int64_t *first, int64_t *last);
// d_s[j - slot0] = ROP(X[i], VOP(X[i], Y[c])) for every edge slot j of the processed rows
int edge_scalars(const Args &a, val_t *d_s, int64_t slot0, DeviceState *d, hipStream_t stream);
// the rest of the pipeline (VOP, MOP, AOP) with per-edge scalars d_s[j - slot0]
int accumulate_with_scalars(const Args &a, val_t *d_s, int64_t slot0, hipStream_t stream);
int launch_apply_sop(val_t *s, int64_t n, int sop_kind, const val_t *tab, int num_cu, hipStream_t stream);
int launch_zero_rows(val_t *z, int64_t m, int64_t k, int64_t ldz, int num_cu, hipStream_t stream);

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

// ---- fusedmm_launch.hip, one object per unit ----------------------------------------
// The three kernels of a call (classify, fused, merge) for the op and SOP body of the
// unit: sopk >= 0 names a body fixed at compile time, -1 the run-time switch.
enum : int { kUnitGcn = 0, kUnitSpmm, kUnitDotSigmoid, kUnitDotAny, kUnitDistTdist, kUnitDistFr, kUnitDistAny,
             kUnitGeneric, kUnits };
int launch_unit_gcn(const Params<idx_t> &p, const Shape &s, const Launch &l);
int launch_unit_spmm(const Params<idx_t> &p, const Shape &s, const Launch &l);
int launch_unit_dot_sigmoid(const Params<idx_t> &p, const Shape &s, const Launch &l);
int launch_unit_dot_any(const Params<idx_t> &p, const Shape &s, const Launch &l);
int launch_unit_dist_tdist(const Params<idx_t> &p, const Shape &s, const Launch &l);
int launch_unit_dist_fr(const Params<idx_t> &p, const Shape &s, const Launch &l);
int launch_unit_dist_any(const Params<idx_t> &p, const Shape &s, const Launch &l);
int launch_unit_generic(const Params<idx_t> &p, const Shape &s, const Launch &l);

// ---- fusedmm_staging.hip ----------------------------------------------------------
int stage_up(const Args &h, const Plan &pl, Args *a, int64_t *slots_out);
int stage_down(const Args &h, const Args &a);
int run_staged(const Args &h, const Plan &pl, int sop_kind);

// ---- fusedmm_host_stages.hip ------------------------------------------------------
struct StageFns {
   fusedMM_amd_vop_fn vop;
   fusedMM_amd_rop_fn rop;
   fusedMM_amd_sop_fn sop;
   fusedMM_amd_vsc_fn vsc;
   fusedMM_amd_aop_fn aop;
};
int run_host_sop(const Args &a, const idx_t *h_pb, const idx_t *h_pe, const Plan &pl, fusedMM_amd_sop_fn fn);
int run_host_stages(const Args &a, const idx_t *h_pb, const idx_t *h_pe, const Plan &pl, const StageFns &f, int sop_kind);

}  // namespace fmm_host
