// From the op tuple to the kernels of one call: validation and pattern match of the
// tuple (reference fusedMM.c:512-628), the kernel shape for (K, alignment)
// (reference kernels/src/kernels.c:456-631 picks by K/VLEN), queue sizing, the
// launch, and the column slabs of rows wider than one kernel instance holds.
#include "fusedmm_host.hpp"
#include "fusedmm_aux_kernels.h"

namespace fmm_host {

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

namespace {

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
   p.pack_rows = (g.pack != 1 && sh.V == 4 && sh.L <= 16) ? 1 : 0;
   // Finished rows of Z wait in LDS for a common store tick (82 us) where the gathered matrix is several times the
   // 256 MiB last-level cache, 1 GiB and more: there the gathers run at the memory's own rate and a thin stream of
   // stores between them costs several times its share (2^23 rows of 16 edges, K = 64 ... 256: 9-14 % of the call).
   // Where much of Y is served from that cache the stores are not what limits, and the bookkeeping costs half a
   // per cent (sigmoid K=128 on 2^20 nodes, Y of 512 MiB).
   // The period is the longest one a wavefront's share of LDS still covers: 82 us, or 41 us where rows average
   // fewer than 10 edges and the shares fill twice as fast (2^21 rows of 4 edges at K=512: 4.43 ms at 41 us, 4.57 at
   // 82, 4.77 with rows written as they finish; rows of 16 edges: 13.8, 12.7, 14.6).
   if (g.store_shift >= 0) p.store_shift = g.store_shift;
   else if (a.n * a.ldy * (int64_t)kValBytes < (1ll << 30)) p.store_shift = 0;
   else p.store_shift = (a.m > 0 && a.nnz / a.m < 10) ? 12 : 13;

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
      case OP_GCN: st = launch_unit_gcn(p, sh, l); break;
      case OP_SPMM: st = launch_unit_spmm(p, sh, l); break;
      case OP_DOT:
         if (sop_kind == SOP_SIGMOID) st = launch_unit_dot_sigmoid(p, sh, l);
         else st = launch_unit_dot_any(p, sh, l);
         break;
      case OP_DIST:
         if (sop_kind == SOP_TDIST) st = launch_unit_dist_tdist(p, sh, l);
         else if (sop_kind == SOP_FR) st = launch_unit_dist_fr(p, sh, l);
         else st = launch_unit_dist_any(p, sh, l);
         break;
      default: st = launch_unit_generic(p, sh, l); break;
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

}  // namespace

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
// ---- per-edge scalars over edge slots ------------------------------------------------
namespace {

template <int V, int L, int R, bool EXACT, int U>
int launch_edge_scalar(const Params<idx_t> &p, val_t *s_out, int accumulate, int num_cu, hipStream_t stream)
{
   int64_t blocks = (p.m + kWavesPerBlock - 1) / kWavesPerBlock;
   if (blocks > (int64_t)num_cu * 8) blocks = (int64_t)num_cu * 8;
   hipLaunchKernelGGL((edge_scalar_kernel<V, L, R, EXACT, U, idx_t>), dim3((unsigned int)blocks), dim3(kBlockThreads), 0,
                      stream, p, s_out, accumulate);
   return hip_status(hipGetLastError(), "edge scalar launch");
}

// a pointer `slot0` elements before `base`, for kernels that index by absolute edge slot;
// nothing below slot0 is ever dereferenced through it
inline val_t *biased(val_t *base, int64_t slot0)
{
   return (val_t *)((uintptr_t)base - (uintptr_t)slot0 * sizeof(val_t));
}

}  // namespace

void slot_range(const idx_t *h_pb, const idx_t *h_pe, int64_t m, int64_t *first, int64_t *last)
{
   int64_t lo = INT64_MAX, hi = 0;
   for (int64_t i = 0; i < m; i++)
   {
      const int64_t b = (int64_t)h_pb[i], e = (int64_t)h_pe[i];
      if (e <= b) continue;
      if (b < lo) lo = b;
      if (e > hi) hi = e;
   }
   if (hi <= 0 || lo >= hi) lo = hi = 0;
   *first = lo;
   *last = hi;
}

// d_s[j - slot0] = ROP(X[i], VOP(X[i], Y[c])) for every edge slot j of the processed rows,
// column slab by column slab when k exceeds what one kernel instance holds.
int edge_scalars(const Args &a, val_t *d_s, int64_t slot0, DeviceState *d, hipStream_t stream)
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
      st = launch_edge_scalar<V_, L_, R_, (X_ != 0), U_>(p, biased(d_s, slot0), off > 0 ? 1 : 0, d->num_cu, stream);
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

int launch_apply_sop(val_t *s, int64_t n, int sop_kind, const val_t *tab, int num_cu, hipStream_t stream)
{
   hipLaunchKernelGGL(apply_sop_kernel, dim3((unsigned int)(num_cu * 4)), dim3(kBlockThreads), 0, stream, s, n, sop_kind, tab);
   return hip_status(hipGetLastError(), "apply sop launch");
}

int launch_zero_rows(val_t *z, int64_t m, int64_t k, int64_t ldz, int num_cu, hipStream_t stream)
{
   hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned int)(num_cu * 8)), dim3(kBlockThreads), 0, stream, z, m, k, ldz);
   return hip_status(hipGetLastError(), "zero rows launch");
}

namespace {

bool column_separable(const Plan &pl, int32_t imsg)
{
   return pl.op == OP_GCN || pl.op == OP_SPMM || (pl.op == OP_GENERIC && GET_ROP_FLAG(imsg) == ROP_NOOP);
}

}  // namespace

// Rest of the pipeline (VOP, MOP, AOP) with per-edge scalars already in d_s[j - slot0].
int accumulate_with_scalars(const Args &a, val_t *d_s, int64_t slot0, hipStream_t stream)
{
   Args a2 = a;
   a2.val = biased(d_s, slot0);
   a2.imessage = GET_VOP_FLAG(a.imessage) | ROP_NOOP | SOP_COPY | GET_VSC_FLAG(a.imessage) | GET_AOP_FLAG(a.imessage);
   Plan p2;
   int st = make_plan(a2.imessage, 0, &p2);   // general rule: accumulate (Z is cleared first when it must be overwritten)
   if (st) return st;
   return run_on_device(a2, p2, FUSEDMM_SOP_KIND_IDENTITY, stream);
}

namespace {

// k > kMaxK with a reduction over the whole row (dot / distance tuples): the
// per-edge scalar is assembled from column slabs, the device SOP applied to it,
// then the accumulate stage runs slab by slab.  Synchronous (needs the range of
// edge slots in use, read back from the row pointers).
int run_wide_reduction(const Args &a, const Plan &pl, int sop_kind)
{
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   std::vector<idx_t> hb((size_t)a.m), he((size_t)a.m);
   FMM_HIP(hipMemcpy(hb.data(), a.pntrb, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
   FMM_HIP(hipMemcpy(he.data(), a.pntre, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
   int64_t slot0 = 0, slot1 = 0;
   slot_range(hb.data(), he.data(), a.m, &slot0, &slot1);
   if (pl.opt_rule && a.beta == 0.0f)
   {
      st = launch_zero_rows(a.z, a.m, a.k, a.ldz, d->num_cu, 0);
      if (st) return st;
   }
   if (slot1 <= slot0) return FUSEDMM_SUCCESS_RETURN;
   const int64_t slots = slot1 - slot0;
   st = grow(d->stage[7], (size_t)slots * kValBytes);
   if (st) return st;
   val_t *d_s = (val_t *)d->stage[7].ptr;
   st = edge_scalars(a, d_s, slot0, d, 0);
   if (st) return st;
   if (pl.needs_sop)
   {
      // slots of the range that no processed row uses hold whatever the buffer held: the SOP is applied
      // to them too and nothing reads the result
      st = launch_apply_sop(d_s, slots, sop_kind, (const val_t *)d->sigmoid_table, d->num_cu, 0);
      if (st) return st;
   }
   return accumulate_with_scalars(a, d_s, slot0, 0);
}

}  // namespace

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

}  // namespace fmm_host
