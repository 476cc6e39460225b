// The three kernels of a call -- classify, fused, merge -- for one op and SOP body:
// this file is compiled once per unit (-DFMM_LAUNCH_UNIT=0..7), each object holding
// the fused kernel's instances over every row shape for that unit, so that the
// library's objects build side by side.
#include "fusedmm_host.hpp"

#ifndef FMM_LAUNCH_UNIT
#error "compile with -DFMM_LAUNCH_UNIT=<0..7>"
#endif

namespace fmm_host {

namespace {

template <int V, int L, int R, bool EXACT, int OP, int SOPK, int U>
int launch_instance(const Params<idx_t> &p, const Launch &l)
{
   // persistent grid: as many blocks as stay resident; waves share out the
   // queued segments, then claim rows
   static int occ = 0, occ_staged = 0, stage_lds = 0;
   if (occ == 0)
   {
      const auto kernel = fused_kernel<V, L, R, EXACT, OP, SOPK, U, idx_t>;
      FMM_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, kBlockThreads, 0));
      if (occ < 1) occ = 1;
      // Dynamic LDS for the rows that wait for the store tick: what a CU's 160 KiB leave each of the workgroups
      // that are resident anyway (four at most) beside the kernel's own static LDS, within the 64 KiB one
      // workgroup may have; then checked against the runtime's own count, and shrunk until residency is kept.
      hipFuncAttributes attr;
      FMM_HIP(hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kernel)));
      const int want = occ < 4 ? occ : 4;
      int lds = 163840 / want - (int)attr.sharedSizeBytes - 512;
      if (lds > 65536 - (int)attr.sharedSizeBytes) lds = 65536 - (int)attr.sharedSizeBytes;
      lds = lds > 0 ? lds / 1024 * 1024 : 0;
      if (OP == OP_GENERIC) lds = 0;   // the general pipeline's instances write rows as they finish
      int got = occ;
      while (lds > 0)
      {
         got = 0;
         if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&got, kernel, kBlockThreads, (size_t)lds) == hipSuccess && got >= want) break;
         (void)hipGetLastError();
         lds -= 1024;
      }
      if (lds > 49152) (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      (void)hipGetLastError();
      stage_lds = lds > 0 ? lds : 0;
      occ_staged = lds > 0 ? got : occ;
   }
   const bool staged = p.store_shift > 0 && stage_lds > 0;
   const int dyn_lds = staged ? stage_lds : 0;
   const int occ_now = staged ? occ_staged : occ;
   // enough blocks for the rows, or for the segments the caller's nnz could give rise to
   int64_t need = (p.m + kWavesPerBlock - 1) / kWavesPerBlock;
   const int64_t need_segs = (l.nnz_hint / p.seg_len + kWavesPerBlock - 1) / kWavesPerBlock;
   if (need < need_segs) need = need_segs;
   // Four workgroups (16 waves) per CU at most: with 8-16 gathers in flight per wave
   // that saturates the memory system, and more waves only evict each other's lines
   // (measured on the sigmoid K=128 benchmark: 1.307 ms at 4 per CU, 1.314 at 5, 1.335 at 6).
   // (FUSEDMM_BLOCKS_PER_CU is capped at what stays resident: segments are dealt to the grid's waves by number, so a
   // workgroup that has to wait for a free slot would hold its segments back until then)
   const int resident = occ_now < 4 ? occ_now : 4;
   int64_t gr = (int64_t)l.num_cu * (l.blocks_per_cu > 0 ? (l.blocks_per_cu < occ_now ? l.blocks_per_cu : occ_now) : resident);
   if (gr > need) gr = need;
   if (gr < 1) gr = 1;
   Params<idx_t> pr = p;
   pr.stage_vecs = dyn_lds / (kWavesPerBlock * (int)sizeof(real4));
   if (!staged) pr.store_shift = 0;
   const int64_t nchunks = (p.m + kRowsPerClaim - 1) / kRowsPerClaim;
   if (nchunks <= gr * kWavesPerBlock) pr.row_counters = 0;   // one chunk per wave at most: static
   else pr.row_counters = (gr * kWavesPerBlock >= kRowCounters) ? kRowCounters : 1;
   int64_t gc = (p.m + kBlockThreads - 1) / kBlockThreads;
   if (gc > (int64_t)l.num_cu * 8) gc = (int64_t)l.num_cu * 8;
   if (l.ev) FMM_HIP(hipEventRecord(l.ev[0], l.stream));
   hipLaunchKernelGGL((classify_kernel<idx_t>), dim3((unsigned int)gc), dim3(kBlockThreads), 0, l.stream, p);
   if (l.ev) FMM_HIP(hipEventRecord(l.ev[1], l.stream));
   hipLaunchKernelGGL((fused_kernel<V, L, R, EXACT, OP, SOPK, U, idx_t>), dim3((unsigned int)gr), dim3(kBlockThreads), (size_t)dyn_lds, l.stream, pr);
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

}  // namespace

#if FMM_LAUNCH_UNIT == 0
int launch_unit_gcn(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_GCN, -1>(p, s, l); }
#elif FMM_LAUNCH_UNIT == 1
int launch_unit_spmm(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_SPMM, -1>(p, s, l); }
#elif FMM_LAUNCH_UNIT == 2
int launch_unit_dot_sigmoid(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_DOT, SOP_SIGMOID>(p, s, l); }
#elif FMM_LAUNCH_UNIT == 3
int launch_unit_dot_any(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_DOT, -1>(p, s, l); }
#elif FMM_LAUNCH_UNIT == 4
int launch_unit_dist_tdist(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_DIST, SOP_TDIST>(p, s, l); }
#elif FMM_LAUNCH_UNIT == 5
int launch_unit_dist_fr(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_DIST, SOP_FR>(p, s, l); }
#elif FMM_LAUNCH_UNIT == 6
int launch_unit_dist_any(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_DIST, -1>(p, s, l); }
#elif FMM_LAUNCH_UNIT == 7
int launch_unit_generic(const Params<idx_t> &p, const Shape &s, const Launch &l) { return launch_op<OP_GENERIC, -1>(p, s, l); }
#else
#error "FMM_LAUNCH_UNIT out of range"
#endif

}  // namespace fmm_host
