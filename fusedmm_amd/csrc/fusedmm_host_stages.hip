// Stages of the op tuple that are the caller's own host functions: SOP_UDEF_FUNC
// (always enabled in the reference, fusedMM.h:131) and, for callers who built the
// reference with the matching switches, VOP/ROP/VSC/AOP_UDEF_FUNC (fusedMM.h:129-143).
// The library's own stages stay on the GPU; per-edge scalars and vectors cross to the
// host for the caller's functions only.  Per-edge buffers cover the edge slots from the
// first to the last one the processed rows use, not the whole CSR arrays.
#include <thread>

#include "fusedmm_host.hpp"
#include "fusedmm_stage_kernels.h"

namespace fmm_host {

namespace {

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

}  // namespace

// ---- SOP_UDEF evaluated by the caller's host function ---------------------------------------
// The reference calls SOP_UDEF_FUNC once per edge from inside its kernels
// (genkern.base:487, 554; fusedMM.c:729).  Here: pass 1 on the GPU writes the
// ROP result of every edge, the host applies the function to each of them,
// pass 2 on the GPU runs the rest of the pipeline (MOP, AOP) with those
// scalars as edge values.  Synchronous; device operands `a`, host copies of
// the row pointers in h_pb / h_pe.
int run_host_sop(const Args &a, const idx_t *h_pb, const idx_t *h_pe, const Plan &pl, fusedMM_amd_sop_fn fn)
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
   {
      st = launch_zero_rows(a.z, a.m, a.k, a.ldz, d->num_cu, 0);
      if (st) return st;
   }
   int64_t slot0 = 0, slot1 = 0;
   slot_range(h_pb, h_pe, a.m, &slot0, &slot1);
   if (slot1 <= slot0) return hip_status(hipStreamSynchronize(0), "hipStreamSynchronize");
   const int64_t slots = slot1 - slot0;
   st = grow(d->stage[7], (size_t)slots * kValBytes);
   if (st) return st;
   val_t *d_s = (val_t *)d->stage[7].ptr;

   // pass 1
   st = edge_scalars(a, d_s, slot0, d, 0);
   if (st) return st;
   std::vector<val_t> hs((size_t)slots);
   FMM_HIP(hipMemcpyAsync(hs.data(), d_s, (size_t)slots * kValBytes, hipMemcpyDeviceToHost, 0));
   FMM_HIP(hipStreamSynchronize(0));

   // host SOP, rows dealt to a few threads (the function must be thread-safe, reference fusedMM.h:125-126)
   for_row_ranges(a.m, [&](int64_t lo, int64_t hi) {
      for (int64_t i = lo; i < hi; i++)
         for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
         {
            val_t out = hs[(size_t)(j - slot0)];
            (void)fn(hs[(size_t)(j - slot0)], &out);
            hs[(size_t)(j - slot0)] = out;
         }
   });
   FMM_HIP(hipMemcpyAsync(d_s, hs.data(), (size_t)slots * kValBytes, hipMemcpyHostToDevice, 0));

   // pass 2: same VOP / MOP / AOP, the scalar comes in as the edge value
   st = accumulate_with_scalars(a, d_s, slot0, 0);
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
int run_host_stages(const Args &a, const idx_t *h_pb, const idx_t *h_pe, const Plan &pl, const StageFns &f, int sop_kind)
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
   int64_t slot0 = 0, slot1 = 0;
   slot_range(h_pb, h_pe, a.m, &slot0, &slot1);
   if (slot1 <= slot0) return FUSEDMM_SUCCESS_RETURN;   // no processed row has an edge: Z is left alone (general rule)
   const int64_t slots = slot1 - slot0;
   const int vop = GET_VOP_FLAG(a.imessage), rop = GET_ROP_FLAG(a.imessage), sop = GET_SOP_FLAG(a.imessage),
             vsc = GET_VSC_FLAG(a.imessage), aop = GET_AOP_FLAG(a.imessage);
   (void)vop;
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

   // host copies (indexed by j - slot0), made when a host stage first needs them
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
      FMM_HIP(hipMemcpy(hidx.data(), a.indx + slot0, (size_t)slots * sizeof(idx_t), hipMemcpyDeviceToHost));
      // the host function is handed rows of a host copy of Y: as many rows as the processed edges reach
      // (n is not trusted: the reference never reads it)
      int64_t y_rows = 0;
      for (int64_t i = 0; i < m; i++)
         for (int64_t j = (int64_t)h_pb[i]; j < (int64_t)h_pe[i]; j++)
         {
            const int64_t c = (int64_t)hidx[(size_t)(j - slot0)];
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
               (void)f.vop((idx_t)k, hX.data() + i * a.ldx, (idx_t)k, hY.data() + (int64_t)hidx[(size_t)(j - slot0)] * a.ldy,
                           (idx_t)k, hT.data() + (size_t)(j - slot0) * (size_t)k);
      });
      T_host = true;
   }
   else
   {
      hipLaunchKernelGGL(stage_vop_kernel<idx_t>, grid, block, 0, 0, p, d_T, slot0);
      st = hip_status(hipGetLastError(), "stage kernel launch"); if (st) return st;
      T_dev = true;
   }

   // ---- ROP: the scalar starts as the edge value (fusedMM.c:717)
   if (a.val) FMM_HIP(hipMemcpyAsync(d_s, a.val + slot0, (size_t)slots * kValBytes, hipMemcpyDeviceToDevice, 0));
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
               (void)f.rop((idx_t)k, hX.data() + i * a.ldx, (idx_t)k, hT.data() + (size_t)(j - slot0) * (size_t)k,
                           &hs[(size_t)(j - slot0)]);
      });
      s_dev = false;
   }
   else if (rop != ROP_NOOP)
   {
      st = need_T_dev(); if (st) return st;
      hipLaunchKernelGGL(stage_rop_kernel<idx_t>, grid, block, 0, 0, p, (const val_t *)d_T, d_s, slot0);
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
                  val_t out = hs[(size_t)(j - slot0)];
                  (void)f.sop(hs[(size_t)(j - slot0)], &out);
                  hs[(size_t)(j - slot0)] = out;
               }
         });
         s_dev = false;
      }
      else
      {
         st = need_s_dev(); if (st) return st;
         st = launch_apply_sop(d_s, slots, sop_kind, (const val_t *)d->sigmoid_table, d->num_cu, 0);
         if (st) return st;
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
               val_t *t = hT.data() + (size_t)(j - slot0) * (size_t)k;
               (void)f.vsc((idx_t)k, t, hs[(size_t)(j - slot0)], (idx_t)k, t);
            }
      });
      T_dev = false;
   }
   else if (vsc != VSC_NOOP)
   {
      st = need_T_dev(); if (st) return st;
      st = need_s_dev(); if (st) return st;
      hipLaunchKernelGGL(stage_vsc_kernel<idx_t>, grid, block, 0, 0, p, d_T, (const val_t *)d_s, slot0);
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
               (void)f.aop((idx_t)k, hT.data() + (size_t)(j - slot0) * (size_t)k, (idx_t)k, hZ.data() + i * a.ldz);
      });
      FMM_HIP(hipMemcpy(a.z, hZ.data(), hZ.size() * kValBytes, hipMemcpyHostToDevice));
   }
   else if (aop != AOP_NOOP)
   {
      st = need_T_dev(); if (st) return st;
      hipLaunchKernelGGL(stage_aop_kernel<idx_t>, grid, block, 0, 0, p, (const val_t *)d_T, slot0);
      st = hip_status(hipGetLastError(), "stage kernel launch"); if (st) return st;
   }
   return hip_status(hipStreamSynchronize(0), "hipStreamSynchronize");
}

}  // namespace fmm_host
