// The five stages as separate kernels over materialised edges (tuples in which a stage is
// the caller's host function).  Included by the one translation unit that launches them.
#pragma once
#include "fusedmm_kernels.h"

namespace fmm {

// ---- the pipeline stage by stage over materialised edges ---------------------------
// For tuples in which VOP, ROP, VSC or AOP is the caller's host function: the
// per-edge vector T[j - slot0][0..k) and scalar s[j - slot0] live in device buffers indexed
// by edge slot (slot0: the first slot any processed row uses, so that a window of rows high
// in the CSR arrays costs its own edges only), so that a host pass can stand in for any
// stage while the library's own
// stages stay on the GPU.  One wavefront per row.  Every built-in stage evaluates in
// the reference's own order (fusedMM.c:28-333: element by element, sums left to
// right, separate multiply and add), so the results are the reference's bits.

// T[j] = VOP(X[i], Y[indx[j]])
template <typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void stage_vop_kernel(const Params<IdxT> p, real_t *T, int64_t slot0)
{
   const int lane = threadIdx.x & 63;
   const int vop = p.imessage & 0xF;
   const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   for (int64_t i = wave0; i < p.m; i += (int64_t)gridDim.x * kWavesPerBlock)
   {
      const real_t *xr = p.x + i * p.ldx;
      for (int64_t j = (int64_t)p.pntrb[i]; j < (int64_t)p.pntre[i]; j++)
      {
         const real_t *yr = p.y + (int64_t)p.indx[j] * p.ldy;
         real_t *t = T + (j - slot0) * p.k;
         for (int e = lane; e < p.k; e += 64)
         {
            const real_t a = xr[e], b = yr[e];
            real_t v;
            switch (vop)
            {
               case kVopCopyLhs: v = a; break;
               case kVopCopyRhs: v = b; break;
               case kVopAdd: v = a + b; break;
               case kVopSubl: v = -a + b; break;
               case kVopSubr: v = a - b; break;
               case kVopMax: v = a > b ? a : b; break;   // the reference's own fmax/fmin are these ternaries (fusedMM.c:18-19)
               default: v = a < b ? a : b; break;
            }
            t[e] = v;
         }
      }
   }
}

// s[j] = ROP(X[i], T[j]); a lane owns an edge and sums its k terms left to right.
// (ROP_NOOP is not launched: s[j] stays the edge value.)
template <typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void stage_rop_kernel(const Params<IdxT> p, const real_t *T, real_t *s, int64_t slot0)
{
   const int lane = threadIdx.x & 63;
   const int rop = p.imessage & 0xF0;
   const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   for (int64_t i = wave0; i < p.m; i += (int64_t)gridDim.x * kWavesPerBlock)
   {
      const real_t *xr = p.x + i * p.ldx;
      for (int64_t j = (int64_t)p.pntrb[i] + lane; j < (int64_t)p.pntre[i]; j += 64)
      {
         const real_t *t = T + (j - slot0) * p.k;
         real_t acc = (real_t)0;
         for (int e = 0; e < p.k; e++)
         {
            real_t term;
            switch (rop)
            {
               case kRopDot: term = xr[e] * t[e]; break;
               case kRopAddLhs: term = xr[e]; break;
               case kRopAddRhs: term = t[e]; break;
               case kRopNormL: term = xr[e] * xr[e]; break;
               default: term = t[e] * t[e]; break;   // kRopNormR
            }
            acc = acc + term;
         }
         s[j - slot0] = acc;
      }
   }
}

// T[j] = VSC(s[j], T[j]) for the edge slots of the processed rows
template <typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void stage_vsc_kernel(const Params<IdxT> p, real_t *T, const real_t *s, int64_t slot0)
{
   const int lane = threadIdx.x & 63;
   const int vsc = p.imessage & 0xF000;
   const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   for (int64_t i = wave0; i < p.m; i += (int64_t)gridDim.x * kWavesPerBlock)
      for (int64_t j = (int64_t)p.pntrb[i]; j < (int64_t)p.pntre[i]; j++)
      {
         const real_t d = s[j - slot0];
         real_t *t = T + (j - slot0) * p.k;
         for (int e = lane; e < p.k; e += 64) t[e] = (vsc == kVscMul) ? d * t[e] : d + t[e];
      }
}

// Z[i] = AOP(Z[i], T[j]) over the row's edges in order; a lane owns a column.
template <typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void stage_aop_kernel(const Params<IdxT> p, const real_t *T, int64_t slot0)
{
   const int lane = threadIdx.x & 63;
   const int aop = p.imessage & 0xF0000;
   const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   for (int64_t i = wave0; i < p.m; i += (int64_t)gridDim.x * kWavesPerBlock)
   {
      const int64_t jb = (int64_t)p.pntrb[i], je = (int64_t)p.pntre[i];
      if (je <= jb) continue;
      real_t *zr = p.z + i * p.ldz;
      for (int e = lane; e < p.k; e += 64)
      {
         real_t z = zr[e];
         for (int64_t j = jb; j < je; j++)
         {
            const real_t t = T[(j - slot0) * p.k + e];
            if (aop == kAopAdd) z = z + t;
            else if (aop == kAopMax) z = z > t ? z : t;
            else z = z < t ? z : t;
         }
         zr[e] = z;
      }
   }
}

}  // namespace fmm
