// Kernels around the fused one: the per-edge scalar pass of the host-function SOP and of
// rows wider than one kernel instance, the device SOP over a scalar array, the optional
// operand check, and clearing Z.  Included by the one translation unit that launches them.
#pragma once
#include "fusedmm_kernels.h"

namespace fmm {

// ---- host-callback SOP, pass 1: s[j] = ROP(X[i], VOP(X[i], Y[c])) for every edge slot ----
// One wave per row (static stride; this path exists for compatibility, the
// host evaluates the caller's SOP_UDEF_FUNC on s[] before the accumulate pass).
template <int V, int L, int R, bool EXACT, int U, typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void edge_scalar_kernel(const Params<IdxT> p, real_t *s_out, int accumulate)
{
   constexpr int S = 64 / L;
   const int lane = threadIdx.x & 63;
   const int sub = lane / L, sl = lane % L;
   const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
   const int vop = p.imessage & 0xF, rop = p.imessage & 0xF0;
   for (int64_t row = wave0; row < p.m; row += nwaves)
   {
      const IdxT jb = wave_uniform<IdxT>(p.pntrb[row]);
      const IdxT je = wave_uniform<IdxT>(p.pntre[row]);
      Slice<R> xs;
      load_slice<V, L, R, EXACT>(xs, p.x + row * p.ldx, sl, p.k);
      // slot numbers in 64 bits: an int32 slot next to 2^31 must not wrap when stepped past je
      const int64_t je64 = (int64_t)je;
      for (int64_t j0 = (int64_t)jb; j0 < je64; j0 += S * U)
      {
#pragma unroll
         for (int u = 0; u < U; u++)
         {
            const int64_t j = j0 + sub + u * S;
            if (j < je64)
            {
               Slice<R> ys, t;
               load_slice<V, L, R, EXACT>(ys, p.y + (int64_t)p.indx[j] * p.ldy, sl, p.k);
               const real_t scal = vop_rop<L, R>(t, xs, ys, p.val ? p.val[j] : (real_t)0, vop, rop);
               // every ROP is a sum over elements, so column slabs of a wide row add up
               if (sl == 0) s_out[j] = accumulate ? s_out[j] + scal : scal;
            }
         }
      }
   }
}

// d[j] = SOP(s[j]) in place, for the wide-row path where the ROP result is
// assembled from column slabs before the scalar op can be applied.
__global__ __launch_bounds__(kBlockThreads) void apply_sop_kernel(real_t *s, int64_t n, int sop_kind, const real_t *tab)
{
   for (int64_t i = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlockThreads)
      s[i] = sop_eval(sop_kind, s[i], tab);
}

// Optional operand check (off by default, like the reference, which trusts its
// caller): a column id outside [0, n) or a row with pntre < pntrb would make the
// kernels read outside Y.  Sets flag[0] when anything is wrong.
template <typename IdxT>
__global__ __launch_bounds__(kBlockThreads) void validate_kernel(const Params<IdxT> p, int64_t n, unsigned int *flag)
{
   const int lane = threadIdx.x & 63;
   const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
   const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
   bool bad = false;
   for (int64_t row = wave0; row < p.m; row += nwaves)
   {
      const IdxT jb = p.pntrb[row], je = p.pntre[row];
      if (je < jb || jb < 0) { bad = true; continue; }
      for (int64_t j = (int64_t)jb + lane; j < (int64_t)je; j += 64)   // 64-bit: no wrap next to 2^31
      {
         const IdxT c = p.indx[j];
         if (c < 0 || (int64_t)c >= n) bad = true;
      }
   }
   if (bad) atomicOr(flag, 1u);
}

// Z[i, 0:k] = 0 for i < m (the overwrite rule of the pattern tuples, when the
// accumulate pass that follows can only add).
__global__ __launch_bounds__(kBlockThreads) void zero_rows_kernel(real_t *z, int64_t m, int64_t k, int64_t ldz)
{
   const int64_t total = m * k;
   for (int64_t i = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlockThreads)
      z[(i / k) * ldz + (i % k)] = (real_t)0;
}

}  // namespace fmm
