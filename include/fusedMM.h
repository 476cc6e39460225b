/*
 * fusedMM.h -- host API of the MI355X (gfx950) build of FusedMM.
 *
 * Drop-in for the reference's fusedMM.h: same macro names and values for the
 * five-stage op tuple (reference fusedMM.h:18-73), same fusedMM_csr prototype
 * (:76-97), same status codes (:103-112), same user-function prototypes
 * (:135-143).  As there, the includer chooses the ABI by defining INDEXTYPE
 * (int32_t or int64_t) and VALUETYPE (float) before the include and links the
 * matching library: libfusedmm_amd_i32.so or libfusedmm_amd_i64.so.
 *
 * Additions that have no counterpart in the reference are in fusedmm_amd.h.
 */
#ifndef FUSEDMM_AMD_FUSEDMM_H
#define FUSEDMM_AMD_FUSEDMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * imessage: one 4-bit field per stage, low to high
 *     bits  0-3  VOP   T = vop(X[i], Y[c])              vector, vector -> vector
 *     bits  4-7  ROP   s = rop(X[i], T)                 reduction to a scalar
 *     bits  8-11 SOP   d = sop(s)                       scalar -> scalar
 *     bits 12-15 VSC   T = vsc(d, T)    (a.k.a. MOP)    scalar, vector -> vector
 *     bits 16-19 AOP   Z[i] = aop(Z[i], T)              accumulate
 */

/* ---- VOP ------------------------------------------------------------- */
#define VOP_NOOP      0x0
#define VOP_COPY_LHS  0x1   /* T = X[i]                                   */
#define VOP_COPY_RHS  0x2   /* T = Y[c]                                   */
#define VOP_ADD       0x3   /* T = X[i] + Y[c]                            */
#define VOP_SUBL      0x4   /* T = Y[c] - X[i]  (what the reference's code computes) */
#define VOP_SUBR      0x5   /* T = X[i] - Y[c]  (what the reference's code computes) */
#define VOP_MAX       0x6
#define VOP_MIN       0x7
#define VOP_UDEF      0xF
#define VOP_MASK(bvec)   ((bvec) & 0xF)
#define VOP_CLEAR(bvec)  (((bvec) >> 4) << 4)
#define GET_VOP_FLAG(imsg)        VOP_MASK(imsg)
#define SET_VOP_FLAG(imsg, vflag) (imsg = (VOP_CLEAR(imsg) | vflag))

/* ---- ROP ------------------------------------------------------------- */
#define ROP_NOOP      0x00  /* s = val[j]                                 */
#define ROP_DOT       0x10  /* s = <X[i], T>                              */
#define ROP_ADD_LHS   0x20  /* s = sum X[i]                               */
#define ROP_ADD_RHS   0x30  /* s = sum T                                  */
#define ROP_NORML     0x40  /* s = sum X[i]^2                             */
#define ROP_NORMR     0x50  /* s = sum T^2                                */
#define ROP_UDEF      0xF0
#define ROP_MASK(bvec)   ((bvec) & 0xF0)
#define ROP_CLEAR(bvec)  ((bvec) & (~((int32_t)0xF0)))
#define GET_ROP_FLAG(imsg)        ROP_MASK(imsg)
#define SET_ROP_FLAG(imsg, vflag) (imsg = (ROP_CLEAR(imsg) | vflag))

/* ---- SOP ------------------------------------------------------------- */
#define SOP_NOOP      0x000
#define SOP_COPY      0x100 /* d = s                                      */
#define SOP_UDEF      0xF00 /* d = SOP_UDEF_FUNC(s)                       */
#define SOP_MASK(bvec)   ((bvec) & 0xF00)
#define SOP_CLEAR(bvec)  ((bvec) & (~((int32_t)0xF00)))
#define GET_SOP_FLAG(imsg)        SOP_MASK(imsg)
#define SET_SOP_FLAG(imsg, vflag) (imsg = (SOP_CLEAR(imsg) | vflag))

/* ---- VSC / MOP ------------------------------------------------------- */
#define VSC_NOOP      0x0000
#define VSC_MUL       0x1000 /* T = d * T                                 */
#define VSC_ADD       0x2000 /* T = d + T                                 */
#define VSC_UDEF      0xF000
#define VSC_MASK(bvec)   ((bvec) & 0xF000)
#define VSC_CLEAR(bvec)  ((bvec) & (~((int32_t)0xF000)))
#define GET_VSC_FLAG(imsg)        VSC_MASK(imsg)
#define SET_VSC_FLAG(imsg, vflag) (imsg = (VSC_CLEAR(imsg) | vflag))

/* ---- AOP ------------------------------------------------------------- */
#define AOP_NOOP      0x00000
#define AOP_ADD       0x10000 /* Z[i] += T                                */
#define AOP_MAX       0x20000 /* Z[i] = max(Z[i], T)                      */
#define AOP_MIN       0x30000 /* Z[i] = min(Z[i], T)                      */
#define AOP_UDEF      0xF0000
#define AOP_MASK(bvec)   ((bvec) & 0xF0000)
#define AOP_CLEAR(bvec)  ((bvec) & (~((int32_t)0xF0000)))
#define GET_AOP_FLAG(imsg)        AOP_MASK(imsg)
#define SET_AOP_FLAG(imsg, vflag) (imsg = (AOP_CLEAR(imsg) | vflag))

/* ---- status codes (reference fusedMM.h:103-112) ----------------------- */
#define FUSEDMM_SUCCESS_RETURN            0
#define FUSEDMM_FAIL_RETURN               1
#define FUSEDMM_VOP_FAIL_RETURN           2
#define FUSEDMM_ROP_FAIL_RETURN           4
#define FUSEDMM_AOP_FAIL_RETURN           8
#define FUSEDMM_SOP_FAIL_RETURN          16
#define FUSEDMM_VSC_FAIL_RETURN          32
#define FUSEDMM_NOT_ENOUGH_MEM           -1
#define FUSEDMM_UNDEFINED_USER_FUNCTION  64
#define FUSEDMM_NO_OPT_IMPL             128

/*
 * Z[i,:] = aop-fold over j in [pntrb[i], pntre[i]) of vsc(sop(rop(X[i], T)), T),
 * T = vop(X[i], Y[indx[j]]), for i in [0, m).   Replaces reference fusedMM.c:487-744.
 *
 * Pointers may be host memory (staged to the GPU and back inside the call) or
 * device memory (used in place); all seven must be of the same kind.  The call
 * returns after the result is complete.
 *
 * The four op tuples the reference pattern-matches (fusedMM.c:523-583: gcn,
 * spmm, sigmoid, t-dist/FR) follow its optimised kernels: beta == 0 overwrites
 * Z, any other beta accumulates into Z.  Every other tuple follows its general
 * pipeline: always accumulates into Z.  alpha, nnz, rows and cols are not read
 * except that nnz, when positive, sizes an internal work queue.
 */
int fusedMM_csr
(
   const int32_t imessage,    /* op tuple                                          */
   const INDEXTYPE m,         /* rows of X and Z to compute                        */
   const INDEXTYPE n,         /* rows of Y                                         */
   const INDEXTYPE k,         /* feature dimension                                 */
   const VALUETYPE alpha,     /* unused, as in the reference                       */
   const INDEXTYPE nnz,       /* edges of the sparse matrix                        */
   const INDEXTYPE rows,      /* rows of the sparse matrix                         */
   const INDEXTYPE cols,      /* columns of the sparse matrix                      */
   const VALUETYPE *val,      /* edge values                                       */
   const INDEXTYPE *indx,     /* column ids                                        */
   const INDEXTYPE *pntrb,    /* first edge slot of each row                       */
   const INDEXTYPE *pntre,    /* one past the last edge slot of each row           */
   const VALUETYPE *x,        /* dense X [m, ldx]                                  */
   const INDEXTYPE ldx,
   const VALUETYPE *y,        /* dense Y [n, ldy]                                  */
   const INDEXTYPE ldy,
   const VALUETYPE beta,      /* 0: overwrite Z, otherwise accumulate (see above)  */
   VALUETYPE *z,              /* dense Z [m, ldz]                                  */
   const INDEXTYPE ldz
);

/*
 * User functions (reference fusedMM.h:129-143).  Only SOP_UDEF_FUNC is honoured,
 * as in the reference's default configuration (SOP_UDEF_IMPL on, the other four
 * off).  A GPU kernel cannot call a host symbol per edge: select a built-in
 * device body with fusedMM_amd_set_sop_kind() (fusedmm_amd.h), or leave the
 * kind at "host" and the library evaluates the caller's SOP_UDEF_FUNC on the
 * host between a GPU reduction pass and a GPU accumulate pass.
 */
#define SOP_UDEF_IMPL 1

int VOP_UDEF_FUNC(INDEXTYPE lhs_dim, const VALUETYPE *lhs, INDEXTYPE rhs_dim,
                  const VALUETYPE *rhs, INDEXTYPE out_dim, VALUETYPE *out);
int ROP_UDEF_FUNC(INDEXTYPE lhs_dim, const VALUETYPE *lhs, INDEXTYPE rhs_dim,
                  const VALUETYPE *rhs, VALUETYPE *out);
int SOP_UDEF_FUNC(VALUETYPE val, VALUETYPE *out);
int VSC_UDEF_FUNC(INDEXTYPE rhs_dim, const VALUETYPE *rhs, VALUETYPE scal,
                  INDEXTYPE out_dim, VALUETYPE *out);
int AOP_UDEF_FUNC(INDEXTYPE rhs_dim, const VALUETYPE *rhs, INDEXTYPE out_dim,
                  VALUETYPE *out);

#ifdef __cplusplus
}
#endif

#endif /* FUSEDMM_AMD_FUSEDMM_H */
