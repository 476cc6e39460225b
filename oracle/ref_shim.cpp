/*
 * ref_shim.cpp -- extern "C" doorway into the REAL reference, for tests only.
 *
 * Built by oracle/Makefile together with two reference translation units taken
 * where they lie under /root/reference (never copied into this repository):
 *   test/fusedMMtime.cpp  (harness: trusted kernels :159-365, sigmoid table and
 *                          SOP_UDEF_FUNC bodies :586-674, mytest_csr :704-762,
 *                          its main renamed with -Dmain=ref_harness_main)
 *   fusedMM.c             (generic fusedMM_csr, :487-744, built the way the
 *                          reference builds its non-"Opt" executables)
 * The reference's optimised kernels need its code generator's output and are
 * therefore not part of this build.  One library per (SOP body, precision,
 * index width), like the reference's one executable per kind.
 *
 * This file contains no reference code: it only declares the reference's
 * symbols and forwards to them.
 */
#include <cstdint>
#include <cstring>
#include <string>

#include "include/CSC.h"
#include "include/CSR.h"
#include "include/commonutility.h"

#ifndef INDEXTYPE
#error "build with -DINDEXTYPE=int32_t or int64_t"
#endif
#ifdef DREAL   /* the reference's switch for double precision */
#define VALUETYPE double
#else
#define VALUETYPE float
#endif

#define REF_CSR_ARGS                                                                   \
   const char tkern, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,          \
      const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows,                \
      const INDEXTYPE cols, const VALUETYPE *val, const INDEXTYPE *indx,               \
      const INDEXTYPE *pntrb, const INDEXTYPE *pntre, const VALUETYPE *a,              \
      const INDEXTYPE lda, const VALUETYPE *b, const INDEXTYPE ldb,                    \
      const VALUETYPE beta, VALUETYPE *c, const INDEXTYPE ldc
#define REF_CSR_PASS                                                                   \
   tkern, m, n, k, alpha, nnz, rows, cols, val, indx, pntrb, pntre, a, lda, b, ldb,    \
      beta, c, ldc

/* defined in the reference harness (C++ linkage) */
void mytrusted_csr(REF_CSR_ARGS);
void mytest_csr(REF_CSR_ARGS);
extern VALUETYPE *SM_TABLE;
void uinit_SM_TABLE();

/* defined in the reference library / harness (C linkage) */
extern "C" int SOP_UDEF_FUNC(VALUETYPE val, VALUETYPE *out);
extern "C" int fusedMM_csr(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n,
                           const INDEXTYPE k, const VALUETYPE alpha, const INDEXTYPE nnz,
                           const INDEXTYPE rows, const INDEXTYPE cols, const VALUETYPE *val,
                           const INDEXTYPE *indx, const INDEXTYPE *pntrb,
                           const INDEXTYPE *pntre, const VALUETYPE *x, const INDEXTYPE ldx,
                           const VALUETYPE *y, const INDEXTYPE ldy, const VALUETYPE beta,
                           VALUETYPE *z, const INDEXTYPE ldz);

static CSR<INDEXTYPE, VALUETYPE> *g_csr = nullptr;

extern "C" {

int ref_index_bytes(void) { return (int)sizeof(INDEXTYPE); }
int ref_value_bytes(void) { return (int)sizeof(VALUETYPE); }

/* the harness's trusted kernel for tkern in {t,s,m,g,f} */
void ref_trusted_csr(REF_CSR_ARGS) { mytrusted_csr(REF_CSR_PASS); }

/* the harness's call into fusedMM_csr for tkern in {t,f,s,m,g} */
void ref_test_csr(REF_CSR_ARGS) { mytest_csr(REF_CSR_PASS); }

/* fusedMM_csr itself, any op tuple (generic five-stage pipeline) */
int ref_fusedMM_csr(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n,
                    const INDEXTYPE k, const VALUETYPE alpha, const INDEXTYPE nnz,
                    const INDEXTYPE rows, const INDEXTYPE cols, const VALUETYPE *val,
                    const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                    const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y,
                    const INDEXTYPE ldy, const VALUETYPE beta, VALUETYPE *z,
                    const INDEXTYPE ldz)
{
   if (!SM_TABLE) uinit_SM_TABLE();
   return fusedMM_csr(imessage, m, n, k, alpha, nnz, rows, cols, val, indx, pntrb, pntre,
                      x, ldx, y, ldy, beta, z, ldz);
}

/* the 2048-entry table exactly as the harness builds it */
void ref_sm_table(VALUETYPE *out)
{
   if (!SM_TABLE) uinit_SM_TABLE();
   std::memcpy(out, SM_TABLE, sizeof(VALUETYPE) * 2048);
}

/* the SOP_UDEF_FUNC body this library was compiled with */
void ref_sop_array(const VALUETYPE *in, VALUETYPE *out, int64_t n)
{
   if (!SM_TABLE) uinit_SM_TABLE();
   for (int64_t i = 0; i < n; i++) SOP_UDEF_FUNC(in[i], &out[i]);
}

/* .mtx -> CSC -> CSR through the reference's own loader
 * (commonutility.h:26-44, IO.h:62-162, CSC.h:147-189, CSR.h:154-186) */
int ref_load_mtx(const char *path, int64_t *rows, int64_t *cols, int64_t *nnz)
{
   CSC<INDEXTYPE, VALUETYPE> csc;
   SetInputMatricesAsCSC(csc, std::string(path));
   csc.Sorted();
   delete g_csr;
   g_csr = new CSR<INDEXTYPE, VALUETYPE>(csc);
   g_csr->Sorted();
   *rows = g_csr->rows;
   *cols = g_csr->cols;
   *nnz = g_csr->nnz;
   return 0;
}

void ref_get_csr(INDEXTYPE *rowptr, INDEXTYPE *colids, VALUETYPE *values)
{
   if (!g_csr) return;
   std::memcpy(rowptr, g_csr->rowptr, sizeof(INDEXTYPE) * (size_t)(g_csr->rows + 1));
   std::memcpy(colids, g_csr->colids, sizeof(INDEXTYPE) * (size_t)g_csr->nnz);
   std::memcpy(values, g_csr->values, sizeof(VALUETYPE) * (size_t)g_csr->nnz);
}

} /* extern "C" */
