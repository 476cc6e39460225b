// C doorway to the tester's .mtx loader (mtx_csr.hpp) so that it can be checked
// from outside C++.  Replaces, for tests, direct use of the reference's
// SetInputMatricesAsCSC + CSR(CSC) (test/include/commonutility.h:26-44, CSR.h:154-186).
#include <cstring>
#include <string>

#ifndef INDEXTYPE
#error "compile with -DINDEXTYPE=int32_t or -DINDEXTYPE=int64_t"
#endif
#include "mtx_csr.hpp"

static fmm_host::CsrMatrix<INDEXTYPE> g_last;
static std::string g_err;

extern "C" {

int fmm_load_mtx(const char *path, int64_t *rows, int64_t *cols, int64_t *nnz)
{
   g_last = fmm_host::CsrMatrix<INDEXTYPE>();
   g_err = fmm_host::load_mtx<INDEXTYPE>(path, g_last);
   if (!g_err.empty()) return 1;
   *rows = g_last.rows;
   *cols = g_last.cols;
   *nnz = g_last.nnz;
   return 0;
}

const char *fmm_load_error(void) { return g_err.c_str(); }

void fmm_get_csr(INDEXTYPE *rowptr, INDEXTYPE *colids, float *values)
{
   std::memcpy(rowptr, g_last.rowptr.data(), g_last.rowptr.size() * sizeof(INDEXTYPE));
   std::memcpy(colids, g_last.colids.data(), g_last.colids.size() * sizeof(INDEXTYPE));
   std::memcpy(values, g_last.values.data(), g_last.values.size() * sizeof(float));
}

}
