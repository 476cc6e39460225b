/*
 * A caller written exactly as for the reference library: plain C, includes
 * fusedMM.h only, defines its own SOP_UDEF_FUNC, passes host arrays.  Nothing
 * here knows about the GPU.  Link with -rdynamic so the library can find
 * SOP_UDEF_FUNC the way the reference's kernels do (by symbol).
 *
 *   gcc -DINDEXTYPE=int64_t -DVALUETYPE=float dropin_example.c -rdynamic \
 *       -L.. -lfusedmm_amd_i64 -Wl,-rpath,'$ORIGIN/..' -lm -o xdropin_example
 *
 * Computes the sigmoid-embedding update on a ring graph with a logistic SOP and
 * compares against a direct evaluation; then a tuple whose accumulate stage is the
 * caller's own AOP_UDEF_FUNC (what a reference built with AOP_UDEF_IMPL binds,
 * fusedMM.h:129-143), found by the library by name in the same way; prints PASSED
 * or FAILED.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "../../include/fusedMM.h"

/* the user's scalar op: exact logistic instead of the tester's table */
int SOP_UDEF_FUNC(VALUETYPE val, VALUETYPE *out)
{
   *out = (VALUETYPE)(1.0 - 1.0 / (1.0 + exp(-(double)val)));
   return FUSEDMM_SUCCESS_RETURN;
}

/* the user's accumulate stage: largest magnitude seen per column */
int AOP_UDEF_FUNC(INDEXTYPE rhs_dim, const VALUETYPE *rhs, INDEXTYPE out_dim, VALUETYPE *out)
{
   (void)rhs_dim;
   for (INDEXTYPE t = 0; t < out_dim; t++)
   {
      const VALUETYPE a = rhs[t] < 0 ? -rhs[t] : rhs[t];
      if (a > out[t]) out[t] = a;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

int main(void)
{
   const INDEXTYPE n = 1000, k = 48, deg = 6;
   const INDEXTYPE nnz = n * deg;
   INDEXTYPE *rowptr = malloc(sizeof(INDEXTYPE) * (n + 1));
   INDEXTYPE *col = malloc(sizeof(INDEXTYPE) * nnz);
   VALUETYPE *val = malloc(sizeof(VALUETYPE) * nnz);
   VALUETYPE *x = malloc(sizeof(VALUETYPE) * n * k), *y = malloc(sizeof(VALUETYPE) * n * k);
   VALUETYPE *z = calloc((size_t)(n * k), sizeof(VALUETYPE)), *w = calloc((size_t)(n * k), sizeof(VALUETYPE));
   unsigned s = 12345u;
   for (INDEXTYPE i = 0; i <= n; i++) rowptr[i] = i * deg;
   for (INDEXTYPE i = 0; i < n; i++)
      for (INDEXTYPE d = 0; d < deg; d++)
      {
         col[i * deg + d] = (i + 1 + d * 37) % n;
         val[i * deg + d] = 1.0f;
      }
   for (INDEXTYPE i = 0; i < n * k; i++)
   {
      s = s * 1664525u + 1013904223u; x[i] = (VALUETYPE)((s >> 8) / 16777216.0 - 0.5);
      s = s * 1664525u + 1013904223u; y[i] = (VALUETYPE)((s >> 8) / 16777216.0 - 0.5);
   }
   int32_t imsg = VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD;
   int rc = fusedMM_csr(imsg, n, n, k, 1.0f, nnz, n, n, val, col, rowptr, rowptr + 1, x, k, y, k, 0.0f, z, k);
   if (rc != FUSEDMM_SUCCESS_RETURN) { printf("FAILED: fusedMM_csr returned %d\n", rc); return 1; }
   double worst = 0;
   for (INDEXTYPE i = 0; i < n; i++)
      for (INDEXTYPE j = rowptr[i]; j < rowptr[i + 1]; j++)
      {
         double dot = 0, d;
         for (INDEXTYPE t = 0; t < k; t++) dot += (double)x[i * k + t] * y[col[j] * k + t];
         d = 1.0 - 1.0 / (1.0 + exp(-(double)(float)dot));
         for (INDEXTYPE t = 0; t < k; t++) w[i * k + t] += (VALUETYPE)(d * y[col[j] * k + t]);
      }
   for (INDEXTYPE i = 0; i < n * k; i++)
   {
      double e = fabs((double)z[i] - (double)w[i]);
      if (e > worst) worst = e;
   }
   printf("max |dz| = %.3e\n", worst);

   /* Z[i] = max over the row's edges of |X[i] - Y[c]|, element by element, through AOP_UDEF_FUNC */
   for (INDEXTYPE i = 0; i < n * k; i++) z[i] = w[i] = 0;
   imsg = VOP_SUBR | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_UDEF;
   rc = fusedMM_csr(imsg, n, n, k, 1.0f, nnz, n, n, val, col, rowptr, rowptr + 1, x, k, y, k, 0.0f, z, k);
   if (rc != FUSEDMM_SUCCESS_RETURN) { printf("FAILED: fusedMM_csr with AOP_UDEF returned %d\n", rc); return 1; }
   long differ = 0;
   for (INDEXTYPE i = 0; i < n; i++)
      for (INDEXTYPE j = rowptr[i]; j < rowptr[i + 1]; j++)
         for (INDEXTYPE t = 0; t < k; t++)
         {
            const VALUETYPE d = x[i * k + t] - y[col[j] * k + t], a = d < 0 ? -d : d;
            if (a > w[i * k + t]) w[i * k + t] = a;
         }
   for (INDEXTYPE i = 0; i < n * k; i++) differ += (z[i] != w[i]);
   printf("user accumulate stage: %ld elements differ\n%s\n", differ, (worst < 1e-5 && differ == 0) ? "PASSED" : "FAILED");
   return (worst < 1e-5 && differ == 0) ? 0 : 1;
}
