/* Links against the CMake target `fusedmm` and includes fusedMM.h only; INDEXTYPE
 * and VALUETYPE come from the target.  gcn op on a ring graph with Y = 1: every
 * Z entry must equal the row's degree. */
#include <stdio.h>
#include <stdlib.h>

#include "fusedMM.h"

int main(void)
{
   const INDEXTYPE n = 4096, k = 64, deg = 5;
   INDEXTYPE *ptr = malloc(sizeof(INDEXTYPE) * (size_t)(n + 1)), *col = malloc(sizeof(INDEXTYPE) * (size_t)(n * deg));
   VALUETYPE *y = malloc(sizeof(VALUETYPE) * (size_t)(n * k)), *z = malloc(sizeof(VALUETYPE) * (size_t)(n * k));
   for (INDEXTYPE i = 0; i <= n; i++) ptr[i] = i * deg;
   for (INDEXTYPE j = 0; j < n * deg; j++) col[j] = (j / deg + 1 + (j % deg) * 97) % n;
   for (INDEXTYPE i = 0; i < n * k; i++) { y[i] = 1; z[i] = -7; }
   const int32_t gcn = VOP_COPY_RHS | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_ADD;
   int rc = fusedMM_csr(gcn, n, n, k, 1, n * deg, n, n, NULL, col, ptr, ptr + 1, NULL, k, y, k, 0, z, k);
   long bad = 0;
   for (INDEXTYPE i = 0; i < n * k; i++) bad += (z[i] != (VALUETYPE)deg);
   printf("fusedMM_csr returned %d, %ld wrong entries\n%s\n", rc, bad, (rc == 0 && bad == 0) ? "PASSED" : "FAILED");
   return (rc == 0 && bad == 0) ? 0 : 1;
}
