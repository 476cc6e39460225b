/*
 * ref_partition_probe.c -- makes the REAL reference show which thread it gives
 * each row to.  Test infrastructure only.
 *
 * Built by oracle/Makefile together with /root/reference/fusedMM.c compiled
 * where it lies with -DPTTIME -DLOAD_BALANCE -DNTHREADS=<n>, i.e. with the
 * nnz-balanced row partition of fusedMM.c:633-676 switched on.  The reference
 * does not return its partition, but it calls the caller's SOP_UDEF_FUNC once
 * per edge from the thread that owns the edge's row (fusedMM.c:696-729).  The
 * SOP_UDEF_FUNC below is that caller-side function: fed the tuple
 * VOP_COPY_RHS | ROP_NOOP | SOP_UDEF | VSC_MUL | AOP_ADD with val[j] = id of the
 * row slot j belongs to (ROP_NOOP leaves scal = val[j], :717), it receives the
 * row id and records omp_get_thread_num() for it.
 *
 * This file contains no reference code: it declares the reference's entry
 * point and forwards to it.
 */
#include <omp.h>
#include <stdint.h>

#ifndef INDEXTYPE
#error "build with -DINDEXTYPE=int32_t or int64_t"
#endif
#define VALUETYPE float

int fusedMM_csr(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
                const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
                const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
                const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz);

static int32_t *probe_owner; /* [rows] thread that evaluated the row's edges, -1: none seen */
static int32_t *probe_calls; /* [rows] edges evaluated for the row (every edge exactly once?) */
static int32_t probe_mixed;  /* rows seen from more than one thread */

int SOP_UDEF_FUNC(VALUETYPE val, VALUETYPE *out)
{
   const int64_t row = (int64_t)val;
   const int32_t me = (int32_t)omp_get_thread_num();
   /* a row belongs to one thread, so these stores never race between threads
    * unless the partition is broken, which probe_mixed then reports */
   const int32_t before = __atomic_exchange_n(&probe_owner[row], me, __ATOMIC_RELAXED);
   if (before != -1 && before != me) __atomic_fetch_add(&probe_mixed, 1, __ATOMIC_RELAXED);
   __atomic_fetch_add(&probe_calls[row], 1, __ATOMIC_RELAXED);
   *out = val;
   return 0;
}

int ref_probe_index_bytes(void) { return (int)sizeof(INDEXTYPE); }

int ref_probe_threads(void) { return NTHREADS; }

/* Runs the reference's fusedMM_csr over the m rows described by pntrb/pntre
 * (k = 1; every operand supplied by the caller: val[j] = row id of slot j,
 * indx[j] = 0, y[0] = 1, x unused by the tuple but indexed, z[m]).  owner[] must
 * come in as -1, calls[] as 0.  Returns the reference's status, or -1000 - count
 * when some row was evaluated by more than one thread. */
int ref_partition_probe(INDEXTYPE m, INDEXTYPE nnz, const VALUETYPE *val, const INDEXTYPE *indx,
                        const INDEXTYPE *pntrb, const INDEXTYPE *pntre, const VALUETYPE *x, const VALUETYPE *y,
                        VALUETYPE *z, int32_t *owner, int32_t *calls)
{
   probe_owner = owner;
   probe_calls = calls;
   probe_mixed = 0;
   /* VOP_COPY_RHS 0x2 | ROP_NOOP 0x00 | SOP_UDEF 0xF00 | VSC_MUL 0x1000 | AOP_ADD 0x10000 (fusedMM.h:18-73) */
   const int st = fusedMM_csr(0x11F02, m, 1, 1, 1.0f, nnz, m, 1, val, indx, pntrb, pntre, x, 1, y, 1, 0.0f, z, 1);
   if (probe_mixed) return -1000 - probe_mixed;
   return st;
}
