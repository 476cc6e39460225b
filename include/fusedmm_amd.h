/*
 * fusedmm_amd.h -- entry points of libfusedmm_amd_i{32,64}.so beyond the
 * reference's fusedMM.h.  Plain C ABI: pointers, sizes and ints only.
 * Define INDEXTYPE / VALUETYPE before including, as for fusedMM.h.
 */
#ifndef FUSEDMM_AMD_H
#define FUSEDMM_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Device-native bodies for the SOP_UDEF stage.  They restate, expression for
 * expression, the SOP_UDEF_FUNC bodies the reference's tester compiles, one
 * per executable (reference test/fusedMMtime.cpp:626-674).
 */
#define FUSEDMM_SOP_KIND_HOST     (-1) /* call the host symbol SOP_UDEF_FUNC per edge (three passes) */
#define FUSEDMM_SOP_KIND_IDENTITY   0  /* d = s                          (:668-673) */
#define FUSEDMM_SOP_KIND_SIGMOID    1  /* d = 1 - table_sigmoid(s)       (:606-611, 628-632) */
#define FUSEDMM_SOP_KIND_TDIST      2  /* d = clamp(-2/(1+s), -5, 5)     (:613-618, 642-646) */
#define FUSEDMM_SOP_KIND_FR         3  /* d = 1 + 1/s                    (:635-639) */
#define FUSEDMM_SOP_KIND_LL         4  /* d = log2(1 + sqrt(s))          (:649-653) */
#define FUSEDMM_SOP_KIND_FA         5  /* d = sqrt(s) + 1/s              (:656-660) */
/* The t-distribution weight as it is usually written, d = 1/(1+s): the tester's body (kind 2) is this times
 * the constant -2, clamped to [-5, 5], which never binds for s >= 0.  No body of the tester computes it; a
 * caller who wants it from the reference writes it as a SOP_UDEF_FUNC, and this kind gives the bits such a
 * function written with the tester's conventions gives: (VALUETYPE)(1.0 / (1.0 + s)), formed in double. */
#define FUSEDMM_SOP_KIND_TDIST_PLAIN 6

/*
 * Choose what SOP_UDEF means for later fusedMM_csr calls of this process.
 * Replaces the reference's link-time choice of a SOP_UDEF_FUNC body
 * (kernels/CONFIG/make.base:339-345 builds one executable per -D<KIND>_UDEF).
 * Returns the previous kind, or -2 for an unknown kind.  The initial kind comes
 * from the environment variable FUSEDMM_SOP_KIND (host, identity, sigmoid,
 * tdist, fr, ll, fa, tdist_plain) and is "host" when that is unset.  A call of this function
 * overrides the variable, whenever it is made (the same holds for every setter below whose
 * setting also has a variable).
 */
int fusedMM_amd_set_sop_kind(int kind);
int fusedMM_amd_get_sop_kind(void);

/*
 * Register the host SOP function used by FUSEDMM_SOP_KIND_HOST.  When never
 * called, the library looks up the symbol SOP_UDEF_FUNC in the process, which
 * is how the reference binds it (fusedMM.h:139; genkern.base:487, 554).
 */
typedef int (*fusedMM_amd_sop_fn)(VALUETYPE val, VALUETYPE *out);
void fusedMM_amd_set_sop_callback(fusedMM_amd_sop_fn fn);

/*
 * VOP_UDEF, ROP_UDEF, VSC_UDEF, AOP_UDEF: the caller's host functions, with the
 * reference's prototypes (fusedMM.h:135-143), called as the reference calls them
 * (fusedMM.c:696-740): VOP(k, X[i], k, Y[c], k, T); ROP(k, X[i], k, T, &scal) with
 * scal starting as the edge value; VSC(k, T, out, k, T); AOP(k, T, k, Z[i]), the
 * last in edge order within a row.  A tuple that names such a stage is served by
 * the synchronous entry point when the process defines <STAGE>_UDEF_FUNC (looked up
 * by name, as SOP_UDEF_FUNC is) or a function was registered here (NULL: look the
 * name up); otherwise it returns FUSEDMM_UNDEFINED_USER_FUNCTION, which is what the
 * reference's default build, compiled without <STAGE>_UDEF_IMPL, makes of it
 * (fusedMM.h:129-133, fusedMM_internal.h:50-84).  The library's own stages of such
 * a tuple run on the GPU, over per-edge buffers (k values per edge slot of device
 * memory); only the caller's functions run on the host, rows dealt to a few
 * threads, so they must be thread-safe as the reference requires
 * (fusedMM.h:125-126).  Their return values are ignored, as in the reference's
 * release build.
 */
typedef int (*fusedMM_amd_vop_fn)(INDEXTYPE lhs_dim, const VALUETYPE *lhs, INDEXTYPE rhs_dim, const VALUETYPE *rhs,
                                  INDEXTYPE out_dim, VALUETYPE *out);
typedef int (*fusedMM_amd_rop_fn)(INDEXTYPE lhs_dim, const VALUETYPE *lhs, INDEXTYPE rhs_dim, const VALUETYPE *rhs,
                                  VALUETYPE *out);
typedef int (*fusedMM_amd_vsc_fn)(INDEXTYPE rhs_dim, const VALUETYPE *rhs, VALUETYPE scal, INDEXTYPE out_dim,
                                  VALUETYPE *out);
typedef int (*fusedMM_amd_aop_fn)(INDEXTYPE rhs_dim, const VALUETYPE *rhs, INDEXTYPE out_dim, VALUETYPE *out);
void fusedMM_amd_set_stage_callbacks(fusedMM_amd_vop_fn vop, fusedMM_amd_rop_fn rop, fusedMM_amd_vsc_fn vsc,
                                     fusedMM_amd_aop_fn aop);

/*
 * fusedMM_csr on a caller-supplied HIP stream: every pointer is device memory,
 * work is enqueued on `stream` (a hipStream_t; NULL is the default stream) and
 * the call returns without waiting.  No counterpart in the reference; it is what
 * a framework that already keeps its tensors on the GPU binds (the reference's
 * CMakeLists.txt:1-14 packages fusedMM_csr for DGL).  Every call on a GPU uses
 * that GPU's one set of work queues, so the library runs calls enqueued on
 * different streams one after the other (each waits for the previous call's last
 * kernel).  Under HIP graph capture that ordering is the caller's, and a call
 * whose work queues would have to grow returns FUSEDMM_NOT_ENOUGH_MEM: run one
 * call of the same size before capturing; a later, larger call re-allocates the
 * queues and invalidates graphs captured earlier (fusedMM_csr_stream_noalloc has
 * neither restriction).
 * A stream that carried an eager call must not
 * enter a capture while a call on ANOTHER stream may still have to be ordered after it: that
 * call is refused with FUSEDMM_FAIL_RETURN (an event recorded on a capturing stream would
 * become a node of the caller's graph), and succeeds once the capture has ended.
 * FUSEDMM_SOP_KIND_HOST is
 * not available here (it needs the host between passes): returns
 * FUSEDMM_UNDEFINED_USER_FUNCTION.
 */
int fusedMM_csr_stream
(
   const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
   const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
   const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
   const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
   const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz, void *stream
);

/*
 * fusedMM_csr_stream for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference.  Same arguments, results (bit for bit) and rules
 * as fusedMM_csr_stream, but the call's work queues (counters, queued-row bitmap,
 * heavy-row queue, segment descriptors, partial results of split rows) and the
 * sigmoid table live in a static device array of fusedMM_amd_noalloc_capacity()
 * bytes (32 MiB) that every GPU the library runs on holds until the process ends;
 * the call allocates and frees nothing.  A call whose queues, sized from m, nnz
 * and k exactly as fusedMM_csr_stream sizes them, do not fit returns
 * FUSEDMM_NOT_ENOUGH_MEM with a message on stderr and touches nothing; so does
 * k > 2048 and m > 2^25.  (The first 4 MiB hold the table, the counters and one
 * bit per row; the sigmoid benchmark at K=128 with 2^20 rows and 2^24 edges needs
 * 10.9 MiB in all.)  Pass the true nnz: it sizes the queues.  The first call on a device
 * looks up the array's address and copies the 2048-entry table there; do that
 * ahead of time, outside any capture, with fusedMM_amd_init().  All calls on a
 * GPU share the one array: calls enqueued on different streams are ordered one
 * after the other by the library, except while a stream is being captured, where
 * the caller must keep them from overlapping.
 */
int fusedMM_csr_stream_noalloc
(
   const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
   const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
   const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
   const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
   const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz, void *stream
);
int64_t fusedMM_amd_noalloc_capacity(void);

/* Set up the current device ahead of the first call: small fixed allocations of
 * the ordinary entry points (sigmoid table, counters) and the static array of
 * fusedMM_csr_stream_noalloc.  Optional outside HIP graph capture, where every
 * entry point does its part of this on first use; required before a device's
 * first call is captured (that call returns FUSEDMM_FAIL_RETURN otherwise, as the
 * set-up copies and clears with blocking calls).  Operand validation
 * (fusedMM_amd_set_validate) waits for the GPU too: a captured call is refused
 * while it is switched on.  Returns a fusedMM status code. */
int fusedMM_amd_init(void);

/* The part of fusedMM_amd_init() that fusedMM_csr_stream_noalloc needs, for callers that must not
 * allocate device memory at set-up either: looks up the static array's address on the current
 * device, copies the sigmoid table there and clears its counters (blocking copies: not inside a
 * capture).  No hipMalloc; the ordinary entry points still make their small allocations on their
 * own first use.  No counterpart in the reference.  Returns a fusedMM status code. */
int fusedMM_amd_init_noalloc(void);

/*
 * The reference's second-level entry (kernels/include/kernels.h:32-37,
 * kernels/src/kernels.c:456-631): tkern 'g' gcn, 'm' spmm, 's' sigmoid,
 * 't' t-dist/FR.  Same pointer rules as fusedMM_csr.  Exported by the
 * single-precision libraries.
 */
void sgfusedMM_csr
(
   const char tkern, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
   const float alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
   const float *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
   const float *a, const INDEXTYPE lda, const float *b, const INDEXTYPE ldb,
   const float beta, float *c, const INDEXTYPE ldc
);

/* The same for the double-precision libraries (kernels/include/kernels.h:17-22). */
void dgfusedMM_csr
(
   const char tkern, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
   const double alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
   const double *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
   const double *a, const INDEXTYPE lda, const double *b, const INDEXTYPE ldb,
   const double beta, double *c, const INDEXTYPE ldc
);

/* sizeof(INDEXTYPE) and sizeof(VALUETYPE) this library was built for (4 or 8 each).
 * Libraries: libfusedmm_amd_i32.so, _i64.so (float; the reference's default
 * build) and libfusedmm_amd_d_i32.so, _d_i64.so (double; its -DDREAL build). */
int fusedMM_amd_index_bytes(void);
int fusedMM_amd_value_bytes(void);

/* 1: pattern-matched tuples use the optimised kernels' write-back rule
 * (default, the reference's ENABLE_OPT_FUSEDMM build, fusedMM.c:512-605);
 * 0: every tuple follows the general pipeline (always accumulates);
 * 2: as 1, and a tuple that matches no optimised kernel is refused with
 * FUSEDMM_NO_OPT_IMPL (the reference built with MUST_OPT_FUSEDMM,
 * fusedMM.c:599-604).  Returns the previous setting. */
int fusedMM_amd_set_opt(int enable);

/* 1: before each call, check on the device that every row has pntrb <= pntre
 * and every column id lies in [0, n); a call with bad operands then returns
 * FUSEDMM_FAIL_RETURN instead of reading outside Y.  Off by default (the
 * reference does not check either); also enabled by FUSEDMM_VALIDATE=1.
 * Costs one pass over the CSR arrays and a synchronisation.  Returns the
 * previous setting. */
int fusedMM_amd_set_validate(int enable);

/*
 * Host-pointer calls (fusedMM_csr with ordinary host arrays) upload every
 * operand on every call, because the caller may have changed it: the reference
 * keeps no state either.  fusedMM_amd_set_cache(1) (or FUSEDMM_CACHE=1) keeps a
 * device mirror of each read-only operand (val, indx, pntrb, pntre, x, y), keyed
 * by host address and size, and reuses it on later calls; only z then travels.
 * The caller promises not to change those arrays, or calls
 * fusedMM_amd_invalidate() after changing them (it drops every mirror; at most
 * 32 are kept per GPU, the one used longest ago goes first).  Off by default.
 * Returns the previous setting.
 */
int fusedMM_amd_set_cache(int enable);
void fusedMM_amd_invalidate(void);

/* Upload, kernel and download time in milliseconds of the last fusedMM_csr call
 * that took host pointers; FUSEDMM_FAIL_RETURN when there was none. */
int fusedMM_amd_last_host_phases(double *upload_ms, double *kernels_ms, double *download_ms);

/* Tuning knobs of the heavy-row split: rows with more than `heavy_deg` edges
 * are cut into segments of `seg_len` edges (0, 0 restores the K-dependent
 * defaults).  For tests and experiments. */
void fusedMM_amd_set_split(int64_t heavy_deg, int seg_len);
/* The values in force (0: the K-dependent default): what fusedMM_amd_set_split() last set, or else what
 * the environment variable FUSEDMM_SPLIT=heavy_deg,seg_len gave. */
void fusedMM_amd_get_split(int64_t *heavy_deg, int *seg_len);

/* Short rows one per group of lanes.  For K <= 64 a wavefront holds S = 8 (K <= 32) or 4 neighbour rows at a time and
 * keeps U = 8 gathers (4 in double precision) in flight for each.  A group of S consecutive CSR rows (row numbers
 * g*S .. g*S+S-1) whose longest row has md <= S*U edges and ceil(md / U) <= (rows of the group that have edges) is
 * processed with one row per group of lanes, every row's edges in order, instead of one row after the other across
 * the whole wavefront.  1 (default; also FUSEDMM_PACK_ROWS=on|auto) enables it, 0 (FUSEDMM_PACK_ROWS=off) disables
 * it.  Which rows are taken that way depends on the row pointers only; it changes the order in which such a row's
 * edges are summed (same values to rounding) and nothing else.  Returns the previous setting. */
int fusedMM_amd_set_pack_rows(int enable);

/* When finished rows of Z are written.  Where the gathered matrix Y is 1 GiB or more, a finished row waits in the
 * compute unit's local memory and every wavefront of a call writes its waiting rows when the same tick of the
 * device's constant 100 MHz counter passes (the counter shifted right by `shift` bits: 13, a period of 82 us; 12
 * where the caller's nnz / m is below 10), or earlier when its share of that memory is full: the stores of the whole
 * grid reach memory in short common bursts instead of a steady trickle between the gathers, which the memory system
 * serves faster.  Results do not change, bit for bit.  shift = 0 (FUSEDMM_STORE_TICK=off) writes every row as it
 * finishes; 8 ... 24 sets the period and holds rows whatever the size of Y; -1 (FUSEDMM_STORE_TICK=auto) restores
 * the rule above.  Rows too wide for two of them to fit the wavefront's share, and the general pipeline's rows, are
 * always written at once.  Returns the previous setting.  For tests and experiments. */
int fusedMM_amd_set_store_tick(int shift);

/*
 * Per-kernel timing with HIP events on the stream the kernels run on.
 * enable = n > 0 starts a fresh recording of every n-th call (1: every call; up
 * to 512 calls are kept); 0 stops.  Event records between a call's kernels keep
 * them from being dispatched back to back (about 20 us per call on an MI355X), so
 * a caller that also times whole calls samples, e.g. every 4th.  The summary
 * waits for the recorded events and returns the number of calls recorded and the
 * summed milliseconds of the three kernels of those calls: classify (queues heavy
 * rows), fused (all the gathering and arithmetic), merge (folds split rows).
 */
void fusedMM_amd_timing(int enable);
int fusedMM_amd_timing_summary(double *classify_ms, double *fused_ms, double *merge_ms);
/* The same for recorded call number i (0-based); returns 0, or FUSEDMM_FAIL_RETURN when i is out of range. */
int fusedMM_amd_timing_call(int i, double *classify_ms, double *fused_ms, double *merge_ms);

/* Counters of the last call on this thread's device: heavy rows queued, edge
 * segments queued, heavy rows that did not fit the queue.  Waits for the device. */
int fusedMM_amd_last_split(unsigned int *heavy_rows, unsigned int *segments, unsigned int *overflow);

/* Where the last call's rows (those not split into segments) had their edges, as its first kernel
 * sampled it (the rows of 32 of its workgroups, scaled down by 64): in the lower and in the upper half
 * of the row space.  When one half holds
 * more than 1.25 times the other (R-MAT graphs, vertices sorted by degree) and rows are claimed
 * dynamically, `scattered` is 1: the row phase then took stretches of 512 rows in a scattered order
 * instead of first to last, so that the GPU works on a mix of dense and sparse rows at any time.
 * Results do not depend on it.  The environment variable FUSEDMM_ROW_ORDER=plain | scattered | auto
 * (read once, at the first call) overrides the choice.  Waits for the GPU. */
int fusedMM_amd_last_row_order(int *scattered, unsigned int *edges_lower_half, unsigned int *edges_upper_half);

/* Release every device buffer the library holds (work queues, staging). */
void fusedMM_amd_finalize(void);

#ifdef __cplusplus
}
#endif

#endif /* FUSEDMM_AMD_H */
