/*
 * fusedmm_oracle.c -- CPU restatement of the reference's fused SDDMM+SpMM path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the tests, the smoke
 * check and the CPU-baseline leg of the benchmark may load it; the shipped
 * library never links, loads or calls anything in this directory.
 *
 * Each function names the reference file:line it restates.  Value-type
 * dependent functions live in fusedmm_oracle_val.inc (float: no suffix, double:
 * _d), index-width dependent ones in fusedmm_oracle_body.inc (suffixes _i32,
 * _i64, _d_i32, _d_i64), mirroring the reference's compile-time INDEXTYPE and
 * SREAL / DREAL.  Every pin below holds for both precisions.
 *
 * Pinning status (what independently checks each function):
 *   orc_sigmoid_table / orc_sigmoid_lookup / orc_sop
 *        - bit-compared with the reference harness's own SM_TABLE and
 *          SOP_UDEF_FUNC bodies through oracle/_ref (tests/test_oracle_ref.py),
 *          committed as tests/golden/sop_*.npz; closed forms sigma(0)=0.5,
 *          saturation beyond +-5, monotonicity.
 *        ORC_SOP_TDIST_PLAIN (1/(1+val); no such body in the harness) - closed
 *          form in exact arithmetic on dyadic arguments; -2 * plain == the TDIST
 *          body bit for bit wherever its clamp does not bind (a power-of-two
 *          factor commutes with the one rounding); dense fp64 brute force of the
 *          whole op; X == Y rows contribute exactly zero.
 *   orc_fusedmm_generic_*  - bit-compared with the reference's generic
 *          fusedMM_csr (compiled from /root/reference/fusedMM.c) on seeded
 *          inputs; scipy CSR @ Y for the spmm/gcn tuples; dense brute force.
 *   orc_fusedmm_generic_udef_* (the general pipeline with the caller's VOP / ROP /
 *          SOP / VSC / AOP functions bound) - bit-compared with the reference's
 *          fusedMM.c built with VOP/ROP/VSC/AOP_UDEF_IMPL switched on and linked with
 *          the same caller-side functions (ref_udef_stages.c, udef_stage_bodies.inc):
 *          all 1344 tuples with a user stage, live, in every precision and index
 *          width (tests/test_oracle_ref.py), 65 of them committed as
 *          tests/golden/udef_stages.npz.  The functions are asymmetric, use the
 *          scalar's start value, work in place and do not commute across edges, so
 *          swapped operands, a missing seed or a changed edge order show.
 *   orc_fusedmm_opt_*      - golden Z from the reference harness's trusted
 *          kernels and generic fusedMM_csr; dense fp64 brute force; invariants.
 *   orc_partition_rows_*   - row for row against the thread the real reference
 *          (fusedMM.c built with -DPTTIME -DLOAD_BALANCE -DNTHREADS=2,3,5,8,16
 *          plus ref_partition_probe.c, whose SOP_UDEF_FUNC records
 *          omp_get_thread_num() per row) evaluates each row on: committed as
 *          tests/golden/partition.npz (30 degree sets: front/back heavy, empty
 *          rows at boundaries, fewer ranges than threads, m < rows, gapped
 *          pointers, Zipf and geometric degrees) and live on fresh random sets
 *          (tests/test_oracle_ref.py).  The vectors separate the rule from its
 *          near misses (quota not recomputed, >= for >, tipping row kept, running
 *          count not restarted); plus hand-computed examples.
 *   orc_gpu_dot / mode 2   - equals the fp64 dot within K*eps*sum|x*y|; equals
 *          the sequential dot exactly for inputs whose products are exactly
 *          representable (small integers), which a wrong lane map would break.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_SM_TABLE_SIZE 2048
#define ORC_SM_BOUND 5.0

/* status codes: fusedMM.h:103-112 */
#define ORC_SUCCESS 0
#define ORC_VOP_FAIL 2
#define ORC_ROP_FAIL 4
#define ORC_AOP_FAIL 8
#define ORC_SOP_FAIL 16
#define ORC_VSC_FAIL 32
#define ORC_UNDEFINED_USER_FUNCTION 64

/* SOP_UDEF_FUNC bodies the reference harness compiles, one per executable
 * (test/fusedMMtime.cpp:626-674).  Numbering is shared with the product's
 * additive API so tests can pass the same integer to both sides. */
enum {
   ORC_SOP_IDENTITY = 0, /* default dummy body: *out = val  (:668-673)  */
   ORC_SOP_SIGMOID = 1,  /* 1 - table_sigmoid(val)          (:628-632)  */
   ORC_SOP_TDIST = 2,    /* clamp(-2/(1+val), +-5)          (:642-646)  */
   ORC_SOP_FR = 3,       /* 1 + 1/val                       (:635-639)  */
   ORC_SOP_LL = 4,       /* log2(1 + sqrt(val))             (:649-653)  */
   ORC_SOP_FA = 5,       /* sqrt(val) + 1/val               (:656-660)  */
   /* Not a body of the harness: the t-distribution weight as usually written,
    * 1/(1+val), i.e. the TDIST body without its constant -2 and its clamp, in the
    * harness's conventions (double literals, one rounding).  Pinned by its closed
    * form and by its exact relation to ORC_SOP_TDIST (tests/test_oracle_pins.py). */
   ORC_SOP_TDIST_PLAIN = 6
};

/* ---- value-type dependent part, compiled for float and double ---- */
#define ORC_VAL float
#define ORC_VFN(name) name
#define ORC_EXP expf
#define ORC_SQRT sqrtf
#define ORC_LOG2 log2f
#define ORC_FMA fmaf
#include "fusedmm_oracle_val.inc"
#undef ORC_VAL
#undef ORC_VFN
#undef ORC_EXP
#undef ORC_SQRT
#undef ORC_LOG2
#undef ORC_FMA

#define ORC_VAL double
#define ORC_VFN(name) name##_d
#define ORC_EXP exp
#define ORC_SQRT sqrt
#define ORC_LOG2 log2
#define ORC_FMA fma
#include "fusedmm_oracle_val.inc"
#undef ORC_VAL
#undef ORC_VFN
#undef ORC_EXP
#undef ORC_SQRT
#undef ORC_LOG2
#undef ORC_FMA

/* Counts the floats v in [-5, 5] for which the reference's bin expression
 * (orc_sigmoid_bin, a double division by 10.0) and the single multiply
 * (int)(((double)v + 5.0) * 204.8) disagree.  The GPU kernels use the multiply;
 * the count must be zero.  Visits every float bit pattern. */
int64_t orc_count_bin_formula_mismatches(int64_t *visited)
{
   int64_t bad = 0, seen = 0;
#pragma omp parallel for reduction(+ : bad, seen) schedule(static)
   for (int64_t u = 0; u < ((int64_t)1 << 32); u++)
   {
      uint32_t bits = (uint32_t)u;
      float v;
      memcpy(&v, &bits, sizeof(v));
      if (!(v >= -5.0f && v <= 5.0f)) continue;
      seen++;
      int want = (int)(((double)v + ORC_SM_BOUND) * ORC_SM_TABLE_SIZE / (2.0 * ORC_SM_BOUND));
      int got = (int)(((double)v + 5.0) * 204.8);
      bad += (want != got);
   }
   if (visited) *visited = seen;
   return bad;
}

int orc_max_threads(void)
{
#ifdef _OPENMP
   return omp_get_max_threads();
#else
   return 1;
#endif
}

/* ---- index-width (and value-type) dependent part: four instances ---- */
#define ORC_VAL float
#define ORC_WIDE double
#define ORC_VFN(name) name
#define ORC_FMA fmaf
#define ORC_IDX int32_t
#define ORC_FN(name) name##_i32
#include "fusedmm_oracle_body.inc"
#undef ORC_IDX
#undef ORC_FN
#define ORC_IDX int64_t
#define ORC_FN(name) name##_i64
#include "fusedmm_oracle_body.inc"
#undef ORC_IDX
#undef ORC_FN
#undef ORC_VAL
#undef ORC_WIDE
#undef ORC_VFN
#undef ORC_FMA

#define ORC_VAL double
#define ORC_WIDE long double
#define ORC_VFN(name) name##_d
#define ORC_FMA fma
#define ORC_IDX int32_t
#define ORC_FN(name) name##_d_i32
#include "fusedmm_oracle_body.inc"
#undef ORC_IDX
#undef ORC_FN
#define ORC_IDX int64_t
#define ORC_FN(name) name##_d_i64
#include "fusedmm_oracle_body.inc"
#undef ORC_IDX
#undef ORC_FN
#undef ORC_VAL
#undef ORC_WIDE
#undef ORC_VFN
#undef ORC_FMA
