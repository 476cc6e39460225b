// Tester + timer for the GPU build of fusedMM_csr, with the command line and
// the CSV line of the reference's test/fusedMMtime.cpp (flags :1807-1954, CSV
// :1758-1804) plus a GPU path:
//
//   xfusedMMtime_i64 -input graph.mtx -K 128 -t s -T 1 -nrep 20 [-M rows]
//                    [-C cacheKB] [-skHd 1] [-ibeta 0|1] [-gpu 0|1] [-opt 1|0|2] [-prof 1]
//
//   -t <t|f|s|m|g>  op kind: t-dist, FR, sigmoid, spmm, gcn.  The reference
//                   builds one executable per kind (-D<KIND>_UDEF); here one
//                   executable selects the op tuple AND the device SOP body.
//                   An executable name containing _tdist_, _fr_, _sigmoid_,
//                   _spmm_ or _gcn_ sets the default the same way.
//   -T 1            run the tester first: scalar "trusted" kernel on the CPU
//                   against fusedMM_csr on the GPU, element by element.
//   -gpu 1          (default) operands resident in device memory while timing;
//   -gpu 0          pass host pointers: every call stages operands over PCIe; the
//                   upload, kernel and download times of the last call are printed.
//   -cache 1        with -gpu 0: keep device mirrors of the read-only operands
//                   between calls (fusedMM_amd_set_cache), so only C travels.
//   -C <KB>         rotate through enough operand copies to exceed this cache
//                   size (reference :1533-1654); default 0 = one copy.
//   -opt 1          (default) tuples with an optimised kernel use it: the reference's
//                   xsOptFusedMMtime_* executables (built with ENABLE_OPT_FUSEDMM);
//   -opt 0          every tuple goes through the general pipeline: its xsFusedMMtime_*;
//   -opt 2          as 1, and a tuple without an optimised kernel is an error (MUST_OPT_FUSEDMM).
//   -prof 1         wrap the phases in roctx ranges for rocprofv3 --marker-trace.
//
// "Trusted" CPU kernels restate test/fusedMMtime.cpp:159-365; inputs follow
// :884-951 (a, b, edge values ~ U[0,1) from a default-seeded
// std::default_random_engine, c = 0).
#include <hip/hip_runtime.h>
#include <omp.h>
#include <rocprofiler-sdk-roctx/roctx.h>

#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#ifndef INDEXTYPE
#define INDEXTYPE int64_t
#endif
#ifdef DREAL       /* double precision, as in the reference's build (-DDREAL) */
#define VALUETYPE double
#else
#define VALUETYPE float
#endif
#include "../../include/fusedMM.h"
#include "../../include/fusedmm_amd.h"
#include "mtx_csr.hpp"

typedef INDEXTYPE IT;
typedef VALUETYPE VT;

static bool g_prof = false;
struct Range {
   explicit Range(const char *name) { if (g_prof) roctxRangePush(name); }
   ~Range() { if (g_prof) roctxRangePop(); }
};

#define HIP_OK(call)                                                                      \
   do {                                                                                   \
      hipError_t e_ = (call);                                                             \
      if (e_ != hipSuccess) {                                                             \
         fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                \
         exit(1);                                                                         \
      }                                                                                   \
   } while (0)

// ---- trusted (scalar) kernels ---------------------------------------------------------
static VT g_table[2048];
static void init_table()
{
   for (int i = 0; i < 2048; i++)
   {
      VT x = (VT)(2.0 * 5.0 * i / 2048 - 5.0);
      VT e = std::exp(-x);               // overload of VALUETYPE, as in the reference's C++ tester
      g_table[i] = (VT)(1.0 / (double)(1 + e));
   }
}
static inline VT table_sigmoid(VT v)
{
   if (v > 5.0) return 1.0;
   if (v < -5.0) return 0.0;
   int i = (int)(((double)v + 5.0) * 2048 / 10.0);
   return g_table[i > 2047 ? 2047 : i];
}

static void trusted(char tkern, IT m, IT k, const VT *val, const IT *indx, const IT *pntrb, const IT *pntre,
                    const VT *a, const VT *b, VT *c)
{
#pragma omp parallel for schedule(dynamic, 64)
   for (IT i = 0; i < m; i++)
   {
      std::vector<VT> T((size_t)k);
      VT *ci = c + (int64_t)i * k;
      const VT *ai = a + (int64_t)i * k;
      for (IT j = pntrb[i]; j < pntre[i]; j++)
      {
         const VT *bj = b + (int64_t)indx[j] * k;
         if (tkern == 'g')
            for (IT t = 0; t < k; t++) ci[t] += bj[t];
         else if (tkern == 'm')
            for (IT t = 0; t < k; t++) ci[t] += val[j] * bj[t];
         else if (tkern == 's')
         {
            VT s = 0;
            for (IT t = 0; t < k; t++) s += ai[t] * bj[t];
            VT d = table_sigmoid(s);
            for (IT t = 0; t < k; t++) ci[t] = (VT)(ci[t] + (1.0 - d) * bj[t]);
         }
         else
         {
            VT s = 0;
            for (IT t = 0; t < k; t++)
            {
               T[t] = ai[t] - bj[t];
               s += T[t] * T[t];
            }
            VT d;
            if (tkern == 't')
            {
               d = (VT)(-2.0 / (1.0 + s));
               d = d > (VT)5.0 ? (VT)5.0 : (d < (VT)-5.0 ? (VT)-5.0 : d);
            }
            else
               d = (VT)(1.0 + 1.0 / s);
            for (IT t = 0; t < k; t++) ci[t] = ci[t] + d * T[t];
         }
      }
   }
}

static int32_t message_for(char tkern)
{
   switch (tkern)
   {
      case 't': case 'f': return VOP_SUBR | ROP_NORMR | SOP_UDEF | VSC_MUL | AOP_ADD;
      case 's': return VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD;
      case 'm': return VOP_COPY_RHS | ROP_NOOP | SOP_COPY | VSC_MUL | AOP_ADD;
      default: return VOP_COPY_RHS | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_ADD;
   }
}
static int sop_kind_for(char tkern)
{
   switch (tkern)
   {
      case 't': return FUSEDMM_SOP_KIND_TDIST;
      case 'f': return FUSEDMM_SOP_KIND_FR;
      case 's': return FUSEDMM_SOP_KIND_SIGMOID;
      default: return FUSEDMM_SOP_KIND_IDENTITY;
   }
}

// flops per edge in the reference's convention (test/fusedMMtime.cpp:806-831)
static double flops_per_edge(char tkern, IT k)
{
   switch (tkern)
   {
      case 's': return 4.0 * k;
      case 't': case 'f': return 5.0 * k;
      case 'm': return 2.0 * k;
      default: return 1.0 * k;
   }
}
static double algorithmic_bytes(char tkern, IT m, IT k, int64_t nnz)
{
   const double F = sizeof(VT), I = sizeof(IT);
   const double vb = tkern == 'm' ? F : 0, xb = (tkern == 's' || tkern == 't' || tkern == 'f') ? F * k : 0;
   return nnz * (F * k + I + vb) + (double)m * (xb + F * k + 2 * I);
}

static void usage()
{
   printf("\nUsage:\n");
   printf("-input <string>, full path of input .mtx file (required)\n");
   printf("-M <number>, rows of S to process (can be less than the rows of S)\n");
   printf("-K <number>, number of cols of A, B and C\n");
   printf("-C <number>, cache size in KB to flush by rotating operand copies (0 = off)\n");
   printf("-nrep <number>, number of repetitions\n");
   printf("-T <0,1>, 1 means run the tester as well\n");
   printf("-t <t,f,s,m,g>, t-distribution, FR, sigmoid, spmm, gcn\n");
   printf("-skHd <1>, 1 means skip the header of the printed results\n");
   printf("-ialpha <1,0,2>, accepted and ignored (alpha is unused)\n");
   printf("-ibeta <1,0>, beta 1.0 or 0.0\n");
   printf("-gpu <0,1>, 1: operands resident on the GPU while timing (default); 0: host pointers\n");
   printf("-cache <0,1>, with -gpu 0: keep device mirrors of the read-only operands between calls\n");
   printf("-opt <1,0,2>, 1: optimised kernels for the tuples that have one (the reference's xsOptFusedMMtime_*), "
          "0: general pipeline for every tuple (its xsFusedMMtime_*), 2: as 1, and a tuple without one is an error\n");
   printf("-prof <0,1>, 1: emit roctx ranges\n");
   printf("-h, show this usage message\n");
}

int main(int narg, char **argv)
{
   std::string inputfile;
   IT M = 0, K = 128;
   int csKB = 0, nrep = 20, isTest = 0, skHd = 0, ibeta = 0, use_gpu_resident = 1, use_cache = 0, opt = 1;
   char tkern = 's';
   const std::string exe = argv[0];
   if (exe.find("_tdist_") != std::string::npos) tkern = 't';
   else if (exe.find("_fr_") != std::string::npos) tkern = 'f';
   else if (exe.find("_spmm_") != std::string::npos) tkern = 'm';
   else if (exe.find("_gcn_") != std::string::npos) tkern = 'g';
   for (int p = 1; p < narg; p++)
   {
      const bool has = p + 1 < narg;
      if (!strcmp(argv[p], "-h")) { usage(); return 1; }
      if (!has) continue;
      if (!strcmp(argv[p], "-input")) inputfile = argv[p + 1];
      else if (!strcmp(argv[p], "-K")) K = (IT)atoll(argv[p + 1]);
      else if (!strcmp(argv[p], "-M")) M = (IT)atoll(argv[p + 1]);
      else if (!strcmp(argv[p], "-C")) csKB = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-nrep")) nrep = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-T")) isTest = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-t")) tkern = argv[p + 1][0];
      else if (!strcmp(argv[p], "-skHd")) skHd = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-ibeta")) ibeta = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-gpu")) use_gpu_resident = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-cache")) use_cache = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-opt")) opt = atoi(argv[p + 1]);
      else if (!strcmp(argv[p], "-prof")) g_prof = atoi(argv[p + 1]) != 0;
   }
   if (inputfile.empty()) { printf("Need input file ??? \n"); return 1; }
   if (!strchr("tfsmg", tkern)) { printf("unknown kernel kind '%c'\n", tkern); return 1; }
   const VT alpha = 1.0, beta = ibeta == 0 ? 0.0 : 1.0;
   if (nrep < 1) nrep = 1;

   fmm_host::CsrMatrix<IT> S;
   {
      Range r("load_mtx");
      std::string err = fmm_host::load_mtx<IT>(inputfile.c_str(), S);
      if (!err.empty()) { fprintf(stderr, "%s: %s\n", inputfile.c_str(), err.c_str()); return 1; }
   }
   const IT N = S.cols;
   if (!M || M > S.rows) M = S.rows;
   assert(N && M && K);
   init_table();
   fusedMM_amd_set_sop_kind(sop_kind_for(tkern));
   fusedMM_amd_set_opt(opt);
   const int32_t imsg = message_for(tkern);

   // inputs as the reference's tester draws them
   std::default_random_engine gen;
   std::uniform_real_distribution<VT> dist(0.0, 1.0);
   const size_t szA = (size_t)M * K, szB = (size_t)N * K, szC = (size_t)M * K;
   std::vector<VT> a(szA), b(szB), c(szC, (VT)0), c0(szC, (VT)0), values((size_t)S.nnz);
   for (auto &v : a) v = dist(gen);
   for (auto &v : b) v = dist(gen);
   for (auto &v : values) v = dist(gen);
   const IT *pb = S.rowptr.data(), *pe = S.rowptr.data() + 1;
   int64_t nnzM = (int64_t)S.rowptr[(size_t)M] - (int64_t)S.rowptr[0];
   int64_t maxdeg = 0;
   for (IT i = 0; i < M; i++) maxdeg = std::max<int64_t>(maxdeg, pe[i] - pb[i]);

   if (isTest)
   {
      Range r("tester");
      fprintf(stdout, "Applying trusted kernel\n");
      trusted(tkern, M, K, values.data(), S.colids.data(), pb, pe, a.data(), b.data(), c0.data());
      fprintf(stdout, "Applying test kernel\n");
      int rc = fusedMM_csr(imsg, M, N, K, alpha, S.nnz, S.rows, S.cols, values.data(), S.colids.data(), pb, pe,
                           a.data(), K, b.data(), K, beta, c.data(), K);
      if (rc) { fprintf(stderr, "fusedMM_csr returned %d\n", rc); return 1; }
      // Bound of the reference's checker (:816-831), 2 * degree * flops-per-element * eps,
      // taken per row.  The table sigmoid is a step function of the dot product: two
      // summation orders of one dot can land in neighbouring bins only when the dot
      // lies within rounding of a bin edge, so only those edges earn their row the
      // height of one table step (times the largest |b| of that edge); every other
      // edge must agree to rounding.  (A blanket per-edge allowance would pass a
      // kernel that picked the wrong bin everywhere.)
      const double eps = sizeof(VT) == 4 ? 1.1920928955078125e-07 : 2.220446049250313e-16;
      const double per = (tkern == 's') ? (4.0 * K + 6) : (tkern == 'm') ? 2.0 * K : (tkern == 'g') ? 1.0 * K : (5.0 * K + 2);
      std::vector<double> row_slack((size_t)M, 0.0);
      int64_t near_edges = 0;
      if (tkern == 's')
      {
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : near_edges)
         for (IT i = 0; i < M; i++)
            for (IT j = pb[i]; j < pe[i]; j++)
            {
               const VT *ai = a.data() + (int64_t)i * K, *bj = b.data() + (int64_t)S.colids[(size_t)j] * K;
               double dot = 0, mag = 0, bmax = 0;
               for (IT t = 0; t < K; t++)
               {
                  dot += (double)ai[t] * (double)bj[t];
                  mag += std::fabs((double)ai[t] * (double)bj[t]);
                  bmax = std::max(bmax, std::fabs((double)bj[t]));
               }
               const double margin = (K + 2.0) * eps * mag + 1e-300;
               if (std::fabs(dot) > 5.0 + margin) continue;                 // saturated either way
               const double pos = (dot + 5.0) * 2048.0 / 10.0;              // bin edges sit at the integers
               const double to_edge = std::fabs(pos - std::nearbyint(pos)) * 10.0 / 2048.0;
               if (to_edge <= margin)
               {
                  const bool at_end = std::fabs(std::fabs(dot) - 5.0) <= margin;   // the step to the saturated value
                  row_slack[(size_t)i] += (at_end ? 6.8e-3 : 1.3e-3) * bmax;
                  near_edges++;
               }
            }
         printf("sigmoid table: %lld of %lld edges have a dot product within rounding of a bin edge; "
                "only their rows are allowed a table step\n", (long long)near_edges, (long long)nnzM);
      }
      int64_t nerr = 0;
      for (size_t i = 0; i < szC; i++)
      {
         const size_t row = i / (size_t)K;
         const double deg = (double)(pe[row] - pb[row]);
         double d = std::fabs((double)c0[i] - (double)c[i]);
         double lim = 2.0 * std::max(1.0, deg) * per * eps * std::max(1.0, std::fabs((double)c0[i])) + row_slack[row];
         if (!(d <= lim) || c[i] != c[i])
         {
            if (nerr < 3) fprintf(stderr, "C(%zu,%zu) : expected=%e, got=%e, diff=%e\n", i / K, i % K, c0[i], c[i], d);
            nerr++;
         }
      }
      if (nerr) { printf("FAILED TEST, %lld ELEMENTS!!!\n", (long long)nerr); return 1; }
      printf("PASSED TEST\n");
      std::fill(c.begin(), c.end(), (VT)0);
      std::fill(c0.begin(), c0.end(), (VT)0);
   }

   // ---- trusted timing (CPU) -------------------------------------------------------------
   double t_trusted;
   {
      Range r("time_trusted");
      trusted(tkern, M, K, values.data(), S.colids.data(), pb, pe, a.data(), b.data(), c0.data());   // warm-up
      const int reps = std::max(1, std::min(nrep, 5));
      double t0 = omp_get_wtime();
      for (int i = 0; i < reps; i++)
         trusted(tkern, M, K, values.data(), S.colids.data(), pb, pe, a.data(), b.data(), c0.data());
      t_trusted = (omp_get_wtime() - t0) / reps;
   }

   // ---- test timing (GPU) ----------------------------------------------------------------
   double t_test, t_kernel = 0.0;
   if (use_gpu_resident)
   {
      // working-set rotation: enough copies to exceed the cache size asked for
      const double ws = (double)sizeof(VT) * (szA + szB + szC + (double)S.nnz) + sizeof(IT) * ((double)S.nnz + 2.0 * (M + 1));
      int ncopies = 1;
      if (csKB > 0 && ws < 1024.0 * csKB) ncopies = (int)std::ceil(1024.0 * csKB / ws);
      struct Dev { VT *a, *b, *c, *val; IT *idx, *ptr; };
      std::vector<Dev> d((size_t)ncopies);
      {
         Range r("h2d");
         for (auto &x : d)
         {
            HIP_OK(hipMalloc((void **)&x.a, szA * sizeof(VT)));
            HIP_OK(hipMalloc((void **)&x.b, szB * sizeof(VT)));
            HIP_OK(hipMalloc((void **)&x.c, szC * sizeof(VT)));
            HIP_OK(hipMalloc((void **)&x.val, std::max<size_t>(1, (size_t)S.nnz) * sizeof(VT)));
            HIP_OK(hipMalloc((void **)&x.idx, std::max<size_t>(1, (size_t)S.nnz) * sizeof(IT)));
            HIP_OK(hipMalloc((void **)&x.ptr, ((size_t)S.rows + 1) * sizeof(IT)));   // rows + 1 pointers
            HIP_OK(hipMemcpy(x.a, a.data(), szA * sizeof(VT), hipMemcpyHostToDevice));
            HIP_OK(hipMemcpy(x.b, b.data(), szB * sizeof(VT), hipMemcpyHostToDevice));
            HIP_OK(hipMemset(x.c, 0, szC * sizeof(VT)));
            HIP_OK(hipMemcpy(x.val, values.data(), (size_t)S.nnz * sizeof(VT), hipMemcpyHostToDevice));
            HIP_OK(hipMemcpy(x.idx, S.colids.data(), (size_t)S.nnz * sizeof(IT), hipMemcpyHostToDevice));
            HIP_OK(hipMemcpy(x.ptr, S.rowptr.data(), ((size_t)S.rows + 1) * sizeof(IT), hipMemcpyHostToDevice));
         }
      }
      auto call = [&](const Dev &x) {
         int rc = fusedMM_csr_stream(imsg, M, N, K, alpha, S.nnz, S.rows, S.cols, x.val, x.idx, x.ptr, x.ptr + 1,
                                     x.a, K, x.b, K, beta, x.c, K, nullptr);
         if (rc) { fprintf(stderr, "fusedMM_csr returned %d\n", rc); exit(1); }
      };
      call(d[0]);   // warm-up, not timed
      HIP_OK(hipDeviceSynchronize());
      {
         Range r("time_test");
         fusedMM_amd_timing(1);
         double t0 = omp_get_wtime();
         for (int i = 0; i < nrep; i++) call(d[(size_t)(i % ncopies)]);
         HIP_OK(hipDeviceSynchronize());
         t_test = (omp_get_wtime() - t0) / nrep;
         double r_ms = 0, s_ms = 0, g_ms = 0;
         int n = fusedMM_amd_timing_summary(&r_ms, &s_ms, &g_ms);
         fusedMM_amd_timing(0);
         if (n > 0) t_kernel = (r_ms + s_ms + g_ms) * 1e-3 / n;
      }
      for (auto &x : d)
      {
         HIP_OK(hipFree(x.a)); HIP_OK(hipFree(x.b)); HIP_OK(hipFree(x.c));
         HIP_OK(hipFree(x.val)); HIP_OK(hipFree(x.idx)); HIP_OK(hipFree(x.ptr));
      }
   }
   else
   {
      Range r("time_test_host_pointers");
      fusedMM_amd_set_cache(use_cache);
      auto call = [&]() {
         int rc = fusedMM_csr(imsg, M, N, K, alpha, S.nnz, S.rows, S.cols, values.data(), S.colids.data(), pb, pe,
                              a.data(), K, b.data(), K, beta, c.data(), K);
         if (rc) { fprintf(stderr, "fusedMM_csr returned %d\n", rc); exit(1); }
      };
      call();
      double t0 = omp_get_wtime();
      for (int i = 0; i < nrep; i++) call();
      t_test = (omp_get_wtime() - t0) / nrep;
      double up = 0, kern = 0, down = 0;
      if (fusedMM_amd_last_host_phases(&up, &kern, &down) == 0)
         fprintf(stderr, "host-pointer call (last of %d, mirrors %s): upload %.3f ms, kernels %.3f ms, download %.3f ms\n",
                 nrep, use_cache ? "kept" : "off", up, kern, down);
      fusedMM_amd_invalidate();
   }
   fusedMM_amd_finalize();

   if (!skHd)
      printf("Filename,NNZ,M,N,K,Trusted_exe_time,Test_exe_time,Speedup_exe_time,"
             "GPU_kernel_time,Edges_per_s,GFLOPS,Alg_GBps,Pct_peak_HBM,CPU_threads\n");
   const double tk = t_kernel > 0 ? t_kernel : t_test;
   const double bytes = algorithmic_bytes(tkern, M, K, nnzM);
   printf("%s,%lld,%lld,%lld,%lld,%e,%e,%f,%e,%e,%f,%f,%f,%d\n", inputfile.c_str(), (long long)S.nnz, (long long)M,
          (long long)N, (long long)K, t_trusted, t_test, t_trusted / t_test, t_kernel, nnzM / t_test,
          flops_per_edge(tkern, K) * nnzM / t_test / 1e9, bytes / tk / 1e9, 100.0 * bytes / tk / 8e12,
          omp_get_max_threads());
   return 0;
}
