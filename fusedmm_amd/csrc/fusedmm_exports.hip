// The entry points of libfusedmm_amd_*.so: the reference's fusedMM_csr
// (fusedMM.h:76-97) and sgfusedMM_csr / dgfusedMM_csr (kernels/include/kernels.h:17-37),
// and the additions of include/fusedmm_amd.h.
#include <dlfcn.h>

#include <new>

#include "fusedmm_host.hpp"

namespace fmm_host {

namespace {

fusedMM_amd_sop_fn host_sop_function()
{
   if (g.sop_fn) return g.sop_fn;
   return (fusedMM_amd_sop_fn)dlsym(RTLD_DEFAULT, "SOP_UDEF_FUNC");
}

int entry_unguarded(const Args &a, bool async, hipStream_t stream, int queues)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   Plan pl;
   int st = make_plan(a.imessage, g.opt, &pl);
   if (st) return st;
   int sop_kind = g.sop_kind;
   if (pl.udef_stages)
   {
      // stages that are the caller's host functions: registered, or found by the names the reference binds
      StageFns f;
      f.vop = g.vop_fn ? g.vop_fn : (fusedMM_amd_vop_fn)dlsym(RTLD_DEFAULT, "VOP_UDEF_FUNC");
      f.rop = g.rop_fn ? g.rop_fn : (fusedMM_amd_rop_fn)dlsym(RTLD_DEFAULT, "ROP_UDEF_FUNC");
      f.vsc = g.vsc_fn ? g.vsc_fn : (fusedMM_amd_vsc_fn)dlsym(RTLD_DEFAULT, "VSC_UDEF_FUNC");
      f.aop = g.aop_fn ? g.aop_fn : (fusedMM_amd_aop_fn)dlsym(RTLD_DEFAULT, "AOP_UDEF_FUNC");
      f.sop = nullptr;
      if (((pl.udef_stages & kUdefVop) && !f.vop) || ((pl.udef_stages & kUdefRop) && !f.rop) ||
          ((pl.udef_stages & kUdefVsc) && !f.vsc) || ((pl.udef_stages & kUdefAop) && !f.aop))
      {
         // what the reference's default build does with such a tuple: its stubs return this code (fusedMM_internal.h:50-84)
         FMM_LOG("the op tuple 0x%x names a *_UDEF stage for which the process defines no <STAGE>_UDEF_FUNC "
                 "(and none was registered with fusedMM_amd_set_stage_callbacks)", a.imessage);
         return FUSEDMM_UNDEFINED_USER_FUNCTION;
      }
      if (pl.needs_sop && sop_kind == FUSEDMM_SOP_KIND_HOST && GET_VSC_FLAG(a.imessage) != VSC_NOOP)
      {
         f.sop = host_sop_function();
         if (!f.sop)
         {
            FMM_LOG("SOP_UDEF: no host SOP_UDEF_FUNC found and no device body selected "
                    "(fusedMM_amd_set_sop_kind / FUSEDMM_SOP_KIND)");
            return FUSEDMM_UNDEFINED_USER_FUNCTION;
         }
      }
      if (async)
      {
         FMM_LOG("a stage evaluated by a host function needs the synchronous entry point");
         return FUSEDMM_UNDEFINED_USER_FUNCTION;
      }
      if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
      if (!a.val) pl.reads_val = false;
      const int where = operand_residence(a);
      if (where < 0) return FUSEDMM_FAIL_RETURN;
      if (where == 1)
      {
         std::vector<idx_t> hb((size_t)a.m), he((size_t)a.m);
         FMM_HIP(hipMemcpy(hb.data(), a.pntrb, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
         FMM_HIP(hipMemcpy(he.data(), a.pntre, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
         return run_host_stages(a, hb.data(), he.data(), pl, f, sop_kind);
      }
      Args dv;
      int64_t slots = 0;
      st = stage_up(a, pl, &dv, &slots);
      if (st) return st;
      st = run_host_stages(dv, a.pntrb, a.pntre, pl, f, sop_kind);
      if (st) return st;
      return stage_down(a, dv);
   }
   if (pl.needs_sop && sop_kind == FUSEDMM_SOP_KIND_HOST)
   {
      if (GET_VSC_FLAG(a.imessage) == VSC_NOOP)
         sop_kind = FUSEDMM_SOP_KIND_IDENTITY;   // the SOP result is never used
      else
      {
         fusedMM_amd_sop_fn fn = host_sop_function();
         if (!fn)
         {
            FMM_LOG("SOP_UDEF: no host SOP_UDEF_FUNC found and no device body selected "
                    "(fusedMM_amd_set_sop_kind / FUSEDMM_SOP_KIND)");
            return FUSEDMM_UNDEFINED_USER_FUNCTION;
         }
         if (async)
         {
            FMM_LOG("SOP_UDEF through a host function needs the synchronous entry point");
            return FUSEDMM_UNDEFINED_USER_FUNCTION;
         }
         if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
         const int where = operand_residence(a);
         if (where < 0) return FUSEDMM_FAIL_RETURN;
         if (where == 1)
         {
            std::vector<idx_t> hb((size_t)a.m), he((size_t)a.m);
            FMM_HIP(hipMemcpy(hb.data(), a.pntrb, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
            FMM_HIP(hipMemcpy(he.data(), a.pntre, (size_t)a.m * sizeof(idx_t), hipMemcpyDeviceToHost));
            return run_host_sop(a, hb.data(), he.data(), pl, fn);
         }
         Args dv;
         int64_t slots = 0;
         st = stage_up(a, pl, &dv, &slots);
         if (st) return st;
         st = run_host_sop(dv, a.pntrb, a.pntre, pl, fn);
         if (st) return st;
         return stage_down(a, dv);
      }
   }
   if (async)
   {
      if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
      if (g.validate)
      {
         // the check reads a flag back and waits for it: impossible inside a capture
         bool capturing = false;
         st = stream_capturing(stream, &capturing);
         if (st) return st;
         if (capturing)
         {
            FMM_LOG("operand validation is switched on and the stream is being captured; "
                    "validate once outside the capture, then switch it off (fusedMM_amd_set_validate(0))");
            return FUSEDMM_FAIL_RETURN;
         }
         st = validate_operands(a, stream, queues);
         if (st) return st;
      }
      return run_on_device(a, pl, sop_kind, stream, queues);
   }
   if (a.m <= 0 || a.k < 1) return FUSEDMM_SUCCESS_RETURN;
   const int where = operand_residence(a);
   if (where < 0) return FUSEDMM_FAIL_RETURN;
   if (where == 1)
   {
      if (g.validate)
      {
         st = validate_operands(a, 0);
         if (st) return st;
      }
      st = run_on_device(a, pl, sop_kind, 0);
      if (st) return st;
      return hip_status(hipStreamSynchronize(0), "hipStreamSynchronize");
   }
   return run_staged(a, pl, sop_kind);
}

// Nothing may leave a C entry point by exception: the host-function paths size
// std::vector buffers from the caller's row pointers and start threads.
int entry(const Args &a, bool async, hipStream_t stream, int queues = kQueuesGrown)
{
   try
   {
      return entry_unguarded(a, async, stream, queues);
   }
   catch (const std::bad_alloc &)
   {
      FMM_LOG("out of host memory");
      return FUSEDMM_NOT_ENOUGH_MEM;
   }
   catch (const std::exception &e)
   {
      FMM_LOG("%s", e.what());
      return FUSEDMM_FAIL_RETURN;
   }
   catch (...)
   {
      FMM_LOG("unexpected failure");
      return FUSEDMM_FAIL_RETURN;
   }
}

}  // namespace

}  // namespace fmm_host

using namespace fmm_host;

// ---- exported C ABI -------------------------------------------------------------------
extern "C" {

int fusedMM_csr(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
                const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
                const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
                const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz)
{
   (void)alpha; (void)rows; (void)cols;
   Args a = {imessage, (int64_t)m, (int64_t)n, (int64_t)k, (int64_t)nnz, val, indx, pntrb, pntre, x, y, z,
             (int64_t)ldx, (int64_t)ldy, (int64_t)ldz, beta};
   return entry(a, false, 0);
}

int fusedMM_csr_stream(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
                       const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
                       const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                       const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
                       const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz, void *stream)
{
   (void)alpha; (void)rows; (void)cols;
   Args a = {imessage, (int64_t)m, (int64_t)n, (int64_t)k, (int64_t)nnz, val, indx, pntrb, pntre, x, y, z,
             (int64_t)ldx, (int64_t)ldy, (int64_t)ldz, beta};
   return entry(a, true, (hipStream_t)stream);
}

int fusedMM_csr_stream_noalloc(const int32_t imessage, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k,
                               const VALUETYPE alpha, const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols,
                               const VALUETYPE *val, const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre,
                               const VALUETYPE *x, const INDEXTYPE ldx, const VALUETYPE *y, const INDEXTYPE ldy,
                               const VALUETYPE beta, VALUETYPE *z, const INDEXTYPE ldz, void *stream)
{
   (void)alpha; (void)rows; (void)cols;
   Args a = {imessage, (int64_t)m, (int64_t)n, (int64_t)k, (int64_t)nnz, val, indx, pntrb, pntre, x, y, z,
             (int64_t)ldx, (int64_t)ldy, (int64_t)ldz, beta};
   return entry(a, true, (hipStream_t)stream, kQueuesStatic);
}

int fusedMM_amd_init(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   return scratch_setup(*d);
}

int fusedMM_amd_init_noalloc(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   return scratch_setup(*d);
}

int64_t fusedMM_amd_noalloc_capacity(void) { return (int64_t)FUSEDMM_AMD_SCRATCH_BYTES; }

#ifdef FMM_DOUBLE
#define FMM_GFUSEDMM dgfusedMM_csr
#else
#define FMM_GFUSEDMM sgfusedMM_csr
#endif
void FMM_GFUSEDMM(const char tkern, const INDEXTYPE m, const INDEXTYPE n, const INDEXTYPE k, const VALUETYPE alpha,
                  const INDEXTYPE nnz, const INDEXTYPE rows, const INDEXTYPE cols, const VALUETYPE *val,
                  const INDEXTYPE *indx, const INDEXTYPE *pntrb, const INDEXTYPE *pntre, const VALUETYPE *a,
                  const INDEXTYPE lda, const VALUETYPE *b, const INDEXTYPE ldb, const VALUETYPE beta, VALUETYPE *c,
                  const INDEXTYPE ldc)
{
   int32_t imsg;
   switch (tkern)
   {
      case 'g': imsg = VOP_COPY_RHS | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_ADD; break;
      case 'm': imsg = VOP_COPY_RHS | ROP_NOOP | SOP_COPY | VSC_MUL | AOP_ADD; break;
      case 's': imsg = VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD; break;
      case 't': imsg = VOP_SUBR | ROP_NORMR | SOP_UDEF | VSC_MUL | AOP_ADD; break;
      default:
         fprintf(stderr, "unknown kernel type!\n");   // reference kernels.c:627-629 only prints
         return;
   }
   (void)fusedMM_csr(imsg, m, n, k, alpha, nnz, rows, cols, val, indx, pntrb, pntre, a, lda, b, ldb, beta, c, ldc);
}

int fusedMM_amd_index_bytes(void) { return (int)sizeof(INDEXTYPE); }

int fusedMM_amd_value_bytes(void) { return (int)sizeof(VALUETYPE); }

int fusedMM_amd_set_sop_kind(int kind)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   if (kind < FUSEDMM_SOP_KIND_HOST || kind > FUSEDMM_SOP_KIND_TDIST_PLAIN) return -2;
   int prev = g.sop_kind;
   g.sop_kind = kind;
   return prev;
}

int fusedMM_amd_get_sop_kind(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   return g.sop_kind;
}

void fusedMM_amd_set_sop_callback(fusedMM_amd_sop_fn fn)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   g.sop_fn = fn;
}

void fusedMM_amd_set_stage_callbacks(fusedMM_amd_vop_fn vop, fusedMM_amd_rop_fn rop, fusedMM_amd_vsc_fn vsc,
                                     fusedMM_amd_aop_fn aop)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   g.vop_fn = vop;
   g.rop_fn = rop;
   g.vsc_fn = vsc;
   g.aop_fn = aop;
}

int fusedMM_amd_set_opt(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   int prev = g.opt;
   g.opt = enable < 0 ? 0 : (enable > 2 ? 2 : enable);
   return prev;
}

int fusedMM_amd_set_cache(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   int prev = g.cache;
   g.cache = enable ? 1 : 0;
   return prev;
}

void fusedMM_amd_invalidate(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   int cur = 0;
   if (hipGetDevice(&cur) != hipSuccess) return;
   for (int dev = 0; dev < kMaxDevices; dev++)
   {
      DeviceState &d = g.dev[dev];
      if (d.mirrors.empty()) continue;
      if (hipSetDevice(dev) != hipSuccess) continue;
      (void)hipDeviceSynchronize();
      for (auto &mi : d.mirrors) (void)hipFree(mi.dev);
      d.mirrors.clear();
   }
   (void)hipSetDevice(cur);
}

int fusedMM_amd_last_host_phases(double *upload_ms, double *kernels_ms, double *download_ms)
{
   std::lock_guard<std::mutex> lock(g.mu);
   if (!g.phase_valid) return FUSEDMM_FAIL_RETURN;
   if (upload_ms) *upload_ms = g.phase_ms[0];
   if (kernels_ms) *kernels_ms = g.phase_ms[1];
   if (download_ms) *download_ms = g.phase_ms[2];
   return FUSEDMM_SUCCESS_RETURN;
}

int fusedMM_amd_set_validate(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   int prev = g.validate;
   g.validate = enable ? 1 : 0;
   return prev;
}

void fusedMM_amd_set_split(int64_t heavy_deg, int seg_len)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();   // so that this call, not FUSEDMM_SPLIT, decides from here on
   g.heavy_deg = heavy_deg > 0 ? heavy_deg : 0;
   g.seg_len = seg_len > 0 ? seg_len : 0;
}

void fusedMM_amd_get_split(int64_t *heavy_deg, int *seg_len)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   if (heavy_deg) *heavy_deg = g.heavy_deg;
   if (seg_len) *seg_len = g.seg_len;
}

int fusedMM_amd_set_pack_rows(int mode)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   const int prev = g.pack == 1 ? 0 : 1;
   g.pack = mode ? 0 : 1;
   return prev;
}

int fusedMM_amd_set_store_tick(int shift)
{
   std::lock_guard<std::mutex> lock(g.mu);
   read_env_once();
   const int prev = g.store_shift;
   g.store_shift = shift == 0 ? 0 : ((shift >= 8 && shift <= 24) ? shift : -1);
   return prev;
}

void fusedMM_amd_timing(int enable)
{
   std::lock_guard<std::mutex> lock(g.mu);
   g.timing = enable > 0 ? enable : 0;
   g.timing_seen = 0;
   g.timing_calls = 0;
   if (g.timing > 0)
   {
      // the events are made here, on the current device, not inside the first timed call
      DeviceState *d = nullptr;
      if (device_basics(&d) == FUSEDMM_SUCCESS_RETURN && !d->ev_made)
      {
         bool ok = true;
         for (int i = 0; i < kTimingSlots && ok; i++)
            for (int e = 0; e < 4 && ok; e++) ok = (hipEventCreate(&d->ev[i][e]) == hipSuccess);
         d->ev_made = ok;
      }
   }
}

int fusedMM_amd_timing_summary(double *classify_ms, double *fused_ms, double *merge_ms)
{
   std::lock_guard<std::mutex> lock(g.mu);
   double t[3] = {0, 0, 0};
   int n = g.timing_calls;
   if (n > 0)
   {
      DeviceState &d = g.dev[g.timing_dev];
      if (hipEventSynchronize(d.ev[n - 1][3]) != hipSuccess) return -1;
      for (int i = 0; i < n; i++)
         for (int e = 0; e < 3; e++)
         {
            float ms = 0.f;
            if (hipEventElapsedTime(&ms, d.ev[i][e], d.ev[i][e + 1]) != hipSuccess) return -1;
            t[e] += ms;
         }
   }
   if (classify_ms) *classify_ms = t[0];
   if (fused_ms) *fused_ms = t[1];
   if (merge_ms) *merge_ms = t[2];
   return n;
}

int fusedMM_amd_timing_call(int i, double *classify_ms, double *fused_ms, double *merge_ms)
{
   std::lock_guard<std::mutex> lock(g.mu);
   if (i < 0 || i >= g.timing_calls) return FUSEDMM_FAIL_RETURN;
   DeviceState &d = g.dev[g.timing_dev];
   if (hipEventSynchronize(d.ev[i][3]) != hipSuccess) return FUSEDMM_FAIL_RETURN;
   double *out[3] = {classify_ms, fused_ms, merge_ms};
   for (int e = 0; e < 3; e++)
   {
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, d.ev[i][e], d.ev[i][e + 1]) != hipSuccess) return FUSEDMM_FAIL_RETURN;
      if (out[e]) *out[e] = ms;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

int fusedMM_amd_last_split(unsigned int *heavy_rows, unsigned int *segments, unsigned int *overflow)
{
   std::lock_guard<std::mutex> lock(g.mu);
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   Counters c;
   memset(&c, 0, sizeof(c));
   FMM_HIP(hipDeviceSynchronize());
   if (d->last_ctr) FMM_HIP(hipMemcpy(&c, d->last_ctr, sizeof(c), hipMemcpyDeviceToHost));
   if (heavy_rows) *heavy_rows = c.last_heavy;
   if (segments) *segments = c.last_seg;
   if (overflow) *overflow = c.last_overflow;
   return FUSEDMM_SUCCESS_RETURN;
}

int fusedMM_amd_last_row_order(int *scattered, unsigned int *edges_lower_half, unsigned int *edges_upper_half)
{
   std::lock_guard<std::mutex> lock(g.mu);
   DeviceState *d = nullptr;
   int st = device_basics(&d);
   if (st) return st;
   Counters c;
   memset(&c, 0, sizeof(c));
   FMM_HIP(hipDeviceSynchronize());
   if (d->last_ctr) FMM_HIP(hipMemcpy(&c, d->last_ctr, sizeof(c), hipMemcpyDeviceToHost));
   if (scattered) *scattered = (int)c.last_scattered;
   if (edges_lower_half) *edges_lower_half = (unsigned int)(c.last_skew & 0xFFFFFFFFull);
   if (edges_upper_half) *edges_upper_half = (unsigned int)(c.last_skew >> 32);
   return FUSEDMM_SUCCESS_RETURN;
}

void fusedMM_amd_finalize(void)
{
   std::lock_guard<std::mutex> lock(g.mu);
   int cur = 0;
   if (hipGetDevice(&cur) != hipSuccess) return;
   for (int dev = 0; dev < kMaxDevices; dev++)
   {
      DeviceState &d = g.dev[dev];
      if (!d.basics) continue;
      if (hipSetDevice(dev) != hipSuccess) continue;
      release_device(d);
   }
   (void)hipSetDevice(cur);
}

}  // extern "C"
