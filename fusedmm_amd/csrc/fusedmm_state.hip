// Per-device state of the library: the settings read from the environment, the
// grow-only work queues of the ordinary entry points, the static array of the entry
// point that allocates nothing, and the ordering of calls that share a set of queues.
#include <math.h>

#include "fusedmm_host.hpp"

// Device memory of the entry point that allocates nothing (fusedMM_csr_stream_noalloc):
// the sigmoid table, the queue and claim counters, the queued-row bitmap, the
// heavy-row queue, the segment descriptors and the partial results of split rows,
// carved out of this array call by call.  Every GPU the library runs on holds its
// own copy until the process ends.  In host code the name is only a handle: the
// address kernels and copies use comes from hipGetSymbolAddress, once per device.
static __device__ __align__(256) unsigned char fmm_scratch[FUSEDMM_AMD_SCRATCH_BYTES];

namespace fmm_host {

Globals g;

namespace {

int sop_kind_from_name(const char *s)
{
   if (!s) return FUSEDMM_SOP_KIND_HOST;
   if (!strcmp(s, "host")) return FUSEDMM_SOP_KIND_HOST;
   if (!strcmp(s, "identity")) return FUSEDMM_SOP_KIND_IDENTITY;
   if (!strcmp(s, "sigmoid")) return FUSEDMM_SOP_KIND_SIGMOID;
   if (!strcmp(s, "tdist")) return FUSEDMM_SOP_KIND_TDIST;
   if (!strcmp(s, "fr")) return FUSEDMM_SOP_KIND_FR;
   if (!strcmp(s, "ll")) return FUSEDMM_SOP_KIND_LL;
   if (!strcmp(s, "fa")) return FUSEDMM_SOP_KIND_FA;
   if (!strcmp(s, "tdist_plain")) return FUSEDMM_SOP_KIND_TDIST_PLAIN;
   FMM_LOG("FUSEDMM_SOP_KIND=%s is not a known kind; using host", s);
   return FUSEDMM_SOP_KIND_HOST;
}

}  // namespace

// Every entry point and every setter reads the environment first (once per process),
// so that a setting made through the API always wins over the variable.
void read_env_once()
{
   if (g.env_read) return;
   g.env_read = true;
   if (const char *e = getenv("FUSEDMM_SOP_KIND")) g.sop_kind = sop_kind_from_name(e);
   if (const char *e = getenv("FUSEDMM_BLOCKS_PER_CU")) g.blocks_per_cu = atoi(e);
   if (const char *e = getenv("FUSEDMM_VALIDATE")) g.validate = atoi(e);
   if (const char *e = getenv("FUSEDMM_CACHE")) g.cache = atoi(e) ? 1 : 0;
   if (const char *e = getenv("FUSEDMM_ROW_ORDER"))   // "auto", "plain" (first to last) or "scattered"
      g.row_order = !strcmp(e, "plain") ? 1 : (!strcmp(e, "scattered") ? 2 : 0);
   if (const char *e = getenv("FUSEDMM_PACK_ROWS"))   // "auto", "off" or "on"
      g.pack = !strcmp(e, "off") ? 1 : (!strcmp(e, "on") ? 2 : 0);
   if (const char *e = getenv("FUSEDMM_STORE_TICK"))   // "auto", "off" or the shift (8 ... 24)
   {
      const int v = atoi(e);
      g.store_shift = !strcmp(e, "off") ? 0 : ((v >= 8 && v <= 24) ? v : -1);
   }
   if (const char *e = getenv("FUSEDMM_SPLIT"))   // "heavy_deg,seg_len", as fusedMM_amd_set_split
   {
      long long h = 0;
      int sl = 0;
      if (sscanf(e, "%lld,%d", &h, &sl) == 2 && h > 0 && sl > 0) { g.heavy_deg = h; g.seg_len = sl; }
   }
}

// The 2048-entry sigmoid table, built with the expressions of the reference's
// tester (test/fusedMMtime.cpp:594-604, a C++ file: exp() resolves to the
// overload of VALUETYPE).  Single precision: x is a float, exp is expf, 1 + e is
// a float sum, the quotient is formed in double and rounded.  Double precision:
// everything is double.
void build_sigmoid_table(val_t *t)
{
   for (int i = 0; i < kSigmoidTableSize; i++)
   {
#ifdef FMM_DOUBLE
      double x = 2.0 * 5.0 * i / kSigmoidTableSize - 5.0;
      t[i] = 1.0 / (1 + exp(-x));
#else
      float x = (float)(2.0 * 5.0 * i / kSigmoidTableSize - 5.0);
      float e = expf(-x);
      float denom = 1 + e;
      t[i] = (float)(1.0 / (double)denom);
#endif
   }
}

// `capturing`: the call is being recorded into a HIP graph.  Replacing a buffer
// then would leave the graph (and any graph captured earlier) with the address
// of freed memory, so the call is refused instead.
int grow(Buffer &b, size_t bytes, bool capturing)
{
   if (bytes <= b.bytes) return FUSEDMM_SUCCESS_RETURN;
   if (capturing)
   {
      FMM_LOG("a work buffer would have to grow (%zu -> %zu bytes) while the stream is being captured; "
              "run one call of this size outside the capture first, or use fusedMM_csr_stream_noalloc",
              b.bytes, bytes);
      return FUSEDMM_NOT_ENOUGH_MEM;
   }
   if (b.ptr) FMM_HIP(hipFree(b.ptr));
   b.ptr = nullptr;
   b.bytes = 0;
   FMM_HIP(hipMalloc(&b.ptr, bytes));
   b.bytes = bytes;
   return FUSEDMM_SUCCESS_RETURN;
}

// What every entry point needs of the current device; allocates no device memory.
int device_basics(DeviceState **out)
{
   int dev = 0;
   FMM_HIP(hipGetDevice(&dev));
   if (dev < 0 || dev >= kMaxDevices) return FUSEDMM_FAIL_RETURN;
   DeviceState &d = g.dev[dev];
   if (!d.basics)
   {
      int cus = 0;
      FMM_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
      d.num_cu = cus > 0 ? cus : 256;
      for (int q = 0; q < 2; q++) FMM_HIP(hipEventCreateWithFlags(&d.order_ev[q], hipEventDisableTiming));
      d.basics = true;
   }
   *out = &d;
   return FUSEDMM_SUCCESS_RETURN;
}

int device_state(DeviceState **out)
{
   DeviceState *dp = nullptr;
   int st0 = device_basics(&dp);
   if (st0) return st0;
   DeviceState &d = *dp;
   if (!d.ready)
   {
      val_t host_tab[kSigmoidTableSize];
      build_sigmoid_table(host_tab);
      FMM_HIP(hipMalloc((void **)&d.sigmoid_table, sizeof(host_tab)));
      FMM_HIP(hipMemcpy(d.sigmoid_table, host_tab, sizeof(host_tab), hipMemcpyHostToDevice));
      FMM_HIP(hipMalloc((void **)&d.ctr, sizeof(Counters)));
      FMM_HIP(hipMemset(d.ctr, 0, sizeof(Counters)));
      d.ready = true;
   }
   *out = &d;
   return FUSEDMM_SUCCESS_RETURN;
}

// Once per device, with that device current: find this device's copy of the
// array, put the sigmoid table at its head and zero the counters.
int scratch_setup(DeviceState &d)
{
   if (d.scratch) return FUSEDMM_SUCCESS_RETURN;
   unsigned char *base = nullptr;
   FMM_HIP(hipGetSymbolAddress((void **)&base, HIP_SYMBOL(fmm_scratch)));
   if (!base) return FUSEDMM_FAIL_RETURN;
   val_t host_tab[kSigmoidTableSize];
   build_sigmoid_table(host_tab);
   FMM_HIP(hipMemcpy(base + kScratchTableOff, host_tab, sizeof(host_tab), hipMemcpyHostToDevice));
   FMM_HIP(hipMemset(base + kScratchCtrOff, 0, kScratchQueuesOff - kScratchCtrOff));   // counters and queued-row bits
   d.scratch = base;
   return FUSEDMM_SUCCESS_RETURN;
}

// Is `stream` being recorded into a HIP graph?  The legacy default stream cannot be.
int stream_capturing(hipStream_t stream, bool *capturing)
{
   *capturing = false;
   if (!stream) return FUSEDMM_SUCCESS_RETURN;
   hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
   FMM_HIP(hipStreamIsCapturing(stream, &cs));
   *capturing = (cs != hipStreamCaptureStatusNone);
   return FUSEDMM_SUCCESS_RETURN;
}

// Make `stream` wait for the work of the previous call that used this set of
// queues, when that call went to another stream.  The event is recorded only now,
// on that earlier stream (it then covers the earlier call and whatever the caller
// enqueued there since): a record after every call would sit between consecutive
// calls of the common one-stream case and keep them from running back to back.
// The earlier stream must not have entered a capture since: an event recorded there
// would become a node of the caller's graph and could not be waited on from outside
// it.  Such a call is refused (the caller's capture is left intact) rather than
// ordered by a device-wide wait, which is illegal while a capture is open.
int order_after_previous(DeviceState &d, int queues, hipStream_t stream)
{
   if (!d.pending[queues] || d.last_stream[queues] == stream) return FUSEDMM_SUCCESS_RETURN;
   hipStream_t prev = d.last_stream[queues];
   if (prev)
   {
      hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
      const hipError_t q = hipStreamIsCapturing(prev, &cs);
      if (q == hipSuccess && cs != hipStreamCaptureStatusNone)
      {
         FMM_LOG("the stream of the previous call on this GPU is now being captured, so this call cannot be ordered "
                 "after it; end the capture first, or make the calls on one stream");
         return FUSEDMM_FAIL_RETURN;
      }
      if (q != hipSuccess) (void)hipGetLastError();   // a destroyed stream: handled below
   }
   hipError_t e = hipEventRecord(d.order_ev[queues], prev);
   if (e == hipSuccess) e = hipStreamWaitEvent(stream, d.order_ev[queues], 0);
   if (e != hipSuccess)
   {
      // the earlier stream is gone (destroyed by the caller; its work still completes)
      (void)hipGetLastError();
      FMM_HIP(hipDeviceSynchronize());
   }
   d.pending[queues] = false;
   return FUSEDMM_SUCCESS_RETURN;
}

void release_device(DeviceState &d)
{
   (void)hipDeviceSynchronize();
   for (int q = 0; q < 2; q++) (void)hipEventDestroy(d.order_ev[q]);
   if (d.sigmoid_table) (void)hipFree(d.sigmoid_table);
   if (d.ctr) (void)hipFree(d.ctr);
   Buffer *bufs[] = {&d.heavy, &d.segs, &d.partial, &d.queued};
   for (Buffer *b : bufs) { if (b->ptr) (void)hipFree(b->ptr); *b = Buffer(); }
   for (Buffer &b : d.stage) { if (b.ptr) (void)hipFree(b.ptr); b = Buffer(); }
   if (d.edge_t.ptr) (void)hipFree(d.edge_t.ptr);
   for (auto &mi : d.mirrors) (void)hipFree(mi.dev);
   d.mirrors.clear();
   if (d.pin[0])
      for (int i = 0; i < 4; i++) { (void)hipHostFree(d.pin[i]); (void)hipEventDestroy(d.pin_ev[i]); }
   if (d.ev_made)
      for (int i = 0; i < kTimingSlots; i++)
         for (int e = 0; e < 4; e++) (void)hipEventDestroy(d.ev[i][e]);
   d = DeviceState();   // also forgets the static array's address: its head is cleared again on next use
}

}  // namespace fmm_host
