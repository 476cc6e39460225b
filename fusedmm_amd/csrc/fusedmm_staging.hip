// Host-pointer mode of the synchronous entry point: the caller's arrays are ordinary
// host memory (what the reference's tester and any plain-C caller pass).  Operands are
// staged to the GPU through pinned buffers, read-only ones optionally mirrored between
// calls, and the first k columns of every Z row are copied back.
#include <chrono>
#include <condition_variable>
#include <thread>

#include "fusedmm_host.hpp"

namespace fmm_host {

namespace {

// ---- host-pointer mode: pinned staging ------------------------------------------------
// The caller's arrays are ordinary pageable memory.  They move through two pinned
// buffers each way, 16 MiB at a time: a few threads copy chunk i+1 between the
// caller's array and a pinned buffer while the DMA engine moves chunk i.
constexpr size_t kPinChunk = (size_t)16 << 20;
constexpr size_t kPinMinBytes = (size_t)1 << 20;   // smaller copies go straight through hipMemcpyAsync

class CopyPool {
 public:
   void copy(void *dst, const void *src, size_t bytes)
   {
      if (bytes < ((size_t)1 << 20) || !start()) { memcpy(dst, src, bytes); return; }
      std::unique_lock<std::mutex> lk(m_);
      dst_ = (char *)dst; src_ = (const char *)src; bytes_ = bytes;
      remaining_ = (int)th_.size();
      generation_++;
      cv_.notify_all();
      done_.wait(lk, [&] { return remaining_ == 0; });
   }
   ~CopyPool()
   {
      {
         std::lock_guard<std::mutex> lk(m_);
         stop_ = true;
         generation_++;
      }
      cv_.notify_all();
      for (auto &t : th_) t.join();
   }

 private:
   bool start()
   {
      if (!th_.empty()) return true;
      unsigned int n = std::thread::hardware_concurrency();
      n = n < 2 ? 0 : (n > 8 ? 8 : n);
      for (unsigned int i = 0; i < n; i++) th_.emplace_back([this, i, n] { work(i, n); });
      return n > 0;
   }
   void work(unsigned int i, unsigned int n)
   {
      int seen = 0;
      for (;;)
      {
         std::unique_lock<std::mutex> lk(m_);
         cv_.wait(lk, [&] { return generation_ != seen; });
         seen = generation_;
         if (stop_) return;
         char *d = dst_; const char *s = src_; const size_t b = bytes_;
         lk.unlock();
         const size_t lo = b / n * i, hi = (i + 1 == n) ? b : b / n * (i + 1);
         memcpy(d + lo, s + lo, hi - lo);
         lk.lock();
         if (--remaining_ == 0) done_.notify_one();
      }
   }
   std::vector<std::thread> th_;
   std::mutex m_;
   std::condition_variable cv_, done_;
   char *dst_ = nullptr; const char *src_ = nullptr; size_t bytes_ = 0;
   int generation_ = 0, remaining_ = 0;
   bool stop_ = false;
};
CopyPool copy_pool;

int pinned_buffers(DeviceState &d)
{
   if (d.pin[0]) return FUSEDMM_SUCCESS_RETURN;
   for (int i = 0; i < 4; i++)
   {
      FMM_HIP(hipHostMalloc(&d.pin[i], kPinChunk, hipHostMallocDefault));
      FMM_HIP(hipEventCreateWithFlags(&d.pin_ev[i], hipEventDisableTiming));
      d.pin_busy[i] = false;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

// host -> device, enqueued on `s`; returns when the host array has been read
int upload(DeviceState &d, void *dev, const void *host, size_t bytes, hipStream_t s)
{
   if (bytes == 0) return FUSEDMM_SUCCESS_RETURN;
   if (bytes < kPinMinBytes) { FMM_HIP(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, s)); return FUSEDMM_SUCCESS_RETURN; }
   int st = pinned_buffers(d);
   if (st) return st;
   int b = 0;
   for (size_t off = 0; off < bytes; off += kPinChunk, b ^= 1)
   {
      const size_t n = bytes - off < kPinChunk ? bytes - off : kPinChunk;
      if (d.pin_busy[b]) FMM_HIP(hipEventSynchronize(d.pin_ev[b]));   // its previous DMA has drained
      copy_pool.copy(d.pin[b], (const char *)host + off, n);
      FMM_HIP(hipMemcpyAsync((char *)dev + off, d.pin[b], n, hipMemcpyHostToDevice, s));
      FMM_HIP(hipEventRecord(d.pin_ev[b], s));
      d.pin_busy[b] = true;
   }
   return FUSEDMM_SUCCESS_RETURN;
}

// device -> host through the other two pinned buffers; returns when `host` holds the data
int download(DeviceState &d, void *host, const void *dev, size_t bytes, hipStream_t s)
{
   if (bytes == 0) return FUSEDMM_SUCCESS_RETURN;
   if (bytes < kPinMinBytes)
   {
      FMM_HIP(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, s));
      return hip_status(hipStreamSynchronize(s), "hipStreamSynchronize");
   }
   int st = pinned_buffers(d);
   if (st) return st;
   size_t prev_off = 0, prev_n = 0;
   int b = 2, prev_b = -1;
   for (size_t off = 0; off < bytes; off += kPinChunk)
   {
      const size_t n = bytes - off < kPinChunk ? bytes - off : kPinChunk;
      FMM_HIP(hipMemcpyAsync(d.pin[b], (const char *)dev + off, n, hipMemcpyDeviceToHost, s));
      FMM_HIP(hipEventRecord(d.pin_ev[b], s));
      if (prev_b >= 0)
      {
         FMM_HIP(hipEventSynchronize(d.pin_ev[prev_b]));
         copy_pool.copy((char *)host + prev_off, d.pin[prev_b], prev_n);
      }
      prev_b = b; prev_off = off; prev_n = n;
      b = (b == 2) ? 3 : 2;
   }
   FMM_HIP(hipEventSynchronize(d.pin_ev[prev_b]));
   copy_pool.copy((char *)host + prev_off, d.pin[prev_b], prev_n);
   d.pin_busy[2] = d.pin_busy[3] = false;
   return FUSEDMM_SUCCESS_RETURN;
}

// Device copy of a read-only host operand.  With the mirror cache off (the
// default) it is uploaded into the staging buffer `stage` on every call, as
// the caller may have changed it.  With the cache on, a mirror keyed by host
// address and size is kept and reused until fusedMM_amd_invalidate().
int device_copy(DeviceState &d, Buffer &stage, const void *host, size_t bytes, size_t copy_bytes, hipStream_t s, const void **out)
{
   if (!g.cache)
   {
      int st = grow(stage, bytes);
      if (st) return st;
      *out = stage.ptr;
      return upload(d, stage.ptr, host, copy_bytes, s);
   }
   for (auto &mi : d.mirrors)
      if (mi.host == host && mi.bytes == copy_bytes)
      {
         mi.last_use = ++g.cache_clock;
         *out = mi.dev;
         return FUSEDMM_SUCCESS_RETURN;
      }
   if (d.mirrors.size() >= 32)   // drop the mirror used longest ago
   {
      size_t victim = 0;
      for (size_t i = 1; i < d.mirrors.size(); i++)
         if (d.mirrors[i].last_use < d.mirrors[victim].last_use) victim = i;
      (void)hipFree(d.mirrors[victim].dev);
      d.mirrors.erase(d.mirrors.begin() + (long)victim);
   }
   void *dev = nullptr;
   FMM_HIP(hipMalloc(&dev, bytes > 0 ? bytes : 16));
   d.mirrors.push_back(DeviceState::Mirror{host, copy_bytes, dev, ++g.cache_clock});
   *out = dev;
   return upload(d, dev, host, copy_bytes, s);
}

}  // namespace

// Host-pointer mode: copy the operands to the GPU.  On return `a` holds device
// addresses and `slots` is one past the last edge slot any processed row uses.
int stage_up(const Args &h, const Plan &pl, Args *a, int64_t *slots_out)
{
   if (h.n <= 0) { FMM_LOG("n (rows of Y) must be positive for host operands"); return FUSEDMM_FAIL_RETURN; }
   if (h.ldy < h.k || h.ldz < h.k || (pl.reads_x && h.ldx < h.k))
   {
      FMM_LOG("leading dimension smaller than k");
      return FUSEDMM_FAIL_RETURN;
   }
   if (!h.indx || !h.pntrb || !h.pntre || !h.y || !h.z || (pl.reads_x && !h.x))
   {
      FMM_LOG("NULL operand");
      return FUSEDMM_FAIL_RETURN;
   }
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   if (g.validate)
   {
      st = validate_host_pointers(h);
      if (st) return st;
   }
   int64_t slots = 0;
   for (int64_t i = 0; i < h.m; i++)
      if ((int64_t)h.pntre[i] > slots) slots = (int64_t)h.pntre[i];
   const bool need_val = pl.reads_val;
   if (need_val && !h.val) { FMM_LOG("NULL operand"); return FUSEDMM_FAIL_RETURN; }
   const size_t b_ptr = (size_t)h.m * sizeof(idx_t);
   const size_t b_idx = (size_t)(slots > 0 ? slots : 1) * sizeof(idx_t);
   const size_t b_val = (size_t)(slots > 0 ? slots : 1) * kValBytes;
   const size_t b_x = (size_t)h.m * (size_t)h.ldx * kValBytes;
   const size_t b_y = (size_t)h.n * (size_t)h.ldy * kValBytes;
   const size_t b_z = (size_t)h.m * (size_t)h.ldz * kValBytes;
   // the caller's arrays need not extend past the last element the reference reads:
   // (rows - 1) * ld + k elements, not rows * ld
   hipStream_t s = 0;
   const void *dp[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
   st = device_copy(*d, d->stage[0], h.pntrb, b_ptr, b_ptr, s, &dp[0]); if (st) return st;
   st = device_copy(*d, d->stage[1], h.pntre, b_ptr, b_ptr, s, &dp[1]); if (st) return st;
   st = device_copy(*d, d->stage[2], h.indx, b_idx, (size_t)slots * sizeof(idx_t), s, &dp[2]); if (st) return st;
   if (need_val) { st = device_copy(*d, d->stage[3], h.val, b_val, (size_t)slots * kValBytes, s, &dp[3]); if (st) return st; }
   st = device_copy(*d, d->stage[5], h.y, b_y, b_y - (size_t)(h.ldy - h.k) * kValBytes, s, &dp[5]); if (st) return st;
   if (pl.reads_x)
   {
      if ((const void *)h.x == (const void *)h.y && h.ldx == h.ldy && b_x <= b_y) dp[4] = dp[5];   // A = B: one copy serves both
      else { st = device_copy(*d, d->stage[4], h.x, b_x, b_x - (size_t)(h.ldx - h.k) * kValBytes, s, &dp[4]); if (st) return st; }
   }
   st = grow(d->stage[6], b_z); if (st) return st;
   const bool overwrite = pl.opt_rule && h.beta == 0.0f;
   if (!overwrite)   // one contiguous copy, padding columns included (they are never written back)
   {
      st = upload(*d, d->stage[6].ptr, h.z, b_z - (size_t)(h.ldz - h.k) * kValBytes, s);
      if (st) return st;
   }
   *a = h;
   a->pntrb = (const idx_t *)dp[0];
   a->pntre = (const idx_t *)dp[1];
   a->indx = (const idx_t *)dp[2];
   a->val = need_val ? (const val_t *)dp[3] : nullptr;
   a->x = pl.reads_x ? (const val_t *)dp[4] : nullptr;
   a->y = (const val_t *)dp[5];
   a->z = (val_t *)d->stage[6].ptr;
   if (a->nnz <= 0 || a->nnz > slots) a->nnz = slots;
   *slots_out = slots;
   return FUSEDMM_SUCCESS_RETURN;
}

// Only the first k columns of each Z row are written back, as the reference
// touches nothing else.  With ldz == k that is one contiguous copy; otherwise
// the block is fetched contiguously and the k columns of every row are copied
// out on the host (a strided device copy of millions of short rows is far
// slower than either).
int stage_down(const Args &h, const Args &a)
{
   DeviceState *d = nullptr;
   int st = device_state(&d);
   if (st) return st;
   const size_t span = ((size_t)h.m * (size_t)h.ldz - (size_t)(h.ldz - h.k)) * kValBytes;
   if (h.ldz == h.k) return download(*d, h.z, a.z, span, 0);
   std::vector<val_t> tmp(span / kValBytes);
   st = download(*d, tmp.data(), a.z, span, 0);
   if (st) return st;
   for (int64_t i = 0; i < h.m; i++)
      memcpy(h.z + i * h.ldz, tmp.data() + i * h.ldz, (size_t)h.k * kValBytes);
   return FUSEDMM_SUCCESS_RETURN;
}

int run_staged(const Args &h, const Plan &pl, int sop_kind)
{
   if (h.m <= 0 || h.k < 1) return FUSEDMM_SUCCESS_RETURN;
   typedef std::chrono::steady_clock clk;
   auto ms = [](clk::time_point a, clk::time_point b) { return std::chrono::duration<double, std::milli>(b - a).count(); };
   g.phase_valid = false;
   const clk::time_point t0 = clk::now();
   Args a;
   int64_t slots = 0;
   int st = stage_up(h, pl, &a, &slots);
   if (st) return st;
   FMM_HIP(hipStreamSynchronize(0));
   const clk::time_point t1 = clk::now();
   if (g.validate)
   {
      st = validate_operands(a, 0);
      if (st) return st;
   }
   st = run_on_device(a, pl, sop_kind, 0);
   if (st) return st;
   FMM_HIP(hipStreamSynchronize(0));
   const clk::time_point t2 = clk::now();
   st = stage_down(h, a);
   if (st) return st;
   const clk::time_point t3 = clk::now();
   g.phase_ms[0] = ms(t0, t1); g.phase_ms[1] = ms(t1, t2); g.phase_ms[2] = ms(t2, t3);
   g.phase_valid = true;
   return FUSEDMM_SUCCESS_RETURN;
}

}  // namespace fmm_host
