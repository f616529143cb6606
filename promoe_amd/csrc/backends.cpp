// Device backends of the engine: HIP (HBM slot pool, side-stream copies) and a
// host stand-in used by the CPU tests of the cache logic.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <thread>

#include "engine_internal.h"

namespace {

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

#define HIPC(call)                                        \
  do {                                                    \
    if (int rc_ = moe_check_hip((call), #call)) return rc_; \
  } while (0)

struct HipBackend : Backend {
  int dev = 0;
  hipStream_t compute = nullptr, copy = nullptr;
  bool own_compute = false, own_copy = false;
  // VMM pool
  std::vector<hipMemGenericAllocationHandle_t> handles;
  void *va = nullptr;
  size_t va_size = 0, mapped = 0;
  void *slab = nullptr;
  std::vector<void *> dev_allocs, host_allocs;
  std::vector<hipEvent_t> events;
  bool ok = true;

  HipBackend(void *compute_stream, bool cache_only) {
    if (hipGetDevice(&dev) != hipSuccess) { moe_set_error("no HIP device"); ok = false; return; }
    if (compute_stream) compute = (hipStream_t)compute_stream;
    else {
      // prefetcher.cpp:407-413: a private non-blocking compute stream, default priority
      if (hipStreamCreateWithFlags(&compute, hipStreamNonBlocking) != hipSuccess) { moe_set_error("hipStreamCreate failed"); ok = false; return; }
      own_compute = true;
    }
    if (cache_only) copy = compute;  // prefetcher.cpp:420-424
    else {
      if (hipStreamCreateWithFlags(&copy, hipStreamNonBlocking) != hipSuccess) { moe_set_error("hipStreamCreate failed"); ok = false; return; }
      own_copy = true;
    }
  }
  ~HipBackend() override {
    if (copy) (void)hipStreamSynchronize(copy);
    for (auto e : events) (void)hipEventDestroy(e);
    if (va) {
      if (mapped) (void)hipMemUnmap(va, mapped);
      for (auto h : handles) (void)hipMemRelease(h);
      (void)hipMemAddressFree(va, va_size);
    }
    if (slab) (void)hipFree(slab);
    for (auto p : dev_allocs) (void)hipFree(p);
    for (auto p : host_allocs) (void)hipHostFree(p);
    if (own_copy) (void)hipStreamDestroy(copy);
    if (own_compute) (void)hipStreamDestroy(compute);
  }

  // Slot pool.  vmm: one virtual range reserved for the full expert population
  // (reserve_slots), physical memory created in granularity-sized pieces and mapped
  // back to back for the first n_slots only, so slots are packed (no per-slot rounding
  // to the 2 MiB granularity) and the pool can grow in place.
  // Reference: model_loader.cpp:81-116 (cuMem* wrappers), :236-275 (per-expert handles).
  int alloc_pool(size_t slot_bytes, size_t n_slots, size_t reserve_slots, bool vmm, void **base, size_t *stride) override {
    *stride = round_up(slot_bytes, 256);
    const size_t need = *stride * n_slots;
    if (!vmm) {
      HIPC(hipMalloc(&slab, need));
      HIPC(hipMemset(slab, 0, need));
      *base = slab;
      return MOE_OK;
    }
    hipMemAllocationProp prop;
    memset(&prop, 0, sizeof prop);
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = dev;
    size_t gran = 0;
    HIPC(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended));
    if (gran == 0) gran = 2u << 20;
    const size_t piece = round_up((size_t)64 << 20, gran);
    va_size = round_up(*stride * (reserve_slots > n_slots ? reserve_slots : n_slots), piece);
    HIPC(hipMemAddressReserve(&va, va_size, gran, nullptr, 0));
    const size_t want = round_up(need, gran);
    size_t off = 0;
    while (off < want) {
      const size_t sz = (want - off) < piece ? (want - off) : piece;
      hipMemGenericAllocationHandle_t h;
      HIPC(hipMemCreate(&h, sz, &prop, 0));
      handles.push_back(h);
      HIPC(hipMemMap((char *)va + off, sz, 0, h, 0));
      off += sz;
    }
    mapped = want;
    hipMemAccessDesc acc;
    memset(&acc, 0, sizeof acc);
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = dev;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    HIPC(hipMemSetAccess(va, mapped, &acc, 1));
    *base = va;
    return MOE_OK;
  }
  int alloc_table(size_t n, uint64_t **d, uint64_t **h) override {
    void *dp = nullptr, *hp = nullptr;
    HIPC(hipMalloc(&dp, n * sizeof(uint64_t)));
    dev_allocs.push_back(dp);
    HIPC(hipMemset(dp, 0, n * sizeof(uint64_t)));
    HIPC(hipHostMalloc(&hp, n * sizeof(uint64_t), hipHostMallocDefault));
    host_allocs.push_back(hp);
    *d = (uint64_t *)dp; *h = (uint64_t *)hp;
    return MOE_OK;
  }
  int copy_h2d(void *dst, const void *src, size_t n) override {
    HIPC(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, copy));  // worker.cpp:92-96
    return MOE_OK;
  }
  int copy_sync() override { HIPC(hipStreamSynchronize(copy)); return MOE_OK; }  // worker.cpp:103
  int flush_table(uint64_t *d, const uint64_t *h, size_t n, void *stream) override {
    HIPC(hipMemcpyAsync(d, h, n * sizeof(uint64_t), hipMemcpyHostToDevice, (hipStream_t)stream));
    return MOE_OK;
  }
  void *event_create() override {
    hipEvent_t e;
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) return nullptr;  // model_loader.cpp:18
    events.push_back(e);
    return e;
  }
  int event_record(void *ev, void *stream) override { HIPC(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream)); return MOE_OK; }
  int event_sync(void *ev) override { HIPC(hipEventSynchronize((hipEvent_t)ev)); return MOE_OK; }
  bool event_done(void *ev) override { return hipEventQuery((hipEvent_t)ev) == hipSuccess; }
  void *compute_stream() override { return compute; }
  void *copy_stream() override { return copy; }
  bool is_pinned(const void *p) override {
    hipPointerAttribute_t a;
    if (hipPointerGetAttributes(&a, p) != hipSuccess) { (void)hipGetLastError(); return false; }
    return a.type == hipMemoryTypeHost;
  }
};

struct HostBackend : Backend {
  std::vector<void *> allocs;
  long delay_us = 0;
  HostBackend() {
    if (const char *e = getenv("MOE_HOST_COPY_DELAY_US")) delay_us = atol(e);
  }
  ~HostBackend() override { for (auto p : allocs) free(p); }
  int alloc_pool(size_t slot_bytes, size_t n, size_t, bool, void **base, size_t *stride) override {
    *stride = round_up(slot_bytes, 256);
    void *p = nullptr;
    if (posix_memalign(&p, 256, *stride * n ? *stride * n : 256)) { moe_set_error("out of host memory"); return MOE_ENOMEM; }
    memset(p, 0, *stride * n);
    allocs.push_back(p);
    *base = p;
    return MOE_OK;
  }
  int alloc_table(size_t n, uint64_t **d, uint64_t **h) override {
    *d = (uint64_t *)calloc(n, sizeof(uint64_t));
    *h = (uint64_t *)calloc(n, sizeof(uint64_t));
    allocs.push_back(*d); allocs.push_back(*h);
    return (*d && *h) ? MOE_OK : MOE_ENOMEM;
  }
  int copy_h2d(void *dst, const void *src, size_t n) override {
    if (delay_us) std::this_thread::sleep_for(std::chrono::microseconds(delay_us));
    memcpy(dst, src, n);
    return MOE_OK;
  }
  int copy_sync() override { return MOE_OK; }
  int flush_table(uint64_t *d, const uint64_t *h, size_t n, void *) override { memcpy(d, h, n * sizeof(uint64_t)); return MOE_OK; }
  void *event_create() override { return (void *)1; }
  int event_record(void *, void *) override { return MOE_OK; }
  int event_sync(void *) override { return MOE_OK; }
  bool event_done(void *) override { return true; }
  void *compute_stream() override { return nullptr; }
  void *copy_stream() override { return nullptr; }
  bool is_pinned(const void *) override { return true; }
};

}  // namespace

Backend *moe_make_hip_backend(void *compute_stream, bool cache_only) {
  auto *b = new HipBackend(compute_stream, cache_only);
  if (!b->ok) { delete b; return nullptr; }
  return b;
}
Backend *moe_make_host_backend() { return new HostBackend(); }

extern "C" void *moe_host_alloc(size_t nbytes) {
  void *p = nullptr;
  if (nbytes == 0) nbytes = 1;
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) == hipSuccess && ndev > 0) {
    if (hipHostMalloc(&p, nbytes, hipHostMallocDefault) == hipSuccess) return p;
    moe_set_error("hipHostMalloc(%zu) failed", nbytes);
    (void)hipGetLastError();
    return nullptr;
  }
  (void)hipGetLastError();
  // no GPU in this process: plain aligned memory, tagged so that moe_host_free can tell
  if (posix_memalign(&p, 4096, nbytes)) { moe_set_error("out of host memory"); return nullptr; }
  return p;
}

extern "C" void moe_host_free(void *p) {
  if (!p) return;
  hipPointerAttribute_t a;
  if (hipPointerGetAttributes(&a, p) == hipSuccess && a.type == hipMemoryTypeHost) { (void)hipHostFree(p); return; }
  (void)hipGetLastError();
  free(p);
}
