// The one entry point of the library that brings its own scratch memory.
//
// Every other entry point takes its index scratch (count tables, the row mover's int32 position plane) from a
// caller-provided workspace, which the caller has to allocate.  Some callers cannot: code under HIP graph
// capture, serving loops that must not touch the allocator, harnesses that forbid hipMalloc.  For them
// terrace_k1_arrival_static runs the Hop-B arrival chain with that scratch in a file-scope device array.
//
// The array's name is only a host-side handle: its device address is looked up once per device with
// hipGetSymbolAddress (each GPU holds its own copy of the array at its own address) and only that address is
// ever handed to a kernel.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU race.
// Nothing in it has to start at zero -- the count kernel writes every table entry and the rank kernel every
// position before either is read -- so a call never depends on what the last one left behind.
//
// The look-up is a runtime call that may load the code object, so it must not happen while a stream is being
// captured: terrace_static_init() does it for the current device ahead of time (the first
// terrace_k1_arrival_static call on a device does the same when nobody called it).
#include <atomic>
#include <mutex>

#include "common.hpp"

namespace terrace {
size_t k1_workspace(int64_t R, int quota, int rpn);
int run_k1_arrival(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                   int gate_bytes, int quota, int epr, int rpn, int my_local, void *send_buf, void *gate_pairs,
                   int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *pair_pos, int32_t *status, void *ws,
                   size_t ws_bytes, int64_t slot_pitch, int64_t gate_pitch, int64_t *meta, const int64_t *tags_in,
                   int64_t *tags_out, hipStream_t s);
}  // namespace terrace

static __device__ __align__(256) unsigned char scratch[TERRACE_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_lock;
std::atomic<void *> g_scratch_of[kMaxDevices];

// Device address of this GPU's copy of `scratch`, or nullptr with *rc set.
void *scratch_of_current_device(int *rc) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        *rc = TERRACE_EINVAL;
        return nullptr;
    }
    void *p = g_scratch_of[dev].load(std::memory_order_acquire);
    if (p) return p;
    std::lock_guard<std::mutex> hold(g_lock);
    p = g_scratch_of[dev].load(std::memory_order_relaxed);
    if (p) return p;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
        (void)hipGetLastError();
        *rc = TERRACE_ELAUNCH;
        return nullptr;
    }
    g_scratch_of[dev].store(p, std::memory_order_release);
    return p;
}

}  // namespace

extern "C" {

size_t terrace_static_scratch_bytes(void) { return (size_t)TERRACE_STATIC_SCRATCH_BYTES; }

int terrace_static_init(void) {
    int rc = TERRACE_OK;
    return scratch_of_current_device(&rc) ? TERRACE_OK : rc;
}

int terrace_k1_arrival_static(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                              int gate_bytes, int quota, int epr, int rpn, int my_local, void *send_buf,
                              void *gate_pairs, int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *pair_pos,
                              int32_t *status, terrace_stream_t stream) {
    if (R < 0 || quota <= 0 || rpn <= 0) return TERRACE_EINVAL;
    if (R > (((int64_t)1 << 31) - 1) / quota) return TERRACE_EINVAL;
    if (terrace::k1_workspace(R, quota, rpn) > (size_t)TERRACE_STATIC_SCRATCH_BYTES) return TERRACE_E2BIG;
    int rc = TERRACE_OK;
    void *ws = scratch_of_current_device(&rc);
    if (!ws) return rc;
    return terrace::run_k1_arrival(rx, rslot, rgate, R, row_bytes, gate_bytes, quota, epr, rpn, my_local, send_buf,
                                   gate_pairs, r_idx, slot_idx, i_send, pair_pos, status, ws,
                                   (size_t)TERRACE_STATIC_SCRATCH_BYTES, quota, quota, nullptr, nullptr, nullptr,
                                   (hipStream_t)stream);
}

}  // extern "C"
