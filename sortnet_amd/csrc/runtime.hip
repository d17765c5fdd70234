// Library runtime: error reporting, device queries, fill kernel and the verification exports.
#include <atomic>
#include <cmath>
#include <mutex>
#include <vector>
#include "common.h"

namespace sd {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(e));
        return SD_ERR_HIP;
    }
    return SD_OK;
}

static thread_local char g_fwd_kernel[64] = "";

void note_forward_kernel(const char* kind, int tb, int tm) {
    snprintf(g_fwd_kernel, sizeof(g_fwd_kernel), "%s<%d,%d>", kind, tb, tm);
}

struct TermNote { const unsigned long long* counts; int kind; double denom0, denom1; unsigned long long limit0; };
static thread_local TermNote g_term_note = {nullptr, 0, 1.0, 1.0, 0ull};

void note_term_counts(const unsigned long long* counts, int kind, double denom0, double denom1, unsigned long long limit0) {
    g_term_note = TermNote{counts, kind, denom0, denom1, limit0};
}

// sd_time_forward_kernels / sd_last_forward_kernel_ms: two events per thread, created on first use
static thread_local bool g_time_kernels = false, g_timed = false, g_time_ev_made = false;
static thread_local hipEvent_t g_time_ev[2];

void forward_kernel_timer(hipStream_t stream, bool after) {
    if (!g_time_kernels) return;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) { (void)hipGetLastError(); return; }
    if (cap != hipStreamCaptureStatusNone) return;
    if (!g_time_ev_made) {
        if (hipEventCreate(&g_time_ev[0]) != hipSuccess || hipEventCreate(&g_time_ev[1]) != hipSuccess) {
            (void)hipGetLastError();
            return;
        }
        g_time_ev_made = true;
    }
    if (hipEventRecord(g_time_ev[after ? 1 : 0], stream) != hipSuccess) { (void)hipGetLastError(); return; }
    g_timed = after;
}

static std::recursive_mutex g_call_mu;
CallGuard::CallGuard() { g_call_mu.lock(); }
CallGuard::~CallGuard() { g_call_mu.unlock(); }

int num_cus() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

void* workspace(size_t bytes, hipStream_t stream) {
    struct Slot { int dev; hipStream_t stream; void* buf; size_t cap; };
    static std::mutex mu;
    static std::vector<Slot> slots;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) { set_error("workspace: no current device"); return nullptr; }
    std::lock_guard<std::mutex> lock(mu);
    Slot* slot = nullptr;
    for (Slot& c : slots) if (c.dev == dev && c.stream == stream) { slot = &c; break; }
    if (!slot) { slots.push_back(Slot{dev, stream, nullptr, 0}); slot = &slots.back(); }
    if (slot->cap < bytes) {
        // nothing may be allocated or waited for while the stream records a graph: the caller runs the same
        // call once on this stream beforehand, which sizes the buffer
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();
        if (cap != hipStreamCaptureStatusNone) {
            set_error("workspace: %zu bytes needed while the stream is capturing; run the call once on this stream before the capture", bytes);
            return nullptr;
        }
        // kernels queued on this stream may still use the old buffer: release it only after they are done
        if (slot->buf) { (void)hipStreamSynchronize(stream); (void)hipFree(slot->buf); slot->buf = nullptr; slot->cap = 0; }
        size_t want = bytes + bytes / 4;
        void* p = nullptr;
        if (hipMalloc(&p, want) != hipSuccess) { (void)hipGetLastError(); set_error("workspace: hipMalloc of %zu bytes failed", want); return nullptr; }
        slot->buf = p; slot->cap = want;
    }
    return slot->buf;
}

namespace {
constexpr int kHintRing = 4;   // outcomes of a layer that may be on their way to the host at once
constexpr size_t kHintSlots = 256;   // layers (site, weight matrix) the hints remember at a time
struct HintSlot {
    int dev, site, B, CO, CI;
    const void* weight;         // the layer: same shapes with other weights are other layers
    unsigned long long* host;   // pinned: kHintRing flags
    hipEvent_t ev[kHintRing];   // recorded behind the copy of flag i
    int head, queued;           // oldest outcome not yet looked at, and how many are queued
    int stale;                  // of the queued outcomes, how many belong to the layer the slot stood for before
    int streak, skip_left;
    unsigned long long used;    // g_hint_clock at the slot's last use: the least recently used slot is given away
};
std::mutex g_hint_mu;
std::vector<HintSlot> g_hints;
unsigned long long g_hint_clock = 0;

bool capturing(hipStream_t stream) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) { (void)hipGetLastError(); return false; }
    return cap != hipStreamCaptureStatusNone;
}

// A slot that is handed to another layer keeps its pinned memory and events (copies into them may still be on their
// way); what is queued at that moment is counted as stale and thrown away when it arrives.
void hint_rekey(HintSlot& h, int dev, int site, const void* weight, int B, int CO, int CI) {
    h.dev = dev; h.site = site; h.weight = weight; h.B = B; h.CO = CO; h.CI = CI;
    h.stale = h.queued;
    h.streak = h.skip_left = 0;
}

HintSlot* hint_slot(int site, const void* weight, int B, int CO, int CI, bool create) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    HintSlot* same_weight = nullptr;
    for (HintSlot& h : g_hints) {
        if (h.dev != dev || h.site != site || h.weight != weight) continue;
        if (h.B == B && h.CO == CO && h.CI == CI) { h.used = ++g_hint_clock; return &h; }
        same_weight = &h;
    }
    if (!create) return nullptr;
    // the same address with another shape: the memory holds another layer now, the old one's history is dropped
    if (same_weight) { hint_rekey(*same_weight, dev, site, weight, B, CO, CI); same_weight->used = ++g_hint_clock; return same_weight; }
    if (g_hints.size() >= kHintSlots) {
        HintSlot* oldest = nullptr;
        for (HintSlot& h : g_hints)
            if (h.dev == dev && (!oldest || h.used < oldest->used)) oldest = &h;   // events belong to their device
        if (!oldest) return nullptr;
        hint_rekey(*oldest, dev, site, weight, B, CO, CI);
        oldest->used = ++g_hint_clock;
        return oldest;
    }
    HintSlot h{};
    if (hipHostMalloc(reinterpret_cast<void**>(&h.host), kHintRing * sizeof(unsigned long long), hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    for (int i = 0; i < kHintRing; i++) {
        h.host[i] = 0;
        if (hipEventCreateWithFlags(&h.ev[i], hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            for (int k = 0; k < i; k++) (void)hipEventDestroy(h.ev[k]);   // nothing has been recorded on them yet
            (void)hipHostFree(h.host);
            return nullptr;
        }
    }
    hint_rekey(h, dev, site, weight, B, CO, CI);
    h.used = ++g_hint_clock;
    g_hints.push_back(h);
    return &g_hints.back();
}
}  // namespace

bool hint_build_tables(int site, const void* weight, int B, int CO, int CI, hipStream_t stream) {
    if (capturing(stream)) return true;
    std::lock_guard<std::mutex> lock(g_hint_mu);
    HintSlot* h = hint_slot(site, weight, B, CO, CI, false);
    if (!h) return true;
    // outcomes that have arrived, oldest first (the host may run several calls ahead of the device)
    while (h->queued > 0) {
        if (hipEventQuery(h->ev[h->head]) != hipSuccess) { (void)hipGetLastError(); break; }   // not ready: next call
        if (h->stale > 0) h->stale--;   // an outcome of the layer this slot stood for before
        else {
            h->streak = h->host[h->head] != 0ull ? h->streak + 1 : 0;
            // the streak is long enough (or the probe after a stretch without tables came out the same): no tables
            // for the next kHintSkip calls, then one call probes again
            h->skip_left = h->streak >= kHintStreak ? kHintSkip : 0;
        }
        h->head = (h->head + 1) % kHintRing;
        h->queued--;
    }
    if (h->skip_left > 0) { h->skip_left--; return false; }
    return true;
}

void hint_record(int site, const void* weight, int B, int CO, int CI, const unsigned long long* every_term_ran,
                 hipStream_t stream) {
    if (capturing(stream)) return;
    std::lock_guard<std::mutex> lock(g_hint_mu);
    HintSlot* h = hint_slot(site, weight, B, CO, CI, true);
    if (!h || h->queued == kHintRing) return;
    const int i = (h->head + h->queued) % kHintRing;
    if (hipMemcpyAsync(h->host + i, every_term_ran, sizeof(unsigned long long), hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipEventRecord(h->ev[i], stream) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    h->queued++;
}

__global__ void __launch_bounds__(256) fill_zero_kernel(uint32_t* __restrict__ p, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    size_t n4 = n / 4;
    uint4* p4 = reinterpret_cast<uint4*>(p);
    for (size_t k = i; k < n4; k += stride) p4[k] = make_uint4(0u, 0u, 0u, 0u);
    for (size_t k = n4 * 4 + i; k < n; k += stride) p[k] = 0u;
}

__global__ void __launch_bounds__(256) fill_zero2_kernel(uint4* __restrict__ a, size_t na4, uint4* __restrict__ b,
                                                         size_t nb4) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
    for (size_t k = i; k < na4; k += stride) a[k] = make_uint4(0u, 0u, 0u, 0u);
    for (size_t k = i; k < nb4; k += stride) b[k] = make_uint4(0u, 0u, 0u, 0u);
}

int fill_zero2(void* a, size_t na_words, void* b, size_t nb_words, hipStream_t stream) {
    if (na_words % 4 != 0 || nb_words % 4 != 0 || reinterpret_cast<uintptr_t>(a) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(b) % 16 != 0) {   // not two runs of whole 16-byte words: one launch each
        int rc = fill_zero(a, na_words, stream);
        return rc ? rc : fill_zero(b, nb_words, stream);
    }
    const size_t n4 = (na_words > nb_words ? na_words : nb_words) / 4;
    if (n4 == 0) return SD_OK;
    size_t blocks = (n4 + 255) / 256;
    const size_t cap = (size_t)num_cus() * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(fill_zero2_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<uint4*>(a),
                       na_words / 4, reinterpret_cast<uint4*>(b), nb_words / 4);
    return check_launch("fill_zero2");
}

int fill_zero(void* ptr, size_t n_words, hipStream_t stream) {
    if (n_words == 0) return SD_OK;
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) {
        set_error("fill_zero: buffer must be 16-byte aligned");
        return SD_ERR_ARG;
    }
    size_t blocks = (n_words / 4 + 255) / 256;
    size_t cap = (size_t)num_cus() * 16;
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       reinterpret_cast<uint32_t*>(ptr), n_words);
    return check_launch("fill_zero");
}

}  // namespace sd

extern "C" {

int sd_version(void) { return 100; }

const char* sd_last_error(void) { return sd::g_err; }

const char* sd_last_forward_kernel(void) { return sd::g_fwd_kernel; }

int sd_time_forward_kernels(int on) { sd::g_time_kernels = on != 0; sd::g_timed = false; return SD_OK; }

float sd_last_forward_kernel_ms(void) {
    if (!sd::g_timed) return -1.f;
    float ms = -1.f;
    if (hipEventSynchronize(sd::g_time_ev[1]) != hipSuccess ||
        hipEventElapsedTime(&ms, sd::g_time_ev[0], sd::g_time_ev[1]) != hipSuccess) {
        (void)hipGetLastError();
        return -1.f;
    }
    return ms;
}

float sd_last_forward_term_share(sd_stream_t stream) {
    const sd::TermNote n = sd::g_term_note;
    if (n.kind == 0 || !n.counts) return 1.f;
    unsigned long long c[4] = {0ull, 0ull, 0ull, 0ull};
    // waits for the stream, so the call that left the counters has run and nothing has overwritten them yet
    if (hipMemcpyAsync(c, n.counts, sizeof(c), hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)) != hipSuccess ||
        hipStreamSynchronize(static_cast<hipStream_t>(stream)) != hipSuccess) {
        (void)hipGetLastError();
        return -1.f;
    }
    if (n.kind == 1) return c[1] != 0ull ? 1.f : (float)((double)c[0] / n.denom0);
    if (n.kind == 3) return c[1] != 0ull ? 1.f : c[2] != 0ull ? (float)((double)c[0] / n.denom0) : (float)((double)c[3] / n.denom1);
    if (c[2] != 0ull) return 1.f;
    return c[0] <= n.limit0 ? (float)((double)c[0] / n.denom0) : (float)((double)c[1] / n.denom1);
}

uint32_t sd_rng_word(uint32_t seed, uint32_t stream_id, uint32_t row, uint32_t col) {
    return sd::rng_word(sd::rng_row_key(seed, stream_id, row), col);
}

uint32_t sd_mask_threshold8(float q) {
    double t = std::floor((double)q * 256.0 + 0.5);
    if (t < 0) t = 0;
    if (t > 256) t = 256;
    return (uint32_t)t;
}

uint32_t sd_mask_threshold16(float q) {
    double t = std::floor(std::sqrt((double)q) * 65536.0 + 0.5);
    if (t < 0) t = 0;
    if (t > 65536) t = 65536;
    return (uint32_t)t;
}

}  // extern "C"
