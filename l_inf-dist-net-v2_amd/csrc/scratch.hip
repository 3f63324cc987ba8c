// Temporary device memory of the launchers.
//
// hipMallocAsync / hipFreeAsync wait on the host until the work queued before them on the stream has finished
// (measured on ROCm 7.2: a loop of kernel + hipMallocAsync + hipFreeAsync runs at the kernel's pace on the host
// side too, whatever the pool's release threshold), so a launcher that takes its scratch from the stream-ordered pool
// turns every call into a synchronous one and a training loop loses the overlap of host and device work.
//
// Instead the library keeps arenas: blocks of device memory that stay allocated and are handed out again call after
// call.  An arena belongs to one (device, stream) and serves one call at a time; work queued on a stream runs in
// order, so the next call on that stream may reuse the bytes the previous one used without any wait.  Two host
// threads that call on the same stream at the same time get two arenas.  Within a call the allocations are
// released in reverse order (a stack).  The blocking hipMalloc / hipFree appear only while an arena is still
// growing towards the largest request of its stream, i.e. in the first calls of each shape.
//
// Callers that cannot allocate at all use the entry point that takes its scratch from a fixed array in device
// memory instead (static scratch, below): while a StaticScratchScope is alive on the calling thread, scratch_alloc
// hands out pieces of that array and never touches the arenas or the HIP allocator.
#include <atomic>
#include <mutex>
#include <vector>

#include "ndist_common.h"

namespace ndist {

// Scratch of the entry point that allocates nothing: one array per device, part of the code object, alive until the
// process ends.  Host code never uses the array's name as an address: the device address is looked up once per
// device with hipGetSymbolAddress (static_scratch_base) and passed to the kernels like any other buffer.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr size_t kAlign = 256;

std::atomic<long> g_mallocs{0}, g_frees{0};  // hipMalloc / hipFree calls made for the arenas (scratch_counters)

thread_local StaticScratchScope* t_static = nullptr;  // lives on the stack of the entry point

struct Block {
    char* base;
    size_t size, used;
};

struct Arena {
    int device;
    hipStream_t stream;
    bool busy;
    std::vector<Block> blocks;  // normally one; more while a call outgrows the first
    size_t live;                // allocations of the current call not yet released
    size_t high;                // largest total the arena had in use during a call
    size_t cur;                 // total in use now
};

std::mutex g_mu;
std::vector<Arena*> g_arenas;  // never shrinks; arenas are reused

struct Current {
    Arena* arena = nullptr;
};
thread_local Current t_cur;

size_t aligned(size_t n) { return (n + kAlign - 1) / kAlign * kAlign; }

void free_blocks(Arena* a) {
    for (Block& b : a->blocks) {
        (void)hipFree(b.base);  // hipFree waits for the device: nothing still reads the block
        g_frees++;
    }
    a->blocks.clear();
}

// The arena of (device, stream) for a new call: an idle one, with a single block large enough for what its calls
// have needed so far.
Arena* acquire(hipStream_t st) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    Arena* a = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        for (Arena* c : g_arenas)
            if (!c->busy && c->device == dev && c->stream == st) { a = c; break; }
        if (a == nullptr) {
            a = new Arena{dev, st, false, {}, 0, 0, 0};
            g_arenas.push_back(a);
        }
        a->busy = true;
    }
    // a call that spilled into further blocks: one block of the whole size from now on
    if (a->blocks.size() > 1 || (a->blocks.size() == 1 && a->blocks[0].size < a->high)) {
        free_blocks(a);
        char* p = nullptr;
        const size_t want = aligned(a->high + a->high / 4);
        if (hipMalloc((void**)&p, want) == hipSuccess) {
            a->blocks.push_back(Block{p, want, 0});
            g_mallocs++;
        } else {
            (void)hipGetLastError();  // the blocks come back one request at a time
        }
    }
    a->live = 0;
    a->cur = 0;
    for (Block& b : a->blocks) b.used = 0;
    return a;
}

void release(Arena* a) {
    std::lock_guard<std::mutex> lock(g_mu);
    a->busy = false;
}

}  // namespace

bool stream_is_capturing(hipStream_t st) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    // an error here (e.g. the legacy stream while another stream captures globally) also means "do not touch it"
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return cs != hipStreamCaptureStatusNone;
}

// may_query == false (the stream is being captured): only an address that an earlier call has already looked up
// is returned; the lookup itself is not made from inside a capture
hipError_t static_scratch_base(char** out, bool may_query) {
    constexpr int kMaxDev = 64;
    static char* base[kMaxDev] = {};
    static std::mutex mu;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDev) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (base[dev] == nullptr && !may_query) return hipErrorStreamCaptureUnsupported;
    if (base[dev] == nullptr) {
        // once per device, with that device current: every device holds its own copy of the array
        char* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (ptr == nullptr) return hipErrorInvalidSymbol;
        base[dev] = ptr;
    }
    *out = base[dev];
    return hipSuccess;
}

StaticScratchScope::StaticScratchScope(bool may_query) : status(hipSuccess), base(nullptr), used(0), live(0) {
    status = static_scratch_base(&base, may_query);
    if (status == hipSuccess) t_static = this;
}
StaticScratchScope::~StaticScratchScope() {
    if (t_static == this) t_static = nullptr;
}
bool static_scratch_active() { return t_static != nullptr; }

void scratch_counters(long* mallocs, long* frees) {
    *mallocs = g_mallocs.load();
    *frees = g_frees.load();
}

hipError_t scratch_alloc(void** out, size_t bytes, hipStream_t st) {
    *out = nullptr;
    if (t_static != nullptr) {
        // pieces of the fixed array, stack-ordered like the arena's; no allocation, no query of the stream
        const size_t need = aligned(bytes == 0 ? 1 : bytes);
        if (need > kStaticScratchBytes - t_static->used) return hipErrorOutOfMemory;
        *out = t_static->base + t_static->used;
        t_static->used += need;
        t_static->live++;
        return hipSuccess;
    }
    // A stream that is being captured into a graph must see neither an allocation (hipMalloc is not permitted
    // during a capture, and a later hipFree of the block would leave the graph with a dangling address) nor a
    // block address that only this call's arena guarantees: calls that need scratch refuse to run under capture.
    if (stream_is_capturing(st)) return hipErrorStreamCaptureUnsupported;
    if (t_cur.arena != nullptr && t_cur.arena->stream != st) {
        // a call that failed between a request and its release left its arena attached to this thread
        release(t_cur.arena);
        t_cur.arena = nullptr;
    }
    if (t_cur.arena == nullptr) {
        t_cur.arena = acquire(st);
        if (t_cur.arena == nullptr) return hipErrorInvalidDevice;
    }
    Arena* a = t_cur.arena;
    const size_t need = aligned(bytes == 0 ? 1 : bytes);
    Block* blk = a->blocks.empty() ? nullptr : &a->blocks.back();
    if (blk == nullptr || blk->size - blk->used < need) {
        // a further block; hipMalloc does not wait for queued work and nothing queued can know the new address
        char* p = nullptr;
        const hipError_t e = hipMalloc((void**)&p, need);
        if (e != hipSuccess) {
            if (a->live == 0) { release(a); t_cur.arena = nullptr; }
            return e;
        }
        g_mallocs++;
        a->blocks.push_back(Block{p, need, 0});
        blk = &a->blocks.back();
    }
    *out = blk->base + blk->used;
    blk->used += need;
    a->live++;
    a->cur += need;
    if (a->cur > a->high) a->high = a->cur;
    return hipSuccess;
}

hipError_t scratch_free(void* p, hipStream_t) {
    if (t_static != nullptr) {
        char* c = static_cast<char*>(p);
        if (p == nullptr || t_static->live == 0 || c < t_static->base || c >= t_static->base + t_static->used)
            return hipErrorInvalidValue;
        t_static->used = (size_t)(c - t_static->base);
        t_static->live--;
        return hipSuccess;
    }
    Arena* a = t_cur.arena;
    if (p == nullptr || a == nullptr || a->live == 0) return hipErrorInvalidValue;
    // stack order: p is the most recent allocation still alive, at the end of the last block in use
    for (size_t i = a->blocks.size(); i-- > 0;) {
        Block& b = a->blocks[i];
        char* c = static_cast<char*>(p);
        if (c >= b.base && c < b.base + b.used) {
            a->cur -= (size_t)(b.base + b.used - c);
            b.used = (size_t)(c - b.base);
            break;
        }
    }
    if (--a->live == 0) {
        release(a);
        t_cur.arena = nullptr;
    }
    return hipSuccess;
}

int scratch_release_all() {
    std::lock_guard<std::mutex> lock(g_mu);
    int rc = 0;
    int keep = 0;
    if (hipGetDevice(&keep) != hipSuccess) return 4;
    for (Arena* a : g_arenas) {
        if (a->busy) continue;
        if (hipSetDevice(a->device) != hipSuccess) { rc = 4; continue; }
        free_blocks(a);
        a->high = 0;
    }
    (void)hipSetDevice(keep);
    return rc;
}

}  // namespace ndist
