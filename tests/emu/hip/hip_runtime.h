// Test infrastructure, not a HIP runtime: a CPU stand-in for the few pieces of <hip/hip_runtime.h> that the plain
// (no matrix-core, no LDS-DMA) kernels of hodu_amd/csrc use, so that a kernel's UNMODIFIED source can be compiled
// for the host and run there -- a CPU build for checking indexing, masks and reductions without a GPU.
//
// Execution model: a launch runs its workgroups one after the other (so __shared__ can be a plain static).  A
// wavefront is a host thread; its 64 lanes are contexts of their own on that thread, each run until it reaches a point
// where the wavefront has to meet (a cross-lane operation such as __shfl_xor, which exchanges through a per-wavefront
// buffer) or the workgroup has to (__syncthreads), and resumed when the others have arrived.  Arithmetic is the host's: expf / exp
// are libm's, bf16 / f16 conversions the host compiler's (round to nearest even), so results agree with the device
// to rounding, not to the bit.  The 8-bit float conversions are written out below.  Nothing here knows about MFMA,
// DPP, LDS-DMA or buffer instructions; stand-ins for
// those the tile kernels use are in gfx950_insn_emu.hpp, for the translation units that want them.
#pragma once

#include <sys/mman.h>
#include <ucontext.h>

#include <chrono>
#include <cmath>
#include <condition_variable>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
// A kernel's static __shared__ arrays become statics (workgroups run one at a time).  The dynamically sized LDS
// (HODU_DYNAMIC_LDS(name) in the kernels) is one 160 KiB array that belongs to the workgroup that is running.
#define __shared__ static
namespace emu {
constexpr unsigned kLdsBytes = 160 * 1024;
char *lds_base();
}  // namespace emu
#define HODU_DYNAMIC_LDS(name) char *const name = emu::lds_base()
#define __align__(n) __attribute__((aligned(n)))

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct emu_uint3 { unsigned x = 0, y = 0, z = 0; };

// ---- the runtime API the library's host code calls: one device, one implicit stream, everything synchronous --------
typedef void *hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0, hipErrorOutOfMemory = 2, hipErrorInvalidValue = 1;
struct hipDeviceProp_t {
    char name[64] = "CPU build of the kernels";
    char gcnArchName[64] = "gfx950:emulated";
    int multiProcessorCount = 256;
    int clockRate = 2400000;
    size_t totalGlobalMem = (size_t)288 << 30;
};
namespace emu {
// "device" memory: host memory between two inaccessible pages, the allocation's last 16-byte unit ending where the
// second one begins (emu_alloc_tight(0): its first byte following the first one instead)
void *device_alloc(size_t bytes);
bool device_free(void *p);
}  // namespace emu
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipSetDevice(int) { return hipSuccess; }
inline const char *hipGetErrorString(hipError_t e) { return e == hipErrorOutOfMemory ? "out of memory" : "emulated runtime error"; }
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
inline hipError_t hipFuncSetAttribute(const void *, hipFuncAttribute, int) { return hipSuccess; }
inline hipError_t hipGetDeviceCount(int *n) { *n = 1; return hipSuccess; }
inline hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int) { *p = hipDeviceProp_t(); return hipSuccess; }
constexpr unsigned hipStreamNonBlocking = 1;
inline hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { *s = nullptr; return hipSuccess; }
inline hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
// Graphs: while the (one) stream is being captured, a kernel launch or a memset is recorded instead of run; launching
// the instantiated graph runs the recorded nodes in order.
struct emu_graph { std::vector<std::function<void()>> nodes; };
typedef emu_graph *hipGraph_t;
typedef emu_graph *hipGraphExec_t;
typedef void *hipGraphNode_t;
namespace emu {
inline emu_graph *&capturing() { static emu_graph *g = nullptr; return g; }
}  // namespace emu
enum hipStreamCaptureStatus { hipStreamCaptureStatusNone = 0, hipStreamCaptureStatusActive = 1 };
enum hipStreamCaptureMode { hipStreamCaptureModeGlobal = 0, hipStreamCaptureModeThreadLocal = 1, hipStreamCaptureModeRelaxed = 2 };
inline hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus *st) {
    *st = emu::capturing() ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
    return hipSuccess;
}
inline hipError_t hipStreamBeginCapture(hipStream_t, hipStreamCaptureMode) {
    if (emu::capturing()) return hipErrorInvalidValue;
    emu::capturing() = new emu_graph;
    return hipSuccess;
}
inline hipError_t hipStreamEndCapture(hipStream_t, hipGraph_t *g) {
    *g = emu::capturing();
    emu::capturing() = nullptr;
    return *g ? hipSuccess : hipErrorInvalidValue;
}
inline hipError_t hipGraphInstantiate(hipGraphExec_t *exec, hipGraph_t g, hipGraphNode_t *, char *, size_t) {
    *exec = new emu_graph(*g);
    return hipSuccess;
}
inline hipError_t hipGraphLaunch(hipGraphExec_t exec, hipStream_t) {
    for (auto &node : exec->nodes) node();
    return hipSuccess;
}
inline hipError_t hipGraphExecDestroy(hipGraphExec_t exec) { delete exec; return hipSuccess; }
inline hipError_t hipGraphDestroy(hipGraph_t g) { delete g; return hipSuccess; }
template <class T> inline hipError_t hipMalloc(T **p, size_t bytes) {
    *p = (T *)emu::device_alloc(bytes);
    return *p ? hipSuccess : hipErrorOutOfMemory;
}
inline hipError_t hipFree(void *p) { return (!p || emu::device_free(p)) ? hipSuccess : hipErrorInvalidValue; }
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
inline hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind, hipStream_t) { memmove(dst, src, bytes); return hipSuccess; }
inline hipError_t hipMemcpy(void *dst, const void *src, size_t bytes, hipMemcpyKind) { memmove(dst, src, bytes); return hipSuccess; }
inline hipError_t hipMemsetAsync(void *dst, int byte, size_t bytes, hipStream_t) {
    if (emu::capturing()) emu::capturing()->nodes.push_back([=] { memset(dst, byte, bytes); });
    else memset(dst, byte, bytes);
    return hipSuccess;
}
// a __device__ variable is an ordinary one here, and its "device address" its address
#define HIP_SYMBOL(x) (x)
template <class T> inline hipError_t hipGetSymbolAddress(void **p, T &symbol) { *p = (void *)&symbol; return hipSuccess; }
// events: the host's clock at the moment of recording (everything before it on the one stream has run by then)
struct emu_event { std::chrono::steady_clock::time_point at; };
typedef emu_event *hipEvent_t;
inline hipError_t hipEventCreate(hipEvent_t *e) { *e = new emu_event{std::chrono::steady_clock::now()}; return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t) { e->at = std::chrono::steady_clock::now(); return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float *ms, hipEvent_t a, hipEvent_t b) {
    *ms = std::chrono::duration<float, std::milli>(b->at - a->at).count();
    return hipSuccess;
}
inline hipError_t hipEventDestroy(hipEvent_t e) { delete e; return hipSuccess; }

namespace emu {
constexpr int kWave = 64, kMaxBlock = 1024;

// a barrier whose parties may leave for good (here: the wavefronts' threads of one workgroup)
class Barrier {
public:
    void reset(unsigned parties) { parties_ = parties; waiting_ = 0; phase_ = 0; }
    void wait() {
        std::unique_lock<std::mutex> hold(mu_);
        const unsigned my = phase_;
        if (++waiting_ >= parties_) {
            waiting_ = 0;
            phase_++;
            cv_.notify_all();
            return;
        }
        cv_.wait(hold, [&] { return phase_ != my; });
    }
    void leave() {
        std::unique_lock<std::mutex> hold(mu_);
        parties_--;
        if (parties_ > 0 && waiting_ >= parties_) {
            waiting_ = 0;
            phase_++;
            cv_.notify_all();
        }
    }
private:
    std::mutex mu_;
    std::condition_variable cv_;
    unsigned parties_ = 0, waiting_ = 0, phase_ = 0;
};

// A lane is a context of its own (stack, registers) that runs until it reaches a point where the wavefront or the
// workgroup has to meet, and is resumed when everyone it waits for has arrived; a lane that has returned from the
// kernel is waited for by nobody, as on the GPU.
enum LaneState { kRunnable, kAtWaveMeet, kAtBlockBarrier, kDone };
struct PendingDma { const char *src; unsigned lds_addr; };
struct Lane {
    ucontext_t uc;
    LaneState state = kDone;
    emu_uint3 tid;
    unsigned flat = 0;
    // per-wavefront registers and queues of the LDS-DMA model (gfx950_insn_emu.hpp), kept per lane
    unsigned m0 = 0;
    bool m0_written = false;
    unsigned wide_phase = 0;
    std::vector<PendingDma> dma_queue;
};
struct Block {
    Barrier all;  // __syncthreads, between the wavefronts' threads
    alignas(16) unsigned char xchg[kMaxBlock / kWave][kWave][16];
    alignas(16) unsigned char wide[2][kMaxBlock / kWave][kWave][64];  // operands of wavefront-wide instructions, two sets
};
struct WaveRun {
    ucontext_t sched;
    Lane lanes[kWave];
    const std::function<void()> *kernel = nullptr;
};
inline Block *&current() { static Block *b = nullptr; return b; }
inline thread_local Lane *t_lane = nullptr;
inline thread_local WaveRun *t_wave = nullptr;
inline thread_local emu_uint3 b_idx, b_dim, g_dim;

// stacks of all lanes of a workgroup, allocated once, an inaccessible page below each
constexpr size_t kStackBytes = 1u << 20, kStackStride = kStackBytes + 4096;
inline char *lane_stack(unsigned flat) {
    static char *pool = [] {
        void *p = mmap(nullptr, kStackStride * kMaxBlock, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        if (p == MAP_FAILED) { perror("emu: lane stacks"); abort(); }
        for (unsigned i = 0; i < (unsigned)kMaxBlock; i++) mprotect((char *)p + i * kStackStride, 4096, PROT_NONE);
        return (char *)p;
    }();
    return pool + flat * kStackStride + 4096;
}
inline void lane_entry() {
    (*t_wave->kernel)();
    t_lane->state = kDone;  // returning resumes the scheduler (uc_link)
}
inline void lane_yield(LaneState why) {
    t_lane->state = why;
    swapcontext(&t_lane->uc, &t_wave->sched);
}
// every running lane of the wavefront arrives here before any goes on
inline void wave_meet() { lane_yield(kAtWaveMeet); }

inline void run_wave(Block &blk, const std::function<void()> &kernel, unsigned w, dim3 block) {
    std::unique_ptr<WaveRun> owned(new WaveRun);
    WaveRun &run = *owned;
    run.kernel = &kernel;
    t_wave = &run;
    for (unsigned l = 0; l < (unsigned)kWave; l++) {
        Lane &ln = run.lanes[l];
        const unsigned t = w * kWave + l;
        ln.flat = t;
        ln.tid.x = t % block.x; ln.tid.y = (t / block.x) % block.y; ln.tid.z = t / (block.x * block.y);
        ln.m0 = 0; ln.m0_written = false; ln.wide_phase = 0; ln.dma_queue.clear();
        getcontext(&ln.uc);
        ln.uc.uc_stack.ss_sp = lane_stack(t);
        ln.uc.uc_stack.ss_size = kStackBytes;
        ln.uc.uc_link = &run.sched;
        makecontext(&ln.uc, lane_entry, 0);
        ln.state = kRunnable;
    }
    for (;;) {
        for (unsigned l = 0; l < (unsigned)kWave; l++)
            if (run.lanes[l].state == kRunnable) {
                t_lane = &run.lanes[l];
                swapcontext(&run.sched, &run.lanes[l].uc);
            }
        unsigned meet = 0, barrier = 0, done = 0;
        for (unsigned l = 0; l < (unsigned)kWave; l++) {
            meet += run.lanes[l].state == kAtWaveMeet;
            barrier += run.lanes[l].state == kAtBlockBarrier;
            done += run.lanes[l].state == kDone;
        }
        if (done == (unsigned)kWave) break;
        if (meet != 0 && barrier != 0) {
            fprintf(stderr, "emu: wavefront %u diverged: %u lanes at a wavefront-wide instruction, %u at a workgroup barrier\n", w, meet, barrier);
            abort();
        }
        if (barrier != 0) blk.all.wait();
        for (unsigned l = 0; l < (unsigned)kWave; l++)
            if (run.lanes[l].state != kDone) run.lanes[l].state = kRunnable;
    }
    t_lane = nullptr;
    t_wave = nullptr;
    blk.all.leave();
}

inline void run_grid(const std::function<void()> &call, dim3 grid, dim3 block) {
    static Block blk;  // (workgroups, and launches, run one at a time)
    current() = &blk;
    const unsigned waves = block.x * block.y * block.z / kWave;
    // The threads of wavefronts 1.. live for the whole launch and are handed one workgroup after the other (the
    // calling thread is wavefront 0): `turn` counts the workgroups started, `finished` the wavefronts done with the
    // current one.
    struct Shift {
        std::mutex mu;
        std::condition_variable cv;
        unsigned long turn = 0;
        unsigned finished = 0;
        bool over = false;
        emu_uint3 idx;
    } shift;
    auto body = [&](unsigned w, emu_uint3 idx) {
        b_idx = idx;
        b_dim.x = block.x; b_dim.y = block.y; b_dim.z = block.z;
        g_dim.x = grid.x; g_dim.y = grid.y; g_dim.z = grid.z;
        run_wave(blk, call, w, block);
    };
    std::vector<std::thread> pool;
    pool.reserve(waves - 1);
    for (unsigned w = 1; w < waves; w++)
        pool.emplace_back([&, w] {
            unsigned long seen = 0;
            for (;;) {
                emu_uint3 idx;
                {
                    std::unique_lock<std::mutex> hold(shift.mu);
                    shift.cv.wait(hold, [&] { return shift.over || shift.turn != seen; });
                    if (shift.over) return;
                    seen = shift.turn;
                    idx = shift.idx;
                }
                body(w, idx);
                {
                    std::lock_guard<std::mutex> hold(shift.mu);
                    shift.finished++;
                }
                shift.cv.notify_all();
            }
        });
    for (unsigned bz = 0; bz < grid.z; bz++)
        for (unsigned by = 0; by < grid.y; by++)
            for (unsigned bx = 0; bx < grid.x; bx++) {
                blk.all.reset(waves);
                emu_uint3 idx;
                idx.x = bx; idx.y = by; idx.z = bz;
                {
                    std::lock_guard<std::mutex> hold(shift.mu);
                    shift.idx = idx;
                    shift.finished = 0;
                    shift.turn++;
                }
                shift.cv.notify_all();
                body(0, idx);
                std::unique_lock<std::mutex> hold(shift.mu);
                shift.cv.wait(hold, [&] { return shift.finished == waves - 1; });
            }
    {
        std::lock_guard<std::mutex> hold(shift.mu);
        shift.over = true;
    }
    shift.cv.notify_all();
    for (auto &th : pool) th.join();
    current() = nullptr;
}

template <class K, class... Args> void launch(K kernel, dim3 grid, dim3 block, Args... args) {
    const unsigned nthreads = block.x * block.y * block.z;
    if (nthreads == 0 || nthreads > (unsigned)kMaxBlock || nthreads % kWave != 0) {
        fprintf(stderr, "emu: a workgroup of %u threads is not whole wavefronts\n", nthreads);
        abort();
    }
    const std::function<void()> call = [=] { kernel(args...); };
    if (emu_graph *g = capturing()) g->nodes.push_back([=] { run_grid(call, grid, block); });  // recorded, run at graph launch
    else run_grid(call, grid, block);
}
inline unsigned flat_tid() { return t_lane->flat; }
}  // namespace emu

#define threadIdx (emu::t_lane->tid)
#define blockIdx (emu::b_idx)
#define blockDim (emu::b_dim)
#define gridDim (emu::g_dim)
// the parenthesised kernel name of a template instantiation arrives as one macro argument
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) emu::launch(kernel, grid, block, __VA_ARGS__)

inline void __syncthreads() { emu::lane_yield(emu::kAtBlockBarrier); }

// every lane of the wavefront that is still running calls it; a lane that has returned from the kernel is not waited
// for (its slot keeps what it wrote last)
template <class T> inline T __shfl_xor(T v, int lane_mask, int width = 64) {
    static_assert(sizeof(T) <= 16, "exchange slot");
    (void)width;
    emu::Block *b = emu::current();
    const unsigned tid = emu::flat_tid(), w = tid / emu::kWave, lane = tid % emu::kWave;
    memcpy(b->xchg[w][lane], &v, sizeof(T));
    emu::wave_meet();
    T out;
    memcpy(&out, b->xchg[w][(lane ^ (unsigned)lane_mask) % emu::kWave], sizeof(T));
    emu::wave_meet();
    return out;
}

// HIP's device headers put the classification functions at global scope
using std::isinf;
using std::isnan;
using std::isfinite;

inline float __uint_as_float(unsigned u) { float f; memcpy(&f, &u, 4); return f; }
inline unsigned __float_as_uint(float f) { unsigned u; memcpy(&u, &f, 4); return u; }

// An instruction without a CPU stand-in: a kernel that reaches one counts it here and goes on with zeros, and the test
// that ran it fails on the count.
namespace emu {
inline int &no_such_instruction_hits() { static int n = 0; return n; }
inline const char *&no_such_instruction_first() { static const char *what = ""; return what; }
inline int no_such_instruction(const char *what = "?") {
    if (no_such_instruction_hits() == 0) no_such_instruction_first() = what;
    return ++no_such_instruction_hits();
}

// The 8-bit float conversions of gfx950 (OCP formats): e4m3 has no infinities and one NaN per sign (0x7F), e5m2 is
// IEEE-like.  Narrowing rounds to nearest even; what lies beyond the largest finite value becomes NaN (e4m3) or
// infinity (e5m2) -- the kernels clamp first, so that only matters for non-finite inputs.
template <int EBITS, int MBITS> inline float f8_decode(unsigned v) {
    constexpr int BIAS = (1 << (EBITS - 1)) - 1, EMAX = (1 << EBITS) - 1;
    const unsigned e = (v >> MBITS) & EMAX, m = v & ((1u << MBITS) - 1);
    const float sign = (v & 0x80u) ? -1.f : 1.f;
    if (EBITS == 4 ? (e == (unsigned)EMAX && m == (1u << MBITS) - 1) : (e == (unsigned)EMAX && m != 0)) return NAN;
    if (EBITS == 5 && e == (unsigned)EMAX) return sign * INFINITY;
    if (e == 0) return sign * std::ldexp((float)m, 1 - BIAS - MBITS);
    return sign * std::ldexp(1.f + (float)m / (1 << MBITS), (int)e - BIAS);
}
template <int EBITS, int MBITS> inline unsigned f8_encode(float f) {
    constexpr int BIAS = (1 << (EBITS - 1)) - 1, EMAX = (1 << EBITS) - 1;
    constexpr unsigned NAN_CODE = 0x7F, INF_CODE = EBITS == 5 ? (unsigned)EMAX << MBITS : NAN_CODE;
    const unsigned sign = std::signbit(f) ? 0x80u : 0u;
    if (f != f) return sign | NAN_CODE;
    const double a = std::fabs((double)f);
    if (std::isinf(a)) return sign | INF_CODE;
    unsigned code;
    if (a < std::ldexp(1.0, 1 - BIAS)) {
        code = (unsigned)std::nearbyint(a * std::ldexp(1.0, BIAS - 1 + MBITS));  // units of the smallest subnormal
    } else {
        int e;
        const double m = std::frexp(a, &e) * 2.0;  // [1, 2)
        e -= 1;
        unsigned q = (unsigned)std::nearbyint((m - 1.0) * (1 << MBITS));
        if (q == (1u << MBITS)) { q = 0; e += 1; }
        if (e + BIAS > EMAX) return sign | INF_CODE;
        code = ((unsigned)(e + BIAS) << MBITS) | q;
    }
    if (EBITS == 4 ? code >= 0x7F : code >= INF_CODE) return sign | INF_CODE;
    return sign | code;
}
inline int cvt_pk_f8(unsigned lo, unsigned hi_code, int old, bool high_half) {
    const unsigned pk = lo | (hi_code << 8);
    return high_half ? (int)(((unsigned)old & 0xFFFFu) | (pk << 16)) : (int)(((unsigned)old & 0xFFFF0000u) | pk);
}
inline float fmed3(float a, float b, float c) { return std::fmax(std::fmin(a, b), std::fmin(std::fmax(a, b), c)); }
}  // namespace emu
#define __builtin_amdgcn_cvt_f32_fp8(word, sel) (emu::f8_decode<4, 3>(((unsigned)(word) >> (8 * (sel))) & 0xFFu))
#define __builtin_amdgcn_cvt_f32_bf8(word, sel) (emu::f8_decode<5, 2>(((unsigned)(word) >> (8 * (sel))) & 0xFFu))
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, hi) (emu::cvt_pk_f8(emu::f8_encode<4, 3>(a), emu::f8_encode<4, 3>(b), old, hi))
#define __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, hi) (emu::cvt_pk_f8(emu::f8_encode<5, 2>(a), emu::f8_encode<5, 2>(b), old, hi))
#define __builtin_amdgcn_fmed3f(a, b, c) (emu::fmed3(a, b, c))
