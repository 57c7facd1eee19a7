// A CPU stand-in for <hip/hip_runtime.h>: test infrastructure, never part of the library.
//
// The kernel sources of tenmo_amd/csrc compile against this header with a host compiler (clang++ for x86, which knows
// the vector extensions they use) into a CPU build of the whole library whose "device memory" is host memory.  A kernel
// launch runs here and now: every workgroup of the grid, every thread of a workgroup as a fibre (a stack of its own,
// switched cooperatively), so that the threads of a wavefront can meet at the operations that involve the whole
// wavefront (MFMA, shuffles) and the wavefronts of a workgroup at its barriers, in exactly the places where the source
// says so.  What this buys:
//   * every global address a kernel touches is a real host access: under AddressSanitizer (or next to a guard page)
//     an access one byte outside an operand is reported with the kernel, workgroup and thread that made it — the
//     check to run BEFORE a kernel is launched on a GPU with a new shape;
//   * the direct global->LDS loads and their s_waitcnt are modelled (a load lands in LDS no earlier than its issue and,
//     in the "late" mode, no earlier than the wait that covers it), so that a missing wait or a ring stage refilled too
//     early shows up as wrong numbers;
//   * barrier counts are checked: a workgroup whose wavefronts do not all arrive is reported as a deadlock;
//   * the results are the real kernel arithmetic in fp32, so that parity tests run without a GPU (slowly: small shapes).
// What it does not model: timing, occupancy, caches, the hardware's register limits, LDS bank conflicts, and any
// difference between the instruction sequence the GPU compiler emits and the C++ it was given.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <functional>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>

// ---- qualifiers ---------------------------------------------------------------------------------------------------
#define __host__
#define __device__
#define __global__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static thread_local
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

namespace replay {

constexpr int WAVE = 64;
constexpr int MAX_PENDING = 64; // the hardware's vmcnt holds 63

struct Wave {
    int live = 0, arrived = 0;
    uint64_t gen = 0;
    // hand-over slots of the wavefront-wide operations, two sets used in turn
    float a[2][WAVE], b[2][WAVE];
    uint64_t x[2][WAVE];
    bool alive[WAVE]; // lanes that exist and have not finished
};

struct Workgroup {
    dim3 bid, bdim, gdim;
    int live = 0, arrived = 0;
    uint64_t gen = 0;
    const char* kernel = "";
};

struct PendingLoad { char* dst; const char* src; };

struct Lane {
    dim3 tid;
    int lane = 0;      // within the wavefront
    int index = 0;     // within the workgroup
    Wave* wave = nullptr;
    Workgroup* wg = nullptr;
    void* sp = nullptr;          // saved stack pointer while switched out
    int state = 0;               // 0 runnable, 1 waits for its wavefront, 2 waits for the workgroup, 3 done
    uint64_t wait_gen = 0;
    unsigned turn = 0;           // which set of hand-over slots the next wavefront-wide operation uses
    PendingLoad pending[MAX_PENDING];
    int pend_head = 0, pend_count = 0;
};

extern thread_local Lane* cur;
extern int late_loads; // 1: a direct load reaches LDS at the wait that covers it (the latest the hardware may), 0: at issue

void wave_sync();                // every live lane of the wavefront arrives
void wg_barrier();               // every live lane of the workgroup arrives
void complete_loads(int leave);  // this lane's direct loads land until at most `leave` are outstanding
void check_global(const void* p, size_t bytes, bool write, const char* what);
void fail(const char* fmt, ...) __attribute__((noreturn));

// v_mfma_f32_32x32x2_f32: lane l brings A[i = l % 32][k = l / 32] and B[k = l / 32][j = l % 32]; it receives, in
// element e of its 16, D[8 (e / 4) + 4 (l / 32) + e % 4][l % 32]
template <class V>
inline V mfma32x32x2(float a, float b, V c) {
    Lane* l = cur;
    Wave* w = l->wave;
    const unsigned p = l->turn++ & 1;
    w->a[p][l->lane] = a;
    w->b[p][l->lane] = b;
    wave_sync();
    const int col = l->lane & 31, h = l->lane >> 5;
    const float b0 = w->b[p][col], b1 = w->b[p][32 + col];
    for (int e = 0; e < 16; ++e) {
        const int row = 8 * (e >> 2) + 4 * h + (e & 3);
        c[e] = std::fmaf(w->a[p][32 + row], b1, std::fmaf(w->a[p][row], b0, c[e]));
    }
    return c;
}

template <class T>
inline T exchange(T v, int src_lane) { // every lane gives v and takes the value of src_lane (its own when out of range)
    static_assert(sizeof(T) <= 8, "values of up to 8 bytes");
    Lane* l = cur;
    Wave* w = l->wave;
    const unsigned p = l->turn++ & 1;
    uint64_t bits = 0;
    std::memcpy(&bits, &v, sizeof(T));
    w->x[p][l->lane] = bits;
    wave_sync();
    if (src_lane < 0 || src_lane >= WAVE) src_lane = l->lane;
    T out;
    std::memcpy(&out, &w->x[p][src_lane], sizeof(T));
    return out;
}

inline int vote(bool pred, bool all) { // __any / __all over the live lanes of the wavefront
    Lane* l = cur;
    Wave* w = l->wave;
    const unsigned p = l->turn++ & 1;
    w->x[p][l->lane] = pred ? 1 : 0;
    wave_sync();
    int yes = 0, n = 0;
    for (int i = 0; i < WAVE; ++i)
        if (w->alive[i]) { ++n; yes += (int)w->x[p][i]; }
    return all ? yes == n : yes > 0;
}

inline void waitcnt(int imm) { complete_loads((imm & 0xF) | (((imm >> 14) & 3) << 4)); } // the gfx9 encoding of vmcnt

} // namespace replay

// ---- built-in variables and device functions ------------------------------------------------------------------------
#define threadIdx (replay::cur->tid)
#define blockIdx (replay::cur->wg->bid)
#define blockDim (replay::cur->wg->bdim)
#define gridDim (replay::cur->wg->gdim)

#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) replay::mfma32x32x2((a), (b), (c))
#define __builtin_amdgcn_s_waitcnt(imm) replay::waitcnt(imm)
#define __builtin_amdgcn_s_barrier() replay::wg_barrier()

inline void __syncthreads() { replay::wg_barrier(); }
template <class T> inline T __shfl_xor(T v, int mask, int width = 64) { (void)width; return replay::exchange(v, replay::cur->lane ^ mask); }
template <class T> inline T __shfl_down(T v, unsigned delta, int width = 64) { (void)width; return replay::exchange(v, replay::cur->lane + (int)delta); }
template <class T> inline T __shfl(T v, int src, int width = 64) { (void)width; return replay::exchange(v, src); }
inline int __any(int pred) { return replay::vote(pred != 0, false); }
inline int __all(int pred) { return replay::vote(pred != 0, true); }
inline float __expf(float x) { return std::exp(x); }
inline float __logf(float x) { return std::log(x); }
inline float unsafeAtomicAdd(float* p, float v) {
    uint32_t* q = reinterpret_cast<uint32_t*>(p);
    uint32_t old_bits = __atomic_load_n(q, __ATOMIC_RELAXED), want_bits;
    float old;
    do {
        std::memcpy(&old, &old_bits, 4);
        const float want = old + v;
        std::memcpy(&want_bits, &want, 4);
    } while (!__atomic_compare_exchange_n(q, &old_bits, want_bits, true, __ATOMIC_RELAXED, __ATOMIC_RELAXED));
    return old;
}
inline float atomicAdd(float* p, float v) { return unsafeAtomicAdd(p, v); }
inline unsigned atomicAdd(unsigned* p, unsigned v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); } // the fences around it order it
inline void __threadfence() { __atomic_thread_fence(__ATOMIC_SEQ_CST); }

// HIP's device-side min / max for mixed integer types
template <class A, class B, class = std::enable_if_t<std::is_arithmetic<A>::value && std::is_arithmetic<B>::value>>
inline constexpr std::common_type_t<A, B> min(A a, B b) { using T = std::common_type_t<A, B>; return (T)a < (T)b ? (T)a : (T)b; }
template <class A, class B, class = std::enable_if_t<std::is_arithmetic<A>::value && std::is_arithmetic<B>::value>>
inline constexpr std::common_type_t<A, B> max(A a, B b) { using T = std::common_type_t<A, B>; return (T)a < (T)b ? (T)b : (T)a; }

// ---- the gfx950 assembly pieces (tenmo_amd/csrc/gfx950_asm.hpp), modelled ------------------------------------------
#define TENMO_GFX950_ASM_HPP
namespace tenmo {
inline void direct_load_16B(float* lds, uint32_t block_byte_off, uint32_t lane_byte_off, const float* src) {
    replay::Lane* l = replay::cur;
    char* dst = reinterpret_cast<char*>(lds) + block_byte_off + 16 * l->lane;
    const char* s = reinterpret_cast<const char*>(src) + lane_byte_off;
    replay::check_global(s, 16, false, "direct load");
    if (l->pend_count == replay::MAX_PENDING) replay::fail("more than %d direct loads outstanding in one wavefront", replay::MAX_PENDING - 1);
    l->pending[(l->pend_head + l->pend_count++) % replay::MAX_PENDING] = replay::PendingLoad{dst, s};
    if (!replay::late_loads) replay::complete_loads(0);
}
inline void direct_load_16B_where(float* lds, uint32_t block_byte_off, uint32_t lane_byte_off, const float* src, bool ok) {
    if (ok) { direct_load_16B(lds, block_byte_off, lane_byte_off, src); return; }
    // a masked lane moves nothing, but the wavefront's load still counts in vmcnt
    replay::Lane* l = replay::cur;
    if (l->pend_count == replay::MAX_PENDING) replay::fail("more than %d direct loads outstanding in one wavefront", replay::MAX_PENDING - 1);
    l->pending[(l->pend_head + l->pend_count++) % replay::MAX_PENDING] = replay::PendingLoad{nullptr, nullptr};
    if (!replay::late_loads) replay::complete_loads(0);
}
template <class V> inline void keep_alive(const V&, const V&, const V&, const V&) {}
} // namespace tenmo

// ---- the runtime API (what the library's host side calls) ------------------------------------------------------------
typedef int hipError_t;
enum : int { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2, hipErrorIllegalAddress = 700, hipErrorUnknown = 999 };
typedef struct replayStream* hipStream_t;
typedef struct replayEvent* hipEvent_t;
typedef struct replayGraph* hipGraph_t;
typedef struct replayGraphExec* hipGraphExec_t;
enum hipMemcpyKind { hipMemcpyHostToHost = 0, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3, hipMemcpyDefault = 4 };
enum hipStreamCaptureMode { hipStreamCaptureModeGlobal = 0, hipStreamCaptureModeThreadLocal = 1, hipStreamCaptureModeRelaxed = 2 };
struct hipDeviceProp_t {
    char name[256];
    char gcnArchName[256];
    int multiProcessorCount;
    size_t totalGlobalMem;
};

// (C linkage, as in the real runtime: a plain C program can call them)
extern "C" {
hipError_t hipGetDeviceCount(int* n);
hipError_t hipSetDevice(int d);
hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int d);
hipError_t hipMalloc(void** p, size_t bytes);
hipError_t hipFree(void* p);
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind);
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind kind, hipStream_t s);
hipError_t hipMemcpy2DAsync(void* dst, size_t dpitch, const void* src, size_t spitch, size_t width, size_t height, hipMemcpyKind kind, hipStream_t s);
hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t s);
hipError_t hipMemset(void* dst, int value, size_t bytes);
hipError_t hipStreamCreate(hipStream_t* s);
hipError_t hipStreamDestroy(hipStream_t s);
hipError_t hipStreamSynchronize(hipStream_t s);
hipError_t hipDeviceSynchronize();
hipError_t hipEventCreate(hipEvent_t* e);
hipError_t hipEventDestroy(hipEvent_t e);
hipError_t hipEventRecord(hipEvent_t e, hipStream_t s);
hipError_t hipEventSynchronize(hipEvent_t e);
hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b);
hipError_t hipGetLastError();
const char* hipGetErrorString(hipError_t e);
hipError_t hipGetSymbolAddress(void** p, const void* symbol);
hipError_t hipStreamBeginCapture(hipStream_t s, hipStreamCaptureMode mode);
hipError_t hipStreamEndCapture(hipStream_t s, hipGraph_t* g);
hipError_t hipGraphInstantiate(hipGraphExec_t* exec, hipGraph_t g, void*, void*, size_t);
hipError_t hipGraphDestroy(hipGraph_t g);
hipError_t hipGraphExecDestroy(hipGraphExec_t e);
hipError_t hipGraphLaunch(hipGraphExec_t e, hipStream_t s);
} // extern "C"
template <class T> inline hipError_t hipMalloc(T** p, size_t bytes) { return hipMalloc(reinterpret_cast<void**>(p), bytes); }

namespace replay {
// what a real launch would put into the kernel's argument block: the arguments converted to the kernel's parameter types, each at
// its natural alignment (the layout of these plain structs is the same on the host and on the GPU), and the kernel function itself
struct KernelArgs {
    const void* fn = nullptr;
    std::vector<unsigned char> bytes;
};
template <class T, size_t I, class Tuple>
inline T nth_argument_or_zero(const Tuple& given) {
    // (a trailing parameter the launch leaves to its default: every such default in the library is a null pointer or 0)
    if constexpr (I < std::tuple_size_v<Tuple>) return static_cast<T>(std::get<I>(given));
    else return T{};
}
template <class... P, size_t... I, class Tuple>
inline void pack_each(KernelArgs& k, std::index_sequence<I...>, const Tuple& given) {
    auto put = [&k](auto value) {
        using T = decltype(value);
        const size_t at = (k.bytes.size() + alignof(T) - 1) / alignof(T) * alignof(T);
        k.bytes.resize(at + sizeof(T));
        std::memcpy(k.bytes.data() + at, &value, sizeof(T));
    };
    (put(nth_argument_or_zero<std::remove_cv_t<P>, I>(given)), ...);
}
template <class... P, class... A>
inline KernelArgs pack_args(void (*fn)(P...), const A&... a) {
    KernelArgs k;
    k.fn = reinterpret_cast<const void*>(fn);
    pack_each<P...>(k, std::index_sequence_for<P...>{}, std::forward_as_tuple(a...));
    return k;
}
void enqueue(hipStream_t s, const char* name, dim3 grid, dim3 block, std::function<void()> body, KernelArgs args);
}
// the arguments are evaluated now and copied into the launch, as the real launch copies them into the kernel's argument block
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...)                                                                 \
    replay::enqueue((stream), #kernel, dim3(grid), dim3(block), replay::bind_kernel([](auto... a) { kernel(a...); }, __VA_ARGS__), \
                    replay::pack_args(kernel, __VA_ARGS__))

namespace replay {
template <class F, class... Args>
inline std::function<void()> bind_kernel(F f, Args... args) {
    return [=]() { f(args...); };
}
} // namespace replay
