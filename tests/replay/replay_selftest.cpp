// Self-test of the CPU replay (hip/hip_runtime.h in this directory): tiny kernels that are wrong on purpose — on the
// CPU, where that is harmless — to show that each kind of mistake is caught, and one that is right.
//   replay_selftest ok | overread | overwrite | direct_overread | divergent_collective | lenient_wait
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

extern "C" void replay_set_late_loads(int on);
#include "../../tenmo_amd/csrc/gfx950_asm.hpp" // (pre-empted by the stand-in: declares nothing new)

namespace {

// out[i] = in[i] + in[i + shift]: shift = 1 reads one element past the end in the last thread
__global__ void shifted_sum(const float* in, float* out, int n, int shift) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = in[i] + in[i + shift];
}

__global__ void store_past(float* out, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i <= n) out[i] = 1.f; // one too many
}

// every lane copies 16 bytes of `in` into LDS with a direct load and reads its neighbour's; `wait` = outstanding loads
// the kernel tolerates before reading (must be 0); `extra` shifts the source (1: the last lane reads past the end)
template <int WAIT>
__global__ void direct_copy(const float* in, float* out, int extra) {
    __shared__ __attribute__((aligned(1024))) float stage[256];
    const int lane = threadIdx.x;
    tenmo::direct_load_16B(stage, 0, (uint32_t)(lane * 16 + extra * 16), in);
    __builtin_amdgcn_s_waitcnt(WAIT); // vmcnt in the low bits of the gfx9 encoding
    __syncthreads();
    out[lane] = stage[4 * ((lane + 1) % 64)];
}

// half of a wavefront waits for an exchange with the other half, which waits at the workgroup barrier: neither arrives
__global__ void divergent_collective(float* out) {
    float v = (float)threadIdx.x;
    if (threadIdx.x < 32) v = __shfl_xor(v, 1, 64);
    else __syncthreads();
    out[threadIdx.x] = v;
}

} // namespace

int main(int argc, char** argv) {
    const char* what = argc > 1 ? argv[1] : "ok";
    const int n = 256;
    float *in, *out;
    hipMalloc(&in, n * sizeof(float));
    hipMalloc(&out, n * sizeof(float));
    for (int i = 0; i < n; ++i) { in[i] = (float)i; out[i] = 0.f; }
    if (!strcmp(what, "ok")) {
        hipLaunchKernelGGL(shifted_sum, dim3(n / 64), dim3(64), 0, nullptr, in, out, n, 0);
        for (int i = 0; i < n; ++i) if (out[i] != (float)(2 * i)) { printf("wrong sum at %d\n", i); return 1; }
        replay_set_late_loads(1);
        hipLaunchKernelGGL((direct_copy<0>), dim3(1), dim3(64), 0, nullptr, in, out, 0);
        for (int i = 0; i < 64; ++i) if (out[i] != (float)(4 * ((i + 1) % 64))) { printf("wrong copy at %d: %g\n", i, out[i]); return 1; }
        printf("ok\n");
        return 0;
    }
    if (!strcmp(what, "overread")) hipLaunchKernelGGL(shifted_sum, dim3(n / 64), dim3(64), 0, nullptr, in, out, n, 1);
    else if (!strcmp(what, "overwrite")) hipLaunchKernelGGL(store_past, dim3(n / 64 + 1), dim3(64), 0, nullptr, out, n);
    else if (!strcmp(what, "direct_overread")) hipLaunchKernelGGL((direct_copy<0>), dim3(1), dim3(64), 0, nullptr, in + n - 256, out, 1);
    else if (!strcmp(what, "divergent_collective")) hipLaunchKernelGGL(divergent_collective, dim3(1), dim3(64), 0, nullptr, out);
    else if (!strcmp(what, "lenient_wait")) {
        replay_set_late_loads(1);
        hipLaunchKernelGGL((direct_copy<1>), dim3(1), dim3(64), 0, nullptr, in, out, 0);
        for (int i = 0; i < 64; ++i) if (out[i] != (float)(4 * ((i + 1) % 64))) { printf("stale data at %d\n", i); return 3; }
    }
    printf("not caught\n");
    return 0;
}
