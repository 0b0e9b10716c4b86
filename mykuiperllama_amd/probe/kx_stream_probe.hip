// Measurement only (not part of the drop-in boundary): a kernel that reads given device buffers once with
// plain 16-byte loads and does nothing else, and a kernel that does nothing at all.  bench.py times it over the very tensors of a projection, with
// the same cold rotation and graph replay as the GEMV, and reports the result as the streaming floor of
// that shape on this machine: what the memory system, the dispatcher and a kernel boundary cost when no
// arithmetic, reduction or exchange is in the way.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kLoads = 4;  // 16-byte loads per thread: a workgroup reads 32 KiB, like a GEMV workgroup's tile

struct Segments {
    const u32x4* p[3];
    unsigned long long n16[3];    // 16-byte pieces in each buffer
    unsigned int first_block[4];  // workgroups [first_block[i], first_block[i + 1]) read buffer i
};

__global__ __launch_bounds__(kThreads) void stream_read_kernel(Segments s, uint32_t* sink) {
    int seg = 0;
    if (blockIdx.x >= s.first_block[1]) seg = 1;
    if (blockIdx.x >= s.first_block[2]) seg = 2;
    const u32x4* p = s.p[seg];
    const unsigned long long n16 = s.n16[seg];
    const unsigned long long base =
        static_cast<unsigned long long>(blockIdx.x - s.first_block[seg]) * kThreads * kLoads + threadIdx.x;
    u32x4 v[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
        const unsigned long long at = base + static_cast<unsigned long long>(i) * kThreads;
        v[i] = __builtin_nontemporal_load(p + (at < n16 ? at : n16 - 1));  // clamped: no branch around a load
    }
    uint32_t fold = 0;
#pragma unroll
    for (int i = 0; i < kLoads; i++) fold ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    if (fold == 0x9E3779B9u && sink) sink[0] = fold;  // keeps the loads alive; all but never taken
}

// A launch that does nothing: what the dispatcher and a kernel boundary cost on their own.
__global__ __launch_bounds__(kThreads) void empty_kernel(uint32_t* sink) {
    if (sink && blockIdx.x == 0xffffffffu) sink[0] = threadIdx.x;  // never taken
}

}  // namespace

// Launches `blocks` workgroups of 512 threads that do nothing.  Returns 0 or a hipError_t.
extern "C" int kx_probe_empty_launch(int blocks, void* sink, void* stream) {
    if (blocks < 1) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(empty_kernel, dim3(blocks), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint32_t*>(sink));
    return static_cast<int>(hipGetLastError());
}

// Reads up to three device buffers (16-byte aligned, sizes rounded down to 16 bytes; a null or empty buffer is
// skipped) once on `stream`.  `sink` is one writable device word, or null.  Returns 0 or a hipError_t.
extern "C" int kx_probe_stream_read(const void* a, size_t a_bytes, const void* b, size_t b_bytes, const void* c,
                                    size_t c_bytes, void* sink, void* stream) {
    const void* ptr[3] = {a, b, c};
    const size_t bytes[3] = {a_bytes, b_bytes, c_bytes};
    Segments s{};
    unsigned int blocks = 0;
    for (int i = 0; i < 3; i++) {
        const unsigned long long n16 = ptr[i] ? bytes[i] / 16 : 0;
        if (reinterpret_cast<uintptr_t>(ptr[i]) % 16) return static_cast<int>(hipErrorInvalidValue);
        s.p[i] = static_cast<const u32x4*>(ptr[i]);
        s.n16[i] = n16;
        s.first_block[i] = blocks;
        blocks += static_cast<unsigned int>((n16 + kThreads * kLoads - 1) / (kThreads * kLoads));
    }
    s.first_block[3] = blocks;
    // an empty buffer owns no workgroup; give it a valid pointer anyway so that nothing dereferences null
    for (int i = 0; i < 3; i++) {
        if (s.n16[i] == 0) {
            s.p[i] = s.p[0] ? s.p[0] : (s.p[1] ? s.p[1] : s.p[2]);
            s.n16[i] = 1;
        }
    }
    if (blocks == 0) return 0;
    hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(kThreads), 0, static_cast<hipStream_t>(stream), s,
                       static_cast<uint32_t*>(sink));
    return static_cast<int>(hipGetLastError());
}
