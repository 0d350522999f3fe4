// Measurement probes for bench.py --ceiling: what this GPU does with a plain stream and with the primitives a
// single-launch backward would need.  Built into libthnprobe.so, a library of its own: nothing here is part of the
// operator ABI (include/thnorm.h) and no operator calls it.  gfx950 only.
//
//   thnp_empty         an empty kernel: what one launch costs, from launch to launch
//   thnp_copy          the row loop of the norm kernels with the arithmetic taken out: 256 workgroups of 256 threads,
//                      four 16-byte vectors per thread and step, the next step requested before the current one is
//                      stored, streaming loads and stores; optionally the time at which every workgroup started, had
//                      its first vectors, left its loop and had its last store acknowledged (100 MHz device clock)
//   thnp_atomic_burst  every workgroup adds to ONE counter with device-scope atomics, n times: the rate at which one
//                      address takes them (a ticket counter for dynamic row assignment, or the arrival counter of a
//                      grid-wide second stage, is such an address)
//   thnp_atomic_chain  one lane, n dependent device-scope atomics: the round trip of one
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

__global__ void empty_kernel() {}

constexpr int kBlock = 256, kVecs = 4;

__global__ void __launch_bounds__(kBlock) copy_kernel(const char* __restrict__ src, char* __restrict__ dst, int64_t nvec,
                                                      uint64_t* ts) {
    uint64_t t0 = 0;
    if (ts) t0 = wall_clock64();
    const int64_t step = static_cast<int64_t>(gridDim.x) * kBlock * kVecs;
    int64_t base = static_cast<int64_t>(blockIdx.x) * kBlock * kVecs + threadIdx.x;
    const int64_t last = nvec - 1;
    u32x4 cur[kVecs], nxt[kVecs];
#pragma unroll
    for (int k = 0; k < kVecs; ++k) {
        const int64_t v = base + k * kBlock;
        cur[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + (v < last ? v : last) * 16));
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
    uint64_t t1 = 0;
    if (ts) t1 = wall_clock64();
    for (; base < nvec; base += step) {
        const int64_t nb = base + step;
#pragma unroll
        for (int k = 0; k < kVecs; ++k) {
            const int64_t v = nb + k * kBlock;
            nxt[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + (v < last ? v : last) * 16));
        }
#pragma unroll
        for (int k = 0; k < kVecs; ++k) {
            const int64_t v = base + k * kBlock;
            __builtin_nontemporal_store(cur[k], reinterpret_cast<u32x4*>(dst + (v < last ? v : last) * 16));
        }
#pragma unroll
        for (int k = 0; k < kVecs; ++k) cur[k] = nxt[k];
    }
    if (ts) {
        const uint64_t t2 = wall_clock64();
        __builtin_amdgcn_s_waitcnt(0x0F70);
        const uint64_t t3 = wall_clock64();
        if (threadIdx.x == 0) {
            ts[blockIdx.x * 4 + 0] = t0;
            ts[blockIdx.x * 4 + 1] = t1;
            ts[blockIdx.x * 4 + 2] = t2;
            ts[blockIdx.x * 4 + 3] = t3;
        }
    }
}

__global__ void atomic_burst_kernel(uint32_t* counter, int n) {
    if (threadIdx.x == 0) {
        for (int i = 0; i < n; ++i) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// counter[0], counter[1]: which of the two the next atomic goes to depends on the value the previous one returned
__global__ void atomic_chain_kernel(uint32_t* counter, uint64_t* ticks, int n) {
    const uint64_t t0 = wall_clock64();
    uint32_t v = 0;
    for (int i = 0; i < n; ++i) v = __hip_atomic_fetch_add(counter + (v & 1u), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t t1 = wall_clock64();
    ticks[0] = t1 - t0;
    ticks[1] = v;
}

int launched() { return hipGetLastError() == hipSuccess ? 0 : -1; }

}  // namespace

extern "C" {

int thnp_empty(int blocks, int threads, void* stream) {
    hipLaunchKernelGGL(empty_kernel, dim3(blocks), dim3(threads), 0, static_cast<hipStream_t>(stream));
    return launched();
}

// bytes: a multiple of 16, at least 16; ts: NULL or 4 * 256 uint64 in device memory
int thnp_copy(const void* src, void* dst, int64_t bytes, uint64_t* ts, void* stream) {
    if (bytes < 16 || bytes % 16 != 0 || src == nullptr || dst == nullptr) return -2;
    hipLaunchKernelGGL(copy_kernel, dim3(256), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                       static_cast<const char*>(src), static_cast<char*>(dst), bytes / 16, ts);
    return launched();
}

int thnp_atomic_burst(uint32_t* counter, int per_workgroup, void* stream) {
    if (counter == nullptr || per_workgroup < 0) return -2;
    hipLaunchKernelGGL(atomic_burst_kernel, dim3(256), dim3(64), 0, static_cast<hipStream_t>(stream), counter, per_workgroup);
    return launched();
}

int thnp_atomic_chain(uint32_t* counter, uint64_t* ticks, int n, void* stream) {
    if (counter == nullptr || ticks == nullptr || n < 0) return -2;
    hipLaunchKernelGGL(atomic_chain_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), counter, ticks, n);
    return launched();
}

int thnp_wall_clock_khz(void) {
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return -1;
    return khz;
}

}  // extern "C"
