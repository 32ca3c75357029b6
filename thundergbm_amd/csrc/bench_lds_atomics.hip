// Microbenchmark of LDS atomic throughput on gfx950: float vs 32/64-bit integer adds, random vs
// conflict-free vs same-address, 256/512/1024-thread groups. It is the measurement behind the
// fixed-point histogram of tree_kernels.hip; built as bin/bench_lds_atomics, not linked into the library.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); return 1; } } while (0)
constexpr int NBINS = 14336;  // floats (56 KB)
constexpr int ITERS = 2048;

template <int MODE>
__global__ __launch_bounds__(1024) void k(float *out, int iters) {
    extern __shared__ float lds[];
    for (int i = threadIdx.x; i < NBINS; i += blockDim.x) lds[i] = 0.f;
    __syncthreads();
    unsigned s = (blockIdx.x * blockDim.x + threadIdx.x) * 2654435761u + 12345u;
    unsigned lane = threadIdx.x & 63;
    float v = 1.0f + lane * 1e-3f;
    for (int it = 0; it < iters; ++it) {
        s = s * 1664525u + 1013904223u;
        unsigned r = (s >> 8) % NBINS;
        if (MODE == 0) unsafeAtomicAdd(&lds[r], v);                              // float, random
        if (MODE == 1) atomicAdd((unsigned *)&lds[r], 1u);                       // uint, random
        if (MODE == 2) unsafeAtomicAdd(&lds[(it * 64 + lane) % NBINS], v);       // float, conflict free
        if (MODE == 3) atomicAdd((unsigned *)&lds[(it * 64 + lane) % NBINS], 1u);// uint, conflict free
        if (MODE == 4) unsafeAtomicAdd(&lds[it % NBINS], v);                     // float, same address
        if (MODE == 5) { float o = atomicAdd(&lds[r], v); v += o * 1e-30f; }     // float with return
        if (MODE == 6) atomicAdd((unsigned long long *)&lds[(r & ~1u)], 1ull);   // u64 random
        if (MODE == 7) lds[r] = v;                                               // plain store random
        if (MODE == 8) v += lds[r];                                              // plain load random
        if (MODE == 9) { lds[r] += v; }                                          // non-atomic rmw random
        if (MODE == 10) unsafeAtomicAdd(&lds[(r & ~31u) | (lane & 31)], v);      // float, random rows, bank = lane%32 (2-way)
        if (MODE == 11) atomicAdd((int *)&lds[r], 3);                            // int add random
        if (MODE == 12) atomicAdd((unsigned long long *)&lds[((it * 64 + lane) * 2) % NBINS], 1ull);  // u64 conflict free
    }
    __syncthreads();
    float acc = v;
    for (int i = threadIdx.x; i < NBINS; i += blockDim.x) acc += lds[i];
    if (acc == 123.456f) out[0] = acc;
}

// The histogram kernel's own instruction mix: every lane holds one dword of four bin bytes per step (eight
// lanes = one row of 28+4 features, 256 bins of 8 bytes per feature) and issues four 64-bit adds; the bytes
// are refreshed with one rotate-and-add per dword, so address arithmetic stays at the kernel's two to three
// vector instructions per add. CHECK adds the kernel's "bin != missing" test (compare + exec mask) per add.
template <bool CHECK, int WIDTH>
__global__ __launch_bounds__(1024) void k_mix(float *out, int iters) {
    extern __shared__ float lds[];
    unsigned long long *h = reinterpret_cast<unsigned long long *>(lds);
    for (int i = threadIdx.x; i < NBINS; i += blockDim.x) lds[i] = 0.f;
    __syncthreads();
    unsigned w = (blockIdx.x * blockDim.x + threadIdx.x) * 2654435761u + 12345u;
    w ^= w >> 15; w *= 2246822519u; w ^= w >> 13;
    const unsigned q = threadIdx.x & 7;
    const unsigned o0 = (q * 4 + 0) % 28 * 256, o1 = (q * 4 + 1) % 28 * 256, o2 = (q * 4 + 2) % 28 * 256,
                   o3 = (q * 4 + 3) % 28 * 256;
    const unsigned long long add = ((unsigned long long)(threadIdx.x + 1) << 32) + 3u;
    for (int it = 0; it < iters; ++it) {
        w = ((w >> 8) | (w << 24)) + 0x9e3779b9u;
        const unsigned b0 = w & 0xff, b1 = (w >> 8) & 0xff, b2 = (w >> 16) & 0xff, b3 = w >> 24;
        if (WIDTH == 8) {
            if (!CHECK || b0 != 255u) atomicAdd(h + o0 + b0, add);
            if (!CHECK || b1 != 255u) atomicAdd(h + o1 + b1, add);
            if (!CHECK || b2 != 255u) atomicAdd(h + o2 + b2, add);
            if (!CHECK || b3 != 255u) atomicAdd(h + o3 + b3, add);
        } else {
            unsigned *h32 = reinterpret_cast<unsigned *>(lds);
            if (!CHECK || b0 != 255u) atomicAdd(h32 + o0 + b0, (unsigned)add);
            if (!CHECK || b1 != 255u) atomicAdd(h32 + o1 + b1, (unsigned)add);
            if (!CHECK || b2 != 255u) atomicAdd(h32 + o2 + b2, (unsigned)add);
            if (!CHECK || b3 != 255u) atomicAdd(h32 + o3 + b3, (unsigned)add);
        }
    }
    __syncthreads();
    float acc = 0;
    for (int i = threadIdx.x; i < NBINS; i += blockDim.x) acc += lds[i];
    if (acc == 123.456f) out[0] = acc;
}

// The same work with the histogram interleaved by feature (slot = bin * 32 + feature, so a feature owns one
// pair of banks) and the four features of a lane taken in an order rotated by the row's position in the
// wavefront: every instruction then touches each of the 32 features from exactly two lanes.
__global__ __launch_bounds__(1024) void k_mix_rotated(float *out, int iters) {
    extern __shared__ float lds[];
    unsigned long long *h = reinterpret_cast<unsigned long long *>(lds);
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) lds[i] = 0.f;
    __syncthreads();
    unsigned w = (blockIdx.x * blockDim.x + threadIdx.x) * 2654435761u + 12345u;
    w ^= w >> 15; w *= 2246822519u; w ^= w >> 13;
    const unsigned q = threadIdx.x & 7, r = (threadIdx.x >> 3) & 7;
    const unsigned k0 = r & 3, k1 = (r + 1) & 3, k2 = (r + 2) & 3, k3 = (r + 3) & 3;
    const unsigned f0 = q * 4 + k0, f1 = q * 4 + k1, f2 = q * 4 + k2, f3 = q * 4 + k3;
    const unsigned s0 = k0 * 8, s1 = k1 * 8, s2 = k2 * 8, s3 = k3 * 8;
    const unsigned long long add = ((unsigned long long)(threadIdx.x + 1) << 32) + 3u;
    for (int it = 0; it < iters; ++it) {
        w = ((w >> 8) | (w << 24)) + 0x9e3779b9u;
        atomicAdd(h + ((w >> s0) & 0xff) * 32 + f0, add);
        atomicAdd(h + ((w >> s1) & 0xff) * 32 + f1, add);
        atomicAdd(h + ((w >> s2) & 0xff) * 32 + f2, add);
        atomicAdd(h + ((w >> s3) & 0xff) * 32 + f3, add);
    }
    __syncthreads();
    float acc = 0;
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) acc += lds[i];
    if (acc == 123.456f) out[0] = acc;
}

int run_mix_rotated(const char *name, float *d_out) {
    hipEvent_t a, b;
    CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
    const int grid = 512, block = 1024, iters = ITERS / 4;
    k_mix_rotated<<<grid, block, 65536>>>(d_out, 16);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(a));
    k_mix_rotated<<<grid, block, 65536>>>(d_out, iters);
    CK(hipEventRecord(b));
    CK(hipEventSynchronize(b));
    float ms; CK(hipEventElapsedTime(&ms, a, b));
    double ops = (double)grid * block * iters * 4;
    printf("%-40s %8.3f ms  %8.1f G lane-ops/s  %.2f lane-ops/clk/CU (2.4GHz, 256 CU)\n", name, ms, ops / ms / 1e6,
           ops / (ms * 1e-3) / 256 / 2.4e9);
    return 0;
}

template <bool CHECK, int WIDTH>
int run_mix(const char *name, float *d_out) {
    hipEvent_t a, b;
    CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
    const int grid = 512, block = 1024, iters = ITERS / 4;
    k_mix<CHECK, WIDTH><<<grid, block, NBINS * 4>>>(d_out, 16);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(a));
    k_mix<CHECK, WIDTH><<<grid, block, NBINS * 4>>>(d_out, iters);
    CK(hipEventRecord(b));
    CK(hipEventSynchronize(b));
    float ms; CK(hipEventElapsedTime(&ms, a, b));
    double ops = (double)grid * block * iters * 4;
    printf("%-40s %8.3f ms  %8.1f G lane-ops/s  %.2f lane-ops/clk/CU (2.4GHz, 256 CU)\n", name, ms, ops / ms / 1e6,
           ops / (ms * 1e-3) / 256 / 2.4e9);
    return 0;
}

template <int MODE>
int run(const char *name, float *d_out, int block = 256) {
    hipEvent_t a, b;
    CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
    const int grid = 2048 * 256 / block;
    k<MODE><<<grid, block, NBINS * 4>>>(d_out, 16);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(a));
    k<MODE><<<grid, block, NBINS * 4>>>(d_out, ITERS);
    CK(hipEventRecord(b));
    CK(hipEventSynchronize(b));
    float ms; CK(hipEventElapsedTime(&ms, a, b));
    double ops = (double)grid * block * ITERS;
    printf("%-40s %8.3f ms  %8.1f G lane-ops/s  %.2f lane-ops/clk/CU (2.4GHz, 256 CU)\n", name, ms, ops / ms / 1e6,
           ops / (ms * 1e-3) / 256 / 2.4e9);
    return 0;
}

int main() {
    float *d; CK(hipMalloc(&d, 64));
    run<0>("float add, random", d);
    run<1>("uint add, random", d);
    run<2>("float add, conflict free", d);
    run<3>("uint add, conflict free", d);
    run<4>("float add, same address", d);
    run<5>("float add rtn, random", d);
    run<6>("u64 add, random", d);
    run<7>("plain store, random", d);
    run<8>("plain load, random", d);
    run<9>("non-atomic rmw, random", d);
    run<10>("float add, 2-way bank", d);
    run<11>("int add, random", d);
    run<12>("u64 add, conflict free", d);
    run<6>("u64 add, random, block 512", d, 512);
    run<6>("u64 add, random, block 1024", d, 1024);
    run<12>("u64 add, conflict free, block 1024", d, 1024);
    run<1>("uint add, random, block 1024", d, 1024);
    run<0>("float add, random, block 1024", d, 1024);
    run_mix<true, 8>("histogram mix, u64, missing check", d);
    run_mix<false, 8>("histogram mix, u64, no check", d);
    run_mix<true, 4>("histogram mix, u32, missing check", d);
    run_mix<false, 4>("histogram mix, u32, no check", d);
    run_mix_rotated("histogram mix, u64, one bank pair per feature", d);
    return 0;
}
