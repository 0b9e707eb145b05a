// What the single-pass transposed normalisation (f16 [8192 rows x 4096 cols], input with the rows
// contiguous and a column pitch of 8192 elements, output row-major) can hope for: the time of its
// LOAD phase and of its STORE phase alone, for the ways a compute unit's 256 KB register tile can be
// cut. Every kernel moves exactly what the real kernel moves (16 vectors of 16 bytes per thread,
// 1024 threads, 256 workgroups = one per compute unit) and nothing else, so the figures are ceilings
// for the corresponding arrangement. The numbers explain the planner's choices in layout.cpp
// (plan_normalize, transposed plans) and are summarised under profiles/.
//
//   build: python -m hpt_amd.build          (hipcc --offload-arch=gfx950)
//   run:   hpt_amd/lib/transposed_access_patterns
#include <hip/hip_runtime.h>

#include <cstdio>
#include <vector>

#define CK(x)                                                                      \
    do {                                                                           \
        hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                    \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);  \
            return 1;                                                              \
        }                                                                          \
    } while (0)

typedef uint32_t u4 __attribute__((ext_vector_type(4)));
constexpr int R = 8192, C = 4096;

// LOAD variants. Every thread loads 16 vectors, then folds them into one word nobody reads.
//   1  32 rows x 4096 cols per workgroup: 64-byte segments (4 lanes along the rows); the two workgroups
//      that share every 128-byte line run on the same XCD (transposed_tile_kernel's arrangement)
//   5  the same without the pairing (the partner runs on another XCD)
//   4  the same, but only every second row block exists: half the bytes, nobody reads the other half lines
//   2  64 rows x 2048 cols per workgroup: whole 128-byte lines (8 lanes along the rows)
//   3  64 rows x 2048 cols per workgroup, read as two passes of 64-byte segments
template <int LV> __global__ void __launch_bounds__(1024) load_phase(const _Float16* __restrict__ in, uint32_t* __restrict__ sink) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    u4 v[16];
    if (LV == 1 || LV == 4 || LV == 5) {
        const int rg = lane & 3, cgl = lane >> 2;
        int b = blockIdx.x;
        if (LV == 1) {
            const int x = b & 7, q = b >> 3;
            b = ((x + 8 * (q >> 1)) << 1) | (q & 1);
        }
        if (LV == 4) b *= 2;
        const int r0 = (b * 4 + rg) * 8, cb = w * 256 + cgl * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 8; ++i) v[h * 8 + i] = *(const u4*)(in + (size_t)(cb + h * 128 + i) * R + r0);
    } else if (LV == 2) {
        const int rg = lane & 7, cgl = lane >> 3;
        const int b = blockIdx.x >> 1, half = blockIdx.x & 1;
        const int r0 = (b * 8 + rg) * 8, cb = half * 2048 + w * 128 + cgl * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 8; ++i) v[h * 8 + i] = *(const u4*)(in + (size_t)(cb + h * 64 + i) * R + r0);
    } else {
        const int rg = lane & 3, cgl = lane >> 2;
        const int b = blockIdx.x >> 1, half = blockIdx.x & 1;
        const int cb = half * 2048 + w * 128 + cgl * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int r0 = (b * 8 + h * 4 + rg) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) v[h * 8 + i] = *(const u4*)(in + (size_t)(cb + i) * R + r0);
        }
    }
    u4 a = v[0];
#pragma unroll
    for (int j = 1; j < 16; ++j) a ^= v[j];
    if ((a.x ^ a.y ^ a.z ^ a.w) == 0x12345u) sink[threadIdx.x] = a.x;  // (never: the inputs are zero)
}

// STORE variants: every thread stores 16 vectors of the [R][C] output.
//   1  4 rows x 256 bytes per instruction (the register-tile transpose with 4 lanes along the rows)
//   2  8 rows x 128 bytes per instruction (the same with 8 lanes along the rows)
//   3  1 row x 1 KiB per instruction, non-temporal (what a transposition through LDS gives)
//   4  1 row x 1 KiB per instruction, plain stores
//   9  nothing: the cost of a launch
template <int SV> __global__ void __launch_bounds__(1024) store_phase(_Float16* __restrict__ out) {
    if (SV == 9) return;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const u4 val = {(uint32_t)lane, (uint32_t)w, 0u, 1u};
    if (SV == 1) {
        const int rg = lane & 3, cgl = lane >> 2;
        const int r0 = (blockIdx.x * 4 + rg) * 8, cb = w * 256 + cgl * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int k = 0; k < 8; ++k) __builtin_nontemporal_store(val, (u4*)(out + (size_t)(r0 + k) * C + cb + h * 128));
    } else if (SV == 2) {
        const int rg = lane & 7, cgl = lane >> 3;
        const int b = blockIdx.x >> 1, half = blockIdx.x & 1;
        const int r0 = (b * 8 + rg) * 8, cb = half * 2048 + w * 128 + cgl * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int k = 0; k < 8; ++k) __builtin_nontemporal_store(val, (u4*)(out + (size_t)(r0 + k) * C + cb + h * 64));
    } else {
        // a workgroup owns 32 rows x 8 KiB; wave w writes rows 2w and 2w + 1: 16 instructions of 1 KiB
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            u4* p = (u4*)(out + (size_t)(blockIdx.x * 32 + 2 * w + (j >> 3)) * C + (j & 7) * 512 + lane * 8);
            if (SV == 3) __builtin_nontemporal_store(val, p);
            else *p = val;
        }
    }
}

int main() {
    const size_t bytes = (size_t)R * C * 2;
    const int NBUF = 6;  // 768 MB in rotation: nothing is served from the 256 MB Infinity Cache
    std::vector<_Float16*> in(NBUF), out(NBUF);
    for (int i = 0; i < NBUF; ++i) {
        CK(hipMalloc(&in[i], bytes));
        CK(hipMemset(in[i], 0, bytes));
        CK(hipMalloc(&out[i], bytes));
    }
    uint32_t* sink;
    CK(hipMalloc(&sink, 1 << 16));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    auto run = [&](const char* name, double moved, auto launch) {
        for (int i = 0; i < 5; ++i) launch(i % NBUF);
        (void)hipDeviceSynchronize();
        (void)hipEventRecord(e0);
        const int N = 100;
        for (int i = 0; i < N; ++i) launch(i % NBUF);
        (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        printf("%-52s %8.2f us  %8.1f GB/s\n", name, ms * 1e3 / N, moved * N / (ms * 1e-3) / 1e9);
        fflush(stdout);
    };
    run("launch only", 0, [&](int) { store_phase<9><<<dim3(1), dim3(64)>>>(nullptr); });
    run("load 1: 64 B segments, line partners on one XCD", bytes, [&](int k) { load_phase<1><<<dim3(256), dim3(1024)>>>(in[k], sink); });
    run("load 5: 64 B segments, partners on different XCDs", bytes, [&](int k) { load_phase<5><<<dim3(256), dim3(1024)>>>(in[k], sink); });
    run("load 4: 64 B segments, half the row blocks only", bytes / 2, [&](int k) { load_phase<4><<<dim3(128), dim3(1024)>>>(in[k], sink); });
    run("load 2: whole 128 B lines, 64 rows x 2048 cols", bytes, [&](int k) { load_phase<2><<<dim3(256), dim3(1024)>>>(in[k], sink); });
    run("load 3: 64 B segments twice, 64 rows x 2048 cols", bytes, [&](int k) { load_phase<3><<<dim3(256), dim3(1024)>>>(in[k], sink); });
    run("store 1: 4 rows x 256 B per instruction", bytes, [&](int k) { store_phase<1><<<dim3(256), dim3(1024)>>>(out[k]); });
    run("store 2: 8 rows x 128 B per instruction", bytes, [&](int k) { store_phase<2><<<dim3(256), dim3(1024)>>>(out[k]); });
    run("store 3: 1 row x 1 KiB per instruction, non-temporal", bytes, [&](int k) { store_phase<3><<<dim3(256), dim3(1024)>>>(out[k]); });
    run("store 4: 1 row x 1 KiB per instruction, plain", bytes, [&](int k) { store_phase<4><<<dim3(256), dim3(1024)>>>(out[k]); });
    return 0;
}
