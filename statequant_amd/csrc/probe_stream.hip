// Memory-system probe for the decode step's access pattern: how fast can the codes of one layer step -- 8192 tiles of
// 16 KB, one per (slot, value head), found through a shuffled slot index inside slot blobs of the headline layout
// (583 680 bytes per slot, codes at offset 43 008) -- be read by kernels that do nothing else?  Each variant runs
// over 24 layer buffers back to back, as bench.py steps its 24 layer states.  The figures bound what any step kernel
// can reach on this access pattern; the last line is the shader clock under a streaming load.
//
//     python -m statequant_amd.csrc.build --probes     # writes statequant_amd/probe_stream
//     statequant_amd/probe_stream                      # or: python bench.py --calibrate-stream
//
// Variants (a workgroup of four wavefronts per tile unless noted; every wavefront 4 KB):
//   coalesced           each load instruction of a wavefront covers 1 KB of consecutive addresses
//   coalesced nt        the same with non-temporal loads (what the step kernels use)
//   half lines nt       lane (n, kb) loads 16 bytes of row 16 s + n at chunk kb + 4 j of 128-byte rows: an
//                       instruction covers 16 rows x 64 bytes (the shape a 16x16x64 matrix operand would want)
//   rows of 64 B nt     the same lane order on 64-byte rows: an instruction covers 1 KB of consecutive addresses
//   + N small           N extra one-dword-per-lane loads per wavefront from 64 bytes that the wavefronts of a head
//                       pair share (cache hits: they add load instructions, hardly any bytes)
//   resident 4 / CU     40 KB of LDS per workgroup, as the int8 step kernel has: four workgroups per compute unit
// The last variants read what a KDA step reads of an int4 / group-32 slot (32 heads, 128 x 128, 8 buffer slots of
// which 4 are live; 509 056 bytes per slot, fields in the reference's order): per head 8 KB of codes, 1 KB of scales,
// 2 KB of fp32 decays, 512 B of running decay, 512 B each of buffered keys and values, from seven places of the slot
// -- one wavefront per head as the KDA kernel has it, every load covering consecutive bytes.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <algorithm>
#include <numeric>
#include <random>
#include <vector>

typedef uint32_t v4u __attribute__((ext_vector_type(4)));

constexpr size_t SLOT_BYTES = 583680, CODES_AT = 43008, TILE = 16384;
constexpr int SLOTS = 256, HEADS = 32, LAYERS = 24, TILES = SLOTS * HEADS;

struct Args {
    const uint8_t* base;
    const int* idx;
    uint32_t* sink;
    int per_xcd;
};

__device__ __forceinline__ const uint8_t* slot_ptr(const Args& a, int wg, int& h) {
    const int tile = (wg & 7) * a.per_xcd + (wg >> 3);       // every XCD walks a contiguous range of tiles
    h = tile & (HEADS - 1);
    return a.base + size_t(a.idx[tile / HEADS]) * SLOT_BYTES;
}

template <bool NT>
__device__ __forceinline__ v4u ld(const uint8_t* p) {
    const v4u* q = reinterpret_cast<const v4u*>(p);
    return NT ? __builtin_nontemporal_load(q) : *q;
}

// SHAPE 0: coalesced; 1: half lines of 128-byte rows; 2: rows of 64 bytes in the same lane order.
// SMALL: extra one-dword loads per wavefront from 64 bytes shared by a head pair.
template <bool NT, int SHAPE, int SMALL>
__global__ __launch_bounds__(256) void probe(Args a) {
    int h;
    const uint8_t* slot = slot_ptr(a, blockIdx.x, h);
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63, n = lane & 15, kb = lane >> 4;
    const uint8_t* mine = slot + CODES_AT + size_t(h) * TILE + w * 4096;
    uint32_t sm[SMALL > 0 ? SMALL : 1] = {0};
#pragma unroll
    for (int j = 0; j < SMALL; ++j) {
        const uint8_t* p = slot + (j * 256 + (h / 2) * 64) % 40960 + n * 4;
        sm[j] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
    }
    v4u x[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if constexpr (SHAPE == 0) x[j] = ld<NT>(mine + j * 1024 + lane * 16);
        else if constexpr (SHAPE == 1) x[j] = ld<NT>(mine + (16 * (j >> 1) + n) * 128 + 16 * (kb + 4 * (j & 1)));
        else x[j] = ld<NT>(mine + (16 * j + n) * 64 + 16 * kb);
    }
    uint32_t acc = 0;
#pragma unroll
    for (int j = 0; j < SMALL; ++j) acc ^= sm[j];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc ^= x[j].x ^ x[j].y ^ x[j].z ^ x[j].w;
    if (acc == 0x12345678u) a.sink[blockIdx.x] = acc;        // never true for the buffer's contents: keeps the loads
}

// KDA: offsets of the fields inside a slot, bytes per head of each
constexpr size_t KDA_SLOT = 509056, KDA_GB = 0, KDA_GCUR = 131072, KDA_SC = 147584, KDA_S = 181376, KDA_KB = 443520,
                 KDA_UB = 476288;
constexpr int KDA_LIVE = 4;
constexpr double KDA_BYTES = 8192 + 1024 + KDA_LIVE * 512 + 512 + KDA_LIVE * 128 + KDA_LIVE * 128;
template <bool WIDE>
__global__ __launch_bounds__(64) void probe_kda(Args a) {
    const int wg = blockIdx.x;
    const int tile = (wg & 7) * a.per_xcd + (wg >> 3);
    const int h = tile & (HEADS - 1), lane = threadIdx.x;
    const uint8_t* slot = a.base + size_t(a.idx[tile / HEADS]) * KDA_SLOT;
    uint32_t acc = 0;
    auto eat = [&](const v4u& x) { acc ^= x.x ^ x.y ^ x.z ^ x.w; };
    const uint8_t* codes = slot + KDA_S + size_t(h) * 8192;
    if constexpr (WIDE) {                                    // 1 KB per load
#pragma unroll
        for (int j = 0; j < 8; ++j) eat(ld<true>(codes + j * 1024 + lane * 16));
    } else {                                                 // 512 B per load, as the kernel's row-shaped loads
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            typedef uint32_t v2 __attribute__((ext_vector_type(2)));
            const v2 x = __builtin_nontemporal_load(reinterpret_cast<const v2*>(codes + j * 512 + lane * 8));
            acc ^= x.x ^ x.y;
        }
    }
    eat(ld<true>(slot + KDA_SC + size_t(h) * 1024 + lane * 16));
#pragma unroll
    for (int j = 0; j < KDA_LIVE / 2; ++j) eat(ld<false>(slot + KDA_GB + size_t(h) * 4096 + j * 1024 + lane * 16));
    eat(ld<false>(slot + KDA_GCUR + size_t(h) * 512 + (lane & 31) * 16));
    eat(ld<false>(slot + KDA_KB + size_t(h) * 1024 + (lane & 31) * 16));
    eat(ld<false>(slot + KDA_UB + size_t(h) * 1024 + (lane & 31) * 16));
    if (acc == 0x12345678u) a.sink[blockIdx.x] = acc;
}

// shader clock: the core clock counter against the 100 MHz real-time counter over a streaming read
__global__ __launch_bounds__(256) void clock_probe(const v4u* src, uint64_t* out, uint32_t* sink, int iters) {
    const uint64_t c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    uint32_t acc = 0;
    const v4u* p = src + size_t(blockIdx.x) * 256 * iters + threadIdx.x;
    for (int i = 0; i < iters; ++i) {
        const v4u v = __builtin_nontemporal_load(p + i * 256);
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    const uint64_t c1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    if (threadIdx.x == 0) {
        out[2 * blockIdx.x] = c1 - c0;
        out[2 * blockIdx.x + 1] = r1 - r0;
    }
    if (acc == 0x12345678u) sink[0] = acc;
}

#define CHECK(x)                                                                     \
    do {                                                                             \
        hipError_t e_ = (x);                                                         \
        if (e_ != hipSuccess) {                                                      \
            printf("%s: %s\n", #x, hipGetErrorString(e_));                           \
            return 1;                                                                \
        }                                                                            \
    } while (0)

struct Variant {
    const char* name;
    void (*kernel)(Args);
    int lds;
};

int main() {
    static_assert(KDA_SLOT <= SLOT_BYTES, "the KDA variants reuse the buffer: slot pitch of the larger layout");
    const size_t per_layer = size_t(SLOTS + 1) * SLOT_BYTES;
    uint8_t* buf;
    uint32_t* sink;
    int* idx;
    CHECK(hipMalloc(&buf, per_layer * LAYERS));
    CHECK(hipMalloc(&sink, TILES * 4));
    CHECK(hipMalloc(&idx, SLOTS * 4));
    CHECK(hipMemset(buf, 1, per_layer * LAYERS));
    std::vector<int> perm(SLOTS);
    std::iota(perm.begin(), perm.end(), 1);
    std::mt19937 g(0);
    std::shuffle(perm.begin(), perm.end(), g);
    CHECK(hipMemcpy(idx, perm.data(), SLOTS * 4, hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    const Variant vs[] = {
        {"coalesced", probe<false, 0, 0>, 0},
        {"coalesced nt", probe<true, 0, 0>, 0},
        {"coalesced nt, resident 4 / CU", probe<true, 0, 0>, 40960},
        {"half lines nt", probe<true, 1, 0>, 0},
        {"rows of 64 B nt", probe<true, 2, 0>, 0},
        {"coalesced nt + 8 small", probe<true, 0, 8>, 0},
        {"coalesced nt + 16 small", probe<true, 0, 16>, 0},
    };
    const double code_bytes = double(TILES) * TILE;
    for (const Variant& v : vs) {
        CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(v.kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
        auto launch = [&](int layer) {
            Args a{buf + layer * per_layer, idx, sink, TILES / 8};
            hipLaunchKernelGGL(v.kernel, dim3(TILES), dim3(256), v.lds, 0, a);
        };
        for (int r = 0; r < 2; ++r)
            for (int layer = 0; layer < LAYERS; ++layer) launch(layer);
        CHECK(hipDeviceSynchronize());
        const int reps = 10;
        CHECK(hipEventRecord(e0));
        for (int r = 0; r < reps; ++r)
            for (int layer = 0; layer < LAYERS; ++layer) launch(layer);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        const double us = ms * 1e3 / (reps * LAYERS);
        printf("%-34s %7.2f us per launch  %7.1f GB/s\n", v.name, us, code_bytes / us * 1e-3);
        fflush(stdout);
    }
    for (int wide = 0; wide < 2; ++wide) {
        auto launch = [&](int layer) {
            Args a{buf + layer * per_layer, idx, sink, TILES / 8};
            if (wide) hipLaunchKernelGGL(probe_kda<true>, dim3(TILES), dim3(64), 0, 0, a);
            else hipLaunchKernelGGL(probe_kda<false>, dim3(TILES), dim3(64), 0, 0, a);
        };
        for (int r = 0; r < 2; ++r)
            for (int layer = 0; layer < LAYERS; ++layer) launch(layer);
        CHECK(hipDeviceSynchronize());
        const int reps = 10;
        CHECK(hipEventRecord(e0));
        for (int r = 0; r < reps; ++r)
            for (int layer = 0; layer < LAYERS; ++layer) launch(layer);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        const double us = ms * 1e3 / (reps * LAYERS);
        printf("%-34s %7.2f us per launch  %7.1f GB/s\n", wide ? "kda fields, 1 KB code loads" : "kda fields, 512 B code loads", us,
               KDA_BYTES * TILES / us * 1e-3);
        fflush(stdout);
    }
    {
        const int blocks = 8192, iters = 64;                 // 2 GiB
        uint64_t* out;
        CHECK(hipMalloc(&out, blocks * 16));
        for (int r = 0; r < 3; ++r)
            hipLaunchKernelGGL(clock_probe, dim3(blocks), dim3(256), 0, 0, reinterpret_cast<const v4u*>(buf), out, sink, iters);
        CHECK(hipDeviceSynchronize());
        std::vector<uint64_t> h(2 * blocks);
        CHECK(hipMemcpy(h.data(), out, blocks * 16, hipMemcpyDeviceToHost));
        double c = 0, r = 0;
        for (int b = 0; b < blocks; ++b) {
            c += double(h[2 * b]);
            r += double(h[2 * b + 1]);
        }
        printf("%-34s %7.0f MHz\n", "shader clock under streaming load", c / r * 100.0);
    }
    return 0;
}
