// Microbenchmark: how fast does one MI355X fetch isolated cache lines at random addresses?
//
// The pull and push kernels of the sparse table read one 64-byte bucket and one 64..128-byte row per
// cold key, each in a 128-byte line of its own somewhere in tens of GB. This program measures the
// ceiling of exactly that access pattern, apart from any table logic: `lines` random line addresses
// in a buffer of `gib` GiB, `bytes` (16..128) consecutive bytes read from each line by bytes/16
// neighbouring lanes with one 16-byte load each, `depth` independent loads in flight per lane, all
// compute units busy. It prints fetched lines per second and the useful bytes per second, next to a
// plain streaming read of the same buffer.
//
//   line_gather_bench [gib=16] [lines=4194304]
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                                          \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            std::fprintf(stderr, "%s:%d %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            std::exit(1);                                                                 \
        }                                                                                 \
    } while (0)

namespace {

__device__ __forceinline__ uint64_t mix(uint64_t x) {  // MurmurHash3's 64-bit finaliser
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdull;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ull;
    x ^= x >> 33;
    return x;
}

// Lane group of LPL lanes (LPL * 16 bytes of a line) takes DEPTH lines per round.
template <int LPL, int DEPTH>
__global__ __launch_bounds__(256) void gather_kernel(const uint4* __restrict__ buf, uint64_t n_lines_in_buf,
                                                      uint32_t lines, uint32_t seed, uint32_t* __restrict__ sink) {
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t nthreads = gridDim.x * blockDim.x;
    const uint32_t grp = tid / LPL, sub = tid % LPL, ngrp = nthreads / LPL;
    uint32_t acc = 0;
    for (uint32_t i0 = grp; i0 < lines; i0 += ngrp * DEPTH) {
        uint4 v[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const uint32_t i = i0 + d * ngrp;
            const uint64_t line = mix(((uint64_t)seed << 32) | (i < lines ? i : 0u)) % n_lines_in_buf;
            v[d] = buf[line * 8 + sub];  // a 128-byte line holds eight 16-byte units
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) acc += v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
    }
    if (acc == 0x12345678u) sink[0] = acc;  // keeps the loads alive, practically never taken
}

__global__ __launch_bounds__(256) void stream_kernel(const uint4* __restrict__ buf, uint64_t units,
                                                      uint32_t* __restrict__ sink) {
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t nthreads = (uint64_t)gridDim.x * blockDim.x;
    uint32_t acc = 0;
    for (uint64_t i = tid; i < units; i += 4 * nthreads) {
        uint4 v[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) v[d] = buf[i + d * nthreads < units ? i + d * nthreads : i];
#pragma unroll
        for (int d = 0; d < 4; ++d) acc += v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
    }
    if (acc == 0x12345678u) sink[0] = acc;
}

template <int LPL, int DEPTH>
void run(const uint4* buf, uint64_t n_lines, uint32_t lines, uint32_t* sink, int blocks) {
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    float best = 1e30f;
    for (int rep = 0; rep < 6; ++rep) {  // a new set of lines every time: nothing is cached from the last
        CHECK(hipEventRecord(a, 0));
        gather_kernel<LPL, DEPTH><<<blocks, 256>>>(buf, n_lines, lines, 100u + rep, sink);
        CHECK(hipEventRecord(b, 0));
        CHECK(hipEventSynchronize(b));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, a, b));
        if (rep && ms < best) best = ms;
    }
    std::printf("bytes/line %3d  loads in flight/lane %d  blocks %5d : %8.2f us  %6.2f G lines/s  %7.1f GB/s useful  %7.1f GB/s of 128-byte lines\n",
                LPL * 16, DEPTH, blocks, best * 1e3, lines / (best * 1e6), (double)lines * LPL * 16 / (best * 1e6),
                (double)lines * 128 / (best * 1e6));
}

}  // namespace

int main(int argc, char** argv) {
    const uint64_t gib = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 16;
    const uint32_t lines = argc > 2 ? (uint32_t)std::strtoul(argv[2], nullptr, 10) : (1u << 22);
    const uint64_t bytes = gib << 30, n_lines = bytes / 128;
    uint4* buf = nullptr;
    uint32_t* sink = nullptr;
    CHECK(hipMalloc(&buf, bytes));
    CHECK(hipMalloc(&sink, 4));
    CHECK(hipMemset(buf, 1, bytes));
    CHECK(hipDeviceSynchronize());
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    std::printf("%s, %d compute units; buffer %llu GiB, %u random lines per launch (best of 5)\n", prop.name, cus,
                (unsigned long long)gib, lines);
    for (int per_cu : {4, 8}) {  // workgroups of 256 threads per compute unit: 16 and 32 wavefronts
        const int blocks = cus * per_cu;
        run<4, 1>(buf, n_lines, lines, sink, blocks);
        run<4, 2>(buf, n_lines, lines, sink, blocks);
        run<4, 4>(buf, n_lines, lines, sink, blocks);
        run<4, 8>(buf, n_lines, lines, sink, blocks);
        run<8, 1>(buf, n_lines, lines, sink, blocks);
        run<8, 4>(buf, n_lines, lines, sink, blocks);
        run<8, 8>(buf, n_lines, lines, sink, blocks);
        run<1, 8>(buf, n_lines, lines, sink, blocks);
    }
    {
        hipEvent_t a, b;
        CHECK(hipEventCreate(&a));
        CHECK(hipEventCreate(&b));
        float best = 1e30f;
        for (int rep = 0; rep < 4; ++rep) {
            CHECK(hipEventRecord(a, 0));
            stream_kernel<<<cus * 8, 256>>>(buf, bytes / 16, sink);
            CHECK(hipEventRecord(b, 0));
            CHECK(hipEventSynchronize(b));
            float ms = 0;
            CHECK(hipEventElapsedTime(&ms, a, b));
            if (rep && ms < best) best = ms;
        }
        std::printf("streaming read of the whole buffer: %.2f ms  %.1f GB/s\n", best, (double)bytes / (best * 1e6));
    }
    CHECK(hipFree(buf));
    CHECK(hipFree(sink));
    return 0;
}
