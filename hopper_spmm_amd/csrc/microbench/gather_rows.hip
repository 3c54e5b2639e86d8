// Measurement program (make microbench): what the memory system delivers for random gathers of 256-byte
// rows - the access pattern of the gather kernels (spmm_mfma_kernel.hpp) - with the rows landing in
// registers (global_load_dwordx4) or in LDS (global_load_lds_dwordx4, gfx950's direct-to-LDS load).
// 16 M gathers per launch, 16 waves per compute unit, eight loads per lane in flight; tables of 2 MiB (fits
// every L2) and 256 MiB; indices uniform or skewed like the columns of an R-MAT graph (20 bits, each set with
// probability 0.24).  Prints TB/s of gathered bytes per variant.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("%s: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__); std::exit(1); } } while (0)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// rows into LDS: a quarter-wave per row, UNROLL instructions of 1 KB per wave in flight, then one read of them
template <int UNROLL, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gather_to_lds(const char *__restrict__ table, const uint32_t *__restrict__ idx,
                                                            size_t per_wave, uint32_t *out)
{
    __shared__ __attribute__((aligned(16))) char smem[WAVES * UNROLL * 1024];
    const uint32_t lane = threadIdx.x & 63u, g = lane >> 4, j = lane & 15u, w = threadIdx.x >> 6;
    const uint32_t *my = idx + (size_t(blockIdx.x) * WAVES + w) * per_wave;
    char *mine = smem + w * UNROLL * 1024;
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = 0; i < per_wave; i += 4 * UNROLL) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const char *p = table + size_t(my[i + 4 * u + g]) * 256u + j * 16u;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p,
                                             (__attribute__((address_space(3))) void *)(mine + u * 1024), 16, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0);
        acc ^= *reinterpret_cast<const u32x4 *>(mine + lane * 16u);
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[0] = 1;
}

// rows into registers
template <int UNROLL>
__global__ __launch_bounds__(256) void gather_to_registers(const char *__restrict__ table, const uint32_t *__restrict__ idx,
                                                           size_t per_wave, uint32_t *out)
{
    const uint32_t lane = threadIdx.x & 63u, g = lane >> 4, j = lane & 15u;
    const uint32_t *my = idx + (size_t(blockIdx.x) * 4 + (threadIdx.x >> 6)) * per_wave;
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = 0; i < per_wave; i += 4 * UNROLL) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = *reinterpret_cast<const u32x4 *>(table + size_t(my[i + 4 * u + g]) * 256u + j * 16u);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[0] = 1;
}

int main()
{
    const size_t gathers = size_t(16) << 20;              // x 256 B = 4 GiB per launch
    const int waves = 256 * 16;
    uint32_t *d_out, *d_idx;
    CHECK(hipMalloc(&d_out, 4));
    CHECK(hipMalloc(&d_idx, gathers * 4));
    std::vector<uint32_t> h(gathers);
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a)); CHECK(hipEventCreate(&b));
    for (int skew = 0; skew < 2; ++skew)
        for (size_t mib : {size_t(2), size_t(256)}) {
            const size_t rows = mib * 1024 * 1024 / 256;
            char *table;
            CHECK(hipMalloc(&table, rows * 256)); CHECK(hipMemset(table, 1, rows * 256));
            uint64_t s = 88172645463325252ull;
            auto next = [&] { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return s; };
            for (auto &x : h) {
                if (!skew) x = uint32_t(next() % rows);
                else { uint32_t c = 0; for (int bit = 0; bit < 20; ++bit) c = (c << 1) | ((next() & 0xFFFFu) < 15729u); x = c % rows; }
            }
            CHECK(hipMemcpy(d_idx, h.data(), h.size() * 4, hipMemcpyHostToDevice));
            const char *names[] = {"registers, 8 in flight", "LDS, 8 in flight, 4 waves per group", "LDS, 8 in flight, 16 waves per group",
                                   "LDS, 4 in flight, 16 waves per group"};
            for (int variant = 0; variant < 4; ++variant) {
                float best = 1e9f;
                for (int rep = 0; rep < 4; ++rep) {
                    CHECK(hipEventRecord(a));
                    if (variant == 0) gather_to_registers<8><<<waves / 4, 256>>>(table, d_idx, gathers / waves, d_out);
                    if (variant == 1) gather_to_lds<8, 4><<<waves / 4, 256>>>(table, d_idx, gathers / waves, d_out);
                    if (variant == 2) gather_to_lds<8, 16><<<waves / 16, 1024>>>(table, d_idx, gathers / waves, d_out);
                    if (variant == 3) gather_to_lds<4, 16><<<waves / 16, 1024>>>(table, d_idx, gathers / waves, d_out);
                    CHECK(hipGetLastError());
                    CHECK(hipEventRecord(b)); CHECK(hipEventSynchronize(b));
                    float ms;
                    CHECK(hipEventElapsedTime(&ms, a, b));
                    if (ms < best) best = ms;
                }
                std::printf("%s indices, table %3zu MiB, rows to %-38s: %.3f ms  %.2f TB/s\n", skew ? "skewed " : "uniform", mib, names[variant],
                            best, double(gathers) * 256.0 / (best * 1e-3) / 1e12);
                std::fflush(stdout);
            }
            CHECK(hipFree(table));
        }
    return 0;
}
