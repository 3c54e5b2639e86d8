// Measurement program (not part of the library): what a gfx950 compute unit sustains on the inner step of
// the LDS-panel kernels (spmm_panel_kernel.hpp) - 16 ds_read_b64_tr_b16 that feed 8 v_mfma_f32_16x16x32_f16 -
// with nothing else going on: no global loads, no barriers.  Every wave runs the same loop on rows of an
// LDS image 288 bytes apart whose numbers differ mod 8 inside the two 16-lane blocks served together (no bank
// conflicts, as the plan arranges it).  Printed per variant and waves per compute unit: cycles per step and
// wave (2.4 GHz assumed) and how busy the MFMA pipes would be.  Built by `make microbench` in this folder's
// parent; run it on the GPU as ./lds_mfma_microbench.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef short tr16x4 __attribute__((ext_vector_type(4)));
typedef tr16x4 __attribute__((address_space(3))) *lds_tr_ptr;
typedef __attribute__((address_space(3))) char *lds_char_ptr;
template <int MODE>   // 0: reads and MFMAs as the compiler orders them (8 + 4 + 8 + 4), 1: all 16 reads first, 2: MFMAs only, 3: reads only
__global__ __launch_bounds__(1024) void k(uint32_t iters, float *out, uint32_t seed)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    for (uint32_t i = threadIdx.x; i < 36864; i += blockDim.x) reinterpret_cast<uint32_t *>(smem)[i] = 0x3c003c00u;
    __syncthreads();
    const uint32_t blk = lane >> 4, i = lane & 15u;
    f32x4 acc[8];
    for (int p = 0; p < 8; ++p) acc[p] = f32x4{0, 0, 0, 0};
    u32x4 A = {0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
    uint32_t r0 = (blk * 4u + (i >> 2) + wave * 16u + seed * 8u) & 255u, r1 = (r0 + 16u) & 255u;
    if (MODE == 4) {
        // reads of step t + 1 in flight during the MFMAs of step t (two sets of operand registers)
        u32x4 b0[8], b1[8];
        auto rd = [&](u32x4 (&b)[8]) __attribute__((always_inline)) {
            const lds_char_ptr a0 = (lds_char_ptr)smem + r0 * 288u + (i & 3u) * 8u;
            const lds_char_ptr a1 = (lds_char_ptr)smem + r1 * 288u + (i & 3u) * 8u;
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const tr16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a0 + 32 * p));
                const tr16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a1 + 32 * p));
                const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                b[p][0] = l2[0]; b[p][1] = l2[1]; b[p][2] = h2[0]; b[p][3] = h2[1];
            }
            r0 = (r0 + 40u) & 255u; r1 = (r1 + 40u) & 255u;
        };
        auto mm = [&](const u32x4 (&b)[8]) __attribute__((always_inline)) {
#pragma unroll
            for (int p = 0; p < 8; ++p) acc[p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, A), __builtin_bit_cast(half8, b[p]), acc[p], 0, 0, 0);
        };
        rd(b0);
        for (uint32_t it = 0; it < iters; it += 2) {
            rd(b1); __builtin_amdgcn_sched_barrier(0);
            mm(b0); __builtin_amdgcn_sched_barrier(0);
            rd(b0); __builtin_amdgcn_sched_barrier(0);
            mm(b1); __builtin_amdgcn_sched_barrier(0);
        }
    } else
    for (uint32_t it = 0; it < iters; ++it) {
        const lds_char_ptr a0 = (lds_char_ptr)smem + r0 * 288u + (i & 3u) * 8u;
        const lds_char_ptr a1 = (lds_char_ptr)smem + r1 * 288u + (i & 3u) * 8u;
        if (MODE == 2) {
#pragma unroll
            for (int p = 0; p < 8; ++p) acc[p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, A), __builtin_bit_cast(half8, A), acc[p], 0, 0, 0);
        } else {
            u32x4 b[8];
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const tr16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a0 + 32 * p));
                const tr16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a1 + 32 * p));
                const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                b[p][0] = l2[0]; b[p][1] = l2[1]; b[p][2] = h2[0]; b[p][3] = h2[1];
                if (MODE == 0) acc[p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, A), __builtin_bit_cast(half8, b[p]), acc[p], 0, 0, 0);
            }
            if (MODE == 1) {
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int p = 0; p < 8; ++p) acc[p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, A), __builtin_bit_cast(half8, b[p]), acc[p], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (MODE == 3) {
#pragma unroll
                for (int p = 0; p < 8; ++p) acc[p][0] += __builtin_bit_cast(float, b[p][0] ^ b[p][3]);
            }
        }
        r0 = (r0 + 40u) & 255u; r1 = (r1 + 40u) & 255u;           // the next step's rows
    }
    float sacc = 0;
    for (int p = 0; p < 8; ++p) sacc += acc[p][0] + acc[p][1] + acc[p][2] + acc[p][3];
    if (sacc == 12345.f) out[threadIdx.x] = sacc;
}
template <int MODE>
void run(const char *name, int threads, float *d_out)
{
    const uint32_t iters = 4000;
    hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
    CK(hipFuncSetAttribute(reinterpret_cast<const void *>(k<MODE>), hipFuncAttributeMaxDynamicSharedMemorySize, 147456));
    float best = 1e9;
    for (int rep = 0; rep < 3; ++rep) {
        CK(hipEventRecord(a));
        k<MODE><<<256, threads, 147456>>>(iters, d_out, rep);
        CK(hipEventRecord(b)); CK(hipEventSynchronize(b));
        float ms; CK(hipEventElapsedTime(&ms, a, b)); if (ms < best) best = ms;
    }
    const double cyc_per_step_per_wave = best * 1e-3 * 2.4e9 / iters;
    const int waves = threads / 64;
    printf("%-44s %2d waves/CU: %.3f ms, %.0f cycles per step and wave, MFMA pipe %.0f %% busy (if 16 cycles each)\n", name, waves, best,
           cyc_per_step_per_wave, MODE == 3 ? 0.0 : 100.0 * (8 * 16.0 * waves / 4) / cyc_per_step_per_wave);
    fflush(stdout);
}
int main()
{
    float *d_out; CK(hipMalloc(&d_out, 4096));
    for (int threads : {256, 512, 768, 1024}) {
        run<0>("16 reads + 8 MFMA, compiler's order", threads, d_out);
        run<1>("16 reads first, then 8 MFMA", threads, d_out);
        run<2>("8 MFMA only", threads, d_out);
        run<3>("16 reads only", threads, d_out);
        run<4>("reads of step t+1 issued before MFMAs of t", threads, d_out);
    }
    return 0;
}
