// gfx950 (MI355X) kernels for C = A * B with A in the condensed 8-row-window
// tile format (reference src/utils/class.h:74-85): the all-shapes scalar kernel,
// the clear kernel, and the dispatch to the MFMA kernels (spmm_mfma_kernel.hpp,
// instantiated in spmm_mfma_<type>_g<n>.hip; spmm_panel_kernel.hpp, instantiated in
// spmm_panel_<type>.hip).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "hspmm_device.h"

namespace hspmm {

// ---------------------------------------------------------------------------
// All-shapes kernel (any N, any alignment): one workgroup per effective window
// and 256-feature slab, one thread per feature, plain fp32 multiply-add, reading
// the format arrays exactly as the caller gave them.  Used when the feature
// dimension rules out the vector loads above (odd N in fp16), and as an
// independent second implementation in tests.
// ---------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<_Float16>(_Float16 v) { return (float)v; }
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__bf16>(__bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ _Float16 from_f32<_Float16>(float v) { return (_Float16)v; }
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __bf16 from_f32<__bf16>(float v) { return (__bf16)v; }

template <typename T, int CW>
__global__ __launch_bounds__(256)
void spmm_scalar_kernel(const KernelArgs ka)
{
    const uint32_t w = blockIdx.x;
    const uint32_t f = blockIdx.y * 256u + threadIdx.x;
    const uint32_t N = ka.N, rows = ka.rows, W = ka.eff_windows;
    const bool active = f < N;
    const T *B = reinterpret_cast<const T *>(ka.B);
    T *C = reinterpret_cast<T *>(ka.C);
    const T *data = reinterpret_cast<const T *>(ka.data);
    float acc[kRowWindow];
#pragma unroll
    for (uint32_t r = 0; r < kRowWindow; ++r) acc[r] = 0.f;
    const uint32_t tb = ka.rowOffset[w], te = ka.rowOffset[w + 1];
    for (uint32_t t = tb; t < te; ++t) {
        for (uint32_t k = 0; k < CW; ++k) {
            const uint32_t c = ka.tcA2B[size_t(t) * CW + k];
            if (c == kIdxMax) continue;
            const float b = active ? to_f32<T>(B[size_t(c) * N + f]) : 0.f;
#pragma unroll
            for (uint32_t r = 0; r < kRowWindow; ++r)
                acc[r] = __builtin_fmaf(to_f32<T>(data[(size_t(t) * kRowWindow + r) * CW + k]), b, acc[r]);
        }
    }
    if (!active) return;
    const uint32_t row0 = ka.rowIdx[w];
#pragma unroll
    for (uint32_t r = 0; r < kRowWindow; ++r)
        if (row0 + r < rows) C[size_t(row0 + r) * N + f] = from_f32<T>(acc[r]);
    const uint32_t next_row = (w + 1u < W) ? ka.rowIdx[w + 1] : rows;
    for (uint32_t r = row0 + kRowWindow; r < next_row; ++r) C[size_t(r) * N + f] = from_f32<T>(0.f);
    if (w == 0u)
        for (uint32_t r = 0; r < row0; ++r) C[size_t(r) * N + f] = from_f32<T>(0.f);
}

// Whole-matrix clear for a matrix without any stored entry (every row of C is 0).  dst is aligned to
// two bytes: one half in front of the first whole word when dst starts inside one, whole words, one half behind.
__global__ __launch_bounds__(256) void fill_zero_kernel(uint16_t *dst, size_t n_halves)
{
    const size_t head = (reinterpret_cast<uintptr_t>(dst) & 2u) ? 1u : 0u;
    const size_t n_words = (n_halves - head) / 2u;
    uint32_t *words = reinterpret_cast<uint32_t *>(dst + head);
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n_words; i += stride) words[i] = 0u;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        if (head) dst[0] = 0;
        if (head + 2u * n_words < n_halves) dst[n_halves - 1u] = 0;
    }
}

// Bitmap tiles -> plain 8 x 16 tiles of 16-bit elements (plans made from the reference's BTCF_MTX arrays, reference
// src/utils/class.h:55-67): one thread per tile element; header and stored elements as the gather kernels read
// them (hspmm_device.h: bm_header).  The kernels that take plain tiles then run on what this wrote.
__global__ __launch_bounds__(256) void expand_bitmap_kernel(const uint32_t *__restrict__ header,
                                                            const uint16_t *__restrict__ vals,
                                                            uint16_t *__restrict__ tiles, uint32_t n_tiles)
{
    const uint32_t t = blockIdx.x * 2u + (threadIdx.x >> 7), b = threadIdx.x & 127u;
    if (t >= n_tiles) return;
    const uint32_t *h = header + size_t(t) * 8u;
    const uint32_t word = b >> 5, w = h[word], bit = b & 31u;
    const uint32_t before = ((h[4] >> (8u * word)) & 0xFFu) + uint32_t(__builtin_popcount(w & ((1u << bit) - 1u)));
    tiles[size_t(t) * 128u + b] = ((w >> bit) & 1u) ? vals[size_t(h[5]) + before] : uint16_t(0);
}

hipError_t launch_expand_bitmap(const uint32_t *header, const void *vals, void *tiles, uint32_t n_tiles, hipStream_t s)
{
    if (!n_tiles) return hipSuccess;
    expand_bitmap_kernel<<<dim3((n_tiles + 1u) / 2u), 256, 0, s>>>(header, static_cast<const uint16_t *>(vals),
                                                                  static_cast<uint16_t *>(tiles), n_tiles);
    return hipGetLastError();
}

#define HSPMM_DECLARE_LAUNCH(name) \
    hipError_t name(int layout, const KernelArgs &ka, int V, int prefetch, bool narrow, int waves_per_group, \
                    hipStream_t s, hipEvent_t mid);
HSPMM_DECLARE_LAUNCH(launch_mfma_f16_g1) HSPMM_DECLARE_LAUNCH(launch_mfma_f16_g2)
HSPMM_DECLARE_LAUNCH(launch_mfma_bf16_g1) HSPMM_DECLARE_LAUNCH(launch_mfma_bf16_g2)
HSPMM_DECLARE_LAUNCH(launch_mfma_f32_g1) HSPMM_DECLARE_LAUNCH(launch_mfma_f32_g2)
#undef HSPMM_DECLARE_LAUNCH

hipError_t launch_mfma_f16_bm(const KernelArgs &ka, int V, int prefetch, bool narrow, int waves_per_group, hipStream_t s,
                              hipEvent_t mid);
hipError_t launch_mfma_bf16_bm(const KernelArgs &ka, int V, int prefetch, bool narrow, int waves_per_group, hipStream_t s,
                               hipEvent_t mid);

hipError_t launch_spmm_mfma(int dtype, int layout, int G, const KernelArgs &ka, int V, int prefetch, bool narrow,
                            int waves_per_group, hipStream_t s, hipEvent_t mid)
{
    if (layout == kLayoutDWB) {
        if (G != 1 || dtype == kDtypeF32) return hipErrorInvalidValue;
        return dtype == kDtypeBf16 ? launch_mfma_bf16_bm(ka, V, prefetch, narrow, waves_per_group, s, mid)
                                   : launch_mfma_f16_bm(ka, V, prefetch, narrow, waves_per_group, s, mid);
    }
    if (dtype == kDtypeF32)
        return G == 2 ? launch_mfma_f32_g2(layout, ka, V, prefetch, narrow, waves_per_group, s, mid)
                      : launch_mfma_f32_g1(layout, ka, V, prefetch, narrow, waves_per_group, s, mid);
    if (dtype == kDtypeBf16)
        return G == 2 ? launch_mfma_bf16_g2(layout, ka, V, prefetch, narrow, waves_per_group, s, mid)
                      : launch_mfma_bf16_g1(layout, ka, V, prefetch, narrow, waves_per_group, s, mid);
    return G == 2 ? launch_mfma_f16_g2(layout, ka, V, prefetch, narrow, waves_per_group, s, mid)
                  : launch_mfma_f16_g1(layout, ka, V, prefetch, narrow, waves_per_group, s, mid);
}

hipError_t launch_panel_f16(int G, bool tall, bool packed, const PanelArgs &pa, const KernelArgs &ka, int waves, hipStream_t s,
                           hipEvent_t mid);
hipError_t launch_panel_bf16(int G, bool tall, bool packed, const PanelArgs &pa, const KernelArgs &ka, int waves, hipStream_t s,
                            hipEvent_t mid);
hipError_t launch_panel_f32(int G, bool split, bool tall, bool packed, const PanelArgs &pa, const KernelArgs &ka, int waves,
                            hipStream_t s, hipEvent_t mid);

hipError_t launch_spmm_panel(int dtype, int G, bool split, bool tall, bool packed, const PanelArgs &pa, const KernelArgs &ka,
                             int waves, hipStream_t s, hipEvent_t mid)
{
    if (dtype == kDtypeF32) return launch_panel_f32(G, split, tall, packed, pa, ka, waves, s, mid);
    if (dtype == kDtypeBf16) return launch_panel_bf16(G, tall, packed, pa, ka, waves, s, mid);
    return launch_panel_f16(G, tall, packed, pa, ka, waves, s, mid);
}

hipError_t launch_spmm_scalar(int dtype, const KernelArgs &ka, hipStream_t s)
{
    const dim3 grid(ka.eff_windows, (ka.N + 255u) / 256u);
    if (dtype == kDtypeF16) spmm_scalar_kernel<_Float16, 16><<<grid, 256, 0, s>>>(ka);
    else if (dtype == kDtypeBf16) spmm_scalar_kernel<__bf16, 16><<<grid, 256, 0, s>>>(ka);
    else spmm_scalar_kernel<float, 8><<<grid, 256, 0, s>>>(ka);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Measurement only: the row gathers of a plan's step stream and nothing else.
// Every wave walks a slice of the stream's column ids and loads, for each id,
// PART bytes of that row of B (PART = 256: a quarter-wave per row, 16 bytes per
// lane; PART = 128: 8 bytes per lane, the part chosen by the XCD the workgroup
// runs on, as the gather kernels do with feature blocks dealt out by XCD), eight
// loads per lane in flight, sixteen waves per compute unit.  The time is the
// floor of any kernel that gathers these rows in this order: what the L2s, the
// fabric and HBM deliver for this id stream.
// ---------------------------------------------------------------------------
template <int PART>
__global__ __launch_bounds__(256)
void gather_rate_kernel(const uint32_t *__restrict__ ids, uint64_t n_ids, uint64_t ids_per_wave, const char *__restrict__ B,
                        uint32_t row_bytes, uint32_t parts, uint32_t *sink)
{
    typedef uint32_t vec_t __attribute__((ext_vector_type(PART / 64)));
    const uint32_t lane = threadIdx.x & 63u, g = lane >> 4, j = lane & 15u;
    uint32_t part = 0, wave;
    if (parts > 1u) {
        // workgroups dealt out as by spmm_mfma_kernel: XCD x = blockIdx % 8 serves part x / (8 / parts)
        const uint32_t per_part = 8u / parts, xcd = blockIdx.x & 7u, set = blockIdx.x >> 3;
        part = xcd / per_part;
        wave = (set * per_part + (xcd - part * per_part)) * 4u + (threadIdx.x >> 6);
    } else {
        wave = blockIdx.x * 4u + (threadIdx.x >> 6);
    }
    const uint64_t begin = uint64_t(wave) * ids_per_wave;
    const uint64_t end = begin + ids_per_wave < n_ids ? begin + ids_per_wave : n_ids;
    const char *lane_base = B + size_t(part) * PART + j * (PART / 16);
    vec_t acc = {};
    for (uint64_t i = begin; i + 32u <= end; i += 32u) {
        vec_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const uint32_t row = ids[i + 4u * u + g];
            v[u] = *reinterpret_cast<const vec_t *>(lane_base + size_t(row) * row_bytes);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u];
    }
    uint32_t x = 0;
#pragma unroll
    for (int k = 0; k < PART / 64; ++k) x ^= acc[k];
    if (x == 0x9E3779B9u && sink) sink[0] = x;      // (keeps the loads; practically never taken)
}

hipError_t launch_gather_rate(const uint32_t *ids, uint64_t n_ids, const void *B, uint32_t row_bytes, uint32_t part_bytes,
                              uint32_t parts, int compute_units, uint32_t *sink, hipStream_t s)
{
    const uint64_t waves = uint64_t(compute_units) * 16u;
    uint64_t per_wave = ((n_ids + waves - 1u) / waves + 31u) & ~uint64_t(31);
    if (per_wave < 32u) per_wave = 32u;
    const uint64_t used = (n_ids + per_wave - 1u) / per_wave;             // waves with work
    const uint64_t per_set = uint64_t(8u / parts) * 4u;
    const uint64_t blocks = parts > 1u ? 8u * ((used + per_set - 1u) / per_set) : (used + 3u) / 4u;
    const char *b = static_cast<const char *>(B);
    if (part_bytes == 256u) gather_rate_kernel<256><<<dim3(unsigned(blocks)), 256, 0, s>>>(ids, n_ids, per_wave, b, row_bytes, parts, sink);
    else gather_rate_kernel<128><<<dim3(unsigned(blocks)), 256, 0, s>>>(ids, n_ids, per_wave, b, row_bytes, parts, sink);
    return hipGetLastError();
}

hipError_t launch_fill_zero(void *dst, size_t bytes, hipStream_t s)
{
    // bytes is a multiple of the element size (2 or 4) and dst is aligned to it
    const size_t halves = bytes / 2;
    if (halves == 0) return hipSuccess;
    size_t blocks = (halves / 2 + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    fill_zero_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(reinterpret_cast<uint16_t *>(dst), halves);
    return hipGetLastError();
}

}  // namespace hspmm
