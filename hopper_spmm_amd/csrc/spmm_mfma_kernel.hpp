// gfx950 (MI355X) MFMA kernel templates for C = A * B with A in the condensed 8-row-window
// tile format (reference src/utils/class.h:74-85).  They replace the reference's
// fp16_spmm_kernel (reference src/fp16.cu:36-175) and supply the fp32-storage
// ("tf32") variant the reference only sketches (src/common.h:26-43).
//
// Design (one wave = one independent pipeline, no LDS, no barriers):
//   * The plan turns the windows into a flat stream of "steps".  A step is one
//     tile of one window or - where two vertically adjacent windows have the same
//     column list, as in block-clustered weights - one tile of each of the two
//     ("paired unit", G = 2): the gathered rows of B are then loaded once and
//     multiplied with both tiles.
//   * A wave owns a contiguous range of steps (a few hundred) and, for feature
//     dimensions wider than one block, one feature block.  Units are contiguous in
//     the step stream, so the loads stream through the range without regard to
//     unit boundaries; only the MFMA stage looks at them (to store a finished
//     window and clear accumulators).
//   * Per fp16 step a lane issues one 16-byte load of four column ids, one load
//     of its part of the sparse tile(s) and the loads of its words of the four B
//     rows those ids name; the 16 lanes of a quarter-wave cover one B row
//     contiguously.
//   * fp16 contraction without any transposition of B: an MFMA operand register
//     holds two k-slots.  A B register as loaded holds features (2c, 2c+1) of one
//     gathered row, i.e. "k-slot pair" = (even feature, odd feature).  The sparse
//     operand is built so that MFMA row 2r holds a[r][k] in the even slot and 0 in
//     the odd one, MFMA row 2r+1 the reverse.  Output row 2r then is window row r
//     for the even features, row 2r+1 for the odd ones: all 16 MFMA rows and all
//     32 k-slots do useful work for an 8-row window, and a lane ends up with
//     contiguous features of two window rows.
//   * fp32 ("tf32") contraction uses v_mfma_f32_16x16x4_f32; one B register per
//     lane per k, no packing issue; MFMA rows 8..15 are zero padding.
//   * Loads for step t+P are issued before the MFMAs of step t (P = prefetch
//     depth, registers as the ring buffer); hardware returns vector loads in
//     order, so the wait before the MFMAs of step t leaves P-1 steps in flight.
//   * Padding columns (id 0xFFFFFFFF) are renamed, in the plan's device copy of the
//     ids, to the real column in front of them; their tile column is all zero.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>
#pragma once
#include "hspmm_device.h"

namespace hspmm {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float    f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int V> struct Vec;
template <> struct Vec<1> { typedef uint32_t type; };
template <> struct Vec<2> { typedef u32x2 type; };
template <> struct Vec<4> { typedef u32x4 type; };

// C is written once per launch; the rows of B are read again and again.  The
// stores are marked non-temporal so that C does not push B out of the L2.
// (Non-temporal loads of the tile / id streams measured slower: not used.)
template <class T>
__device__ __forceinline__ void stream_store(T *p, const T v)
{
    __builtin_nontemporal_store(v, p);
}

template <int V>
__device__ __forceinline__ void store_words(void *p, const uint32_t (&src)[V])
{
    typename Vec<V>::type v;
    if constexpr (V == 1) v = src[0];
    else {
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] = src[i];
    }
    stream_store(reinterpret_cast<typename Vec<V>::type *>(p), v);
}

__device__ __forceinline__ uint32_t pack_half2_rn(float lo, float hi)
{
    // float -> half conversion in the default rounding mode (nearest even), as the
    // reference's store does (src/fp16.cu:167, cvt.rn.f16.f32).
    _Float16 l = (_Float16)lo, h = (_Float16)hi;
    uint16_t lb = __builtin_bit_cast(uint16_t, l), hb = __builtin_bit_cast(uint16_t, h);
    return uint32_t(lb) | (uint32_t(hb) << 16);
}

__device__ __forceinline__ uint32_t umin32(uint32_t a, uint32_t b) { return a < b ? a : b; }

// The two 16-bit element types share everything but the MFMA instruction and the
// rounding of the result: BF = false is IEEE half, BF = true bfloat16 (the
// reference's -DUSE_BF16 build, src/common.h:20-25).  Both round to nearest even.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
template <bool BF> struct HalfOps;
template <> struct HalfOps<false> {
    typedef _Float16 elem_t;
    __device__ static __forceinline__ f32x4 mfma(const u32x4 a, const u32x4 b, const f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi) { return pack_half2_rn(lo, hi); }
};
template <> struct HalfOps<true> {
    typedef __bf16 elem_t;
    __device__ static __forceinline__ f32x4 mfma(const u32x4 a, const u32x4 b, const f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi)
    {
        const __bf16 l = (__bf16)lo, h = (__bf16)hi;
        return uint32_t(__builtin_bit_cast(uint16_t, l)) | (uint32_t(__builtin_bit_cast(uint16_t, h)) << 16);
    }
};

// Device-scope ("agent") accesses of 16 bytes, visible to every XCD: buffer instructions with the sc1
// policy (stores are written through to memory, loads go past the L2 of the XCD).  base is the same in
// every lane, off the lane's byte offset from it (below 2 GB).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t device_scope_buffer(const void *base)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0x7FFFFFFF, 0x00020000);
}
__device__ __forceinline__ void store_device_scope(const __amdgpu_buffer_rsrc_t r, const uint32_t off, const f32x4 v)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, off, 0, 16);
}
__device__ __forceinline__ f32x4 load_device_scope(const __amdgpu_buffer_rsrc_t r, const uint32_t off)
{
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 16));
}
// The stores in front of it are acknowledged (vmcnt(0)); the compiler moves no memory access across it.
__device__ __forceinline__ void wait_stores_acknowledged() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Uniform (per-wave) reads of the small index arrays go through the constant
// address space so that they become scalar loads, which do not share the
// in-order return queue of the vector loads that stream the tiles.
typedef const uint32_t __attribute__((address_space(4))) *const_u32_ptr;
__device__ __forceinline__ const_u32_ptr as_const(const uint32_t *p)
{
    return (const_u32_ptr)(uintptr_t)p;
}

// Where a lane reads its words of B row c.  NARROW: B is smaller than 4 GiB and
// has fewer than 2^24 rows, so one 24-bit multiply-add gives a 32-bit offset
// from a scalar base.
template <bool NARROW>
struct Gather {
    const char *base;        // B (uniform)
    uint32_t row_bytes;      // N * element size
    uint32_t lane_off;       // byte offset of the lane's first feature inside a row
    __device__ __forceinline__ const char *row(uint32_t c) const
    {
        if constexpr (NARROW) {
            const uint32_t off = __umul24(c, row_bytes) + lane_off;
            return base + size_t(off);
        } else {
            return base + (size_t(c) * row_bytes + lane_off);
        }
    }
};

// ---------------------------------------------------------------------------
// Element-type traits: how one step is loaded, multiplied and stored.
// V = 32-bit words of a B row a lane owns, G = windows per unit (1 or 2).
// The plan stores the tiles of a step in lane order (step_stream.hpp,
// lane_order_tiles): what one lane needs of a step is one contiguous load.
// ---------------------------------------------------------------------------

// Common part of the two fp16 layouts: the sparse operand.
//   tiles, G = 1: the caller's tile, [row r][k] halves; lane (g, j) reads
//                 a[j/2][4g..4g+3] = 8 bytes at (r*16 + 4g) halves.
//   tiles, G = 2: [row r][g][window][4 halves]; the lane reads 16 bytes.
template <int G>
struct Fp16Lane {
    typedef typename Vec<2 * G>::type AVec;
    uint32_t g, j;                             // quarter-wave, lane in quarter
    uint32_t half_shift;                       // 16 for the lane that owns the last feature of an odd N alone (mark_half_lane)
    uint32_t sel_lo, sel_hi;                   // byte selectors for the sparse operand
    const uint32_t *a_src;                     // lane's words inside step 0
    const uint32_t *idx_src;                   // lane's ids inside step 0
    const void *a_base;                        // the tile array itself
    __device__ __forceinline__ const void *a_src_base() const { return a_base; }
    __device__ __forceinline__ void init(uint32_t lane, const void *tiles, const uint32_t *ids)
    {
        a_base = tiles;
        g = lane >> 4; j = lane & 15u;
        half_shift = 0u;
        const uint32_t r = j >> 1, parity = j & 1u;
        // v_perm_b32 selectors: bytes 0-3 come from the second source, 0x0c gives 0x00.
        //   even MFMA row: value in the low half  -> {lo: b0 b1 0 0}, {hi: b2 b3 0 0}
        //   odd  MFMA row: value in the high half -> {lo: 0 0 b0 b1}, {hi: 0 0 b2 b3}
        sel_lo = parity ? 0x01000c0cu : 0x0c0c0100u;
        sel_hi = parity ? 0x03020c0cu : 0x0c0c0302u;
        a_src = reinterpret_cast<const uint32_t *>(tiles) + (r * 8u + g * 2u) * G;
        idx_src = ids + g * 4u;
    }
    __device__ __forceinline__ u32x4 load_idx(uint32_t step) const
    {
        return *reinterpret_cast<const u32x4 *>(idx_src + size_t(step) * 16u);
    }
    __device__ __forceinline__ AVec load_a(uint32_t step) const
    {
        return *reinterpret_cast<const AVec *>(a_src + size_t(step) * (64u * G));
    }
    // MFMA row 2r carries a[r][k] in the even k-slot of each pair, row 2r+1 in the odd one.
    template <int W0>
    __device__ __forceinline__ u32x4 sparse_operand(const AVec &a) const
    {
        const uint32_t lo = a[2 * W0], hi = a[2 * W0 + 1];
        u32x4 aw;
        aw[0] = __builtin_amdgcn_perm(0u, lo, sel_lo);
        aw[1] = __builtin_amdgcn_perm(0u, lo, sel_hi);
        aw[2] = __builtin_amdgcn_perm(0u, hi, sel_lo);
        aw[3] = __builtin_amdgcn_perm(0u, hi, sel_hi);
        return aw;
    }
};

// fp16, layout "X4": a lane reads 4*V contiguous bytes of each of its four B rows
// (one wide load per row) and owns 2*V contiguous features.  Any N that is a
// multiple of 2*V.  The B operand of MFMA p is word p of the four loads, which
// costs register moves.
template <int V_, int G_, bool BF = false>
struct Fp16Tile {
    static constexpr int V = V_, G = G_;
    static constexpr int kBlockFeat = 32 * V;      // features one wave covers
    static constexpr int kLaneFeat = 2 * V;        // lane's first feature = j * kLaneFeat
    static constexpr int kElem = 2;
    typedef typename Vec<V>::type BVec;
    typedef u32x4 Idx;                             // four column ids per lane per step
    typedef Fp16Lane<G> Lane;
    typedef typename Lane::AVec AVec;

    __device__ static __forceinline__ Idx load_idx(const Lane &L, uint32_t step) { return L.load_idx(step); }
    // The registers of one step in flight are separate variables of the caller
    // (b0..b3: the lane's words of four B rows, a: its words of the sparse tile(s)).
    template <class GT>
    __device__ static __forceinline__ void load_tile(const Lane &L, uint32_t step, const Idx idx, const GT &gat,
                                                     BVec &b0, BVec &b1, BVec &b2, BVec &b3, AVec &a)
    {
        b0 = *reinterpret_cast<const BVec *>(gat.row(idx[0]));
        b1 = *reinterpret_cast<const BVec *>(gat.row(idx[1]));
        b2 = *reinterpret_cast<const BVec *>(gat.row(idx[2]));
        b3 = *reinterpret_cast<const BVec *>(gat.row(idx[3]));
        a = L.load_a(step);
    }
    template <int p> __device__ static __forceinline__ uint32_t word(const BVec &v)
    {
        if constexpr (V == 1) return v; else return v[p];
    }
    // shift: 16 in the lane whose word was loaded one half early (odd N, see mark_half_lane), else 0
    template <int W0, int p>
    __device__ static __forceinline__ void mma_one(const u32x4 av, const BVec &b0, const BVec &b1, const BVec &b2,
                                                   const BVec &b3, f32x4 (&acc)[G * V], uint32_t shift)
    {
        if constexpr (p < V) {
            u32x4 bw;
            bw[0] = word<p>(b0); bw[1] = word<p>(b1); bw[2] = word<p>(b2); bw[3] = word<p>(b3);
            if constexpr (V == 1) { bw[0] >>= shift; bw[1] >>= shift; bw[2] >>= shift; bw[3] >>= shift; }
            acc[W0 * V + p] = HalfOps<BF>::mfma(av, bw, acc[W0 * V + p]);
        }
    }
    template <int W0>
    __device__ static __forceinline__ void mma_window(const Lane &L, const BVec &b0, const BVec &b1, const BVec &b2,
                                                      const BVec &b3, const AVec &a, f32x4 (&acc)[G * V])
    {
        if constexpr (W0 < G) {
            const u32x4 av = L.template sparse_operand<W0>(a);
            mma_one<W0, 0>(av, b0, b1, b2, b3, acc, L.half_shift); mma_one<W0, 1>(av, b0, b1, b2, b3, acc, 0u);
            mma_one<W0, 2>(av, b0, b1, b2, b3, acc, 0u); mma_one<W0, 3>(av, b0, b1, b2, b3, acc, 0u);
        }
    }
    __device__ static __forceinline__ void mma(const Lane &L, const BVec &b0, const BVec &b1, const BVec &b2,
                                               const BVec &b3, const AVec &a, f32x4 (&acc)[G * V])
    {
        mma_window<0>(L, b0, b1, b2, b3, a, acc);
        mma_window<1>(L, b0, b1, b2, b3, a, acc);
    }
    // acc[W0*V + p][e]: MFMA row 4g+e = window row 2g + e/2, feature lane_feat + 2p + (e & 1).
    template <int W0>
    __device__ static __forceinline__ void store_window(const Lane &L, const f32x4 (&acc)[G * V], char *c_lane,
                                                        size_t row_bytes, uint32_t row0, uint32_t rows, bool active)
    {
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            const uint32_t row = row0 + 2u * L.g + rr;
            uint32_t out[V];
#pragma unroll
            for (int p = 0; p < V; ++p) out[p] = HalfOps<BF>::pack(acc[W0 * V + p][2 * rr], acc[W0 * V + p][2 * rr + 1]);
            if (active && row < rows) {
                if (V == 1 && L.half_shift) stream_store(reinterpret_cast<uint16_t *>(c_lane + size_t(row) * row_bytes), uint16_t(out[0]));
                else store_words<V>(c_lane + size_t(row) * row_bytes, out);
            }
        }
    }
    // Zero rows [r_begin, r_end) of this lane's features.
    __device__ static __forceinline__ void zero_rows(const Lane &L, char *c_lane, size_t row_bytes, uint32_t r_begin,
                                                     uint32_t r_end, bool active)
    {
        uint32_t z[V];
#pragma unroll
        for (int i = 0; i < V; ++i) z[i] = 0u;
        if (!active) return;
        for (uint32_t r = r_begin + L.g; r < r_end; r += 4u) {
            if (V == 1 && L.half_shift) stream_store(reinterpret_cast<uint16_t *>(c_lane + size_t(r) * row_bytes), uint16_t(0));
            else store_words<V>(c_lane + size_t(r) * row_bytes, z);
        }
    }
};

// fp16, layout "DW": a lane reads single words, word p of a row at feature
// 32p + 2j, so that the 16 lanes of a quarter-wave still read 64 contiguous
// bytes, and the four words that form the B operand of MFMA p (one per B row)
// are loaded straight into four consecutive registers: no moves.  Needs N to be
// a multiple of 32*V.
template <int V_, int G_, bool BF = false>
struct Fp16TileDW {
    static constexpr int V = V_, G = G_;
    static constexpr int kBlockFeat = 32 * V;
    static constexpr int kLaneFeat = 2;            // lane's first feature = 2j, then +32 per word
    static constexpr int kElem = 2;
    typedef u32x4 BVec;                            // b_p = word p of the four B rows
    typedef u32x4 Idx;
    typedef Fp16Lane<G> Lane;
    typedef typename Lane::AVec AVec;

    __device__ static __forceinline__ Idx load_idx(const Lane &L, uint32_t step) { return L.load_idx(step); }
    template <class GT>
    __device__ static __forceinline__ void load_tile(const Lane &L, uint32_t step, const Idx idx, const GT &gat,
                                                     BVec &b0, BVec &b1, BVec &b2, BVec &b3, AVec &a)
    {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t *src = reinterpret_cast<const uint32_t *>(gat.row(idx[q]));
            b0[q] = src[0];
            if constexpr (V > 1) b1[q] = src[16];
            if constexpr (V > 2) b2[q] = src[32];
            if constexpr (V > 3) b3[q] = src[48];
        }
        a = L.load_a(step);
    }
    template <int W0>
    __device__ static __forceinline__ void mma_window(const Lane &L, const BVec &b0, const BVec &b1, const BVec &b2,
                                                      const BVec &b3, const AVec &a, f32x4 (&acc)[G * V])
    {
        if constexpr (W0 < G) {
            const u32x4 av = L.template sparse_operand<W0>(a);
            acc[W0 * V] = HalfOps<BF>::mfma(av, b0, acc[W0 * V]);
            if constexpr (V > 1) acc[W0 * V + 1] = HalfOps<BF>::mfma(av, b1, acc[W0 * V + 1]);
            if constexpr (V > 2) acc[W0 * V + 2] = HalfOps<BF>::mfma(av, b2, acc[W0 * V + 2]);
            if constexpr (V > 3) acc[W0 * V + 3] = HalfOps<BF>::mfma(av, b3, acc[W0 * V + 3]);
        }
    }
    __device__ static __forceinline__ void mma(const Lane &L, const BVec &b0, const BVec &b1, const BVec &b2,
                                               const BVec &b3, const AVec &a, f32x4 (&acc)[G * V])
    {
        mma_window<0>(L, b0, b1, b2, b3, a, acc);
        mma_window<1>(L, b0, b1, b2, b3, a, acc);
    }
    // acc[W0*V + p][e]: MFMA row 4g+e = window row 2g + e/2, feature 32p + 2j + (e & 1).
    template <int W0>
    __device__ static __forceinline__ void store_window(const Lane &L, const f32x4 (&acc)[G * V], char *c_lane,
                                                        size_t row_bytes, uint32_t row0, uint32_t rows, bool active)
    {
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            const uint32_t row = row0 + 2u * L.g + rr;
            if (active && row < rows) {
                uint32_t *dst = reinterpret_cast<uint32_t *>(c_lane + size_t(row) * row_bytes);
#pragma unroll
                for (int p = 0; p < V; ++p)
                    stream_store(dst + 16 * p, HalfOps<BF>::pack(acc[W0 * V + p][2 * rr], acc[W0 * V + p][2 * rr + 1]));
            }
        }
    }
    __device__ static __forceinline__ void zero_rows(const Lane &L, char *c_lane, size_t row_bytes, uint32_t r_begin,
                                                     uint32_t r_end, bool active)
    {
        if (!active) return;
        for (uint32_t r = r_begin + L.g; r < r_end; r += 4u) {
            uint32_t *dst = reinterpret_cast<uint32_t *>(c_lane + size_t(r) * row_bytes);
#pragma unroll
            for (int p = 0; p < V; ++p) stream_store(dst + 16 * p, 0u);
        }
    }
};

// fp16 / bf16, layout "DW", single windows, tiles read as bitmap + stored values: the reference's
// bitmap tile format (BTCF_MTX of reference src/utils/class.h:55-67, written by CSR2BTCF,
// src/utils/convert.h:83-101, and never read by the reference's kernel) - per 8 x 16 tile
// 128 bits, bit 16 r + k set for a stored element, and the stored elements of all tiles one
// after the other in ascending bit order.  A lane's four elements a[j/2][4g .. 4g + 3] are four
// consecutive bits, so its stored elements are consecutive too: it counts the tile's bits in
// front of them, loads 8 bytes from there (2-byte aligned) and puts the element of bit i, if
// set, where the dense form has it - the v_perm of the dense form with selectors made from the
// four bits.  A power-law graph stores 16 of a tile's 128 elements: 48 bytes instead of 256.
//   header per step (uniform, scalar loads): the four bitmap words, the counts of words 0, 0..1,
//   0..2 (one byte each, from bit 8 on) and the position of the tile's first stored element.
typedef u32x2 u32x2_unaligned __attribute__((aligned(2)));
struct BitmapHeader { uint32_t d[4]; uint32_t counts; uint32_t first; };

template <int V_, bool BF = false>
struct Fp16TileDWB : Fp16TileDW<V_, 1, BF> {
    typedef Fp16TileDW<V_, 1, BF> Base;
    static constexpr int V = V_, G = 1;
    typedef typename Base::BVec BVec;
    struct Idx { u32x4 ids; BitmapHeader h; };
    struct AVec { u32x2 stored; uint32_t bits; };  // the 8 bytes at the lane's first stored element; its four bits
    struct Lane : Fp16Lane<1> {
        const uint32_t *header;                    // 8 words per step
        uint32_t word, low_mask, shift, sel_base, sel_step;
        __device__ __forceinline__ void init(uint32_t lane, const void *vals, const uint32_t *ids)
        {
            Fp16Lane<1>::init(lane, vals, ids);
            const uint32_t r = this->j >> 1, parity = this->j & 1u;
            word = r >> 1;                          // bitmap word of row r: bits 16 (r & 1) + k
            shift = 16u * (r & 1u) + 4u * this->g;  // the lane's first bit inside that word
            low_mask = (1u << shift) - 1u;
            // v_perm_b32 selector of stored element n (bytes 2n, 2n + 1 of the 8 loaded): into the low half
            // for an even MFMA row, the high half for an odd one; 0x0c gives 0x00
            sel_base = parity ? 0x01000c0cu : 0x0c0c0100u;
            sel_step = parity ? 0x02020000u : 0x00000202u;
        }
        __device__ __forceinline__ void bind_bitmap(const uint32_t *h) { header = h; }
    };
    __device__ static __forceinline__ Idx load_idx(const Lane &L, uint32_t step)
    {
        Idx I;
        I.ids = L.load_idx(step);
        const const_u32_ptr h = as_const(L.header) + size_t(step) * 8u;      // uniform: scalar loads
#pragma unroll
        for (int i = 0; i < 4; ++i) I.h.d[i] = h[i];
        I.h.counts = h[4]; I.h.first = h[5];
        return I;
    }
    template <class GT>
    __device__ static __forceinline__ void load_tile(const Lane &L, uint32_t, const Idx &I, const GT &gat,
                                                     BVec &b0, BVec &b1, BVec &b2, BVec &b3, AVec &a)
    {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t *src = reinterpret_cast<const uint32_t *>(gat.row(I.ids[q]));
            b0[q] = src[0];
            if constexpr (V > 1) b1[q] = src[16];
            if constexpr (V > 2) b2[q] = src[32];
            if constexpr (V > 3) b3[q] = src[48];
        }
        const uint32_t w = L.word == 0u ? I.h.d[0] : L.word == 1u ? I.h.d[1] : L.word == 2u ? I.h.d[2] : I.h.d[3];
        const uint32_t before = __builtin_amdgcn_ubfe(I.h.counts, 8u * L.word, 8u) + uint32_t(__builtin_popcount(w & L.low_mask));
        a.bits = (w >> L.shift) & 15u;
        const char *vals = reinterpret_cast<const char *>(L.a_src_base());
        a.stored = *reinterpret_cast<const u32x2_unaligned *>(vals + 2u * size_t(I.h.first + before));
    }
    __device__ static __forceinline__ u32x4 sparse_operand(const Lane &L, const AVec &a)
    {
        // element i of the four sits at stored position (set bits below bit i), if its bit is set
        const uint32_t n1 = a.bits & 1u, n2 = uint32_t(__builtin_popcount(a.bits & 3u)), n3 = uint32_t(__builtin_popcount(a.bits & 7u));
        const uint32_t none = 0x0c0c0c0cu;
        const uint32_t s0 = (a.bits & 1u) ? L.sel_base : none;
        const uint32_t s1 = (a.bits & 2u) ? L.sel_base + n1 * L.sel_step : none;
        const uint32_t s2 = (a.bits & 4u) ? L.sel_base + n2 * L.sel_step : none;
        const uint32_t s3 = (a.bits & 8u) ? L.sel_base + n3 * L.sel_step : none;
        u32x4 aw;
        aw[0] = __builtin_amdgcn_perm(a.stored[1], a.stored[0], s0);
        aw[1] = __builtin_amdgcn_perm(a.stored[1], a.stored[0], s1);
        aw[2] = __builtin_amdgcn_perm(a.stored[1], a.stored[0], s2);
        aw[3] = __builtin_amdgcn_perm(a.stored[1], a.stored[0], s3);
        return aw;
    }
    __device__ static __forceinline__ void mma(const Lane &L, const BVec &b0, const BVec &b1, const BVec &b2,
                                               const BVec &b3, const AVec &a, f32x4 (&acc)[V])
    {
        const u32x4 av = sparse_operand(L, a);
        acc[0] = HalfOps<BF>::mfma(av, b0, acc[0]);
        if constexpr (V > 1) acc[1] = HalfOps<BF>::mfma(av, b1, acc[1]);
        if constexpr (V > 2) acc[2] = HalfOps<BF>::mfma(av, b2, acc[2]);
        if constexpr (V > 3) acc[3] = HalfOps<BF>::mfma(av, b3, acc[3]);
    }
};
template <class TT> struct TileTraits { static constexpr bool kBitmap = false; };
template <int V, bool BF> struct TileTraits<Fp16TileDWB<V, BF>> { static constexpr bool kBitmap = true; };

// fp32 storage ("tf32" build of the reference): 8x8 tiles, v_mfma_f32_16x16x4_f32.
// MFMA rows 0..7 are the window rows, rows 8..15 zero; lane (g, j) supplies k = g
// and k = g + 4 of a tile and V contiguous features.
//   ids per step, lane order: [g][2] = (id g, id g+4): 8 bytes per lane.
//   tiles per step, lane order: [row r][g][window][2] = (a[r][g], a[r][g+4]) per window.
template <int V_, int G_>
struct Fp32Tile {
    static constexpr int V = V_, G = G_;
    static constexpr int kBlockFeat = 16 * V;
    static constexpr int kLaneFeat = V;
    static constexpr int kElem = 4;
    typedef typename Vec<V>::type BVec;
    typedef u32x2 Idx;                             // two column ids per lane per step
    typedef typename Vec<2 * G>::type AVec;

    struct Lane {
        uint32_t g, j;
        uint32_t a_mask;                           // all ones for MFMA rows 0..7, else 0
        const uint32_t *a_src;
        const uint32_t *idx_src;
        __device__ __forceinline__ void init(uint32_t lane, const void *tiles, const uint32_t *ids)
        {
            g = lane >> 4; j = lane & 15u;
            a_mask = j < 8u ? 0xFFFFFFFFu : 0u;
            a_src = reinterpret_cast<const uint32_t *>(tiles) + ((j & 7u) * 8u + g * 2u) * G;
            idx_src = ids + g * 2u;
        }
    };
    __device__ static __forceinline__ Idx load_idx(const Lane &L, uint32_t step)
    {
        return *reinterpret_cast<const u32x2 *>(L.idx_src + size_t(step) * 8u);
    }
    template <class GT>
    __device__ static __forceinline__ void load_tile(const Lane &L, uint32_t step, const Idx idx, const GT &gat,
                                                     BVec &b0, BVec &b1, BVec &, BVec &, AVec &a)
    {
        b0 = *reinterpret_cast<const BVec *>(gat.row(idx[0]));
        b1 = *reinterpret_cast<const BVec *>(gat.row(idx[1]));
        a = *reinterpret_cast<const AVec *>(L.a_src + size_t(step) * (64u * G));
    }
    template <int p> __device__ static __forceinline__ float word(const BVec &v)
    {
        // (a bit_cast applied directly to a vector element reads element 0: copy first)
        uint32_t w;
        if constexpr (V == 1) w = v; else w = v[p];
        return __builtin_bit_cast(float, w);
    }
    template <int W0, int p>
    __device__ static __forceinline__ void mma_one(const float a, const BVec &b, f32x4 (&acc)[G * V])
    {
        if constexpr (p < V) acc[W0 * V + p] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, word<p>(b), acc[W0 * V + p], 0, 0, 0);
    }
    template <int W0>
    __device__ static __forceinline__ void mma_window(const Lane &L, const BVec &b0, const BVec &b1, const AVec &a,
                                                      f32x4 (&acc)[G * V])
    {
        if constexpr (W0 < G) {
            const uint32_t w0 = a[2 * W0] & L.a_mask, w1 = a[2 * W0 + 1] & L.a_mask;
            const float a0 = __builtin_bit_cast(float, w0), a1 = __builtin_bit_cast(float, w1);
            // first half of k for every accumulator, then the second: an MFMA does not read the
            // result of the one right in front of it
            mma_one<W0, 0>(a0, b0, acc); mma_one<W0, 1>(a0, b0, acc); mma_one<W0, 2>(a0, b0, acc); mma_one<W0, 3>(a0, b0, acc);
            mma_one<W0, 0>(a1, b1, acc); mma_one<W0, 1>(a1, b1, acc); mma_one<W0, 2>(a1, b1, acc); mma_one<W0, 3>(a1, b1, acc);
        }
    }
    __device__ static __forceinline__ void mma(const Lane &L, const BVec &b0, const BVec &b1, const BVec &,
                                               const BVec &, const AVec &a, f32x4 (&acc)[G * V])
    {
        mma_window<0>(L, b0, b1, a, acc);
        mma_window<1>(L, b0, b1, a, acc);
    }
    // acc[W0*V + p][e]: MFMA row 4g+e (a window row when g < 2), feature lane_feat + p.
    template <int W0>
    __device__ static __forceinline__ void store_window(const Lane &L, const f32x4 (&acc)[G * V], char *c_lane,
                                                        size_t row_bytes, uint32_t row0, uint32_t rows, bool active)
    {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t row = row0 + 4u * L.g + e;
            uint32_t out[V];
#pragma unroll
            for (int p = 0; p < V; ++p) { const float f = acc[W0 * V + p][e]; out[p] = __builtin_bit_cast(uint32_t, f); }
            if (active && L.g < 2u && row < rows) store_words<V>(c_lane + size_t(row) * row_bytes, out);
        }
    }
    __device__ static __forceinline__ void zero_rows(const Lane &L, char *c_lane, size_t row_bytes, uint32_t r_begin,
                                                     uint32_t r_end, bool active)
    {
        uint32_t z[V];
#pragma unroll
        for (int i = 0; i < V; ++i) z[i] = 0u;
        if (!active) return;
        for (uint32_t r = r_begin + L.g; r < r_end; r += 4u) store_words<V>(c_lane + size_t(r) * row_bytes, z);
    }
};

// fp32 storage, single windows, tiles read as bitmap + stored values (the fp32 form of Fp16TileDWB above; the
// reference's BTCF_MTX with 8 x 8 tiles, src/utils/class.h:55-67 and src/utils/convert.h:83-101): per tile 64 bits,
// bit 8 r + k set for a stored element, and the stored elements of all tiles one after the other in ascending bit
// order.  Lane (g, j) needs a[j % 8][g] and a[j % 8][g + 4]: it counts the tile's bits in front of each, loads the
// two words from there and keeps those whose bit is set.  A power-law graph stores 8 of a tile's 64 elements:
// 48 bytes instead of 256.
//   header per step (uniform, scalar loads): the two bitmap words (rows 0..3, rows 4..7), the position of the
//   tile's first stored element, the number of its stored elements.
template <int V_>
struct Fp32TileB : Fp32Tile<V_, 1> {
    typedef Fp32Tile<V_, 1> Base;
    static constexpr int V = V_, G = 1;
    typedef typename Base::BVec BVec;
    struct Idx { u32x2 ids; uint32_t lo, hi, first; };
    struct AVec { uint32_t w0, w1, keep0, keep1; };    // the two words at the lane's positions; all ones where the bit is set
    struct Lane : Base::Lane {
        const uint32_t *header;                        // 4 words per step
        const uint32_t *vals;
        uint32_t upper, shift, low_mask;               // rows 4..7; the lane's first bit inside its word; the bits below it
        __device__ __forceinline__ void init(uint32_t lane, const void *values, const uint32_t *ids)
        {
            Base::Lane::init(lane, values, ids);
            vals = static_cast<const uint32_t *>(values);
            const uint32_t r = this->j & 7u;
            upper = r >> 2;
            shift = 8u * (r & 3u) + this->g;
            low_mask = (1u << shift) - 1u;
        }
        __device__ __forceinline__ void bind_bitmap(const uint32_t *h) { header = h; }
    };
    __device__ static __forceinline__ Idx load_idx(const Lane &L, uint32_t step)
    {
        Idx I;
        I.ids = *reinterpret_cast<const u32x2 *>(L.idx_src + size_t(step) * 8u);
        const const_u32_ptr h = as_const(L.header) + size_t(step) * 4u;      // uniform: scalar loads
        I.lo = h[0]; I.hi = h[1]; I.first = h[2];
        return I;
    }
    template <class GT>
    __device__ static __forceinline__ void load_tile(const Lane &L, uint32_t, const Idx &I, const GT &gat,
                                                     BVec &b0, BVec &b1, BVec &, BVec &, AVec &a)
    {
        b0 = *reinterpret_cast<const BVec *>(gat.row(I.ids[0]));
        b1 = *reinterpret_cast<const BVec *>(gat.row(I.ids[1]));
        const uint32_t w = L.upper ? I.hi : I.lo;
        const uint32_t before0 = (L.upper ? uint32_t(__builtin_popcount(I.lo)) : 0u) + uint32_t(__builtin_popcount(w & L.low_mask));
        const uint32_t four = (w >> L.shift) & 31u;                      // bits of columns g .. g + 4
        const uint32_t before1 = before0 + uint32_t(__builtin_popcount(four & 15u));
        // (a position behind the tile's last element, for a bit that is not set, still lies inside the array: it
        // ends with one spare element)
        const uint32_t *src = L.vals + size_t(I.first);
        a.w0 = src[before0];
        a.w1 = src[before1];
        a.keep0 = ((four & 1u) ? 0xFFFFFFFFu : 0u) & L.a_mask;
        a.keep1 = ((four & 16u) ? 0xFFFFFFFFu : 0u) & L.a_mask;
    }
    __device__ static __forceinline__ void mma(const Lane &, const BVec &b0, const BVec &b1, const BVec &,
                                               const BVec &, const AVec &a, f32x4 (&acc)[V])
    {
        const uint32_t w0 = a.w0 & a.keep0, w1 = a.w1 & a.keep1;
        const float a0 = __builtin_bit_cast(float, w0), a1 = __builtin_bit_cast(float, w1);
        Base::template mma_one<0, 0>(a0, b0, acc); Base::template mma_one<0, 1>(a0, b0, acc);
        Base::template mma_one<0, 2>(a0, b0, acc); Base::template mma_one<0, 3>(a0, b0, acc);
        Base::template mma_one<0, 0>(a1, b1, acc); Base::template mma_one<0, 1>(a1, b1, acc);
        Base::template mma_one<0, 2>(a1, b1, acc); Base::template mma_one<0, 3>(a1, b1, acc);
    }
};
template <int V> struct TileTraits<Fp32TileB<V>> { static constexpr bool kBitmap = true; };

// ---------------------------------------------------------------------------
// Main kernel: one wave per (step range, feature block).
// ---------------------------------------------------------------------------
// State of the unit walk (all wave-uniform, kept in scalar registers).  A unit is
// one window, or two adjacent windows with one column list (bit 0 of unitRow).
struct UnitWalk {
    uint32_t u;            // current unit
    uint32_t ustart, uend; // its step span
    uint32_t row;          // its first matrix row | paired bit
    uint32_t next_row;     // first row of the next unit (or rows)
    uint32_t seg_start, seg_end;   // part of the span inside this wave's range
};

// Windows of a unit: the low bits of its row word hold the count less one (1: a pair; the
// LDS-panel kernels also have units of three and four windows).
template <class TT>
__device__ __forceinline__ uint32_t unit_windows(const uint32_t row_word)
{
    return TT::G > 1 ? (row_word & 3u) + 1u : 1u;
}

// Tile classes of the LDS-panel kernels whose lanes own one feature per accumulator (feature 16 p + j of the
// block) keep in `f_valid` how many features of their block lie inside a feature dimension that ends inside the
// block; other classes have no such member and need whole blocks.
template <class LaneT, class = void> struct HasValidCount { static constexpr bool value = false; };
template <class LaneT> struct HasValidCount<LaneT, decltype(void(LaneT::f_valid))> { static constexpr bool value = true; };
template <class TT>
__device__ __forceinline__ void set_valid_features(typename TT::Lane &L, uint32_t N, uint32_t first)
{
    if constexpr (HasValidCount<typename TT::Lane>::value) {
        const uint32_t left = N > first ? N - first : 0u;
        L.f_valid = left < uint32_t(TT::kBlockFeat) ? left : uint32_t(TT::kBlockFeat);
    }
}
// First feature of feature block fb of the LDS-panel kernels.  A feature dimension of one block at least that ends
// inside its last block: that block is moved back to end with the row - features N - block .. N - 1, all of them
// there, every load inside the row - and computes the features it shares with the block in front of it a second
// time (same tiles, same rows of B, same order: the same bits).
__device__ __forceinline__ uint32_t panel_block_first_feature(uint32_t fb, uint32_t block, uint32_t N)
{
    const uint32_t first = fb * block;
    return (first + block > N && N >= block) ? N - block : first;
}

// An odd feature dimension of a 16-bit type (wide-load layout, one word per lane): the lane whose first feature is
// the last one owns that feature alone.  It loads its word one half early - the two last features of the row, so
// that no load leaves the row - and shifts it down, and it stores one half.  Returns the bytes to take off the
// lane's offset into a row of B.  (The launch covers three features at least.)
template <class LaneT, class = void> struct HasHalfLane { static constexpr bool value = false; };
template <class LaneT> struct HasHalfLane<LaneT, decltype(void(LaneT::half_shift))> { static constexpr bool value = true; };
template <class TT>
__device__ __forceinline__ uint32_t mark_half_lane(typename TT::Lane &L, uint32_t N, uint32_t feat)
{
    if constexpr (HasHalfLane<typename TT::Lane>::value && TT::kLaneFeat == 2) {
        if ((N & 1u) && feat + 1u == N) { L.half_shift = 16u; return 2u; }
    }
    return 0u;
}

// Stores the windows W0 .. of a unit (window w covers rows row0 + 8 w .. + 7).
template <class TT, int W0 = 0, int NACC>
__device__ __forceinline__ void store_unit(const typename TT::Lane &L, const f32x4 (&acc)[NACC], char *c_lane,
                                           size_t row_bytes, uint32_t row0, uint32_t nwin, uint32_t rows, bool active)
{
    if (uint32_t(W0) < nwin)
        TT::template store_window<W0>(L, acc, c_lane, row_bytes, row0 + uint32_t(W0) * kRowWindow, rows, active);
    if constexpr (W0 + 1 < TT::G) store_unit<TT, W0 + 1>(L, acc, c_lane, row_bytes, row0, nwin, rows, active);
}

// WAVES: the largest workgroup the kernel is launched with (4, or 8 for the aligned partition); with
// 8 waves half as many workgroups share a compute unit, the waves per SIMD stay what they are.
template <class TT, int P, bool NARROW, int WAVES = kMaxWavesPerGroup>
__global__ __launch_bounds__(WAVES * 64, (P <= 4 ? 4 : 2) * kMaxWavesPerGroup / WAVES)
void spmm_mfma_kernel(const KernelArgs ka)
{
    constexpr int G = TT::G, V = TT::V, NACC = G * V;
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t range, fb;
    if (ka.xcd_split) {
        // Two, four or eight feature blocks, each with XCDs of its own.  The hardware hands consecutive
        // workgroups to the eight XCDs in turn and every XCD has an L2 of its own: with two feature blocks
        // workgroups 0..3 mod 8 take block 0 and workgroups 4..7 mod 8 block 1, so that an L2 only ever
        // holds one part of every B row it caches - that many more rows of a B that does not fit.
        const uint32_t waves = blockDim.x >> 6, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const uint32_t per_fb = 8u / ka.n_feat_blocks;                  // XCDs per feature block: 4, 2, 1
        const uint32_t xcd = blockIdx.x & 7u, set = blockIdx.x >> 3;
        fb = xcd / per_fb;
        range = (set * per_fb + (xcd - fb * per_fb)) * waves + wave;
        if (range >= ka.n_ranges) return;
    } else {
        const uint32_t item = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
        if (item >= ka.n_ranges * ka.n_feat_blocks) return;
        range = item / ka.n_feat_blocks;
        fb = item - range * ka.n_feat_blocks;
    }
    const const_u32_ptr rd = as_const(ka.ranges) + size_t(range) * kRangeWords;
    const const_u32_ptr unitOffset = as_const(ka.unitOffset);
    const const_u32_ptr unitRow = as_const(ka.unitRow);
    const uint32_t t0 = rd[0], t1 = rd[1];
    const uint32_t head_slot = rd[3], tail_slot = rd[4];
    const uint32_t head_split = rd[5], tail_split = rd[6];
    // 1 (for every wave of the workgroup alike): the range is one piece of a unit, as are those of the
    // other waves, and the workgroup adds the pieces in LDS before one sum goes to the slot of wave 0;
    // 2: the pieces are the whole unit, and wave 0 stores it
    const uint32_t combine = rd[7];
    const uint32_t U = ka.n_units, rows = ka.rows;

    typename TT::Lane L;
    L.init(lane, ka.tiles, ka.ids);
    if constexpr (TileTraits<TT>::kBitmap) L.bind_bitmap(ka.bm_header);
    const uint32_t feat = fb * TT::kBlockFeat + L.j * TT::kLaneFeat;
    const bool active = feat < ka.N;
    const size_t row_bytes = size_t(ka.ld) * TT::kElem;
    char *c_lane = reinterpret_cast<char *>(ka.C) + size_t(feat) * TT::kElem;
    Gather<NARROW> gat;
    gat.base = reinterpret_cast<const char *>(ka.B);
    gat.row_bytes = uint32_t(row_bytes);
    gat.lane_off = active ? feat * TT::kElem : 0u;     // lanes past N read (and drop) the row start
    // (a lane that owns the last feature of an odd N alone reads one half early; the host launches odd N from
    // three features on, so that lane's first feature is not the launch's first)
    gat.lane_off -= mark_half_lane<TT>(L, ka.N, feat);

    f32x4 acc[NACC];
#pragma unroll
    for (int p = 0; p < NACC; ++p) acc[p] = f32x4{0.f, 0.f, 0.f, 0.f};

    const uint32_t tlast = t1 - 1u;
    typedef typename TT::BVec BVec;
    typedef typename TT::AVec AVec;
#define HSPMM_FOR_STAGES(X) \
    X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7)
#define HSPMM_DECL(k) BVec b0_##k, b1_##k, b2_##k, b3_##k; AVec a_##k; typename TT::Idx I##k;
#define HSPMM_REGS(k) b0_##k, b1_##k, b2_##k, b3_##k, a_##k
    HSPMM_FOR_STAGES(HSPMM_DECL)
#define HSPMM_PRO_IDX(k) if constexpr (P > k) I##k = TT::load_idx(L, umin32(t0 + k, tlast));
#define HSPMM_PRO_TILE(k) if constexpr (P > k) { \
        TT::load_tile(L, umin32(t0 + k, tlast), I##k, gat, HSPMM_REGS(k)); \
        I##k = TT::load_idx(L, umin32(t0 + P + k, tlast)); \
        __builtin_amdgcn_sched_barrier(0); }
    // The order of the loads below must be the order of the steady state (the
    // compiler derives the steady state's wait counts from both ways into the
    // loop), hence the scheduling barriers.
    HSPMM_FOR_STAGES(HSPMM_PRO_IDX)
    __builtin_amdgcn_sched_barrier(0);
    // The unit the range starts in: looked up while the first ids are on their way (they depend on the range's
    // bounds alone; in front of them these lookups were one more trip to memory before the first gather).
    UnitWalk ww;
    ww.u = rd[2];
    ww.ustart = unitOffset[ww.u];
    ww.uend = unitOffset[ww.u + 1u];
    ww.row = unitRow[ww.u];
    ww.next_row = (ww.u + 1u < U) ? (unitRow[ww.u + 1u] & ~7u) : rows;
    ww.seg_start = t0;
    ww.seg_end = umin32(ww.uend, t1);
    const uint32_t first_row = unitRow[0] & ~7u;
    __builtin_amdgcn_sched_barrier(0);
    HSPMM_FOR_STAGES(HSPMM_PRO_TILE)
    // Rows before the first effective window belong to the wave that starts at step 0.
    if (t0 == 0u) TT::zero_rows(L, c_lane, row_bytes, 0u, first_row, active);

    // MFMAs of `step` from its registers, then the unit bookkeeping.
    auto compute = [&](const BVec &b0, const BVec &b1, const BVec &b2, const BVec &b3, const AVec &a,
                       const uint32_t step) __attribute__((always_inline)) {
        TT::mma(L, b0, b1, b2, b3, a, acc);
        if (step + 1u == ww.seg_end) {
            const uint32_t row0 = ww.row & ~7u;
            const bool paired = (G > 1) && (ww.row & 1u);
            const bool complete = (ww.seg_start == ww.ustart) && (ww.seg_end == ww.uend);
            if (complete) {
                TT::template store_window<0>(L, acc, c_lane, row_bytes, row0, rows, active);
                if constexpr (G > 1) {
                    if (paired) TT::template store_window<G - 1>(L, acc, c_lane, row_bytes, row0 + kRowWindow, rows, active);
                }
            } else {
                const bool head = ww.seg_start == t0;
                const uint32_t slot = head ? head_slot : tail_slot;
                if (slot != kIdxMax && !combine) {
                    f32x4 *slot_sums = reinterpret_cast<f32x4 *>(ka.scratch) + (size_t(slot) * ka.n_feat_blocks + fb) * (NACC * 64u);
                    if (!ka.arrive) {
                        f32x4 *dst = slot_sums + lane;
#pragma unroll
                        for (int p = 0; p < NACC; ++p) dst[p * 64] = acc[p];
                    } else {
                        // The wave that brings the last partial sum of a cut unit adds all of
                        // them, in range order (so the result does not depend on who is last),
                        // and stores the unit.  The partial sums cross the L2s of different
                        // XCDs: they are written and read with device-scope accesses (which go
                        // past the L2 of the XCD), the writes are waited for before the arrival
                        // is counted, and no whole-cache write-back or invalidate is needed.
                        const __amdgpu_buffer_rsrc_t out = device_scope_buffer(slot_sums);
#pragma unroll
                        for (int p = 0; p < NACC; ++p) store_device_scope(out, lane * 16u + uint32_t(p) * 1024u, acc[p]);
                        wait_stores_acknowledged();
                        const uint32_t entry = head ? head_split : tail_split;
                        const uint32_t *fx = ka.split + size_t(entry) * kFixWords;
                        uint32_t *ctr = ka.arrive + size_t(entry) * ka.n_feat_blocks + fb;
                        uint32_t old = 0;
                        if (lane == 0)
                            old = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        old = __builtin_amdgcn_readfirstlane(old);
                        asm volatile("" ::: "memory");      // the loads below stay behind the count they depend on
                        const uint32_t sb = fx[1], sc = fx[2];
                        if (old + 1u == sc) {
#pragma unroll
                            for (int p = 0; p < NACC; ++p) acc[p] = f32x4{0.f, 0.f, 0.f, 0.f};
                            for (uint32_t i = 0; i < sc; ++i) {
                                const uint32_t sl = ka.fix_slots[sb + i];
                                const __amdgpu_buffer_rsrc_t in = device_scope_buffer(
                                    reinterpret_cast<const f32x4 *>(ka.scratch) + (size_t(sl) * ka.n_feat_blocks + fb) * (NACC * 64u));
#pragma unroll
                                for (int p = 0; p < NACC; ++p) acc[p] += load_device_scope(in, lane * 16u + uint32_t(p) * 1024u);
                            }
                            TT::template store_window<0>(L, acc, c_lane, row_bytes, row0, rows, active);
                            if constexpr (G > 1) {
                                if (paired) TT::template store_window<G - 1>(L, acc, c_lane, row_bytes, row0 + kRowWindow, rows, active);
                            }
                            if (lane == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                    }
                }
            }
            if (ww.seg_end == ww.uend) {
                // this wave holds the unit's last step: it also clears the empty
                // windows that follow (rows up to the next effective window)
                const uint32_t gap_begin = row0 + (paired ? 2u * kRowWindow : kRowWindow);
                if (gap_begin < ww.next_row) TT::zero_rows(L, c_lane, row_bytes, gap_begin, ww.next_row, active);
            }
            if (!combine) {                     // (a combining wave ends here and still needs its sums)
#pragma unroll
                for (int p = 0; p < NACC; ++p) acc[p] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            // next unit (the reads are clamped; values past the end are not used)
            ++ww.u;
            ww.ustart = ww.uend;
            ww.uend = unitOffset[umin32(ww.u + 1u, U)];
            ww.row = unitRow[umin32(ww.u, U - 1u)];
            ww.next_row = (ww.u + 1u < U) ? (unitRow[ww.u + 1u] & ~7u) : rows;
            ww.seg_start = ww.seg_end;
            ww.seg_end = umin32(ww.uend, t1);
        }
    };

    // Steady state: every stage computes its step and reloads its registers with
    // the step P further on, without conditions, so that the wait in front of a
    // stage's MFMAs leaves the loads of the P-1 younger stages in flight.
    uint32_t t = t0;
    for (; t + 2u * P <= t1; t += P) {
#define HSPMM_STEADY(k) if constexpr (P > k) { \
        compute(HSPMM_REGS(k), t + k); \
        TT::load_tile(L, t + k + P, I##k, gat, HSPMM_REGS(k)); \
        I##k = TT::load_idx(L, umin32(t + k + 2u * P, tlast)); \
        __builtin_amdgcn_sched_barrier(0); }
        HSPMM_FOR_STAGES(HSPMM_STEADY)
    }
    // Drain: fewer than 2P steps are left; loads stop at the end of the range.
    for (; t < t1; t += P) {
#define HSPMM_DRAIN(k) if constexpr (P > k) { \
        if (t + k < t1) compute(HSPMM_REGS(k), t + k); \
        if (t + k + P < t1) { \
            TT::load_tile(L, t + k + P, I##k, gat, HSPMM_REGS(k)); \
            I##k = TT::load_idx(L, umin32(t + k + 2u * P, tlast)); } }
        HSPMM_FOR_STAGES(HSPMM_DRAIN)
    }
    if (combine) {
        // every wave of the workgroup is here with the sums of its piece: wave 0 adds them in range order
        __shared__ f32x4 pieces[(WAVES - 1) * NACC * 64];
        const uint32_t wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
        if (wave) {
#pragma unroll
            for (int p = 0; p < NACC; ++p) pieces[((wave - 1u) * NACC + p) * 64u + lane] = acc[p];
        }
        __syncthreads();
        if (wave == 0u) {
            for (uint32_t w = 1; w < n_waves; ++w) {
#pragma unroll
                for (int p = 0; p < NACC; ++p) acc[p] += pieces[((w - 1u) * NACC + p) * 64u + lane];
            }
            if (combine == 2u) {
                const uint32_t row = unitRow[rd[2]];
                store_unit<TT>(L, acc, c_lane, row_bytes, row & ~7u, unit_windows<TT>(row), rows, active);
            } else {
                f32x4 *dst = reinterpret_cast<f32x4 *>(ka.scratch) + size_t(head_slot) * (NACC * 64u) + lane;
#pragma unroll
                for (int p = 0; p < NACC; ++p) dst[p * 64] = acc[p];
            }
        }
    }
#undef HSPMM_DRAIN
#undef HSPMM_STEADY
#undef HSPMM_PRO_TILE
#undef HSPMM_PRO_IDX
#undef HSPMM_REGS
#undef HSPMM_DECL
#undef HSPMM_FOR_STAGES
}

// ---------------------------------------------------------------------------
// Second kernel: adds, in range order, the fp32 partial sums of every unit
// whose steps were cut across ranges, and stores its window(s).
// ---------------------------------------------------------------------------
template <class TT>
__global__ __launch_bounds__(kMaxWavesPerGroup * 64)
void spmm_fixup_kernel(const KernelArgs ka)
{
    constexpr int G = TT::G, V = TT::V, NACC = G * V;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t item = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (item >= ka.n_split * ka.n_feat_blocks) return;
    const uint32_t entry = item / ka.n_feat_blocks;
    const uint32_t fb = item - entry * ka.n_feat_blocks;
    // one table entry per cut unit, or (uniform_chunks) every unit cut the same number of ways
    const bool uniform = ka.uniform_chunks != 0u;
    const uint32_t *fx = ka.split + size_t(uniform ? 0u : entry) * kFixWords;
    const uint32_t u = uniform ? entry : fx[0];
    const uint32_t sb = uniform ? entry * ka.uniform_chunks : fx[1];
    const uint32_t sc = uniform ? ka.uniform_chunks : fx[2];

    typename TT::Lane L;
    L.init(lane, ka.tiles, ka.ids);
    // (the sums of the LDS-panel kernels: their last feature block may have been moved back, see above)
    const uint32_t first = uniform ? panel_block_first_feature(fb, uint32_t(TT::kBlockFeat), ka.N) : fb * uint32_t(TT::kBlockFeat);
    set_valid_features<TT>(L, ka.N, first);
    const uint32_t feat = first + L.j * TT::kLaneFeat;
    const bool active = feat < ka.N;
    (void)mark_half_lane<TT>(L, ka.N, feat);
    const size_t row_bytes = size_t(ka.ld) * TT::kElem;
    char *c_lane = reinterpret_cast<char *>(ka.C) + size_t(feat) * TT::kElem;

    f32x4 acc[NACC];
#pragma unroll
    for (int p = 0; p < NACC; ++p) acc[p] = f32x4{0.f, 0.f, 0.f, 0.f};
    // the additions keep the slot order; the loads of four slots are in flight together
#pragma unroll 4
    for (uint32_t i = 0; i < sc; ++i) {
        const uint32_t slot = uniform ? sb + i : ka.fix_slots[sb + i];
        const f32x4 *src = reinterpret_cast<const f32x4 *>(ka.scratch) +
                           (size_t(slot) * ka.n_feat_blocks + fb) * (NACC * 64u) + lane;
#pragma unroll
        for (int p = 0; p < NACC; ++p) acc[p] += src[p * 64];
    }
    const uint32_t row = ka.unitRow[u];
    store_unit<TT>(L, acc, c_lane, row_bytes, row & ~7u, unit_windows<TT>(row), ka.rows, active);
}

// ---------------------------------------------------------------------------
// Launch helpers (host).  The instantiations are spread over several source
// files (one per element type and unit width) so that they compile in parallel.
// ---------------------------------------------------------------------------
template <class TT, bool NARROW>
static hipError_t launch_main_p(const KernelArgs &ka, int prefetch, dim3 grid, dim3 block, hipStream_t s)
{
    constexpr int kDefault = default_prefetch(TT::kElem, TT::G, TT::V);
    if (block.x > 64u * kMaxWavesPerGroup) {
        // workgroups of kAlignedGroupWaves waves (aligned partition): 32-bit offsets, the default depth
        if constexpr (NARROW) {
            if (prefetch != kDefault) return hipErrorInvalidValue;
            spmm_mfma_kernel<TT, kDefault, true, kAlignedGroupWaves><<<grid, block, 0, s>>>(ka);
            return hipGetLastError();
        }
        return hipErrorInvalidValue;
    }
#ifndef HSPMM_EXPERIMENTAL
    if constexpr (!NARROW) {
        // 64-bit gather offsets (a B of 4 GiB or more): the default depth
        if (prefetch != kDefault) return hipErrorInvalidValue;
        spmm_mfma_kernel<TT, kDefault, false><<<grid, block, 0, s>>>(ka);
        return hipGetLastError();
    }
#endif
    switch (prefetch) {
    case 2: spmm_mfma_kernel<TT, 2, NARROW><<<grid, block, 0, s>>>(ka); break;
    case 3: spmm_mfma_kernel<TT, 3, NARROW><<<grid, block, 0, s>>>(ka); break;
    case 4: spmm_mfma_kernel<TT, 4, NARROW><<<grid, block, 0, s>>>(ka); break;
#ifdef HSPMM_EXPERIMENTAL
    case 1: spmm_mfma_kernel<TT, 1, NARROW><<<grid, block, 0, s>>>(ka); break;
    case 6: spmm_mfma_kernel<TT, 6, NARROW><<<grid, block, 0, s>>>(ka); break;
    case 8: spmm_mfma_kernel<TT, 8, NARROW><<<grid, block, 0, s>>>(ka); break;
#endif
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <class TT>
static hipError_t launch_tt(const KernelArgs &ka, int prefetch, bool narrow, int waves_per_group, hipStream_t s,
                            hipEvent_t mid)
{
    const uint32_t items = ka.n_ranges * ka.n_feat_blocks;
    const dim3 block(64u * waves_per_group);
    // (feature blocks dealt out by XCD: sets of eight workgroups, 8 / feature blocks of them per block)
    const uint32_t per_set = (8u / (ka.xcd_split ? ka.n_feat_blocks : 1u)) * uint32_t(waves_per_group);
    const dim3 grid(ka.xcd_split ? 8u * ((ka.n_ranges + per_set - 1u) / per_set)
                                  : (items + waves_per_group - 1) / waves_per_group);
    hipError_t e = narrow ? launch_main_p<TT, true>(ka, prefetch, grid, block, s)
                          : launch_main_p<TT, false>(ka, prefetch, grid, block, s);
    if (e != hipSuccess || ka.n_split == 0 || ka.arrive) return e;
    if (mid && (e = hipEventRecord(mid, s)) != hipSuccess) return e;
    const uint32_t fitems = ka.n_split * ka.n_feat_blocks;
    const uint32_t fwaves = uint32_t(std::min(waves_per_group, kMaxWavesPerGroup));
    const dim3 fgrid((fitems + fwaves - 1) / fwaves);
    spmm_fixup_kernel<TT><<<fgrid, dim3(64u * fwaves), 0, s>>>(ka);
    return hipGetLastError();
}

template <template <int, int> class TTV, int G>
static hipError_t launch_v(const KernelArgs &ka, int V, int prefetch, bool narrow, int waves_per_group, hipStream_t s,
                           hipEvent_t mid)
{
    if (V == 4) return launch_tt<TTV<4, G>>(ka, prefetch, narrow, waves_per_group, s, mid);
    if (V == 2) return launch_tt<TTV<2, G>>(ka, prefetch, narrow, waves_per_group, s, mid);
    return launch_tt<TTV<1, G>>(ka, prefetch, narrow, waves_per_group, s, mid);
}

template <template <int, int> class TTV>
static hipError_t launch_g(const KernelArgs &ka, int G, int V, int prefetch, bool narrow, int waves_per_group,
                           hipStream_t s, hipEvent_t mid)
{
    return G == 2 ? launch_v<TTV, 2>(ka, V, prefetch, narrow, waves_per_group, s, mid)
                  : launch_v<TTV, 1>(ka, V, prefetch, narrow, waves_per_group, s, mid);
}

template <int V, int G> using Fp16X4 = Fp16Tile<V, G, false>;
template <int V, int G> using Fp16DW = Fp16TileDW<V, G, false>;
template <int V, int G> using Bf16X4 = Fp16Tile<V, G, true>;
template <int V, int G> using Bf16DW = Fp16TileDW<V, G, true>;

}  // namespace hspmm
