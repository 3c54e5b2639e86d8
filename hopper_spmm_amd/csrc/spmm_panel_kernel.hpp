// gfx950 (MI355X) kernel family for matrices whose row windows touch a large share
// of all columns (pruned dense weights, block-clustered weights): the rows of B are
// staged through LDS once per workgroup and shared by all its waves, instead of
// every wave gathering its own copy from the L2 (spmm_mfma_kernel.hpp).  It serves
// the same entry point, the reference's fp16_spmm (reference src/fp16.cu:221-281),
// and what the reference sketches with its producer / consumer shared-memory ring
// (src/fp16.cu:56-175).
//
//   * Columns are cut into panels (256 columns for the kernels built on the 16-bit
//     MFMA, 128 for the fp32 MFMA forms).  The plan re-tiles every unit (a window,
//     or a group of adjacent windows with one column list) panel by panel: the
//     unit's columns inside a panel are condensed into steps of their own, so no
//     step straddles a panel; ids are row numbers inside the panel, packed the way
//     the tile type's address arithmetic wants them (PanelOps below).  poff[u][p]
//     is the first step of unit u in panel p.
//   * A workgroup owns up to NC consecutive units (one per consumer wave), one
//     block of 256 bytes of every B row (128 halves / 64 floats of the feature
//     dimension) and a contiguous chunk of panels.  Per panel its producer waves
//     copy the panel's slice of B (coalesced 16-byte loads) to LDS; every consumer
//     wave then runs the steps its unit has in the panel, reading the B rows of
//     its columns from LDS.
//   * Two LDS buffers and one barrier per panel: the producers fill the buffer of
//     panel p+1 while the consumers multiply panel p.
//   * The unit's tiles and ids stream from global memory through a small register
//     ring, as in the gather kernels.
//   * With more than one chunk of panels per unit, every chunk leaves fp32 partial
//     sums in scratch slots that spmm_fixup_kernel adds in chunk order.
#pragma once
#include <type_traits>
#include "spmm_mfma_kernel.hpp"

namespace hspmm {

typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));

// fp32 without the 8 -> 16 row padding of v_mfma_f32_16x16x4_f32 (single windows only):
// v_mfma_f32_4x4x1_16B_f32 multiplies 16 independent 4 x 1 by 1 x 4 blocks.  Block
// b = lane / 4 is rows 4 * (b / 8) .. + 3 of the window times features 4 * (b % 8) .. + 3
// of a group of 32 features; one instruction is one k (one B row) for 8 rows x 32
// features, all of it useful, at the rate of the big instruction.  The B row of a k
// is the same for all lanes, so its panel offset is a scalar.
//   tiles per step: the lane order of Fp32Tile, [row r][8 words: k = 0,4,1,5,2,6,3,7]:
//     a lane reads the 32 bytes of its row.
//   ids per step: four words, word g = offset of row g | offset of row g + 4 << 16
//     (offset = row inside the panel x 256); bits 0..3 of word 0: the panel jump.
struct Fp32Quad {
    static constexpr int V = 2, G = 1;             // two accumulators: features 0..31 and 32..63 of the block
    static constexpr int kBlockFeat = 64;
    static constexpr int kLaneFeat = 1;            // lane's feature = j (+ 32 for the second accumulator)
    static constexpr int kElem = 4;
    static constexpr bool kQuad = true;
    typedef u32x8 AVec;
    struct Lane {
        uint32_t g, j;                             // row quad (0, 1), feature inside the group of 32
        const uint32_t *a_src;
        const uint32_t *idx_src;
        __device__ __forceinline__ void init(uint32_t lane, const void *tiles, const uint32_t *ids)
        {
            g = lane >> 5; j = lane & 31u;
            a_src = reinterpret_cast<const uint32_t *>(tiles) + (4u * g + (lane & 3u)) * 8u;
            idx_src = ids;
        }
    };
    // acc[h][e]: window row 4g + e, feature 32h + j
    template <int W0>
    __device__ static __forceinline__ void store_window(const Lane &L, const f32x4 (&acc)[2], char *c_lane,
                                                        size_t row_bytes, uint32_t row0, uint32_t rows, bool active)
    {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t row = row0 + 4u * L.g + e;
            if (active && row < rows) {
                float *dst = reinterpret_cast<float *>(c_lane + size_t(row) * row_bytes);
                const float lo = acc[0][e], hi = acc[1][e];
                stream_store(dst, lo);
                stream_store(dst + 32, hi);
            }
        }
    }
    __device__ static __forceinline__ void zero_rows(const Lane &L, char *c_lane, size_t row_bytes, uint32_t r_begin,
                                                     uint32_t r_end, bool active)
    {
        if (!active) return;
        for (uint32_t r = r_begin + L.g; r < r_end; r += 2u) {
            float *dst = reinterpret_cast<float *>(c_lane + size_t(r) * row_bytes);
            stream_store(dst, 0.f);
            stream_store(dst + 32, 0.f);
        }
    }
};

// How a consumer wave of the panel kernel reads the ids and tiles of a step and runs it.
template <class TT>
struct PanelOps {
    static_assert(TT::kElem == 4, "the 16-bit types have ops of their own");
    static constexpr uint32_t kRows = kPanelRowsFp32;             // B rows per panel
    static constexpr uint32_t kPitch = kPanelRowBytes;            // bytes from one row of the LDS image to the next
    // a producer's 16 bytes of a B row: column piece c of the image row
    __device__ static __forceinline__ void write_piece(char *row, uint32_t c, const u32x4 x)
    {
        *reinterpret_cast<u32x4 *>(row + c * 16u) = x;
    }
    static constexpr uint32_t kRing = 6;                          // steps of tiles and ids in flight
    static constexpr int kLive = TT::G * TT::V;                   // accumulator registers the step loop keeps
    __device__ static __forceinline__ void fold(f32x4 (&)[kLive]) {}
    typedef uint32_t Idx;                                         // the lane's word of the step's four id words
    typedef typename TT::AVec AVec;
    __device__ static __forceinline__ Idx load_idx(const typename TT::Lane &L, const uint32_t *ids, uint32_t step)
    {
        return ids[size_t(step) * 4u + L.g];
    }
    __device__ static __forceinline__ AVec load_a(const typename TT::Lane &L, uint32_t step)
    {
        return *reinterpret_cast<const AVec *>(L.a_src + size_t(step) * (64u * TT::G));
    }
    __device__ static __forceinline__ uint32_t jump(const Idx I) { return __builtin_amdgcn_readfirstlane(I) >> 28; }
    // A step in two halves (see the consumer loop of spmm_panel_kernel): read_half<H> requests the
    // second operands of half H from LDS, mma_half<H> multiplies them.  Here the first half is the
    // whole step.  img: LDS byte offset of the lane's 16 bytes of row 0 of the current panel image.
    template <int H> struct Half { typename TT::BVec b0, b1; };
    template <int H>
    __device__ static __forceinline__ Half<H> read_half(const typename TT::Lane &, const char *smem, uint32_t img, const Idx I)
    {
        Half<H> B = {};
        if constexpr (H == 0) {
            B.b0 = *reinterpret_cast<const u32x4 *>(smem + img + (__builtin_amdgcn_ubfe(I, 0, 7) << 8));
            B.b1 = *reinterpret_cast<const u32x4 *>(smem + img + (__builtin_amdgcn_ubfe(I, 7, 7) << 8));
        }
        return B;
    }
    template <int H>
    __device__ static __forceinline__ void mma_half(const typename TT::Lane &L, const AVec &A, const Half<H> &B,
                                                    f32x4 (&acc)[kLive])
    {
        if constexpr (H == 0) {
            typename TT::BVec b2 = {}, b3 = {};
            TT::mma(L, B.b0, B.b1, b2, b3, A, acc);
        }
    }
    __device__ static __forceinline__ uint32_t lane_bytes(const typename TT::Lane &L) { return L.j * 16u; }
};

// 16-bit element types: B rows stay row-major in LDS and the transposing LDS read of
// gfx950 (ds_read_b64_tr_b16) turns them into MFMA operands.  In every block of 16 lanes
// that instruction treats the 16 x 4 halves the lanes address as a 4 x 16 matrix (lane i
// supplies columns 4 (i % 4) .. + 3 of row i / 4) and returns column j to lane j: with
// lane i addressing 8 bytes of gathered row i / 4 at features 16 p + 4 (i % 4), lane j
// receives B[row 0..3][16 p + j] - four consecutive k of feature j, which is what
// v_mfma_f32_16x16x32 wants of its second operand.  Two reads give a lane its eight k.
// The rows are gathered by the address alone, so the contraction needs neither the
// even / odd trick of the gather kernels (half of every MFMA multiplies zeros there) nor
// any register moves:
//   * a step is 32 columns of a unit; quarter-wave g covers columns 8g .. 8g + 7;
//   * first operand: the lane's 16 bytes of the plan's tile copy, A[row l % 16 of the
//     unit's 16 rows][columns 8g .. 8g + 7] (rows 8 .. 15 are the second window of a
//     pair, zero for a single window);
//   * accumulator p (of 8): features 16 p .. 16 p + 15 of the block; register e of lane
//     (g, j): unit row 4g + e, feature 16 p + j.
// The rows of the LDS image are 288 bytes apart and the LDS serves two blocks of lanes at a
// time: the eight rows they read lie in different banks when their numbers differ mod 8,
// and the plan orders the columns of a step accordingly (hspmm_create.hip, build_panel_stream).
// Units of three and four windows (G = 4; the third and fourth in a second KB of the step's
// tile copy) run every second operand against two first operands: half the LDS reads per
// row, which is what binds these kernels, with eight consumer waves of twice the
// accumulators.
//   ids per step: 16 words, one per four lanes (word l / 4): bits 4..15 = 9 x (panel row
//     of column 8g + i / 4), bits 16..27 = 9 x (panel row of column 8g + 4 + i / 4)
//     (i = l % 16; x 32 = byte offset in the image); bits 0..3: the panel jump.
typedef short tr16x4 __attribute__((ext_vector_type(4)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));

template <int G_, bool BF>
struct Fp16Tr {
    // G * V accumulators: 8 for the 16 rows of one or two windows; units of up to four windows
    // (G = 4) run every step's second operand against two first operands, rows 0..15 and 16..31
    static constexpr int G = G_, V = G_ == 4 ? 4 : 8 / G_;
    static constexpr int kBlockFeat = 128;
    static constexpr int kLaneFeat = 1;            // lane's feature = j (+ 16 per accumulator)
    static constexpr int kElem = 2;
    typedef u32x4 AVec;
    typedef typename HalfOps<BF>::elem_t elem_t;
    struct Lane {
        uint32_t g, j;
        uint32_t f_valid;                          // features of the block that exist (128 unless N ends inside the block)
        const uint32_t *a_src;
        const uint32_t *idx_src;
        __device__ __forceinline__ void init(uint32_t lane, const void *tiles, const uint32_t *ids)
        {
            g = lane >> 4; j = lane & 15u;
            f_valid = 128u;
            a_src = reinterpret_cast<const uint32_t *>(tiles) + lane * 4u;
            idx_src = ids + (lane >> 2);           // four neighbouring lanes read one word
        }
    };
    // Window W0 of the unit is held by quarter-waves 2 (W0 % 2) and 2 (W0 % 2) + 1 of accumulators
    // 8 (W0 / 2) .. + 7.
    template <int W0>
    __device__ static __forceinline__ void store_window(const Lane &L, const f32x4 (&acc)[G * V], char *c_lane,
                                                        size_t row_bytes, uint32_t row0, uint32_t rows, bool active)
    {
        if ((L.g >> 1) != uint32_t(W0 & 1)) return;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t row = row0 + 4u * (L.g & 1u) + e;
            if (active && row < rows) {
                elem_t *dst = reinterpret_cast<elem_t *>(c_lane + size_t(row) * row_bytes);
#pragma unroll
                for (int p = 0; p < 8; ++p)
                    if (16u * uint32_t(p) + L.j < L.f_valid) stream_store(dst + 16 * p, (elem_t)acc[8 * (W0 >> 1) + p][e]);
            }
        }
    }
    __device__ static __forceinline__ void zero_rows(const Lane &L, char *c_lane, size_t row_bytes, uint32_t r_begin,
                                                     uint32_t r_end, bool active)
    {
        if (!active) return;
        for (uint32_t r = r_begin + L.g; r < r_end; r += 4u) {
            elem_t *dst = reinterpret_cast<elem_t *>(c_lane + size_t(r) * row_bytes);
#pragma unroll
            for (int p = 0; p < 8; ++p)
                if (16u * uint32_t(p) + L.j < L.f_valid) stream_store(dst + 16 * p, (elem_t)0.f);
        }
    }
};

template <int G_, bool BF>
struct PanelOps<Fp16Tr<G_, BF>> {
    typedef Fp16Tr<G_, BF> TT;
    static constexpr uint32_t kRows = kPanelRowsWide;
    static constexpr uint32_t kPitch = kPanelRowBytes + 32u;
    __device__ static __forceinline__ void write_piece(char *row, uint32_t c, const u32x4 x)
    {
        *reinterpret_cast<u32x4 *>(row + c * 16u) = x;
    }
    static constexpr bool kFour = G_ == 4;                        // units of up to four windows
    static constexpr int kConsumers = kFour ? 8 : 12;             // twice the accumulators: fewer, larger waves
    static constexpr uint32_t kRing = kFour ? 3 : 4;              // (registers: a step's second operands are held twice)
    static constexpr int kLive = TT::G * TT::V;
    __device__ static __forceinline__ void fold(f32x4 (&)[kLive]) {}
    typedef uint32_t Idx;
    // the lane's 16 bytes of the step's first 1 KB (rows 0..15), with four windows also of the second (rows 16..31)
    struct AVec { u32x4 r[kFour ? 2 : 1]; };
    __device__ static __forceinline__ Idx load_idx(const typename TT::Lane &L, const uint32_t *, uint32_t step)
    {
        return L.idx_src[size_t(step) * 16u];
    }
    __device__ static __forceinline__ AVec load_a(const typename TT::Lane &L, uint32_t step)
    {
        AVec a;
        const uint32_t *src = L.a_src + size_t(step) * (kFour ? 512u : 256u);
        a.r[0] = *reinterpret_cast<const u32x4 *>(src);
        if constexpr (kFour) a.r[1] = *reinterpret_cast<const u32x4 *>(src + 256);
        return a;
    }
    __device__ static __forceinline__ uint32_t jump(const Idx I) { return __builtin_amdgcn_readfirstlane(I) & 15u; }
    // (waves with two units) the step belongs to the wave's second unit
    __device__ static __forceinline__ bool second_unit(const Idx I) { return (__builtin_amdgcn_readfirstlane(I) >> 28) & 1u; }
    static constexpr uint32_t kPackedRing = 2;                    // steps in flight when the tiles are packed
    // the lane's eight halves from their positions in the packed values (position 0 holds a zero)
    __device__ static __forceinline__ AVec gather_a(const void *vals, const uint32_t (&pos)[8])
    {
        const uint16_t *v = static_cast<const uint16_t *>(vals);
        AVec a;
#pragma unroll
        for (int k = 0; k < 4; ++k) a.r[0][k] = uint32_t(v[pos[2 * k]]) | uint32_t(v[pos[2 * k + 1]]) << 16;
        return a;
    }
    typedef tr16x4 __attribute__((address_space(3))) *lds_tr_ptr;
    // A step in two halves of four accumulators (64 features) each: read_half<H> requests the second
    // operands of half H from LDS, mma_half<H> multiplies them.
    template <int H> struct Half { u32x4 b[4]; };
    template <int H>
    __device__ static __forceinline__ Half<H> read_half(const typename TT::Lane &, const char *smem, uint32_t img, const Idx I)
    {
        typedef __attribute__((address_space(3))) char *lds_char_ptr;
        const lds_char_ptr base = (lds_char_ptr)smem + img;
        const lds_char_ptr a0 = base + (__builtin_amdgcn_ubfe(I, 4, 12) << 5);
        const lds_char_ptr a1 = base + (__builtin_amdgcn_ubfe(I, 16, 12) << 5);
        Half<H> B;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const tr16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a0 + 32 * (4 * H + p)));
            const tr16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a1 + 32 * (4 * H + p)));
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            B.b[p][0] = l2[0]; B.b[p][1] = l2[1]; B.b[p][2] = h2[0]; B.b[p][3] = h2[1];
        }
        return B;
    }
    template <int H>
    __device__ static __forceinline__ void mma_half(const typename TT::Lane &, const AVec &A, const Half<H> &B,
                                                    f32x4 (&acc)[kLive])
    {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            acc[4 * H + p] = HalfOps<BF>::mfma(A.r[0], B.b[p], acc[4 * H + p]);
            if constexpr (kFour) acc[8 + 4 * H + p] = HalfOps<BF>::mfma(A.r[1], B.b[p], acc[8 + 4 * H + p]);
        }
    }
    __device__ static __forceinline__ uint32_t lane_bytes(const typename TT::Lane &L) { return (L.j & 3u) * 8u; }
};

// fp32 storage through the 16-bit MFMA: gfx950 has no tf32 / xf32 matrix instruction, its fp32
// MFMA runs at 1/16 of the bf16 rate, and the reference's "tf32" arithmetic keeps 10 mantissa bits
// of each factor (reference src/ptx/wgmma.h:42-58).  Here every fp32 value v is taken as
// hi + lo with hi = v cut to bf16 (its upper 16 bits: same sign, never overflows) and
// lo = bf16(v - hi) (the difference is exact, its rounding leaves |v - hi - lo| <= 2^-16 |v|), and
// a * b = a_hi b_hi + a_hi b_lo + a_lo b_hi with fp32 accumulation (the fourth product, a_lo b_lo,
// is below 2^-14 |a||b| and is left out): three v_mfma_f32_16x16x32_bf16 where fp32 inputs would
// need eight 16x16x4 instructions of twice the length, and a product exact to 2^-14 where tf32,
// with 10 mantissa bits per factor, is exact to 2^-10.  The sparse values are split by
// the plan, the rows of B by the producer waves on their way into LDS: an image row is
// [64 hi halves][64 lo halves], read through the transposing LDS read like the 16-bit types.
// An infinite or NaN v has lo = 0 (hi carries it).
//   ids per step: as Fp16Tr.  tiles per step: per lane 8 hi halves then 8 lo halves of
//   A[row l % 16][columns 8g .. 8g + 7] (32 bytes).
//   accumulator p (of 4): features 16 p .. 16 p + 15 of the block of 64.
template <int G_>
struct Fp32Split {
    static constexpr int G = G_, V = G_ == 4 ? 2 : 4 / G_;   // G * V = 4 accumulators, 8 for up to four windows
    static constexpr int kBlockFeat = 64;
    static constexpr int kLaneFeat = 1;
    static constexpr int kElem = 4;
    typedef u32x8 AVec;
    struct Lane {
        uint32_t g, j;
        uint32_t f_valid;                          // features of the block that exist (64 unless N ends inside the block)
        const uint32_t *a_src;
        const uint32_t *idx_src;
        __device__ __forceinline__ void init(uint32_t lane, const void *tiles, const uint32_t *ids)
        {
            g = lane >> 4; j = lane & 15u;
            f_valid = 64u;
            a_src = reinterpret_cast<const uint32_t *>(tiles) + lane * 8u;
            idx_src = ids + (lane >> 2);           // four neighbouring lanes read one word
        }
    };
    template <int W0>
    __device__ static __forceinline__ void store_window(const Lane &L, const f32x4 (&acc)[G * V], char *c_lane,
                                                        size_t row_bytes, uint32_t row0, uint32_t rows, bool active)
    {
        if ((L.g >> 1) != uint32_t(W0 & 1)) return;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t row = row0 + 4u * (L.g & 1u) + e;
            if (active && row < rows) {
                float *dst = reinterpret_cast<float *>(c_lane + size_t(row) * row_bytes);
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const float v = acc[4 * (W0 >> 1) + p][e];
                    if (16u * uint32_t(p) + L.j < L.f_valid) stream_store(dst + 16 * p, v);
                }
            }
        }
    }
    __device__ static __forceinline__ void zero_rows(const Lane &L, char *c_lane, size_t row_bytes, uint32_t r_begin,
                                                     uint32_t r_end, bool active)
    {
        if (!active) return;
        for (uint32_t r = r_begin + L.g; r < r_end; r += 4u) {
            float *dst = reinterpret_cast<float *>(c_lane + size_t(r) * row_bytes);
#pragma unroll
            for (int p = 0; p < 4; ++p)
                if (16u * uint32_t(p) + L.j < L.f_valid) stream_store(dst + 16 * p, 0.f);
        }
    }
};

// v - (v cut to bf16): exact; 0 where v is infinite or NaN (hi carries those)
__device__ __forceinline__ float split_rest(const uint32_t v)
{
    const float f = __builtin_bit_cast(float, v);
    const float rest = f - __builtin_bit_cast(float, v & 0xFFFF0000u);
    return __builtin_isfinite(f) ? rest : 0.f;
}
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16_rn(const float a, const float b)
{
    bf16x2_t r;
    r[0] = (__bf16)a; r[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, r);
}

template <int G_>
struct PanelOps<Fp32Split<G_>> {
    typedef Fp32Split<G_> TT;
    static constexpr uint32_t kRows = kPanelRowsWide;
    static constexpr uint32_t kPitch = kPanelRowBytes + 32u;
    // four floats of a row -> four hi halves at [4c .. 4c + 3], four lo halves 128 bytes further on
    __device__ static __forceinline__ void write_piece(char *row, uint32_t c, const u32x4 x)
    {
        u32x2 hi, lo;
        hi[0] = __builtin_amdgcn_perm(x[1], x[0], 0x07060302u);       // the upper halves
        hi[1] = __builtin_amdgcn_perm(x[3], x[2], 0x07060302u);
        lo[0] = pack_bf16_rn(split_rest(x[0]), split_rest(x[1]));
        lo[1] = pack_bf16_rn(split_rest(x[2]), split_rest(x[3]));
        *reinterpret_cast<u32x2 *>(row + c * 8u) = hi;
        *reinterpret_cast<u32x2 *>(row + 128u + c * 8u) = lo;
    }
    static constexpr bool kFour = G_ == 4;
    static constexpr int kConsumers = kFour ? 8 : 12;
    static constexpr uint32_t kRing = kFour ? 3 : 4;
    static constexpr int kLive = TT::G * TT::V;
    __device__ static __forceinline__ void fold(f32x4 (&)[kLive]) {}
    typedef uint32_t Idx;
    // the lane's 32 bytes of the step's first 2 KB (rows 0..15), with four windows also of the second
    struct AVec { u32x8 r[kFour ? 2 : 1]; };
    __device__ static __forceinline__ Idx load_idx(const typename TT::Lane &L, const uint32_t *, uint32_t step)
    {
        return L.idx_src[size_t(step) * 16u];
    }
    __device__ static __forceinline__ AVec load_a(const typename TT::Lane &L, uint32_t step)
    {
        AVec a;
        const uint32_t *src = L.a_src + size_t(step) * (kFour ? 1024u : 512u);
        a.r[0] = *reinterpret_cast<const u32x8 *>(src);
        if constexpr (kFour) a.r[1] = *reinterpret_cast<const u32x8 *>(src + 512);
        return a;
    }
    __device__ static __forceinline__ uint32_t jump(const Idx I) { return __builtin_amdgcn_readfirstlane(I) & 15u; }
    __device__ static __forceinline__ bool second_unit(const Idx I) { return (__builtin_amdgcn_readfirstlane(I) >> 28) & 1u; }
    static constexpr uint32_t kPackedRing = 2;                    // steps in flight when the tiles are packed (four measured slower)
    // the lane's eight values (hi half | lo half << 16) from their positions in the packed values
    // (position 0 holds a zero), rearranged to four words of hi halves and four of lo halves
    __device__ static __forceinline__ AVec gather_a(const void *vals, const uint32_t (&pos)[8])
    {
        const uint32_t *v = static_cast<const uint32_t *>(vals);
        AVec a;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t w0 = v[pos[2 * k]], w1 = v[pos[2 * k + 1]];
            a.r[0][k] = __builtin_amdgcn_perm(w1, w0, 0x05040100u);
            a.r[0][4 + k] = __builtin_amdgcn_perm(w1, w0, 0x07060302u);
        }
        return a;
    }
    typedef tr16x4 __attribute__((address_space(3))) *lds_tr_ptr;
    __device__ static __forceinline__ u32x4 operand(const __attribute__((address_space(3))) char *a0,
                                                    const __attribute__((address_space(3))) char *a1, int off)
    {
        const tr16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a0 + off));
        const tr16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(a1 + off));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        u32x4 b;
        b[0] = l2[0]; b[1] = l2[1]; b[2] = h2[0]; b[3] = h2[1];
        return b;
    }
    // A step in two halves of two accumulators (32 features) each, as for the 16-bit types.
    template <int H> struct Half { u32x4 hi[2], lo[2]; };
    template <int H>
    __device__ static __forceinline__ Half<H> read_half(const typename TT::Lane &, const char *smem, uint32_t img, const Idx I)
    {
        typedef __attribute__((address_space(3))) char *lds_char_ptr;
        const lds_char_ptr base = (lds_char_ptr)smem + img;
        const lds_char_ptr a0 = base + (__builtin_amdgcn_ubfe(I, 4, 12) << 5);
        const lds_char_ptr a1 = base + (__builtin_amdgcn_ubfe(I, 16, 12) << 5);
        Half<H> B;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            B.hi[p] = operand(a0, a1, 32 * (2 * H + p));
            B.lo[p] = operand(a0, a1, 128 + 32 * (2 * H + p));
        }
        return B;
    }
    template <int H>
    __device__ static __forceinline__ void mma_half(const typename TT::Lane &, const AVec &A, const Half<H> &B,
                                                    f32x4 (&acc)[kLive])
    {
        constexpr int kRowSets = kFour ? 2 : 1;
        u32x4 a_hi[kRowSets], a_lo[kRowSets];
#pragma unroll
        for (int h = 0; h < kRowSets; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) { a_hi[h][i] = A.r[h][i]; a_lo[h][i] = A.r[h][4 + i]; }
#pragma unroll
        for (int p = 0; p < 2; ++p) {
#pragma unroll
            for (int h = 0; h < kRowSets; ++h) {
                // small terms first; a_lo * b_lo (below 2^-14 |a||b|, 2^-16 on average) is left out
                const int q = 4 * h + 2 * H + p;
                f32x4 c = HalfOps<true>::mfma(a_lo[h], B.hi[p], acc[q]);
                c = HalfOps<true>::mfma(a_hi[h], B.lo[p], c);
                acc[q] = HalfOps<true>::mfma(a_hi[h], B.hi[p], c);
            }
        }
    }
    __device__ static __forceinline__ uint32_t lane_bytes(const typename TT::Lane &L) { return (L.j & 3u) * 8u; }
};

template <>
struct PanelOps<Fp32Quad> {
    static constexpr uint32_t kRows = kPanelRowsFp32;
    static constexpr uint32_t kPitch = kPanelRowBytes;
    __device__ static __forceinline__ void write_piece(char *row, uint32_t c, const u32x4 x)
    {
        *reinterpret_cast<u32x4 *>(row + c * 16u) = x;
    }
    static constexpr uint32_t kRing = 3;                          // few registers: two workgroups per compute unit
    // Two accumulators per 32-feature half, used in turn: an MFMA then never reads the result of
    // the one two instructions in front of it.  fold() adds the pairs once, at the end of the unit.
    static constexpr int kLive = 4;
    __device__ static __forceinline__ void fold(f32x4 (&acc)[4]) { acc[0] += acc[2]; acc[1] += acc[3]; }
    typedef u32x4 Idx;                                            // all four id words (the same in every lane)
    typedef u32x8 AVec;
    // The address is the same in every lane: the compiler makes this a scalar load.
    __device__ static __forceinline__ Idx load_idx(const Fp32Quad::Lane &, const uint32_t *ids, uint32_t step)
    {
        return *reinterpret_cast<const u32x4 *>(ids + size_t(step) * 4u);
    }
    __device__ static __forceinline__ AVec load_a(const Fp32Quad::Lane &L, uint32_t step)
    {
        return *reinterpret_cast<const u32x8 *>(L.a_src + size_t(step) * 64u);
    }
    __device__ static __forceinline__ uint32_t jump(const Idx I) { return __builtin_amdgcn_readfirstlane(I[0]) & 15u; }
    // The first "half" is the whole step (see the consumer loop of spmm_panel_kernel).
    template <int H> struct Half { float lo[8], hi[8]; };
    template <int H>
    __device__ static __forceinline__ Half<H> read_half(const Fp32Quad::Lane &, const char *smem, uint32_t img, const Idx I)
    {
        Half<H> B = {};
        if constexpr (H == 0) {
            // word w holds the offsets of the rows whose tile values are A[2w] and A[2w + 1]
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t word = I[w];
                const uint32_t sw = __builtin_amdgcn_readfirstlane(word);
                const uint32_t off0 = sw & 0xFF00u, off1 = sw >> 16;
                const float *r0 = reinterpret_cast<const float *>(smem + (img + off0));
                const float *r1 = reinterpret_cast<const float *>(smem + (img + off1));
                B.lo[2 * w] = r0[0]; B.hi[2 * w] = r0[32];
                B.lo[2 * w + 1] = r1[0]; B.hi[2 * w + 1] = r1[32];
            }
        }
        return B;
    }
    template <int H>
    __device__ static __forceinline__ void mma_half(const Fp32Quad::Lane &, const AVec &A, const Half<H> &B, f32x4 (&acc)[4])
    {
        if constexpr (H == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t aw = A[i];
                const float a = __builtin_bit_cast(float, aw);
                acc[2 * (i & 1)] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, B.lo[i], acc[2 * (i & 1)], 0, 0, 0);
                acc[2 * (i & 1) + 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, B.hi[i], acc[2 * (i & 1) + 1], 0, 0, 0);
            }
        }
    }
    __device__ static __forceinline__ uint32_t lane_bytes(const Fp32Quad::Lane &L) { return L.j * 4u; }
};

// The eight lane masks of a step whose tile is stored without its zeros (see spmm_panel_kernel).
struct PackedHeader { uint64_t m[8]; };
typedef const uint64_t __attribute__((address_space(4))) *const_u64_ptr;
__device__ __forceinline__ PackedHeader load_packed_header(const uint64_t *masks, uint32_t step)
{
    const const_u64_ptr mp = (const_u64_ptr)(uintptr_t)masks + size_t(step) * 8u;   // uniform: scalar loads
    PackedHeader h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h.m[i] = mp[i];
    return h;
}

// One barrier of the workgroup with the LDS writes in front of it visible behind it.
__device__ __forceinline__ void panel_barrier()
{
    // (fences for LDS alone: they must not wait for the global loads a wave has in flight)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// NC consumer waves (one unit each) and NPW producer waves that do nothing but copy
// panel images to LDS: the consumers' register ring of tile / id loads then never
// has to wait for a panel load (vector loads return in order, and a wave that had
// both kinds in flight would drain its ring at every panel).
// RAGGED: the feature dimension is no whole number of feature blocks (a build of its own, so that the kernel for
// whole blocks is exactly the one it was: it is sensitive to every register and instruction around its loop).
template <class TT, int NC, int NPW, bool TALL = false, bool PACKED = false, bool RAGGED = false>
__global__ __launch_bounds__((NC + NPW) * 64)
void spmm_panel_kernel(const PanelArgs pa)
{
    constexpr int G = TT::G, V = TT::V, NACC = G * V;
    typedef PanelOps<TT> Ops;
    constexpr uint32_t kPanelRows = Ops::kRows, kPanelBytes = kPanelRows * kPanelRowBytes;
    constexpr int kPieces = int(kPanelBytes / 16u) / (NPW * 64);   // 16-byte pieces of a panel per producer thread
    static_assert(kPieces * NPW * 64 * 16 == int(kPanelBytes), "panel must divide among the producers");
    static_assert(kPieces <= 16, "a producer thread holds a panel's pieces in registers");
    constexpr uint32_t kPitch = Ops::kPitch, kImage = kPanelRows * kPitch;   // one panel image in LDS
    __shared__ __attribute__((aligned(16))) char smem[2 * kImage];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // The hardware hands consecutive workgroups to the eight XCDs in turn, and every XCD has an L2 of
    // its own, filled over a path that delivers about 0.7 TB/s per XCD: what the L2s miss sets the pace
    // of this kernel, so every line should be fetched by as few XCDs as possible.
    //   * The workgroups of one row block and chunk - one per feature block - read the same tiles and
    //     ids: they run on one XCD, adjacent in its launch order, so that one of them fetches the
    //     tile stream and the others hit it.
    //   * A chunk of panels is a range of rows of B: with the chunk as the slowest index an XCD works on
    //     one chunk (or two), and only the XCDs of a chunk fetch its rows of B (every XCD reading all of
    //     B costs 8 x B; the block-clustered matrix at N = 512: 118 of 197 MB per launch).
    //   position in launch order: XCD x = blockIdx % 8 runs blocks x, x + 8, ...; the work items
    //   (chunk, row block, feature block), feature block fastest, are dealt out XCD by XCD.
    constexpr uint32_t kXcds = 8;
    const uint32_t n_blocks = gridDim.x, xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
    const uint32_t item = xcd * (n_blocks / kXcds) + umin32(xcd, n_blocks % kXcds) + slot;
    const uint32_t per_chunk = n_blocks / pa.n_chunks;              // row blocks x feature blocks
    const uint32_t chunk = item / per_chunk;
    const uint32_t rest = item - chunk * per_chunk;
    const uint32_t rb = rest / pa.n_feat_blocks;
    const uint32_t fb = rest - rb * pa.n_feat_blocks;
    const uint32_t p_begin = chunk * pa.panels_per_chunk;
    const uint32_t p_end = umin32(p_begin + pa.panels_per_chunk, pa.n_panels);
    const size_t row_bytes = size_t(pa.N) * TT::kElem;
    // first feature of this block
    const uint32_t feat0 = RAGGED ? panel_block_first_feature(fb, uint32_t(TT::kBlockFeat), pa.N) : fb * uint32_t(TT::kBlockFeat);

    if (wave >= uint32_t(NC)) {
        // ---- producer: panel q goes to buffer q & 1, then the barrier that releases it.
        // Buffer q & 1 was last read for panel q - 2, which every consumer left before
        // the barrier of panel q - 1.
        const uint32_t pt = threadIdx.x - uint32_t(NC) * 64u;       // 0 .. NPW*64-1
        // piece c = pt + i * NPW*64 is bytes [16c, 16c + 16) of the image: row c / 16, 16-byte column c % 16
        const char *b_block = reinterpret_cast<const char *>(pa.B) + size_t(feat0) * TT::kElem;
        // (a feature dimension that ends inside this block: a piece behind a row's end is read from the row's
        // first piece instead - the features it would feed are never stored, and no load leaves the row)
        const uint32_t piece_row0 = pt >> 4;
        const uint32_t col_bytes = (!RAGGED || size_t(feat0) * TT::kElem + (pt & 15u) * 16u < row_bytes) ? (pt & 15u) * 16u : 0u;
        // Addresses: the panel's first row (the same in all lanes) plus 32-bit offsets inside the panel
        // (the host checks that a panel of B spans less than 4 GB).  Rows past the matrix are never
        // referenced: their loads are bent to the matrix's last row.
        const uint32_t row_bytes32 = uint32_t(row_bytes);
        const uint32_t row_off0 = piece_row0 * row_bytes32, row_stride = uint32_t(NPW * 4) * row_bytes32;
        auto panel_base = [&](uint32_t q) __attribute__((always_inline)) -> const char * {
            return b_block + size_t(q) * kPanelRows * row_bytes;
        };
        auto last_row_off = [&](uint32_t q) __attribute__((always_inline)) -> uint32_t {
            return (umin32(pa.cols - q * kPanelRows, kPanelRows) - 1u) * row_bytes32;
        };
        auto load_piece = [&](const char *panel, uint32_t last_off, int i) __attribute__((always_inline)) -> u32x4 {
            const uint32_t off = umin32(row_off0 + uint32_t(i) * row_stride, last_off) + col_bytes;
            return *reinterpret_cast<const u32x4 *>(panel + off);
        };
        // The loads of panel q + 1 are in flight (in registers) while the consumers multiply panel q.
        // A piece's register is reloaded as soon as the piece is written, so that the copy to LDS and
        // the requests for the next panel overlap: one after the other they are most of a barrier
        // period, and the consumers wait for them.  (Three panels in flight, with four producer waves,
        // measured no faster.)
        u32x4 X[kPieces];
        auto copy_piece = [&](char *row, const u32x4 &x) __attribute__((always_inline)) {
            Ops::write_piece(row, pt & 15u, x);
        };
        {
            const char *panel = panel_base(p_begin);
            const uint32_t last_off = last_row_off(p_begin);
#pragma unroll
            for (int i = 0; i < kPieces; ++i) {
                X[i] = load_piece(panel, last_off, i);
                __builtin_amdgcn_sched_barrier(0);                  // in the order they are used
            }
        }
        for (uint32_t q = p_begin; q < p_end; ++q) {
            char *img = smem + (q & 1u) * kImage + piece_row0 * kPitch;
            if (q + 1u < p_end) {
                const char *panel = panel_base(q + 1u);
                const uint32_t last_off = last_row_off(q + 1u);
#pragma unroll
                for (int i = 0; i < kPieces; ++i) {
                    copy_piece(img + uint32_t(i) * (NPW * 4) * kPitch, X[i]);
                    X[i] = load_piece(panel, last_off, i);
                    __builtin_amdgcn_sched_barrier(0);              // in the order the loads return
                }
            } else {
#pragma unroll
                for (int i = 0; i < kPieces; ++i) copy_piece(img + uint32_t(i) * (NPW * 4) * kPitch, X[i]);
            }
            panel_barrier();
        }
        return;
    }

    // ---- consumer
    // TALL: the wave owns two units, 2 su and 2 su + 1 (the second may not exist), with accumulators of
    // their own; the plan has merged their steps panel by panel and marked those of the second unit.
    const uint32_t su = rb * pa.units_per_group + wave;
    const uint32_t u = TALL ? 2u * su : su;
    const bool has_unit = wave < pa.units_per_group && u < pa.n_units;
    const const_u32_ptr poff = as_const(pa.poff) + size_t(has_unit ? su : 0u) * (pa.n_panels + 1u);

    typename TT::Lane L;
    L.init(lane, pa.tiles, pa.ids);
    const uint32_t feat = feat0 + L.j * TT::kLaneFeat;
    char *c_lane = reinterpret_cast<char *>(pa.C) + size_t(feat) * TT::kElem;

    // steps [t0, t1) of the unit lie in this chunk of panels; a wave without a unit has none
    const uint32_t t0 = has_unit ? poff[p_begin] : 0u;
    const uint32_t t1 = has_unit ? poff[p_end] : 0u;
    // loads past the last step are clamped to it (their values are not used)
    const uint32_t tlast = t1 > t0 ? t1 - 1u : umin32(t0, pa.n_steps - 1u);
    // barriers this wave owes: one per panel of the chunk, with or without steps in it
    uint32_t owed = p_end - p_begin;
    // panels in front of the chunk's first step (the count stored with that step refers
    // to its predecessor, which may lie in another chunk)
    uint32_t first_jump = t1 > t0 ? as_const(pa.step_panel)[t0] - p_begin : 0u;

    f32x4 live[Ops::kLive];
    f32x4 live2[TALL ? Ops::kLive : 1];
#pragma unroll
    for (int i = 0; i < Ops::kLive; ++i) live[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < (TALL ? Ops::kLive : 1); ++i) live2[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    typedef typename Ops::AVec AVec;
    typedef typename Ops::Idx Idx;
    auto ring_idx = [&](uint32_t step) __attribute__((always_inline)) -> Idx {
        return Ops::load_idx(L, pa.ids, umin32(step, tlast));
    };
    // PACKED: the step's tile is stored without its zeros.  masks[8 s + i] has bit l set when lane l's
    // i-th value of step s (its column 8 (l / 16) + i of row l % 16) is stored; the stored values follow
    // one another in the order (i, l), those of step s from vals[step_voff[s]] on, and vals[0] is zero
    // (what a lane without the value reads).  The masks are uniform (scalar loads); a lane's position is
    // a count of mask bits below it.  next_val: position of the first value of the next step to load.
    PackedHeader H0 = {}, H1 = {};
    uint32_t next_val = 0;
    if constexpr (PACKED) next_val = as_const(pa.step_voff)[umin32(t0, tlast)];
    auto request = [&](PackedHeader &H, uint32_t step) __attribute__((always_inline)) {
        if constexpr (PACKED) H = load_packed_header(pa.masks, umin32(step, tlast));
    };
    auto ring_a = [&](const PackedHeader &H, uint32_t step) __attribute__((always_inline)) -> AVec {
        if constexpr (PACKED) {
            uint32_t pos[8], base = next_val;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t rank = __builtin_amdgcn_mbcnt_hi(uint32_t(H.m[i] >> 32),
                                                                __builtin_amdgcn_mbcnt_lo(uint32_t(H.m[i]), base));
                pos[i] = __builtin_amdgcn_inverse_ballot_w64(H.m[i]) ? rank : 0u;
                base += uint32_t(__builtin_popcountll(H.m[i]));
            }
            if (step <= tlast) next_val = base;            // (a clamped load repeats the last step)
            return Ops::gather_a(pa.vals, pos);
        } else {
            return Ops::load_a(L, umin32(step, tlast));
        }
    };
    // register ring of kRing steps (separate variables: an array would go to scratch)
#define HSPMM_RING(X) X(0) X(1) X(2) X(3) X(4) X(5)
#define HSPMM_RING2(X) X(0, 1) X(1, 2) X(2, 3) X(3, 4) X(4, 5) X(5, 6)
#define HSPMM_HEADER(k) ((k##u & 1u) ? H1 : H0)
#define HSPMM_OTHER_HEADER(k) ((k##u & 1u) ? H0 : H1)
    // (two sets of accumulators leave registers for fewer steps in flight; packed tiles: see Ops::kPackedRing)
    constexpr uint32_t kRing = [] {
        if constexpr (PACKED) return Ops::kPackedRing;
        else return Ops::kRing;
    }();
    static_assert(kRing >= 1 && kRing <= 6, "ring slots are named variables");
    static_assert(!PACKED || kRing % 2u == 0u, "the two headers alternate with the ring slots");
    // (PACKED: the header of a step is requested one slot ahead of the loads that need it)
    request(H0, t0);
#define HSPMM_RING_DECL(k) Idx I##k = {}; AVec A##k = {}; \
    if constexpr (kRing > k) { request(HSPMM_OTHER_HEADER(k), t0 + k##u + 1u); \
                               I##k = ring_idx(t0 + k##u); A##k = ring_a(HSPMM_HEADER(k), t0 + k##u); }
    HSPMM_RING(HSPMM_RING_DECL)
#undef HSPMM_RING_DECL
    const Idx I6 = {};                                              // (a name for "the slot behind the last"; never read)
    panel_barrier();                                                // panel p_begin is in its buffer
    --owed;
    // the lane's bytes of a row, in the buffer of the current panel
    uint32_t img = (p_begin & 1u) * kImage + Ops::lane_bytes(L);
    const uint32_t img_both = kImage + 2u * Ops::lane_bytes(L);     // img of one buffer + img of the other

    // The barriers between a step and the step in front of it.
    auto enter = [&](const uint32_t jump) __attribute__((always_inline)) {
        for (uint32_t n = jump; n && owed; --n) {                   // never more barriers than the producers pass
            panel_barrier();
            img = img_both - img;
            --owed;
        }
    };
    // A step runs in two halves, and the LDS reads of a half are requested before the MFMAs of the half
    // in front of it are issued: a wave that reads, waits and then multiplies leaves both the LDS and the
    // matrix cores idle for most of a step (the waves of a workgroup leave every barrier in phase).
    // Bq: the second operands of the first half of the step about to run, requested by the step in front
    // of it between its two halves.  Where the next step lies in another panel, the barriers come first:
    // the wave then arrives with its second half still to multiply, which is safe - the operands of that
    // half are in registers (the barrier waits for the wave's LDS reads).
    typename Ops::template Half<0> Bq = {};
    auto mma = [&](auto half, const Idx &I, const AVec &A, const auto &B) __attribute__((always_inline)) {
        constexpr int H = decltype(half)::value;
        if constexpr (TALL) {
            if (Ops::second_unit(I)) Ops::template mma_half<H>(L, A, B, live2);
            else Ops::template mma_half<H>(L, A, B, live);
        } else {
            Ops::template mma_half<H>(L, A, B, live);
        }
    };
    // In: the ids of the next step, jump_next: the barriers in front of it (0 when there is no next step:
    // In then repeats the last step's ids, and what is read for it is not used)
    auto step = [&](const Idx &I, const AVec &A, const Idx &In, const uint32_t jump_next) __attribute__((always_inline)) {
        // (the scheduling barriers keep the compiler from moving the reads behind the MFMAs again)
        const typename Ops::template Half<1> B1 = Ops::template read_half<1>(L, smem, img, I);
        __builtin_amdgcn_sched_barrier(0);
        mma(std::integral_constant<int, 0>{}, I, A, Bq);
        __builtin_amdgcn_sched_barrier(0);
        enter(jump_next);
        Bq = Ops::template read_half<0>(L, smem, img, In);
        __builtin_amdgcn_sched_barrier(0);
        mma(std::integral_constant<int, 1>{}, I, A, B1);
        __builtin_amdgcn_sched_barrier(0);
    };

    uint32_t t = t0;
    if (t0 < t1) {
        enter(first_jump);
        Bq = Ops::template read_half<0>(L, smem, img, I0);
    }
    // Steady state: every slot runs its step and reloads its registers with the step kRing
    // further on, without conditions on the loads.  (After the prologue the header of step
    // t0 + kRing is in H0 / H1 by the parity of kRing, i.e. in slot 0's header.)
    // The step behind slot k's is in slot k + 1, behind the last slot's in slot 0 (just reloaded).
#define HSPMM_NEXT_IDX(k, kn) ((k##u + 1u == kRing) ? I0 : I##kn)
    for (; t + 2u * kRing <= t1; t += kRing) {
#define HSPMM_PANEL_STEADY(k, kn) if constexpr (kRing > k) { \
        step(I##k, A##k, HSPMM_NEXT_IDX(k, kn), Ops::jump(HSPMM_NEXT_IDX(k, kn))); \
        request(HSPMM_OTHER_HEADER(k), t + k##u + kRing + 1u); \
        I##k = ring_idx(t + k##u + kRing); A##k = ring_a(HSPMM_HEADER(k), t + k##u + kRing); }
        HSPMM_RING2(HSPMM_PANEL_STEADY)
#undef HSPMM_PANEL_STEADY
    }
    for (; t < t1; t += kRing) {
#define HSPMM_PANEL_DRAIN(k, kn) if constexpr (kRing > k) { \
        if (t + k##u < t1) step(I##k, A##k, HSPMM_NEXT_IDX(k, kn), t + k##u + 1u < t1 ? Ops::jump(HSPMM_NEXT_IDX(k, kn)) : 0u); \
        request(HSPMM_OTHER_HEADER(k), t + k##u + kRing + 1u); \
        if (t + k##u + kRing < t1) { I##k = ring_idx(t + k##u + kRing); A##k = ring_a(HSPMM_HEADER(k), t + k##u + kRing); } }
        HSPMM_RING2(HSPMM_PANEL_DRAIN)
#undef HSPMM_PANEL_DRAIN
    }
#undef HSPMM_NEXT_IDX
#undef HSPMM_RING
#undef HSPMM_RING2
#undef HSPMM_HEADER
#undef HSPMM_OTHER_HEADER
    // the panels behind the unit's last step
    for (; owed; --owed) panel_barrier();

    if (!has_unit) return;
    // (here, not at the top: nothing of it lives through the steps)
    if constexpr (RAGGED) set_valid_features<TT>(L, pa.N, feat0);
    // Stores unit `unit` from the sums in `sums` (or leaves them as this chunk's partial sums).
    auto finish = [&](const uint32_t unit, f32x4 (&sums)[Ops::kLive]) __attribute__((always_inline)) {
        Ops::fold(sums);
        f32x4 acc[NACC];
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[i] = sums[i];
        const uint32_t row = pa.unitRow[unit];
        const uint32_t row0 = row & ~7u;
        const uint32_t nwin = unit_windows<TT>(row);
        if (pa.n_chunks == 1u) {
            store_unit<TT>(L, acc, c_lane, row_bytes, row0, nwin, pa.rows, true);
        } else if (!pa.arrive) {
            f32x4 *dst = reinterpret_cast<f32x4 *>(pa.scratch) +
                         ((size_t(unit) * pa.n_chunks + chunk) * pa.n_feat_blocks + fb) * (NACC * 64u) + lane;
#pragma unroll
            for (int i = 0; i < NACC; ++i) dst[i * 64] = acc[i];
        } else {
            // The wave that brings the last chunk's sums of a unit adds all of them, in chunk order (so the
            // result does not depend on who is last), and stores the unit.  The sums cross the L2s of
            // different XCDs: they are written and read with device-scope accesses, and the writes are
            // waited for before the arrival is counted.
            const __amdgpu_buffer_rsrc_t sums = device_scope_buffer(
                reinterpret_cast<f32x4 *>(pa.scratch) + (size_t(unit) * pa.n_chunks * pa.n_feat_blocks + fb) * (NACC * 64u));
            const uint32_t chunk_stride = pa.n_feat_blocks * (NACC * 1024u);   // bytes from one chunk's sums to the next
#pragma unroll
            for (int i = 0; i < NACC; ++i) store_device_scope(sums, chunk * chunk_stride + uint32_t(i) * 1024u + lane * 16u, acc[i]);
            wait_stores_acknowledged();
            uint32_t *ctr = pa.arrive + size_t(unit) * pa.n_feat_blocks + fb;
            uint32_t old = 0;
            if (lane == 0) old = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old = __builtin_amdgcn_readfirstlane(old);
            asm volatile("" ::: "memory");                  // the loads below stay behind the count they depend on
            if (old + 1u == pa.n_chunks) {
#pragma unroll
                for (int i = 0; i < NACC; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
                for (uint32_t c = 0; c < pa.n_chunks; ++c) {
#pragma unroll
                    for (int i = 0; i < NACC; ++i) acc[i] += load_device_scope(sums, c * chunk_stride + uint32_t(i) * 1024u + lane * 16u);
                }
                store_unit<TT>(L, acc, c_lane, row_bytes, row0, nwin, pa.rows, true);
                if (lane == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (chunk == 0u) {
            // rows of the windows without entries behind this unit, and in front of the first one
            const uint32_t next_row = (unit + 1u < pa.n_units) ? (pa.unitRow[unit + 1u] & ~7u) : pa.rows;
            const uint32_t gap_begin = row0 + nwin * kRowWindow;
            if (gap_begin < next_row) TT::zero_rows(L, c_lane, row_bytes, gap_begin, next_row, true);
            if (unit == 0u) TT::zero_rows(L, c_lane, row_bytes, 0u, row0, true);
        }
    };
    finish(u, live);
    if constexpr (TALL) {
        if (u + 1u < pa.n_units) finish(u + 1u, live2);
    }
}

// Units (consumer waves) per workgroup: 12 or 14 and two producer waves for panels of 128
// rows (12 + 4 in the shape the 4x4x1 fp32 kernel uses); 12 + 4, or 8 + 4 for units of up
// to four windows, for panels of 256 rows.  Waves go to the four SIMDs of a compute unit
// round-robin, so 8 and 12 consumers spread evenly.

// ka: the arguments of spmm_fixup_kernel for the chunk sums (split table with one
// entry per unit); used only when pa.n_chunks > 1.
template <class TT, int NC, int NPW, bool TALL = false, bool PACKED = false>
static hipError_t launch_panel_tt(const PanelArgs &pa, const KernelArgs &ka, hipStream_t s, hipEvent_t mid)
{
    if (pa.units_per_group < 1u || pa.units_per_group > uint32_t(NC)) return hipErrorInvalidValue;
    const uint32_t wave_units = TALL ? (pa.n_units + 1u) / 2u : pa.n_units;     // what one consumer wave takes
    const uint32_t row_blocks = (wave_units + pa.units_per_group - 1u) / pa.units_per_group;
    const dim3 grid(row_blocks * pa.n_feat_blocks * pa.n_chunks), block((NC + NPW) * 64);
    if (pa.N % uint32_t(TT::kBlockFeat) != 0) spmm_panel_kernel<TT, NC, NPW, TALL, PACKED, true><<<grid, block, 0, s>>>(pa);
    else spmm_panel_kernel<TT, NC, NPW, TALL, PACKED, false><<<grid, block, 0, s>>>(pa);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || pa.n_chunks == 1u || pa.arrive) return e;
    if (mid && (e = hipEventRecord(mid, s)) != hipSuccess) return e;
    const uint32_t fitems = ka.n_split * ka.n_feat_blocks;
    spmm_fixup_kernel<TT><<<dim3((fitems + 3u) / 4u), dim3(256), 0, s>>>(ka);
    return hipGetLastError();
}

template <class TT>
static hipError_t launch_panel_nw(const PanelArgs &pa, const KernelArgs &ka, int units, hipStream_t s, hipEvent_t mid)
{
    // panels of 256 rows need four producer waves to hold one in registers
    if constexpr (PanelOps<TT>::kRows > 128u) return launch_panel_tt<TT, PanelOps<TT>::kConsumers, 4>(pa, ka, s, mid);
    else {
#ifdef HSPMM_EXPERIMENTAL
        if (units == 14) return launch_panel_tt<TT, 14, 2>(pa, ka, s, mid);
        if (units == 13) return launch_panel_tt<TT, 12, 4>(pa, ka, s, mid);      // 12 units, four producer waves
        return launch_panel_tt<TT, 12, 2>(pa, ka, s, mid);
#else
        // the shapes the plans choose: 12 + 4 waves for the 4x4x1 instruction, 14 + 2 for pairs of windows
        if constexpr (std::is_same<TT, Fp32Quad>::value) return units == 13 ? launch_panel_tt<TT, 12, 4>(pa, ka, s, mid) : hipErrorInvalidValue;
        else return units == 14 ? launch_panel_tt<TT, 14, 2>(pa, ka, s, mid) : hipErrorInvalidValue;
#endif
    }
}

#ifdef HSPMM_EXPERIMENTAL
// Waves with two units each (kernels built on the 16-bit MFMA, units of one or two windows); packed: the
// stream holds the tiles without their zeros.
template <class TT>
static hipError_t launch_panel_tall(const PanelArgs &pa, const KernelArgs &ka, bool packed, hipStream_t s, hipEvent_t mid)
{
    static_assert(PanelOps<TT>::kRows > 128u && TT::G <= 2, "two units per wave: 16 rows each");
    // (16-bit types: two sets of eight accumulators and two sets of second operands - eight consumer waves,
    // so that a wave may hold 168 registers)
    constexpr int kTallConsumers = TT::kElem == 2 ? 8 : PanelOps<TT>::kConsumers;
    return packed ? launch_panel_tt<TT, kTallConsumers, 4, true, true>(pa, ka, s, mid)
                  : launch_panel_tt<TT, kTallConsumers, 4, true, false>(pa, ka, s, mid);
}
#endif  // HSPMM_EXPERIMENTAL

}  // namespace hspmm
