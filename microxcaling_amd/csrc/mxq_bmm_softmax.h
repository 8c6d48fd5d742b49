// Attention scores in one kernel: P = softmax(Q(A x B^T)) over the last axis, for packed MX operands
// whose contraction axis is a single K step of 128 eight-bit codes (head_dim 128) and rows of up to
// 2048 columns -- mx.bmm(q, k^T) followed by mx.softmax(dim = -1) with mx_specs['bfloat'] = 16 and
// round-half-away on bf16 tensors (mx/bmm.py:40-59, then mx/softmax.py:26-48).  The logits never
// go to memory: what the separate kernels write and read back (2 x 2 bytes per logit) is the larger
// part of their traffic, and the softmax kernel's input handling a fifth of its instructions.
//
// Work mapping.  A workgroup (4 waves) owns 32 rows of one batch entry and all N columns; wave w
// multiplies the 32 x 32 column tiles w, w + 4, w + 8, ... (32 x 32 x 64 scaled MFMAs, two per tile,
// B tile as the first operand, its rows permuted as in the 256 x 256 GEMM kernel so that a lane ends
// up with two runs of 8 consecutive columns of one row).  The A fragment is loaded once; the B tiles
// stream through a small LDS ring per wave, copied by the memory pipe.  A lane keeps its 256
// logits of the row (lane % 32) as 128 packed bf16 pairs in registers through the three phases:
//   1  product -> bf16, range check, running row maximum
//   2  Q(x); d = Q(x - m); e = Q(exp d); running row sum      (m = Q(row maximum))
//   3  Q(e / Q(sum)) -> memory
// Row maxima and sums: the two lanes of a row inside a wave, then the four waves through LDS in
// wave order.
//
// The quantizer Q on bf16 values (bfloat16, round-half-away, subnormals kept) is "odd significand ->
// next even" on normal numbers and the identity on zeros and subnormals, applied to both halves of
// a dword at once (for exponentials and quotients with the "+ 1" masked by "exponent field not
// zero").  That form serves a workgroup
// whose logits are all finite with 2^-100 <= |x| < 2^100 or x = +0: every later value is then zero
// or positive, or a difference of two such logits.  Any other workgroup (Inf / NaN blocks, extreme
// scales) takes the element-by-element form of the softmax row kernel.  exp: the hardware
// exponential (1 ulp) of half the argument, squared -- correct through the subnormal range, where
// the instruction itself flushes -- so results agree with the separate kernels within the
// tolerance those already have against the CPU chain (exp and the order of the row sum).
#pragma once
#include "mxq_gemm.h"

struct BmmSoftmaxArgs {
    const unsigned char* a;
    const unsigned char* sa;
    const unsigned char* b;
    const unsigned char* sb;
    void* out;                 // bf16 (batch, M, N)
    int M, N;
    int exp2;                  // 1: 2^x instead of e^x (softmax_exp2)
    uint32_t q_nan_from;       // NaN threshold of the bfloat16 quantizer (general form)
    int general_only;          // tests: no packed form
    int64_t batch_a, batch_sa, batch_b, batch_sb, batch_c;
};

namespace {

constexpr int BS_ROWS = 32;                  // rows per workgroup
constexpr int BS_TILES = mxq_addr::S_TILES;  // 32-column tiles per wave: 4 x 16 x 32 = 2048 columns
constexpr int BS_MAX_N = 4 * BS_TILES * 32;
constexpr int BS_TILE_BYTES = mxq_addr::S_TILE_BYTES;   // codes of a B tile
constexpr int BS_RING = mxq_addr::S_RING;    // B tiles per wave in LDS: the one being multiplied and two on their way

template <int CBSZ, int BLGP>
__global__ __launch_bounds__(TPB, 2) void mx_bmm_softmax_kernel(BmmSoftmaxArgs g) {
    __shared__ __attribute__((aligned(16))) unsigned char ring[mxq_addr::S_LDS_BYTES];
    __shared__ float red[2][4][BS_ROWS];
    __shared__ int votes[4];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int fi = lane & 31, fg = lane >> 5;
    const int64_t bz = blockIdx.y;
    const int m0 = blockIdx.x * BS_ROWS;
    const int ntiles = g.N >> 5;

    struct Frag { u32x4 r[4]; };
    struct Scales { int w[1]; };

    // A fragment: row m0 + fi (clamped: rows past M are computed and not stored), the 16-byte
    // columns 2 q + fg of its 128 bytes; the row's four scale bytes shifted so that block fg comes first
    const int arow = min(m0 + fi, g.M - 1);
    Frag af;
    {
        const unsigned char* p = g.a + bz * g.batch_a + (int64_t)arow * 128;
#pragma unroll
        for (int q = 0; q < 4; ++q) af.r[q] = *reinterpret_cast<const u32x4*>(p + (2 * q + fg) * 16);
    }
    Scales sa;
    sa.w[0] = (int)(*reinterpret_cast<const uint32_t*>(g.sa + bz * g.batch_sa + (int64_t)arow * 4) >> (8 * fg));

    // B tiles (32 rows x 128 bytes of codes) come in through LDS: global_load_lds_dwordx4 writes 16
    // bytes per lane straight into a ring of BS_RING tiles per wave (no registers are tied up by
    // loads in flight, so the copy runs several tiles ahead of the multiplication), lane L of load
    // instruction i landing at position L % 8 of row 8 i + L / 8.  The 16-byte column c of row r is kept
    // at position c ^ key(r), which makes the fragment reads below conflict free; the lanes pick
    // their global column accordingly.  A wave only reads what it fetched itself: s_waitcnt orders
    // the two, no barrier.
    const uint32_t ring0 = (uint32_t)(uintptr_t)ring;
    const unsigned char* Bt = g.b + bz * g.batch_b;
    uint32_t boff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) boff[i] = mxq_addr::scores_code_offset(lane, i);
    // tile number i of this wave: the waves take pairs of neighbouring tiles (64 columns = one 128-byte
    // line of output per row) in turn
    auto tile_of = [&](int i) { return mxq_addr::scores_tile_of(wave, i); };
    auto fetch_b = [&](int i) {                               // ... into slot i % BS_RING
        const int t = tile_of(i);
        if (t < ntiles) {                                     // uniform per wave
            const unsigned char* src = Bt + (int64_t)t * BS_TILE_BYTES;
#pragma unroll
            for (int k = 0; k < 4; ++k) dma16(ring0 + mxq_addr::scores_lds_dst(wave, i, k), boff[k], src);
        }
    };
    // fragment row fi is B row (permuted fi) of the tile, see the 256 x 256 kernel: accumulator
    // registers 0-7 of a lane are columns 8 fg .. 8 fg + 7 of the tile, 8-15 columns 16 + 8 fg .. + 7
    const int b_lane = mxq_addr::large_frag_row_b(fi, true);
    int b_addr[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) b_addr[q] = mxq_addr::scores_lds_addr(b_lane, 2 * q + fg);
    const unsigned char* my_ring = ring + wave * (BS_RING * BS_TILE_BYTES);
    // this wave's tiles are numbers 0 .. my_tiles - 1 of its sequence (tile_of grows with i)
    int my_tiles = 0;
#pragma unroll
    for (int i = 0; i < BS_TILES; ++i) my_tiles += tile_of(i) < ntiles ? 1 : 0;
    // the scale bytes of this lane's B rows, all tiles, shifted so that block fg comes first
    int sbw[BS_TILES];
    {
        const unsigned char* SB = g.sb + bz * g.batch_sb + (int64_t)b_lane * 4;
#pragma unroll
        for (int i = 0; i < BS_TILES; ++i) {
            const int t = tile_of(i);
            sbw[i] = t < ntiles ? (int)(*reinterpret_cast<const uint32_t*>(SB + (int64_t)t * (32 * 4)) >> (8 * fg)) : 0;
        }
    }

    auto low_of = [](uint32_t w) { return mxq_float(w << 16); };
    auto high_of = [](uint32_t w) { return mxq_float(w & 0xFFFF0000u); };
    // Q on both halves of a dword.  Normal numbers and zeros of either sign (logits in the plain
    // range and their differences): + 1 on an odd significand; a zero is even.
    auto qpair = [](uint32_t w) { return w + (w & 0x00010001u); };
    // Values >= +0 that may be subnormal (exponentials, quotients): the + 1 only where the exponent
    // field is not zero, i.e. where the half is at least 0x0080 (then adding 0x7F80 sets its top bit)
    auto qpair_nonneg = [](uint32_t w) { return w + (w & ((w + 0x7F807F80u) >> 15) & 0x00010001u); };
    auto Qd = [&](float v) { return mxq_quant_bf16_to_bfloat16_nearest(v, g.q_nan_from); };
    auto Q = [&](float v) { return Qd(mxq_round_bf16(v)); };
    auto Qp = [&](float v) { return mxq_quant_bf16_to_bfloat16_nearest_nonneg(mxq_round_bf16(v)); };

    // ---- phase 1: the products, rounded to bf16 ----------------------------------------------------
    uint32_t lg[BS_TILES][8];
    float mx = -__builtin_inff();
    u16x2 hi = {0, 0}, lo = {0xFFFF, 0xFFFF};                  // largest |x|, smallest |x| - 1 (zero wraps)
    // the A fragment and the scale bytes have arrived before the first tile copy goes out, so that the
    // counter of loads in flight below counts tile copies only
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < BS_RING; ++i) fetch_b(i);
    // the MFMAs of tile i + 1 are issued before the conversion of tile i, so that the matrix pipe works
    // in the shadow of the vector instructions
    auto multiply = [&](int i) {
        v16f acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        if (tile_of(i) < ntiles) {                            // uniform per wave
            // loads complete in order: at most the copies of the tiles fetched after tile i may still
            // be in flight (4 instructions each)
            const int later = min(BS_RING - 1, my_tiles - 1 - i);
            if (later >= 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else if (later == 1) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            Frag bf;
            const unsigned char* slot = my_ring + (i % BS_RING) * BS_TILE_BYTES;
#pragma unroll
            for (int q = 0; q < 4; ++q) bf.r[q] = *reinterpret_cast<const u32x4*>(slot + b_addr[q]);
            Scales sb;
            sb.w[0] = sbw[i];
            acc = mx_mfma32<CBSZ, BLGP>(bf, af, acc, sb, sa, 0);
            acc = mx_mfma32<CBSZ, BLGP>(bf, af, acc, sb, sa, 1);
        }
        return acc;
    };
    v16f acc = multiply(0);
#pragma unroll
    for (int i = 0; i < BS_TILES; ++i) {
        v16f next = acc;
        // the slot of tile i takes tile i + BS_RING once the reads of its fragment have returned their data:
        // the copy is issued by inline assembly, which the compiler may move ahead of the MFMAs and of the
        // wait it puts in front of them, and bytes written into LDS must not overtake a read still on its way
        if (i + BS_RING < BS_TILES) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            fetch_b(i + BS_RING);
        }
        if (i + 1 < BS_TILES) next = multiply(i + 1);
        if (tile_of(i) < ntiles) {                            // uniform per wave
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t w = Pack<MXQ_BF16>::put(acc[2 * j], acc[2 * j + 1]);
                lg[i][j] = w;
                const u16x2 a = __builtin_bit_cast(u16x2, w & 0x7FFF7FFFu);
                hi = __builtin_elementwise_max(hi, a);
                lo = __builtin_elementwise_min(lo, a - u16x2{1, 1});
                mx = fmaxf(mx, fmaxf(low_of(w), high_of(w)));
            }
        }
        acc = next;
    }
    // all logits of the workgroup finite, below 2^100, and zero or at least 2^-100?
    const unsigned short top = hi[0] > hi[1] ? hi[0] : hi[1], bottom = lo[0] < lo[1] ? lo[0] : lo[1];
    const bool wave_plain = __all(top < 0x7180u && bottom >= 0x0D7Fu) && !g.general_only;
    if (lane == 0) votes[wave] = wave_plain ? 1 : 0;
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    if (fg == 0) red[0][wave][fi] = mx;
    __syncthreads();
    const bool plain = (votes[0] & votes[1] & votes[2] & votes[3]) != 0;     // uniform per workgroup

    float sum = 0.0f, m;
    if (plain) {
        // ---- phase 2 ------------------------------------------------------------------------------------
        m = Qd(fmaxf(fmaxf(red[0][0][fi], red[0][1][fi]), fmaxf(red[0][2][fi], red[0][3][fi])));
        const float c = g.exp2 ? 0.5f : 0.72134752f;          // half of 1, or of log2(e)
#pragma unroll
        for (int i = 0; i < BS_TILES; ++i) {
            if (tile_of(i) < ntiles) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t x = qpair(lg[i][j]);
                    const uint32_t d = qpair(Pack<MXQ_BF16>::put(low_of(x) - m, high_of(x) - m));
                    float e0 = __builtin_amdgcn_exp2f(low_of(d) * c), e1 = __builtin_amdgcn_exp2f(high_of(d) * c);
                    e0 *= e0;
                    e1 *= e1;
                    const uint32_t e = qpair_nonneg(Pack<MXQ_BF16>::put(e0, e1));
                    lg[i][j] = e;
                    sum += low_of(e);
                    sum += high_of(e);
                }
            }
        }
    } else {
        // the element-by-element form: NaN sticks to the maximum like torch.max, Inf - Inf = NaN, ...
        float mg = -__builtin_inff();
#pragma unroll
        for (int i = 0; i < BS_TILES; ++i) {
            if (tile_of(i) < ntiles) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float x0 = Qd(low_of(lg[i][j])), x1 = Qd(high_of(lg[i][j]));
                    lg[i][j] = (mxq_bits(x0) >> 16) | (mxq_bits(x1) & 0xFFFF0000u);
                    mg = MaxOp::apply(MaxOp::apply(mg, x0), x1);
                }
            }
        }
        mg = MaxOp::apply(mg, __shfl_xor(mg, 32));
        if (fg == 0) red[1][wave][fi] = mg;
        __syncthreads();
        m = MaxOp::apply(MaxOp::apply(red[1][0][fi], red[1][1][fi]), MaxOp::apply(red[1][2][fi], red[1][3][fi]));
#pragma unroll
        for (int i = 0; i < BS_TILES; ++i) {
            if (tile_of(i) < ntiles) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float d0 = Q(low_of(lg[i][j]) - m), d1 = Q(high_of(lg[i][j]) - m);
                    const float e0 = Qp(g.exp2 ? exp2f(d0) : expf(d0)), e1 = Qp(g.exp2 ? exp2f(d1) : expf(d1));
                    lg[i][j] = (mxq_bits(e0) >> 16) | (mxq_bits(e1) & 0xFFFF0000u);
                    sum += e0;
                    sum += e1;
                }
            }
        }
        __syncthreads();                                      // red[1] is reused for the sums below
    }
    sum += __shfl_xor(sum, 32);
    if (fg == 0) red[1][wave][fi] = sum;
    __syncthreads();
    const float s = Qp(((red[1][0][fi] + red[1][1][fi]) + red[1][2][fi]) + red[1][3][fi]);

    // ---- phase 3: the quotients ---------------------------------------------------------------------
    // one refined reciprocal per row; e * r is within two units in the last place of e / s, which
    // the rounding to bf16 hides except within that distance of a rounding boundary
    const float r0 = __builtin_amdgcn_rcpf(s);
    const float r1 = fmaf(fmaf(-s, r0, 1.0f), r0, r0);
    // A lane holds, of a pair of tiles, four 16-byte pieces of its row's 128-byte line: pieces fg and
    // 2 + fg of either tile.  They go through the wave's (now idle) part of the ring so that the store
    // instructions write whole lines: piece p of row r sits at position p ^ (r & 7) of the row's 128
    // bytes (conflict-free both ways); lane L then picks up piece L % 8 of the rows 8 k + L / 8.
    unsigned char* stage = const_cast<unsigned char*>(my_ring);
    const int srow = lane >> 3, spiece = lane & 7;
    unsigned short* out = reinterpret_cast<unsigned short*>(g.out) + bz * g.batch_c + (int64_t)(m0 + srow) * g.N + 8 * spiece;
#pragma unroll
    for (int k = 0; k < BS_TILES / 2; ++k) {
        const int t0 = tile_of(2 * k);
        if (t0 < ntiles) {                                    // uniform per wave
            unsigned char* buf = stage + (k & 1) * BS_TILE_BYTES;
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int i = 2 * k + p;
                uint32_t o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float e0 = low_of(lg[i][j]), e1 = high_of(lg[i][j]);
                    if (plain) {
                        o[j] = qpair_nonneg(Pack<MXQ_BF16>::put(e0 * r1, e1 * r1));
                    } else {
                        const float q0 = Qp(e0 / s), q1 = Qp(e1 / s);
                        o[j] = (mxq_bits(q0) >> 16) | (mxq_bits(q1) & 0xFFFF0000u);
                    }
                }
                *reinterpret_cast<u32x4*>(buf + mxq_addr::scores_stage_addr(fi, 4 * p + fg)) = u32x4{o[0], o[1], o[2], o[3]};
                *reinterpret_cast<u32x4*>(buf + mxq_addr::scores_stage_addr(fi, 4 * p + 2 + fg)) = u32x4{o[4], o[5], o[6], o[7]};
            }
            const bool second = t0 + 1 < ntiles;              // an odd number of tiles: the last line is half a line
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 8 * r + srow;
                const u32x4 v = *reinterpret_cast<const u32x4*>(buf + mxq_addr::scores_stage_addr(row, spiece));
                if (m0 + row < g.M && (second || spiece < 4))
                    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(out + (int64_t)(8 * r) * g.N + t0 * 32));
            }
        }
    }
}

}  // namespace
