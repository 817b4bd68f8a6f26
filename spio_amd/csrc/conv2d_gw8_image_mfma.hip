// Whole-image MFMA kernel for conv2d_gw8 forward and data gradient on small images (gfx950).
//
// Contract (reference kernel: spio/src/conv2d_gw8.cu:10-225, both modes): the same as the
// row-streaming kernel conv2d_gw8_mfma.hip,
//   fprop : y[n,p,q,k]     = rn16(bias[k] + sum_{c,r,s} x[n,p+r-py,q+s-px,8g+c] * w[k,r,s,c])
//   dgrad : dx[n,h,w,8g+c] = rn16(sum_{j,r,s} dy[n,h-r+py,w-s+px,8g+j] * w[8g+j,r,s,c])
// i.e. "dst = conv(src, filter, effective padding)" with the flipped, group-transposed filter and
// padding (R-1-py, S-1-px) for the data gradient.
//
// Why a second kernel.  The row-streaming kernel synchronises its workgroup once per source row.
// On a 14x14 or 7x7 image a row is a few hundred bytes and one 16-pixel tile per wave: the
// barrier, the LDS round trip and the steps spent on rows above and below the image (R-1 of
// them per block) then cost more than the multiplications, and every workgroup reloads the
// filters of its groups for a single image.  Here a workgroup keeps the filter fragments in
// registers for SPIO_ITERS image blocks and moves whole image blocks through LDS:
//
//   * two input buffers and two output buffers in LDS, each a whole block of SPIO_NB images for
//     SPIO_GB groups; one workgroup barrier per image block (SPIO_DB = 0: one buffer of each and
//     two barriers per block, so that two workgroups fit a CU and overlap each other);
//   * in a phase every thread (a) stores the previous block's output from the other output buffer
//     with coalesced 16-byte stores, (b) multiplies the current block, row by row, with no
//     synchronisation between rows, (c) writes the next block, requested two phases ago, into
//     the other input buffer and (d) requests the block three ahead from global memory: the
//     loads of two blocks are in flight at any time, in two register sets;
//   * an input buffer holds the SH real rows only; rows above and below the image are never
//     staged or multiplied, and of the accumulators of a step only those whose output rows exist
//     are issued (all decided at compile time: the row loop is fully unrolled);
//   * the zero columns left and right of an image are written once, when the buffers are cleared;
//     later phases rewrite the real cells only;
//   * SPIO_TS waves share a group by splitting the accumulators (pairs of output-row slots), not
//     the pixels: each takes NACC/TS of them and reads the same source fragments;
//   * SPIO_MV > 0 adds that many data-mover waves, which do (a), (c) and (d) for the whole
//     workgroup while the other waves only multiply: loads, LDS traffic and stores then flow
//     while a block is multiplied instead of between two blocks.  Measured (MI355X): 3x3 on
//     14x14 images, 384 channels, 11.8 -> 8.6 us; no gain where the multiplications of a block
//     take longer than moving it (7x7 filters: 16.0 -> 16.8 us).
//
// Row layout in LDS, MFMA operand layout, rotating accumulator slots and the output transposition
// are those of the row-streaming kernel:
//   A (16 x 32) = filter: rows m = 8*j + k (two output-row slots j, 8 out channels k),
//                         cols 8*kb + c (four column taps kb, 8 in channels c)
//   B (32 x 16) = source: col n = pixel, rows (tap kb, channel c); lane (n, kb) holds the 16
//                         bytes of pixel n+kb
//   output row p lives in slot p mod NS, NS = 2*ceil(R/2); at source step t (source row t - EPY)
//   slot s takes filter row (t - s) mod NS.
#include "spio_conv_common.h"

using namespace spio;

#ifndef SPIO_IGRAD
#define SPIO_IGRAD 0
#endif
#ifndef SPIO_HAS_BIAS
#define SPIO_HAS_BIAS 0
#endif
#ifndef SPIO_TS
#define SPIO_TS 1
#endif
#ifndef SPIO_NB
#define SPIO_NB 1
#endif
#ifndef SPIO_ITERS
#define SPIO_ITERS 1
#endif
#ifndef SPIO_DB
#define SPIO_DB 1
#endif
#ifndef SPIO_MV
#define SPIO_MV 0
#endif

namespace {

constexpr bool kIgrad = SPIO_IGRAD != 0;
constexpr bool kHasBias = (SPIO_HAS_BIAS != 0) && !kIgrad;
constexpr int SH = kIgrad ? kP : kH;  // source rows / cols
constexpr int SW = kIgrad ? kQ : kW;
constexpr int DH = kIgrad ? kH : kP;  // destination rows / cols
constexpr int DW = kIgrad ? kW : kQ;
constexpr int EPY = kIgrad ? kR - 1 - kPadY : kPadY;
constexpr int EPX = kIgrad ? kS - 1 - kPadX : kPadX;

constexpr int GB = SPIO_GB;        // groups per workgroup
constexpr int NB = SPIO_NB;        // images side by side in one block
constexpr int TS = SPIO_TS;        // waves sharing one group (they split the accumulators)
constexpr int ITERS = SPIO_ITERS;  // image blocks per workgroup
constexpr int MV = SPIO_MV;        // data-mover waves (0: every wave moves data and multiplies)
constexpr int WAVES = GB * TS;     // multiplying waves
constexpr int THREADS = 64 * (WAVES + MV);
constexpr int MTHREADS = MV ? 64 * MV : THREADS;  // threads that move image blocks

constexpr int NS = 2 * ((kR + 1) / 2);  // accumulator row slots
constexpr int NACC = NS / 2;            // accumulators (pairs of slots) per tile
constexpr int APW = NACC / TS;          // accumulators per wave and tile
constexpr int KB = (kS + 3) / 4;        // MFMA K-steps per source row (4 column taps each)
constexpr int WPI = DW + kS - 1;        // padded width of one image in LDS
constexpr int F = NB * WPI;             // flattened pixels of a staged row
constexpr int WT = (F - kS + 1 + 15) / 16;  // 16-pixel tiles per row
constexpr int FP = 16 * WT + 4 * KB - 1;    // pixels any fragment read can touch
constexpr int GS = FP + ((9 - FP % 16) + 16) % 16;  // group stride in pixels, = 9 mod 16
constexpr int ROW_UNITS = GB * GS;                   // 16-byte units per staged source row
constexpr int IN_UNITS = SH * ROW_UNITS;             // one input buffer
constexpr int OSTRIDE = GB * 16 + 16;                // bytes per pixel in an output buffer
constexpr int OUT_ROW_BYTES = 16 * WT * OSTRIDE;
constexpr int OUT_BYTES = DH * OUT_ROW_BYTES;  // one output buffer
// SPIO_DB = 1: two input and two output buffers, one barrier per image block, one workgroup per
// CU for the shapes this kernel is for.  SPIO_DB = 0: one of each and a second barrier per block
// (the block's output leaves, and the next block enters, between the two); half the LDS, so two
// workgroups share a CU and one multiplies while the other moves data.
constexpr int NBUF = SPIO_DB ? 2 : 1;
constexpr int DUMP_UNIT = NBUF * IN_UNITS;  // where moving lanes without a cell write: 32 units, one
constexpr int DUMP_UNITS = 32;              // per lane pair (same-address writes of a wave serialise)
constexpr int OUT_BASE_UNITS = NBUF * IN_UNITS + DUMP_UNITS;
constexpr int FILTER_UNITS = GB * 8 * kR * kS;  // the groups' filters, staged in the output region first
constexpr int OUT_REGION_UNITS = NBUF * OUT_BYTES / 16 > FILTER_UNITS ? NBUF * OUT_BYTES / 16 : FILTER_UNITS;
constexpr int LDS_UNITS = OUT_BASE_UNITS + OUT_REGION_UNITS;
// The multiplying waves fetch the filters (with mover waves these have the image blocks to
// request, and would hold up the first barrier waiting for their share of the filters).
constexpr int FTHREADS = 64 * WAVES;
constexpr int WLPT = (FILTER_UNITS + FTHREADS - 1) / FTHREADS;  // filter units per thread
constexpr int STEPS = DH + kR - 1;

// A block is moved cell by cell (16 bytes: one pixel of one group), the cells numbered as they
// lie in memory ([image][row][col][group of the workgroup]).  A moving thread takes the cells
// mtid + MTHREADS * l; MTHREADS is a multiple of GB, so it stays with one group and its cells
// are CELL_STEP bytes apart in memory: one offset register serves all its loads and stores.
constexpr int IN_CELLS = NB * SH * SW * GB;
constexpr int LPT = (IN_CELLS + MTHREADS - 1) / MTHREADS;
constexpr int OUT_CELLS = NB * DH * DW * GB;
constexpr int SPT = (OUT_CELLS + MTHREADS - 1) / MTHREADS;
constexpr int PIXEL_STEP = MTHREADS / GB;            // pixels between a thread's consecutive cells
constexpr int CELL_STEP = PIXEL_STEP * kGroups * 16;  // and bytes
constexpr int GBLKS = (kGroups + GB - 1) / GB;
constexpr int NBLKS = (kN + NB - 1) / NB;            // image blocks in the batch
constexpr int WGBLKS = (NBLKS + ITERS - 1) / ITERS;  // workgroups along the batch

static_assert(NACC % TS == 0, "the waves of a group split the accumulators evenly");
static_assert(WAVES + MV <= 16 && STEPS <= 64, "bad configuration");
static_assert(MTHREADS % GB == 0, "a moving thread stays with one group");
static_assert(MV == 0 || SPIO_DB, "mover waves work on the other pair of buffers");
static_assert(LDS_UNITS * 16 <= 160 * 1024, "LDS overflow");
static_assert(OUT_ROW_BYTES % 16 == 0, "output rows are read in 16-byte units");

constexpr long long SRC_IMAGE_BYTES = (long long)SH * SW * kC * 2;
constexpr long long DST_IMAGE_BYTES = (long long)DH * DW * kC * 2;
static_assert(NB * SRC_IMAGE_BYTES < (1ll << 30) && NB * DST_IMAGE_BYTES < (1ll << 30) &&
                  (long long)(LPT > SPT ? LPT : SPT) * CELL_STEP < (1ll << 30),
              "an image block must stay far below 2 GiB (32-bit buffer offsets)");
constexpr unsigned OOB = 0x80000000u;    // offset of a lane without data: beyond every descriptor
constexpr int AUX_NT = SPIO_NT ? 2 : 0;  // cache-policy operand of the buffer instructions

typedef __amdgpu_buffer_rsrc_t rsrc_t;
SPIO_DEVICE rsrc_t make_rsrc(const void* base, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

constexpr int pmod(int a, int m) { return ((a % m) + m) % m; }

// Does output-row slot `slot` hold a row of the image at source step t, and does the filter
// have the row it would take there?
constexpr bool slot_is_useful(int t, int slot) {
    const int r = pmod(t - slot, NS);
    const int p = t - r;
    return r < kR && p >= 0 && p < DH;
}
constexpr bool acc_is_useful(int t, int a) { return slot_is_useful(t, 2 * a) || slot_is_useful(t, 2 * a + 1); }

// For the wave that owns accumulators first .. first+APW-1: is anything multiplied at step t
// (the source row exists and at least one of the accumulators is useful)?
constexpr bool step_is_active(int t, int first) {
    const int h = t - EPY;
    if (h < 0 || h >= SH) return false;
    for (int a = 0; a < APW; ++a)
        if (acc_is_useful(t, first + a)) return true;
    return false;
}
constexpr int next_active_step(int t, int first) {
    for (int u = t + 1; u < STEPS; ++u)
        if (step_is_active(u, first)) return u;
    return -1;
}
// which of the two source-fragment sets step t uses: they alternate over the active steps
constexpr int fragment_set(int t, int first) {
    int n = 0;
    for (int u = 0; u < t; ++u) n += step_is_active(u, first) ? 1 : 0;
    return n & 1;
}

typedef __attribute__((address_space(3))) spio_uint4* lds_u4p;
typedef __attribute__((address_space(3))) unsigned char* lds_bytep;

// f(Int<I>{}) for I = BEGIN .. END-1: a loop whose index is a compile-time constant in its body by
// construction (what is multiplied, read and stored at a step is decided per step; a loop left
// to the unroller turns the register arrays into memory when the unroller gives up on its size).
template <int I>
struct Int {
    static constexpr int value = I;
};
template <int BEGIN, int END, class F>
SPIO_DEVICE void static_for(F&& f) {
    if constexpr (BEGIN < END) {
        f(Int<BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// Workgroup -> (channel block, run of ITERS image blocks); channel block fastest, so the
// workgroups in flight cover whole pixels (all channels) of a compact range of images.
SPIO_DEVICE int channel_block() { return block_id() % GBLKS; }
SPIO_DEVICE int first_block() { return (block_id() / GBLKS) * ITERS; }

// ---- the filters: global memory -> registers -> LDS (the output region, free until the first
//      block is multiplied) -> fragments.  Every multiplying thread takes a share; every
//      global byte is fetched once per workgroup, coalesced, as it lies in memory
//      ([group][k or jj][r][s][8 ch]). ----
SPIO_DEVICE void request_filters(spio_uint4 (&wraw)[WLPT], const spio_half* __restrict__ weights, int tid) {
    const int cb = channel_block();
#pragma unroll
    for (int l = 0; l < WLPT; ++l) {
        const int i = imin(tid + FTHREADS * l, FILTER_UNITS - 1);
        const int g = i / (8 * kR * kS);
        const int rem = i % (8 * kR * kS);
        const int gs = cb * GB + g < kGroups ? cb * GB + g : 0;
        wraw[l] = reinterpret_cast<const spio_uint4*>(weights)[(long long)gs * (8 * kR * kS) + rem];
    }
}
SPIO_DEVICE void stage_filters(const spio_uint4 (&wraw)[WLPT], lds_u4p lds, int tid) {
    const lds_u4p wlds = lds + OUT_BASE_UNITS;
#pragma unroll
    for (int l = 0; l < WLPT; ++l) {
        const int i = tid + FTHREADS * l;
        if (i < FILTER_UNITS) wlds[i] = wraw[l];
    }
}
// The input buffers start as zeros: the halo columns and the slack stay zero from here on, later
// blocks rewrite the real cells only.
SPIO_DEVICE void clear_input_buffers(lds_u4p lds, int tid) {
    for (int i = tid; i < NBUF * IN_UNITS + DUMP_UNITS; i += THREADS) lds[i] = spio_uint4{0u, 0u, 0u, 0u};
}

// Filter fragments wfrag[d][u] of the wave with split index WS: what accumulator a of this wave
// (global index WS*APW + a) multiplies at phase ph is wfrag[(ph - 2a) mod NS]; the rotation by
// the wave's first accumulator is folded in here.
template <int WS>
SPIO_DEVICE void load_filter_fragments(spio_half8 (&wfrag)[NS][KB], lds_u4p lds, int wg, int lane) {
    const lds_u4p wlds = lds + OUT_BASE_UNITS;
    constexpr int ROT = 2 * WS * APW;
    if (!kIgrad) {
        // A[m = out channel ch][c] = w[8g+ch][r][s][c]: 16 contiguous bytes per lane.
        // Lane (m = lane%16, kb = lane/16): row slot j = m/8, channel m%8, column tap 4u+kb.
        const int m = lane & 15;
        const int kb = lane >> 4;
        const int j = m >> 3;
        const int ch = m & 7;
#pragma unroll
        for (int d = 0; d < NS; ++d) {
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const int r = pmod(d - ROT - j, NS);
                const int s = 4 * u + kb;
                const int rr = r < kR ? r : 0;
                const int ss = s < kS ? s : 0;
                Pack16 v;
                v.u = wlds[((wg * 8 + ch) * kR + rr) * kS + ss];
                if (!(r < kR && s < kS)) v.u = spio_uint4{0u, 0u, 0u, 0u};
                wfrag[d][u] = v.h;
            }
        }
    } else {
        // A[m = dx channel ch][jj] = w[8g+jj][R-1-r][S-1-s][ch]: the filter transposed within the
        // group, read from the staged copy ([jj][r][s][8 ch]) with the transposing LDS read: in a
        // 16-lane block source lane 4*jr+t supplies 4 channels (half t%2) of row jj = jr for the
        // row slot t/2, and result lane i receives rows jj = 0..3 of column i = 8*slot + ch.
        const int kb = lane >> 4;
        const int jr = (lane & 15) >> 2;
        const int t4 = lane & 3;
        const int src_slot = t4 >> 1;          // slot whose data this lane fetches
        const int my_slot = (lane & 15) >> 3;  // slot of the fragment row this lane receives
        typedef spio_short4 __attribute__((address_space(3))) * lds_ptr;
#pragma unroll
        for (int d = 0; d < NS; ++d) {
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const int s = 4 * u + kb;
                const int r_src = pmod(d - ROT - src_slot, NS);
                const int r_mine = pmod(d - ROT - my_slot, NS);
                // clamp the address of dead taps; their result is discarded below
                const int rr = r_src < kR ? kR - 1 - r_src : 0;
                const int ss = s < kS ? kS - 1 - s : 0;
                const lds_bytep base = (lds_bytep)wlds + ((((wg * 8 + jr) * kR + rr) * kS + ss) * 16) + (t4 & 1) * 8;
                union {
                    spio_short4 q[2];
                    spio_half8 h;
                } v;
                v.q[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)base);
                v.q[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(base + 4 * kR * kS * 16));
                if (!(r_mine < kR && s < kS)) v.h = spio_half8{0, 0, 0, 0, 0, 0, 0, 0};
                wfrag[d][u] = v.h;
            }
        }
    }
}

// ---- moving image blocks: addressing of thread mtid of the MTHREADS moving threads ----
struct BlockMover {
    const spio_uint4* src;
    spio_uint4* dst;
    unsigned voff;     // byte offset of the thread's cell 0 inside an image block (source and
                       // destination blocks are laid out alike); OOB: no such group
    int in_lds[LPT];   // 16-byte unit inside an input buffer; cells without one go to `dump`
    int out_lds[SPT];  // byte offset inside an output buffer
    int dump;

    // what the loads need (so that the first block can be requested before the rest is worked out)
    SPIO_DEVICE void init_global(spio_uint4* dst_, const spio_uint4* src_, int mtid) {
        src = src_;
        dst = dst_;
        const int cb = channel_block();
        const int g = mtid % GB;
        const int pix0 = mtid / GB;
        voff = cb * GB + g < kGroups ? (unsigned)((pix0 * kGroups + cb * GB + g) * 16) : OOB;
    }
    SPIO_DEVICE void init_lds(int mtid) {
        const int g = mtid % GB;
        const int pix0 = mtid / GB;
        dump = DUMP_UNIT + ((mtid & 63) >> 1);
#pragma unroll
        for (int l = 0; l < LPT; ++l) {
            const int pix = pix0 + PIXEL_STEP * l;
            const int img = pix / (SH * SW);
            const int row = (pix / SW) % SH;
            const int f = pix % SW + EPX;  // column in the padded image (negative padding crops)
            in_lds[l] = (img < NB && f >= 0 && f < WPI) ? row * ROW_UNITS + g * GS + img * WPI + f : -1;
        }
#pragma unroll
        for (int s = 0; s < SPT; ++s) {
            const int pix = pix0 + PIXEL_STEP * s;
            const int img = pix / (DH * DW);
            const int row = (pix / DW) % DH;
            const int q = pix % DW;
            out_lds[s] = img < NB ? row * OUT_ROW_BYTES + (img * WPI + q) * OSTRIDE + g * 16 : 0;
        }
    }
    // Image block `blk` of src / dst as a buffer descriptor.  Blocks before the workgroup's first
    // or past the end of the batch get size zero: their loads return zeros, their stores are
    // dropped, and so are the cells past the end of a block, so the phases need no branches
    // around memory instructions.
    SPIO_DEVICE static rsrc_t block_rsrc(const void* base, long long image_bytes, int blk, bool enabled) {
        const int n0 = blk * NB;
        const int images = enabled ? imin(NB, kN - n0) : 0;
        const bool any = images > 0;
        return make_rsrc(reinterpret_cast<const unsigned char*>(base) + (any ? n0 * image_bytes : 0),
                         any ? (int)(images * image_bytes) : 0);
    }
    SPIO_DEVICE void load(spio_uint4 (&regs)[LPT], int blk, bool enabled) const {
        const rsrc_t rs = block_rsrc(src, SRC_IMAGE_BYTES, blk, enabled);
#pragma unroll
        for (int l = 0; l < LPT; ++l) {
            Pack16 v;
            v.i = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(voff + (unsigned)(CELL_STEP * l)), 0, AUX_NT);
            regs[l] = v.u;
        }
    }
    // registers -> input buffer at 16-byte unit `base` (the dump cells lie behind the buffers:
    // not offset by the buffer)
    SPIO_DEVICE void to_lds(const spio_uint4 (&regs)[LPT], lds_u4p lds, int base) const {
#pragma unroll
        for (int l = 0; l < LPT; ++l) lds[in_lds[l] < 0 ? dump : base + in_lds[l]] = regs[l];
    }
    // (Constant scalar-offset operand: the form for which the compiler keeps the data registers
    //  of a 16-byte buffer store untouched for the wait states the hardware needs.)
    SPIO_DEVICE void store(int blk, bool enabled, lds_bytep out) const {
        const rsrc_t rs = block_rsrc(dst, DST_IMAGE_BYTES, blk, enabled);
#pragma unroll
        for (int s = 0; s < SPT; ++s) {
            Pack16 v;
            v.u = *(lds_u4p)(out + out_lds[s]);
            __builtin_amdgcn_raw_buffer_store_b128(v.i, rs, (int)(voff + (unsigned)(CELL_STEP * s)), 0, AUX_NT);
        }
        // (not in the mover waves: a scheduling fence after every block's stores costs them 8 % at
        //  384 channels 14x14; their stores keep the constant-offset form above, for which the
        //  compiler itself leaves the wait state)
        if (MV == 0) store_group_end();
    }
};

// ---- multiplying one image block: input buffer in_cur -> output buffer out_cur, by the wave of
//      group wg with split index WS ----
struct LaneLayout {
    // Accumulator lane layout: D[m = 4*(lane/16)+i][n = lane%16]: pixel n = lane%16,
    // row slot j = lane/32, channels 4*((lane/16)&1) + i.
    int out_j;
    // Byte offset in an output buffer (tile 0, row 0) where the lane writes when the half of the
    // lanes with row slot j holds the finished row: its 8 bytes of the row if that is its own
    // half, else 8 of the 16 spare bytes behind the groups of its pixel, which nobody reads.
    // Both halves then write with the same immediate offsets and no lane-dependent address
    // arithmetic is left in a step.
    int ostage_lane[2];
    int frag_unit;  // unit in an input buffer: tile 0, row 0, tap block 0
    SPIO_DEVICE void init(int wg, int lane) {
        out_j = lane >> 5;
        const int out_kh = (lane >> 4) & 1;
        const int out_n = lane & 15;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            ostage_lane[j] = out_n * OSTRIDE + (out_j == j ? wg * 16 : GB * 16) + out_kh * 8;
        frag_unit = wg * GS + (lane & 15) + (lane >> 4);
    }
};

template <int WS>
SPIO_DEVICE void multiply_block(lds_u4p in_cur, lds_bytep out_cur, const spio_half8 (&wfrag)[NS][KB],
                                const float (&bias_reg)[4], const LaneLayout& ll) {
    // One basic block: no branch depends on the lane, so the scheduler may overlap the LDS reads
    // of a row with the multiplications of the row before (the source fragments are read one
    // active step ahead into a second set).
    spio_float4 acc[WT][APW];
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int a = 0; a < APW; ++a) acc[i][a] = spio_float4{bias_reg[0], bias_reg[1], bias_reg[2], bias_reg[3]};

    constexpr int FIRST = WS * APW;  // this wave's first accumulator (global index)
    spio_half8 bfrag[2][WT][KB];
    auto read_fragments = [&](spio_half8(&frag)[WT][KB], int t) {
        const int h = t - EPY;
#pragma unroll
        for (int i = 0; i < WT; ++i) {
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                Pack16 v;
                v.u = in_cur[h * ROW_UNITS + ll.frag_unit + 16 * i + 4 * u];
                frag[i][u] = v.h;
            }
        }
    };
    {
        constexpr int t0 = next_active_step(-1, FIRST);
        if (t0 >= 0) read_fragments(bfrag[0], t0);
    }

    static_for<0, STEPS>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
        constexpr int ph = t % NS;
        // accumulator (local index) whose row is finished by this step, if it is this wave's
        constexpr int emit_slot = pmod(ph - (kR - 1), NS);
        constexpr int emit_acc = (emit_slot >> 1) / APW == WS ? (emit_slot >> 1) % APW : -1;
        if constexpr (step_is_active(t, FIRST)) {
            constexpr int tn = next_active_step(t, FIRST);
            constexpr int set = fragment_set(t, FIRST);
            if constexpr (tn >= 0) {
                // The next row's fragments are requested before this row is multiplied and stay
                // there: left to itself the scheduler sinks the reads down to their first use,
                // and every row then waits for its own LDS round trip.
                read_fragments(bfrag[set ^ 1], tn);
                __builtin_amdgcn_sched_barrier(0);
            }
            // Tap block by tap block over all accumulators, and the order pinned, so that no
            // multiplication waits for the one issued just before it (the scheduler pairs the
            // two of an accumulator if left alone).  The accumulator that is converted at the
            // end of this step goes first in each round, so that the others cover the latency of
            // its last one.
            static_for<0, KB>([&](auto uc) {
                constexpr int u = decltype(uc)::value;
                static_for<0, APW>([&](auto kc) {
                    constexpr int k = decltype(kc)::value;
                    constexpr int a = emit_acc < 0 ? k : (k == 0 ? emit_acc : (k <= emit_acc ? k - 1 : k));
                    if constexpr (acc_is_useful(t, FIRST + a)) {
                        constexpr int d = pmod(ph - 2 * a, NS);
#pragma unroll
                        for (int i = 0; i < WT; ++i)
                            acc[i][a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wfrag[d][u], bfrag[set][i][u],
                                                                               acc[i][a], 0, 0, 0);
                    }
                });
                __builtin_amdgcn_sched_barrier(0);
            });
        }

        // The output row that received its last tap, if one of this wave's: stage it and reset
        // its slot.  The row sits in one half of the lanes (slot j = lane / 32); the other half
        // converts along, writes into the spare bytes of the row and keeps its accumulators.
        constexpr int ag = emit_slot >> 1;  // accumulator (global index) and half holding the row
        constexpr int j = emit_slot & 1;
        if constexpr (ag / APW == WS) {
            constexpr int a = ag % APW;
            constexpr bool emit = t >= kR - 1;
            constexpr int p = t - (kR - 1);
            const bool mine = ll.out_j == j;
#pragma unroll
            for (int i = 0; i < WT; ++i) {
                if constexpr (emit) {
                    Pack8 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o.h[e] = (spio_half)acc[i][a][e];
                    typedef __attribute__((address_space(3))) spio_uint2* lds_u2p;
                    *(lds_u2p)(out_cur + ll.ostage_lane[j] + (p * OUT_ROW_BYTES + 16 * i * OSTRIDE)) = o.u;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][a][e] = mine ? bias_reg[e] : acc[i][a][e];
            }
        }
    });
}

SPIO_DEVICE void load_bias(float (&bias_reg)[4], const float* __restrict__ bias, int wg, int lane) {
    const int gglob = channel_block() * GB + wg;
    const int out_kh = (lane >> 4) & 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) bias_reg[i] = 0.f;
    if (kHasBias && gglob < kGroups) {  // idle waves compute on zeros; their stores are dropped
#pragma unroll
        for (int i = 0; i < 4; ++i) bias_reg[i] = bias[8 * gglob + 4 * out_kh + i];
    }
}

// ---- SPIO_MV = 0: every wave moves data and multiplies.  WS: the wave's split index
//      (compile-time: which accumulators a wave owns decides which filter fragments it needs at
//      which step). ----
template <int WS>
SPIO_DEVICE void run(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                     const spio_half* __restrict__ weights, const float* __restrict__ bias,
                     lds_u4p lds, int tid, int wg) {
    const int lane = tid & 63;
    const lds_u4p inbuf = lds;
    const lds_bytep outbuf = (lds_bytep)(lds + OUT_BASE_UNITS);
    const int first_blk = first_block();

    // the filters first: everything up to the first multiplication waits for them (global memory
    // -> LDS -> barrier -> fragments), the image blocks are not needed before
    spio_uint4 wraw[WLPT];
    request_filters(wraw, weights, tid);
    __builtin_amdgcn_sched_barrier(0);

    BlockMover mv;
    mv.init_global(dst, src, tid);
    // Two register sets hold the blocks in flight: at any time the loads of two image blocks per
    // workgroup are outstanding (one block per CU does not cover the memory latency: each phase
    // would wait for its block, and the device would run at a fraction of its bandwidth).
    spio_uint4 pre0[LPT], pre1[LPT];
    mv.load(pre0, first_blk, true);
    mv.load(pre1, first_blk + 1, ITERS > 1);
    __builtin_amdgcn_sched_barrier(0);  // both requests leave before anything waits
    mv.init_lds(tid);

    clear_input_buffers(lds, tid);  // while they travel
    stage_filters(wraw, lds, tid);
    block_sync();
    spio_half8 wfrag[NS][KB];
    load_filter_fragments<WS>(wfrag, lds, wg, lane);
    LaneLayout ll;
    ll.init(wg, lane);
    float bias_reg[4];
    load_bias(bias_reg, bias, wg, lane);

    // block 0 into input buffer 0, block 2 on its way.  The barrier also keeps the first output
    // rows from being staged over filters that a slower wave is still reading.
    mv.to_lds(pre0, inbuf, 0);
    mv.load(pre0, first_blk + 2, ITERS > 2);
    block_sync();

    // One phase: block `it`.  `pre` is the register set that holds block it+1 when the phase
    // starts (block it+2 is in flight into the other set) and receives block it+3 at its end.
    auto phase = [&](int it, spio_uint4(&pre)[LPT]) {
        const int cur = SPIO_DB ? (it & 1) : 0;
        const int nxt = SPIO_DB ? (cur ^ 1) : 0;
        // (a) the previous block's output out of the other output buffer
        if (SPIO_DB) mv.store(first_blk + it - 1, it > 0, outbuf + nxt * OUT_BYTES);
        // (b) multiply the current block
        multiply_block<WS>(inbuf + cur * IN_UNITS, outbuf + cur * OUT_BYTES, wfrag, bias_reg, ll);
        __builtin_amdgcn_sched_barrier(0);  // the wait for the next block stays behind the multiplications
        if (!SPIO_DB) {
            // single buffers: everyone is done reading the input and writing the output; this
            // block's output leaves now
            block_sync();
            mv.store(first_blk + it, true, outbuf);
        }
        // (c) the next block, requested two phases ago, into the other input buffer
        mv.to_lds(pre, inbuf, nxt * IN_UNITS);
        // (d) the block three ahead on its way: it has two phases to arrive
        mv.load(pre, first_blk + it + 3, it + 3 < ITERS);
        block_sync();
    };
#pragma nounroll
    for (int it = 0; it < ITERS; it += 2) {
        phase(it, pre1);
        if (it + 1 < ITERS) phase(it + 1, pre0);
    }
    // the last block's output
    if (SPIO_DB) mv.store(first_blk + ITERS - 1, true, outbuf + ((ITERS - 1) & 1) * OUT_BYTES);
}

// ---- SPIO_MV > 0: the two roles.  Both pass the same barriers: two in the set-up (filters
//      staged; block 0 staged and filter fragments read), one per image block. ----
template <int WS>
SPIO_DEVICE void multiplier_role(const spio_half* __restrict__ weights, const float* __restrict__ bias, lds_u4p lds,
                                 int tid, int wg) {
    const int lane = tid & 63;
    const lds_u4p inbuf = lds;
    const lds_bytep outbuf = (lds_bytep)(lds + OUT_BASE_UNITS);
    spio_uint4 wraw[WLPT];
    request_filters(wraw, weights, tid);
    __builtin_amdgcn_sched_barrier(0);
    clear_input_buffers(lds, tid);
    stage_filters(wraw, lds, tid);
    block_sync();
    spio_half8 wfrag[NS][KB];
    load_filter_fragments<WS>(wfrag, lds, wg, lane);
    LaneLayout ll;
    ll.init(wg, lane);
    float bias_reg[4];
    load_bias(bias_reg, bias, wg, lane);
    block_sync();
#pragma nounroll
    for (int it = 0; it < ITERS; ++it) {
        const int cur = it & 1;
        multiply_block<WS>(inbuf + cur * IN_UNITS, outbuf + cur * OUT_BYTES, wfrag, bias_reg, ll);
        block_sync();
    }
}

SPIO_DEVICE void mover_role(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src, lds_u4p lds, int tid) {
    const lds_u4p inbuf = lds;
    const lds_bytep outbuf = (lds_bytep)(lds + OUT_BASE_UNITS);
    const int first_blk = first_block();
    BlockMover mv;
    mv.init_global(dst, src, tid - 64 * WAVES);
    // Three blocks are requested before the first is multiplied (two here, the third once the
    // first is in LDS).  Every workgroup of the device starts at the same time, so the set-up is
    // a stretch in which the memory system only reads; holding the later blocks back until the
    // first has arrived starts the multiplications earlier, but the phases then ask for more
    // bandwidth than there is and the kernel is slower (measured: 16.5 against 15.0 us, 7x7 on
    // 14x14, N=256, C=256).
    spio_uint4 pre0[LPT], pre1[LPT];
    mv.load(pre0, first_blk, true);
    mv.load(pre1, first_blk + 1, ITERS > 1);
    __builtin_amdgcn_sched_barrier(0);
    mv.init_lds(tid - 64 * WAVES);
    clear_input_buffers(lds, tid);
    block_sync();
    mv.to_lds(pre0, inbuf, 0);
    mv.load(pre0, first_blk + 2, ITERS > 2);
    block_sync();
    // while block `it` is multiplied: the output of block it-1 leaves, block it+1 (in `pre`,
    // requested two phases ago) enters the other input buffer, block it+3 is requested
    auto phase = [&](int it, spio_uint4(&pre)[LPT]) {
        const int nxt = (it & 1) ^ 1;
        mv.store(first_blk + it - 1, it > 0, outbuf + nxt * OUT_BYTES);
        mv.to_lds(pre, inbuf, nxt * IN_UNITS);
        mv.load(pre, first_blk + it + 3, it + 3 < ITERS);
        block_sync();
    };
#pragma nounroll
    for (int it = 0; it < ITERS; it += 2) {
        phase(it, pre1);
        if (it + 1 < ITERS) phase(it + 1, pre0);
    }
    mv.store(first_blk + ITERS - 1, true, outbuf + ((ITERS - 1) & 1) * OUT_BYTES);
}

template <int WS>
SPIO_DEVICE void dispatch(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                          const spio_half* __restrict__ weights, const float* __restrict__ bias, lds_u4p lds,
                          int tid, int wg) {
    if (MV == 0)
        run<WS>(dst, src, weights, bias, lds, tid, wg);
    else
        multiplier_role<WS>(weights, bias, lds, tid, wg);
}

}  // namespace

extern "C" __global__ void SPIO_LAUNCH_BOUNDS(THREADS)
SPIO_KERNEL_NAME(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                 const spio_half* __restrict__ weights, const float* __restrict__ bias) {
    // One LDS block: the input buffer(s), the dump cell, the output buffer(s).  The output region
    // first holds the filters of the workgroup's groups.
    __shared__ spio_uint4 lds_block[LDS_UNITS];
    const lds_u4p lds = (lds_u4p)lds_block;
    const int tid = thread_id();
    // the wave index as a scalar: whatever depends on it alone stays in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (MV > 0 && wave >= WAVES) {
        mover_role(dst, src, lds, tid);
        return;
    }
    const int wg = wave % GB;  // group within the workgroup
    const int ws = wave / GB;  // which share of the accumulators
    if (TS == 1 || ws == 0) {
        dispatch<0>(dst, src, weights, bias, lds, tid, wg);
    } else if (TS == 2 || ws == 1) {
        dispatch<(TS > 1 ? 1 : 0)>(dst, src, weights, bias, lds, tid, wg);
    } else if (TS == 3 || ws == 2) {
        dispatch<(TS > 2 ? 2 : 0)>(dst, src, weights, bias, lds, tid, wg);
    } else {
        dispatch<(TS > 3 ? 3 : 0)>(dst, src, weights, bias, lds, tid, wg);
    }
}
