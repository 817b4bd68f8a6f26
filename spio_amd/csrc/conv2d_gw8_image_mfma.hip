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
//     the pixels: each takes NACC/TS of them and reads the same source fragments.
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
constexpr int WAVES = GB * TS;
constexpr int THREADS = 64 * WAVES;

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
constexpr int DUMP_UNIT = NBUF * IN_UNITS;  // where lanes without a cell write: 32 units, one per
constexpr int DUMP_UNITS = 32;              // lane pair (same-address writes of a wave serialise)
constexpr int OUT_BASE_UNITS = NBUF * IN_UNITS + DUMP_UNITS;
constexpr int FILTER_UNITS = GB * 8 * kR * kS;  // the groups' filters, staged in the output region first
constexpr int OUT_REGION_UNITS = NBUF * OUT_BYTES / 16 > FILTER_UNITS ? NBUF * OUT_BYTES / 16 : FILTER_UNITS;
constexpr int LDS_UNITS = OUT_BASE_UNITS + OUT_REGION_UNITS;
constexpr int WLPT = (FILTER_UNITS + THREADS - 1) / THREADS;  // filter units per thread
constexpr int STEPS = DH + kR - 1;

constexpr int IN_CELLS = SH * NB * SW * GB;  // 16-byte cells of a source block that exist in memory
constexpr int LPT = (IN_CELLS + THREADS - 1) / THREADS;
constexpr int OUT_CELLS = DH * NB * DW * GB;
constexpr int SPT = (OUT_CELLS + THREADS - 1) / THREADS;
constexpr int GBLKS = (kGroups + GB - 1) / GB;
constexpr int NBLKS = (kN + NB - 1) / NB;            // image blocks in the batch
constexpr int WGBLKS = (NBLKS + ITERS - 1) / ITERS;  // workgroups along the batch

static_assert(NACC % TS == 0, "the waves of a group split the accumulators evenly");
static_assert(WAVES <= 16 && STEPS <= 64, "bad configuration");
static_assert(LDS_UNITS * 16 <= 160 * 1024, "LDS overflow");
static_assert(OUT_ROW_BYTES % 16 == 0, "output rows are read in 16-byte units");

constexpr long long SRC_IMAGE_BYTES = (long long)SH * SW * kC * 2;
constexpr long long DST_IMAGE_BYTES = (long long)DH * DW * kC * 2;
static_assert(NB * SRC_IMAGE_BYTES < (1ll << 31) && NB * DST_IMAGE_BYTES < (1ll << 31),
              "an image block must stay below 2 GiB (32-bit buffer offsets)");
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

// The kernel body for the wave with split index WS (compile-time: which accumulators a wave owns
// decides which filter fragments it needs at which step).
template <int WS>
SPIO_DEVICE void run(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                     const spio_half* __restrict__ weights, const float* __restrict__ bias,
                     lds_u4p lds, int tid, int wg) {
    const int lane = tid & 63;
    const lds_u4p inbuf = lds;
    const lds_bytep outbuf = (lds_bytep)(lds + OUT_BASE_UNITS);

    // Workgroup -> (channel block, run of ITERS image blocks); channel block fastest, so the
    // workgroups in flight cover whole pixels (all channels) of a compact range of images.
    const int b = block_id();
    const int cb = b % GBLKS;
    const int first_blk = (b / GBLKS) * ITERS;
    const int gglob = cb * GB + wg;
    const bool wave_active = gglob < kGroups;  // idle waves compute on zeros and store nothing

    // ---- the filters first: everything up to the first multiplication waits for them (global
    //      memory -> LDS -> barrier -> fragments), the image blocks are not needed before ----
    // the workgroup's filters as they lie in memory ([group][k or jj][r][s][8 ch]), coalesced
    spio_uint4 wraw[WLPT];
#pragma unroll
    for (int l = 0; l < WLPT; ++l) {
        const int i = imin(tid + THREADS * l, FILTER_UNITS - 1);
        const int g = i / (8 * kR * kS);
        const int rem = i % (8 * kR * kS);
        const int gs = cb * GB + g < kGroups ? cb * GB + g : 0;
        wraw[l] = reinterpret_cast<const spio_uint4*>(weights)[(long long)gs * (8 * kR * kS) + rem];
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- loop-invariant addressing of the cooperative block load and store ----
    unsigned in_voff[LPT];  // byte offset inside the image block
    int in_lds[LPT];        // 16-byte unit inside an input buffer
#pragma unroll
    for (int l = 0; l < LPT; ++l) {
        const int cell = tid + THREADS * l;
        in_voff[l] = OOB;
        in_lds[l] = -1;  // no cell: the lane's dump unit
        if (cell < IN_CELLS) {
            const int g = cell % GB;
            const int col = (cell / GB) % SW;
            const int img = (cell / (GB * SW)) % NB;
            const int row = cell / (GB * SW * NB);
            const int f = col + EPX;  // column in the padded image (negative padding crops)
            if (f >= 0 && f < WPI) {
                in_lds[l] = row * ROW_UNITS + g * GS + img * WPI + f;
                if (cb * GB + g < kGroups)
                    in_voff[l] = (unsigned)((((img * SH + row) * SW + col) * kGroups + cb * GB + g) * 16);
            }
        }
    }
    unsigned out_voff[SPT];  // byte offset inside the image block
    int out_lds[SPT];        // byte offset inside an output buffer
#pragma unroll
    for (int s = 0; s < SPT; ++s) {
        const int cell = tid + THREADS * s;
        out_voff[s] = OOB;
        out_lds[s] = 0;
        if (cell < OUT_CELLS) {
            const int g = cell % GB;
            const int q = (cell / GB) % DW;
            const int img = (cell / (GB * DW)) % NB;
            const int row = cell / (GB * DW * NB);
            out_lds[s] = row * OUT_ROW_BYTES + (img * WPI + q) * OSTRIDE + g * 16;
            if (cb * GB + g < kGroups)
                out_voff[s] = (unsigned)((((img * DH + row) * DW + q) * kGroups + cb * GB + g) * 16);
        }
    }

    // Image block `blk` of src / dst as a buffer descriptor.  Blocks before the workgroup's first
    // or past the end of the batch get size zero: their loads return zeros, their stores are
    // dropped, so the phases need no branches around memory instructions.
    auto block_rsrc = [&](const void* base, long long image_bytes, int blk, bool enabled) {
        const int n0 = blk * NB;
        const int images = enabled ? imin(NB, kN - n0) : 0;
        const bool any = images > 0;
        return make_rsrc(reinterpret_cast<const unsigned char*>(base) + (any ? n0 * image_bytes : 0),
                         any ? (int)(images * image_bytes) : 0);
    };
    auto load_block = [&](spio_uint4(&regs)[LPT], int blk, bool enabled) {
        const rsrc_t rs = block_rsrc(src, SRC_IMAGE_BYTES, blk, enabled);
#pragma unroll
        for (int l = 0; l < LPT; ++l) {
            Pack16 v;
            v.i = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)in_voff[l], 0, AUX_NT);
            regs[l] = v.u;
        }
    };
    // (Constant scalar-offset operand: the form for which the compiler keeps the data registers
    //  of a 16-byte buffer store untouched for the wait states the hardware needs.)
    auto store_block = [&](int blk, bool enabled, lds_bytep out) {
        const rsrc_t rs = block_rsrc(dst, DST_IMAGE_BYTES, blk, enabled);
#pragma unroll
        for (int s = 0; s < SPT; ++s) {
            Pack16 v;
            v.u = *(lds_u4p)(out + out_lds[s]);
            __builtin_amdgcn_raw_buffer_store_b128(v.i, rs, (int)out_voff[s], 0, AUX_NT);
        }
    };

    // ---- the first two blocks on their way ----
    // Two register sets hold the blocks in flight: at any time the loads of two image blocks per
    // workgroup are outstanding (one block per CU does not cover the memory latency: each phase
    // would wait for its block, and the device would run at a fraction of its bandwidth).
    spio_uint4 pre0[LPT], pre1[LPT];
    load_block(pre0, first_blk, true);
    load_block(pre1, first_blk + 1, ITERS > 1);
    __builtin_amdgcn_sched_barrier(0);  // both requests leave before anything waits

    // ---- while they travel: clear the input buffers (halo columns and slack stay zero from
    //      here on) ----
    for (int i = tid; i < NBUF * IN_UNITS + DUMP_UNITS; i += THREADS) inbuf[i] = spio_uint4{0u, 0u, 0u, 0u};

    // ---- filters through LDS (the output region is free until the first block is multiplied):
    //      every global byte is fetched once per workgroup, the fragments are LDS reads ----
    const lds_u4p wlds = lds + OUT_BASE_UNITS;
#pragma unroll
    for (int l = 0; l < WLPT; ++l) {
        const int i = tid + THREADS * l;
        if (i < FILTER_UNITS) wlds[i] = wraw[l];
    }
    block_sync();

    // Filter fragments wfrag[d][u]: what accumulator a of this wave (global index WS*APW + a)
    // multiplies at phase ph is wfrag[(ph - 2a) mod NS]; the rotation by the wave's first
    // accumulator is folded in here.
    spio_half8 wfrag[NS][KB];
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

    // Accumulator lane layout: D[m = 4*(lane/16)+i][n = lane%16]: pixel n = lane%16,
    // row slot j = lane/32, channels 4*((lane/16)&1) + i.
    const int out_j = lane >> 5;
    const int out_kh = (lane >> 4) & 1;
    const int out_n = lane & 15;
    const int ostage_lane = out_n * OSTRIDE + wg * 16 + out_kh * 8;  // tile 0, row 0
    const int frag_unit = wg * GS + (lane & 15) + (lane >> 4);       // tile 0, row 0, tap block 0
    float bias_reg[4] = {0.f, 0.f, 0.f, 0.f};
    if (kHasBias && wave_active) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bias_reg[i] = bias[8 * gglob + 4 * out_kh + i];
    }

    // ---- block 0 into input buffer 0, block 1 on its way.  The barrier also keeps the first
    //      output rows from being staged over filters that a slower wave is still reading. ----
    const int my_dump = DUMP_UNIT + (lane >> 1);
#pragma unroll
    for (int l = 0; l < LPT; ++l) inbuf[in_lds[l] < 0 ? my_dump : in_lds[l]] = pre0[l];
    load_block(pre0, first_blk + 2, ITERS > 2);
    block_sync();

    // One phase: block `it`.  `pre` is the register set that holds block it+1 when the phase
    // starts (block it+2 is in flight into the other set) and receives block it+3 at its end.
    auto phase = [&](int it, spio_uint4(&pre)[LPT]) {
        const int cur = SPIO_DB ? (it & 1) : 0;
        const int nxt = SPIO_DB ? (cur ^ 1) : 0;
        const lds_u4p in_cur = inbuf + cur * IN_UNITS;
        const lds_bytep out_cur = outbuf + cur * OUT_BYTES;

        // (a) the previous block's output out of the other output buffer
        if (SPIO_DB) store_block(first_blk + it - 1, it > 0, outbuf + nxt * OUT_BYTES);

        // (b) multiply the current block.  One basic block: no branch depends on the lane, so
        // the scheduler may overlap the LDS reads of a row with the multiplications of the row
        // before (the source fragments are read one active step ahead into a second set).
        spio_float4 acc[WT][APW];
#pragma unroll
        for (int i = 0; i < WT; ++i)
#pragma unroll
            for (int a = 0; a < APW; ++a)
                acc[i][a] = spio_float4{bias_reg[0], bias_reg[1], bias_reg[2], bias_reg[3]};

        constexpr int FIRST = WS * APW;  // this wave's first accumulator (global index)
        spio_half8 bfrag[2][WT][KB];
        auto read_fragments = [&](spio_half8(&frag)[WT][KB], int t) {
            const int h = t - EPY;
#pragma unroll
            for (int i = 0; i < WT; ++i) {
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    Pack16 v;
                    v.u = in_cur[h * ROW_UNITS + frag_unit + 16 * i + 4 * u];
                    frag[i][u] = v.h;
                }
            }
        };
        {
            constexpr int t0 = next_active_step(-1, FIRST);
            if (t0 >= 0) read_fragments(bfrag[0], t0);
        }

#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const int ph = t % NS;  // compile-time after unrolling, like everything derived from t
            // accumulator (local index) whose row is finished by this step, if it is this wave's
            const int emit_slot = pmod(ph - (kR - 1), NS);
            const int emit_acc = (emit_slot >> 1) / APW == WS ? (emit_slot >> 1) % APW : -1;
            if (step_is_active(t, FIRST)) {
                const int tn = next_active_step(t, FIRST);
                const int set = fragment_set(t, FIRST);
                if (tn >= 0) {
                    // The next row's fragments are requested before this row is multiplied and
                    // stay there: left to itself the scheduler sinks the reads down to their
                    // first use, and every row then waits for its own LDS round trip.
                    read_fragments(bfrag[set ^ 1], tn);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // the accumulator that is converted at the end of this step goes first, so that
                // the other multiplications cover the latency of its last one
#pragma unroll
                for (int k = 0; k < APW; ++k) {
                    const int a = emit_acc < 0 ? k : (k == 0 ? emit_acc : (k <= emit_acc ? k - 1 : k));
                    if (acc_is_useful(t, FIRST + a)) {
                        const int d = pmod(ph - 2 * a, NS);
#pragma unroll
                        for (int i = 0; i < WT; ++i) {
#pragma unroll
                            for (int u = 0; u < KB; ++u)
                                acc[i][a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wfrag[d][u], bfrag[set][i][u],
                                                                                   acc[i][a], 0, 0, 0);
                        }
                    }
                }
            }

            // The output row that received its last tap, if one of this wave's: stage it and
            // reset its slot.  The row sits in one half of the lanes (slot j = lane / 32); the
            // other half converts along, writes to the dump cell and keeps its accumulators.
            {
                const int slot = pmod(ph - (kR - 1), NS);
                const int ag = slot >> 1;  // accumulator (global index) and half holding the row
                const int j = slot & 1;
                if (ag / APW == WS) {
                    const int a = ag % APW;
                    const bool emit = t >= kR - 1;
                    const int p = t - (kR - 1);
                    const bool mine = out_j == j;
#pragma unroll
                    for (int i = 0; i < WT; ++i) {
                        if (emit) {
                            Pack8 o;
#pragma unroll
                            for (int e = 0; e < 4; ++e) o.h[e] = (spio_half)acc[i][a][e];
                            typedef __attribute__((address_space(3))) spio_uint2* lds_u2p;
                            const lds_bytep where =
                                mine ? out_cur + p * OUT_ROW_BYTES + 16 * i * OSTRIDE + ostage_lane
                                     : (lds_bytep)(inbuf + DUMP_UNIT) + lane * 8;
                            *(lds_u2p)where = o.u;
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][a][e] = mine ? bias_reg[e] : acc[i][a][e];
                    }
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // the wait for the next block stays behind the multiplications
        if (!SPIO_DB) {
            // single buffers: everyone is done reading the input and writing the output; this
            // block's output leaves now
            block_sync();
            store_block(first_blk + it, true, outbuf);
        }
        // (c) the next block, requested two phases ago, into the other input buffer
#pragma unroll
        for (int l = 0; l < LPT; ++l) {
            // the dump cells lie behind the buffers: not offset by the buffer
            const int unit = in_lds[l] < 0 ? my_dump : nxt * IN_UNITS + in_lds[l];
            inbuf[unit] = pre[l];
        }
        // (d) the block three ahead on its way: it has two phases to arrive
        load_block(pre, first_blk + it + 3, it + 3 < ITERS);
        block_sync();
    };
#pragma nounroll
    for (int it = 0; it < ITERS; it += 2) {
        phase(it, pre1);
        if (it + 1 < ITERS) phase(it + 1, pre0);
    }
    // the last block's output
    if (SPIO_DB) store_block(first_blk + ITERS - 1, true, outbuf + ((ITERS - 1) & 1) * OUT_BYTES);
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
    const int wg = wave % GB;  // group within the workgroup
    const int ws = wave / GB;  // which share of the accumulators
    if (TS == 1 || ws == 0) {
        run<0>(dst, src, weights, bias, lds, tid, wg);
    } else if (TS == 2 || ws == 1) {
        run<(TS > 1 ? 1 : 0)>(dst, src, weights, bias, lds, tid, wg);
    } else if (TS == 3 || ws == 2) {
        run<(TS > 2 ? 2 : 0)>(dst, src, weights, bias, lds, tid, wg);
    } else {
        run<(TS > 3 ? 3 : 0)>(dst, src, weights, bias, lds, tid, wg);
    }
}
