// Row-streaming MFMA kernel for conv2d_gw8 forward and data gradient (gfx950).
//
// Contract (reference kernel: spio/src/conv2d_gw8.cu:10-225, both modes):
//   fprop : y[n,p,q,k]     = rn16(bias[k] + sum_{c,r,s} x[n,p+r-py,q+s-px,8g+c] * w[k,r,s,c])
//   dgrad : dx[n,h,w,8g+c] = rn16(sum_{j,r,s} dy[n,h-r+py,w-s+px,8g+j] * w[8g+j,r,s,c])
// Both are "dst = conv(src, filter, effective padding)"; dgrad uses the flipped,
// group-transposed filter and padding (R-1-py, S-1-px), which may be negative.
//
// Design
//   * A workgroup owns SPIO_BP output rows of SPIO_NB images for SPIO_GB
//     channel groups.  It streams the BP+R-1 source rows it needs through a
//     two-row LDS ring, one row per step, so every source element is read
//     from HBM once per workgroup and every tap reuses it from LDS/registers.
//   * In LDS a row is stored group-major: [group][flattened pixel][8 ch], the
//     pixels of the NB images laid side by side, each image padded to
//     WPI = DW+S-1 columns so that the zero halo is materialised once and a
//     tap is a plain pixel offset.
//   * One wave owns one group.  Per 16-pixel tile and source row it issues
//     one 16-byte LDS read per lane and ceil(R/2)*ceil(S/4) MFMAs
//     v_mfma_f32_16x16x32_f16 with
//         A (16 x 32) = filter:  rows m = 8*j + k   (two output-row slots j, 8 out channels k)
//                               cols  = 8*kb + c   (four column taps kb, 8 in channels c)
//         B (32 x 16) = source:  col n = pixel, rows = (tap kb, channel c)
//     Lane (n, kb) of B is exactly the 16 bytes of pixel n+kb, so the fragment
//     needs no shuffling.  The two row slots of A belong to two *different*
//     output rows: a source row contributes to R output rows, which live in
//     NS = 2*ceil(R/2) accumulator slots that rotate (slot = output row mod
//     NS); the filter row used for a slot at a step follows from the phase,
//     so accumulators never move between lanes.
//   * A finished output row is converted to fp16, staged through LDS into
//     pixel-major order and stored with one coalesced 16-byte store per lane.
//   * One workgroup barrier per step; global loads run SPIO_PF rows ahead of
//     the row being computed.
//   * Global memory is reached through buffer instructions whose hardware
//     bounds check does the predication: lanes without data carry an
//     out-of-range offset, rows outside the image use a descriptor of size
//     zero.  Such loads return zeros (the zero padding of the convolution) and
//     such stores are dropped, so no memory instruction sits under a branch.
//     Together with the fully unrolled step loop this lets the compiler count
//     the outstanding loads and stores exactly: the wait before a row is used
//     is for that row only.  (A wait counter covers loads and stores alike; a
//     count merged over paths that issue different numbers of them degrades
//     to the smallest, i.e. to waiting for rows that are not needed yet.)
#include "spio_conv_common.h"

using namespace spio;

#ifndef SPIO_IGRAD
#define SPIO_IGRAD 0
#endif
#ifndef SPIO_HAS_BIAS
#define SPIO_HAS_BIAS 0
#endif
#ifndef SPIO_PF
#define SPIO_PF 2
#endif
#ifndef SPIO_PF0
#define SPIO_PF0 SPIO_PF
#endif
#ifndef SPIO_PF_RATE
#define SPIO_PF_RATE 1
#endif
#ifndef SPIO_BP2
#define SPIO_BP2 0
#endif
#ifndef SPIO_BQ
#define SPIO_BQ 0
#endif
#ifndef SPIO_TS
#define SPIO_TS 1
#endif
#ifndef SPIO_NB
#define SPIO_NB 1
#endif
#ifndef SPIO_XCD_CHUNK
#define SPIO_XCD_CHUNK 0
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

constexpr int GB = SPIO_GB;  // groups (waves along channels) per workgroup
constexpr int BP = SPIO_BP;  // output rows per workgroup
// Two tile heights (SPIO_BP2 > 0): the row blocks of an image alternate between BP and BP2 rows;
// the first half of the grid takes the BP-row tiles and the second half the BP2-row tiles.  A
// grid of two workgroups per compute unit is dispatched as two cohorts (ids below half the grid
// land one per CU first, the rest join them a moment later); memory serves requests in arrival
// order, so the first cohort's prefetch burst is served before the second cohort's first row,
// the second cohort trails by that burst for the whole kernel and then finishes alone at one
// workgroup per CU (measured at N=128, C=64, 56x56 with equal tiles: 13.3 us against 18.0 us).
// Taller tiles for the leading cohort and shorter ones for the trailing one let both end together.
constexpr int BP2 = SPIO_BP2;
constexpr int NB = SPIO_NB;  // images per workgroup
constexpr int TS = SPIO_TS;  // waves sharing the tiles of one group
constexpr int PF = SPIO_PF;  // prefetch distance in rows (register buffers for rows in flight)
// The distance is reached by a ramp: PF0 rows are requested before the first step and PF_RATE
// rows per step from then on until the requests run PF rows ahead.  All workgroups of a launch
// start within a fraction of a microsecond of each other and memory serves requests roughly in
// the order they arrive; a workgroup that asks for all PF rows at once gets them before a
// workgroup that started a moment later gets its first row, and the late ones then finish long
// after the others.  With a short first burst every workgroup has its first rows early.
constexpr int PF0 = SPIO_PF0 < SPIO_PF ? SPIO_PF0 : SPIO_PF;
constexpr int PF_RATE = SPIO_PF_RATE;
constexpr int WAVES = GB * TS;
constexpr int THREADS = 64 * WAVES;

constexpr int NS = 2 * ((kR + 1) / 2);  // accumulator row slots
// With an odd filter height every slot rests for one step between two output rows: the finished
// row can then be converted and staged one step after its last tap (see the step loop).
#ifndef SPIO_LATE_EMIT
#define SPIO_LATE_EMIT 1
#endif
constexpr bool kLateEmit = SPIO_LATE_EMIT && NS > kR;
constexpr int NACC = NS / 2;            // accumulators (pairs of slots) per tile
constexpr int KB = (kS + 3) / 4;        // MFMA K-steps per source row (4 column taps each)
// Column blocks (SPIO_BQ > 0): a workgroup owns BQ output columns of its rows and stages the
// BQ + S - 1 source columns they need; the S - 1 extra columns hold the neighbouring blocks'
// pixels, or zeros at the image's edges (reference: block_q / block_w = block_q + S - 1,
// spio/kernels/conv2d_gw8_kernel.py:92-108, and the column halo of spio/src/conv2d_gw8.cu:71-91).
// Rows of any width then fit the LDS ring.  0 = the whole width.
constexpr int BQ = SPIO_BQ > 0 ? SPIO_BQ : DW;
constexpr int QBLKS = (DW + BQ - 1) / BQ;
constexpr int WPI = BQ + kS - 1;        // padded width of one image (block) in LDS
constexpr int F = NB * WPI;             // flattened pixels of a staged row
constexpr int WT = (F - kS + 1 + 15) / 16;  // 16-pixel tiles per row
constexpr int TPW = (WT + TS - 1) / TS;     // tiles per wave
constexpr int FP = 16 * WT + 4 * KB - 1;    // pixels any fragment read can touch
constexpr int GS = FP + ((9 - FP % 16) + 16) % 16;  // group stride in pixels, = 9 mod 16
constexpr int NR = 2;                               // ring rows
constexpr int RING_ROW_UNITS = GB * GS + 1;         // 16-byte units per ring row (+1: dump cell)
constexpr int DUMP_UNIT = GB * GS;                  // where lanes without a cell write
constexpr int OSTRIDE = GB * 16 + 16;               // bytes per pixel in the output stage
constexpr int OUT_ROW_BYTES = 16 * WT * OSTRIDE;
constexpr int IN_CELLS = F * GB;
constexpr int LPT = (IN_CELLS + THREADS - 1) / THREADS;  // source cells per thread per row
constexpr int OUT_CELLS = NB * BQ * GB;
constexpr int SPT = (OUT_CELLS + THREADS - 1) / THREADS;  // stores per thread per row
constexpr int GBLKS = (kGroups + GB - 1) / GB;
constexpr int PAIRS = (DH + BP + BP2 - 1) / (BP + BP2);  // (BP, BP2) pairs of row blocks per image
constexpr int PBLKS = BP2 > 0 ? PAIRS : (DH + BP - 1) / BP;  // row blocks of one height per image
constexpr int NBLKS = (kN + NB - 1) / NB;
constexpr int HALF_BLOCKS = GBLKS * PBLKS * QBLKS * NBLKS;  // workgroups per tile height
constexpr int NUM_BLOCKS = (BP2 > 0 ? 2 : 1) * HALF_BLOCKS;

// The step loop is unrolled completely: every rotation index and every "is there a row to load
// / to store" is then a compile-time fact, and no memory instruction sits in a loop whose entry
// and back edge would disagree about the operations in flight.
#ifndef SPIO_MAX_UNROLL
#define SPIO_MAX_UNROLL 64
#endif
static_assert((BP > BP2 ? BP : BP2) + kR - 1 <= SPIO_MAX_UNROLL, "block_p + R - 1 exceeds the unrolled step limit");
static_assert(PF >= 2 && PF0 >= 2 && PF_RATE >= 1 && WAVES <= 16, "bad configuration");
constexpr int STREAM_UNITS = NR * RING_ROW_UNITS + 2 * OUT_ROW_BYTES / 16;
constexpr int FILTER_UNITS = kIgrad ? GB * 8 * kR * kS : 0;  // staged filters (data gradient only)
constexpr int LDS_UNITS = STREAM_UNITS > FILTER_UNITS ? STREAM_UNITS : FILTER_UNITS;
static_assert(LDS_UNITS * 16 <= 160 * 1024, "LDS overflow");

// Byte extents of the NB-image block a workgroup addresses through one buffer descriptor.
constexpr long long SRC_IMAGE_BYTES = (long long)SH * SW * kC * 2;
constexpr long long DST_IMAGE_BYTES = (long long)DH * DW * kC * 2;
static_assert(NB * SRC_IMAGE_BYTES < (1ll << 31) && NB * DST_IMAGE_BYTES < (1ll << 31),
              "an image block must stay below 2 GiB (32-bit buffer offsets)");
constexpr unsigned OOB = 0x80000000u;  // offset of a lane without data: beyond every descriptor

constexpr int pmod(int a, int m) { return ((a % m) + m) % m; }
constexpr int cmin(int a, int b) { return a < b ? a : b; }
// Source rows requested once step t of `steps` has issued its loads (t = -1: before the first step).
constexpr int rows_requested(int t, int steps) { return cmin(cmin(steps, t + 1 + PF), PF0 + PF_RATE * (t + 1)); }

// Source rows shared with the neighbouring row blocks (the first and last R-1
// steps) can be served from L2 when the neighbour runs on the same XCD;
// SPIO_HALO_CACHED = 1 loads those with the default policy and only the
// interior rows with the non-temporal hint.
#ifndef SPIO_HALO_CACHED
#define SPIO_HALO_CACHED 0
#endif
// Cache-policy operands of the buffer instructions (gfx950: 1 = sc0, 2 = nt, 16 = sc1), one for
// the interior source rows, one for the rows shared with neighbouring row blocks, one for the
// stores.  SPIO_NT = 1 streams with the non-temporal hint unless a policy is given explicitly.
#ifndef SPIO_LD_POLICY
#define SPIO_LD_POLICY (SPIO_NT ? 2 : 0)
#endif
#ifndef SPIO_ST_POLICY
#define SPIO_ST_POLICY (SPIO_NT ? 2 : 0)
#endif
#ifndef SPIO_HALO_POLICY
#define SPIO_HALO_POLICY (SPIO_HALO_CACHED ? 0 : SPIO_LD_POLICY)
#endif
constexpr int AUX_LD = SPIO_LD_POLICY;
constexpr int AUX_HALO = SPIO_HALO_POLICY;
constexpr int AUX_ST = SPIO_ST_POLICY;

typedef __amdgpu_buffer_rsrc_t rsrc_t;
SPIO_DEVICE rsrc_t make_rsrc(const void* base, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// pointers typed in the LDS address space: 32-bit address arithmetic, constant parts of an
// index end up in the instruction's offset field
typedef __attribute__((address_space(3))) spio_uint4* lds_u4p;
typedef __attribute__((address_space(3))) unsigned char* lds_bytep;

// One tile: ROWS output rows starting at row p0 of the NB images from n0 on, channel block cb.
template <int ROWS>
SPIO_DEVICE void conv_rows(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                           const spio_half* __restrict__ weights, const float* __restrict__ bias,
                           const lds_u4p ring, const int p0, const int q0, const int n0, const int cb) {
    constexpr int STEPS = ROWS + kR - 1;
    const lds_bytep ostage = (lds_bytep)(ring + NR * RING_ROW_UNITS);

    const int tid = thread_id();
    const int lane = tid & 63;
    // the wave index as a scalar: whatever depends on it alone stays in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = wave % GB;  // group within the workgroup
    const int ws = wave / GB;  // tile split index
    const int gglob = cb * GB + wg;
    const bool wave_active = gglob < kGroups;  // idle waves compute on zeros and store nothing

    // ---- buffer descriptors: the workgroup's image block of src and of dst ----
    // Offsets are relative to the block's first image; images past the end of the batch lie
    // beyond the descriptor's size, so their loads give zeros and their stores are dropped.
    const int images = imin(NB, kN - n0);
    const rsrc_t rs_src = make_rsrc(reinterpret_cast<const unsigned char*>(src) + n0 * SRC_IMAGE_BYTES,
                                    (int)(images * SRC_IMAGE_BYTES));
    const rsrc_t rs_dst = make_rsrc(reinterpret_cast<const unsigned char*>(dst) + n0 * DST_IMAGE_BYTES,
                                    (int)(images * DST_IMAGE_BYTES));
    const rsrc_t rs_src_none = make_rsrc(reinterpret_cast<const unsigned char*>(src), 0);
    const rsrc_t rs_dst_none = make_rsrc(reinterpret_cast<const unsigned char*>(dst), 0);

    // ---- loop-invariant addressing of the cooperative row load ----
    // Every thread issues the same loads on every step.  Cells that hold no source data (halo
    // columns, missing groups) carry the out-of-range offset: the load returns zeros, which is
    // what the halo must hold.  Threads without a cell write to the row's dump cell.
    unsigned in_voff[LPT];  // byte offset inside the image block; row term excluded
    int in_lds[LPT];        // 16-byte unit inside a ring row
#pragma unroll
    for (int l = 0; l < LPT; ++l) {
        const int cell = tid + THREADS * l;
        in_voff[l] = OOB;
        in_lds[l] = DUMP_UNIT;
        if (cell < IN_CELLS) {
            const int g = cell % GB;
            const int f = cell / GB;
            const int img = f / WPI;
            const int col = q0 + f % WPI - EPX;
            in_lds[l] = g * GS + f;
            if (col >= 0 && col < SW && cb * GB + g < kGroups)
                in_voff[l] = (unsigned)(((img * SH * SW + col) * kGroups + cb * GB + g) * 16);
        }
    }
    constexpr int SRC_ROW_BYTES = SW * kC * 2;
    constexpr int DST_ROW_BYTES = DW * kC * 2;

    // Source row `t` of this workgroup (image row p0 + t - EPY) for every cell of the thread.
    // Rows outside the image read through the empty descriptor: zeros, the vertical padding.
    auto load_row = [&](spio_uint4(&regs)[LPT], int t) {
        const int h = p0 + t - EPY;
        const bool inside = h >= 0 && h < SH;
        const rsrc_t rs = inside ? rs_src : rs_src_none;
        // (readfirstlane: the row offset must stay in a scalar register whatever the optimiser
        //  makes of the clamp)
        const int soff = __builtin_amdgcn_readfirstlane(imin(imax(h, 0), SH - 1) * SRC_ROW_BYTES);
        const bool halo = t < kR - 1 || t >= ROWS;
#pragma unroll
        for (int l = 0; l < LPT; ++l) {
            Pack16 v;
            v.i = halo ? __builtin_amdgcn_raw_buffer_load_b128(rs, (int)in_voff[l], soff, AUX_HALO)
                       : __builtin_amdgcn_raw_buffer_load_b128(rs, (int)in_voff[l], soff, AUX_LD);
            regs[l] = v.u;
        }
    };

    // ---- filter loads, first of all ----
    // Loads of one wave return in order, so what is requested first is what the first
    // multiplication waits for: the filters (a few loads per lane) go ahead of the PF source
    // rows, and the first step can start as soon as source row 0 has landed.  Branch-free: dead
    // taps and idle waves load a valid address and are zeroed when the fragments are built.
    constexpr int WLPT = kIgrad ? (GB * 8 * kR * kS + THREADS - 1) / THREADS : NS * KB;
    spio_uint4 wraw[WLPT];
    if (!kIgrad) {
        // A[m = out channel ch][c] = w[8g+ch][r][s][c]: 16 contiguous bytes per lane.
        // Lane (m = lane%16, kb = lane/16): row slot j = m/8, channel m%8, column tap 4u+kb;
        // the filter row of slot j at distance d is r = (d - j) mod NS (none if r >= R).
        const int m = lane & 15;
        const int kb = lane >> 4;
        const int j = m >> 3;
        const int ch = m & 7;
        const int gsafe = wave_active ? gglob : 0;
#pragma unroll
        for (int d = 0; d < NS; ++d) {
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const int r = (d - j + NS) % NS;
                const int s = 4 * u + kb;
                const int rr = r < kR ? r : 0;
                const int ss = s < kS ? s : 0;
                wraw[d * KB + u] = *reinterpret_cast<const spio_uint4*>(
                    weights + (((long long)(8 * gsafe + ch) * kR + rr) * kS + ss) * 8);
            }
        }
    } else {
        // the workgroup's filters as they lie in memory ([group][jj][r][s][8 ch]), WLPT units per thread
        constexpr int WUNITS = GB * 8 * kR * kS;
#pragma unroll
        for (int l = 0; l < WLPT; ++l) {
            const int i = imin(tid + THREADS * l, WUNITS - 1);
            const int g = i / (8 * kR * kS);
            const int rem = i % (8 * kR * kS);
            const int gs = cb * GB + g < kGroups ? cb * GB + g : 0;
            wraw[l] = reinterpret_cast<const spio_uint4*>(weights)[(long long)gs * (8 * kR * kS) + rem];
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the filter loads ahead of the row loads

    // ---- rows 0..PF-1 into registers: their latency covers the rest of the set-up ----
    spio_uint4 pre[PF][LPT];
#pragma unroll
    for (int t = 0; t < PF0; ++t) load_row(pre[t], imin(t, STEPS - 1));
    __builtin_amdgcn_sched_barrier(0);  // ... and the row loads ahead of everything that waits

    // ---- loop-invariant addressing of the cooperative row store ----
    unsigned out_voff[SPT];  // byte offset inside the image block; row term excluded
    int out_lds[SPT];        // byte offset inside an output-stage row
#pragma unroll
    for (int s = 0; s < SPT; ++s) {
        const int cell = tid + THREADS * s;
        out_voff[s] = OOB;
        out_lds[s] = 0;
        if (cell < OUT_CELLS) {
            const int g = cell % GB;
            const int q = (cell / GB) % BQ;
            const int img = cell / (GB * BQ);
            out_lds[s] = (img * WPI + q) * OSTRIDE + g * 16;
            if (cb * GB + g < kGroups && q0 + q < DW)
                out_voff[s] = (unsigned)(((img * DH * DW + q0 + q) * kGroups + cb * GB + g) * 16);
        }
    }

    // ---- filter fragments: wfrag[d][u], d = (phase - 2*acc) mod NS ----
    spio_half8 wfrag[NS][KB];
    if (!kIgrad) {
        const int m = lane & 15;
        const int kb = lane >> 4;
        const int j = m >> 3;
#pragma unroll
        for (int d = 0; d < NS; ++d) {
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const int r = (d - j + NS) % NS;
                const int s = 4 * u + kb;
                Pack16 v;
                v.u = (r < kR && s < kS) ? wraw[d * KB + u] : spio_uint4{0u, 0u, 0u, 0u};
                wfrag[d][u] = v.h;
            }
        }
    } else {
        // A[m = dx channel ch][jj] = w[8g+jj][R-1-r][S-1-s][ch]: the filter transposed within
        // the group.  The workgroup copies its groups' filters to LDS as they lie in memory
        // ([jj][r][s][8 ch]) and every wave reads its fragments with the transposing LDS read:
        // in a 16-lane block source lane 4*jr+t supplies 4 channels (half t%2) of row jj = jr for
        // the row slot t/2, and result lane i receives rows jj = 0..3 of column i = 8*slot + ch.
        constexpr int WUNITS = GB * 8 * kR * kS;
        const lds_u4p wlds = ring;  // ring and output stage are not in use yet
#pragma unroll
        for (int l = 0; l < WLPT; ++l) {
            const int i = tid + THREADS * l;
            if (i < WUNITS) wlds[i] = wraw[l];
        }
        block_sync();
        const int kb = lane >> 4;
        const int jr = (lane & 15) >> 2;
        const int t4 = lane & 3;
        const int src_slot = t4 >> 1;        // slot whose data this lane fetches
        const int my_slot = (lane & 15) >> 3;  // slot of the fragment row this lane receives
        typedef spio_short4 __attribute__((address_space(3))) * lds_ptr;
#pragma unroll
        for (int d = 0; d < NS; ++d) {
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const int s = 4 * u + kb;
                const int r_src = (d - src_slot + NS) % NS;
                const int r_mine = (d - my_slot + NS) % NS;
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
        block_sync();  // everyone has its fragments before the ring is zero-filled
    }

    // Accumulator lane layout: D[m = 4*(lane/16)+i][n = lane%16]: pixel n = lane%16,
    // row slot j = lane/32, channels 4*((lane/16)&1) + i.
    const int out_j = lane >> 5;
    const int out_kh = (lane >> 4) & 1;
    const int out_n = lane & 15;
    // this lane's place in a staged output row (tile 0 of the wave) and in a ring row
    const lds_bytep ostage_lane = ostage + (16 * ws + out_n) * OSTRIDE + wg * 16 + out_kh * 8;
    const int frag_unit = wg * GS + (lane & 15) + (lane >> 4);
    float bias_reg[4] = {0.f, 0.f, 0.f, 0.f};
    if (kHasBias && wave_active) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bias_reg[i] = bias[8 * gglob + 4 * out_kh + i];
    }
    spio_float4 acc[TPW][NACC];
#pragma unroll
    for (int i = 0; i < TPW; ++i)
#pragma unroll
        for (int a = 0; a < NACC; ++a)
            acc[i][a] = spio_float4{bias_reg[0], bias_reg[1], bias_reg[2], bias_reg[3]};

    // ---- zero the slack cells behind each group's pixels once: fragment reads of the last
    //      tiles touch them (they meet zero filter taps, so they must be finite), nothing ever
    //      writes them ----
    {
        constexpr int SLACK = GS - F;
        for (int i = tid; i < NR * GB * SLACK; i += THREADS) {
            const int row = i / (GB * SLACK);
            const int g = (i / SLACK) % GB;
            ring[row * RING_ROW_UNITS + g * GS + F + i % SLACK] = spio_uint4{0u, 0u, 0u, 0u};
        }
    }

    // ---- row 0 into the ring ----
    block_sync();  // slack zeroed
#pragma unroll
    for (int l = 0; l < LPT; ++l) ring[in_lds[l]] = pre[0][l];
    block_sync();

    // Coalesced store of the output row staged at step `ts` (in stage buffer `obuf`): the row
    // that received its last tap at that step.  Called one step later, after the barrier.  Rows
    // past the end of the image store through the empty descriptor: the instructions are issued
    // all the same and the hardware drops them.
    auto store_output_row = [&](int ts, int obuf) {
        const int p = p0 + ts - (kR - 1);
        const rsrc_t rs = p < DH ? rs_dst : rs_dst_none;
        // The row offset is added to the per-lane offset; the scalar-offset operand stays the
        // constant 0.  A 16-byte buffer store reads its data registers for a few cycles after it
        // issues, and only for the constant form does the compiler keep the next instructions
        // from writing them: with the row offset in a scalar register an accumulator moved into
        // the first data register right behind the store was stored in its place (seen on gfx950
        // as stray values in the first two channels of some pixels of one output row).
        const unsigned row_off = (unsigned)(imin(imax(p, 0), DH - 1) * DST_ROW_BYTES);
#pragma unroll
        for (int s = 0; s < SPT; ++s) {
            Pack16 v;
            v.u = *(lds_u4p)(ostage + obuf * OUT_ROW_BYTES + out_lds[s]);
            __builtin_amdgcn_raw_buffer_store_b128(v.i, rs, (int)(out_voff[s] + row_off), 0, AUX_ST);
        }
        store_group_end();
    };

    // Rows above and below the image are rows of zeros in the ring; their products are skipped (a
    // scalar branch around LDS reads and MFMAs only: with a 7-row filter on a 14-row image they
    // would be 6 of 20 steps).
    auto row_is_live = [&](int t) {
        const int h = p0 + t - EPY;
        return h >= 0 && h < SH;
    };
    spio_half8 bfrag[TPW][KB];
    auto read_fragments = [&](spio_half8(&frag)[TPW][KB], int ring_row) {
        const lds_u4p rrow = ring + ring_row * RING_ROW_UNITS + frag_unit;
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int tile = ws + TS * i;
            if (TS == 1 || tile < WT) {
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    Pack16 v;
                    v.u = rrow[16 * TS * i + 16 * ws + 4 * u];
                    frag[i][u] = v.h;
                }
            }
        }
    };
    // Stages the output row that received its last tap at step `te` (stage buffer te mod 2) and
    // resets its slot to the bias.  The row sits in one half of the lanes (slot j = lane / 32).
    // (Letting the other half convert along and write into spare bytes, which removes the
    // lane-dependent branch, is slower: 1-6 % at the benchmark shapes.)
    auto emit_row = [&](int te) {
        const int slot = pmod(te % NS - (kR - 1), NS);
        const int a = slot >> 1;
        const int j = slot & 1;
        if (out_j == j) {
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                const int tile = ws + TS * i;
                if (TS == 1 || tile < WT) {
                    if (te >= kR - 1) {
                        Pack8 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o.h[e] = (spio_half)acc[i][a][e];
                        typedef __attribute__((address_space(3))) spio_uint2* lds_u2p;
                        *(lds_u2p)(ostage_lane + (te & 1) * OUT_ROW_BYTES + 16 * TS * i * OSTRIDE) = o.u;
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][a][e] = bias_reg[e];
                }
            }
        }
    };
    auto multiply_tile = [&](int ph, int i) {
        const int tile = ws + TS * i;
        if (TS == 1 || tile < WT) {
#pragma unroll
            for (int a = 0; a < NACC; ++a) {
                const int d = pmod(ph - 2 * a, NS);
#pragma unroll
                for (int u = 0; u < KB; ++u)
                    acc[i][a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wfrag[d][u], bfrag[i][u], acc[i][a], 0, 0, 0);
            }
        }
    };
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
        const int ph = t % NS;    // all of these are compile-time constants after unrolling

        // 1. prefetch the next source rows, at most up to row t+PF (whose register buffer is
        //    free: row t is in LDS)
#pragma unroll
        for (int r = rows_requested(t - 1, STEPS); r < rows_requested(t, STEPS); ++r) load_row(pre[r % PF], r);

        // 2. fragment reads of this step's row; a finished output row is stored while they are
        //    in flight
        const bool row_live = row_is_live(t);
        if (row_live) read_fragments(bfrag, t % NR);
        if (kLateEmit) {
            // The row that received its last tap in the previous step is converted and staged
            // now, ahead of this step's multiplications: its results are long complete, and the
            // conversion runs while the fragment reads are on their way instead of behind the
            // MFMAs it would have to wait for.  Its slot rests during this step (NS > R: the
            // slot's filter row is out of range, its A rows are zero), so the values are still
            // there, and the reset takes effect before the slot's next row begins.  The row
            // staged in the previous step goes out.
            if (t >= kR + 1) store_output_row(t - 2, t & 1);
            if (t >= 1) emit_row(t - 1);  // (before the first finished row: resets only)
        } else {
            if (t >= kR) store_output_row(t - 1, (t + 1) & 1);
        }
        // 3. multiply source row t into the live output rows
        if (row_live) {
#pragma unroll
            for (int i = 0; i < TPW; ++i) multiply_tile(ph, i);
        }

        // 4. the row that received its last tap: stage it, reset its slot
        if (!kLateEmit) emit_row(t);

        // 5. the next source row not yet in the ring (loaded earlier) into its ring row
        if (t + 1 < STEPS) {
#pragma unroll
            for (int l = 0; l < LPT; ++l)
                ring[((t + 1) % NR) * RING_ROW_UNITS + in_lds[l]] = pre[(t + 1) % PF][l];
        }

        block_sync();
    }
    if (kLateEmit) {
        // the row staged in the last step goes out, the last row is staged and follows
        if (STEPS >= kR + 1) store_output_row(STEPS - 2, STEPS & 1);
        emit_row(STEPS - 1);
        block_sync();
    }
    store_output_row(STEPS - 1, (STEPS - 1) & 1);  // the last row
}

}  // namespace

extern "C" __global__ void SPIO_LAUNCH_BOUNDS(THREADS)
SPIO_KERNEL_NAME(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                 const spio_half* __restrict__ weights, const float* __restrict__ bias) {
    // One LDS block: the source-row ring, then the two output-stage rows.  The data-gradient
    // mode first uses the same block to stage the filters of the workgroup's groups.
    __shared__ spio_uint4 lds[LDS_UNITS];
    const lds_u4p ring = (lds_u4p)lds;

    // Workgroup -> (image block, channel block, row block), row block fastest.
    // Consecutive workgroup ids are dealt round-robin to the 8 XCDs.  Remap so that runs of
    // SPIO_XCD_CHUNK consecutive tiles land on one XCD (neighbouring row blocks share halo rows
    // through that XCD's L2) while the tiles in flight on the whole device at any moment still
    // form one compact, advancing range of addresses (HBM streams best through such a front;
    // eight distant fronts, one per XCD, cost several per cent).  0 = one contiguous range of
    // tiles per XCD.
    // With two tile heights the two halves of the grid are two such sequences of tiles, one per
    // height, and a tile and the one below it (the other height) have the same index in both:
    // their workgroups run on the same XCD and share their halo rows.
    const int raw = block_id();
    const bool second = BP2 > 0 && raw >= HALF_BLOCKS;
    int b = second ? raw - HALF_BLOCKS : raw;
    {
        constexpr int CH = SPIO_XCD_CHUNK;
        if (CH == 0) {
            if (HALF_BLOCKS % 8 == 0) b = (b & 7) * (HALF_BLOCKS / 8) + (b >> 3);
        } else if (CH > 1 && HALF_BLOCKS % (8 * CH) == 0) {
            const int x = b & 7;   // XCD
            const int k = b >> 3;  // position in that XCD's sequence
            b = (k / CH) * (8 * CH) + x * CH + k % CH;
        }
    }
    // Tile order: row blocks fastest, so that neighbours in a run share halo rows.  Where a
    // workgroup covers only part of a pixel's 128-byte lines (GB * 16 bytes per pixel), the channel
    // blocks that share those lines go fastest instead: dealt to different XCDs, every one of
    // them would fetch the whole lines from memory (measured: twice the algorithmic reads).
    // Column blocks go before the row blocks: neighbours share S - 1 columns of every row.
    constexpr bool kSplitLines = GBLKS > 1 && (GB * 16) % 128 != 0;
    constexpr int TILES = QBLKS * PBLKS;  // tiles of one image and channel block
    const int t = kSplitLines ? (b / GBLKS) % TILES : b % TILES;
    const int cb = kSplitLines ? b % GBLKS : (b / TILES) % GBLKS;
    const int nb = b / (TILES * GBLKS);
    const int pb = t / QBLKS;
    const int q0 = (t % QBLKS) * BQ;
    const int n0 = nb * NB;
    if (BP2 > 0) {
        const int p0 = pb * (BP + BP2);
        if (second)
            conv_rows<(BP2 > 0 ? BP2 : 1)>(dst, src, weights, bias, ring, p0 + BP, q0, n0, cb);
        else
            conv_rows<BP>(dst, src, weights, bias, ring, p0, q0, n0, cb);
    } else {
        conv_rows<BP>(dst, src, weights, bias, ring, pb * BP, q0, n0, cb);
    }
}
