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
#ifndef SPIO_TS
#define SPIO_TS 1
#endif
#ifndef SPIO_NB
#define SPIO_NB 1
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
constexpr int NB = SPIO_NB;  // images per workgroup
constexpr int TS = SPIO_TS;  // waves sharing the tiles of one group
constexpr int PF = SPIO_PF;  // prefetch distance in rows
constexpr int WAVES = GB * TS;
constexpr int THREADS = 64 * WAVES;

constexpr int NS = 2 * ((kR + 1) / 2);  // accumulator row slots
constexpr int NACC = NS / 2;            // accumulators (pairs of slots) per tile
constexpr int KB = (kS + 3) / 4;        // MFMA K-steps per source row (4 column taps each)
constexpr int WPI = DW + kS - 1;        // padded width of one image in LDS
constexpr int F = NB * WPI;             // flattened pixels of a staged row
constexpr int WT = (F - kS + 1 + 15) / 16;  // 16-pixel tiles per row
constexpr int TPW = (WT + TS - 1) / TS;     // tiles per wave
constexpr int FP = 16 * WT + 4 * KB - 1;    // pixels any fragment read can touch
constexpr int GS = FP + ((9 - FP % 16) + 16) % 16;  // group stride in pixels, = 9 mod 16
constexpr int NR = 2;                               // ring rows
constexpr int RING_ROW_UNITS = GB * GS;             // 16-byte units per ring row
constexpr int OSTRIDE = GB * 16 + 16;               // bytes per pixel in the output stage
constexpr int OUT_ROW_BYTES = 16 * WT * OSTRIDE;
constexpr int IN_CELLS = F * GB;
constexpr int LPT = (IN_CELLS + THREADS - 1) / THREADS;  // source cells per thread per row
constexpr int OUT_CELLS = NB * DW * GB;
constexpr int SPT = (OUT_CELLS + THREADS - 1) / THREADS;  // stores per thread per row
constexpr int GBLKS = (kGroups + GB - 1) / GB;
constexpr int PBLKS = (DH + BP - 1) / BP;
constexpr int NBLKS = (kN + NB - 1) / NB;
constexpr int NUM_BLOCKS = GBLKS * PBLKS * NBLKS;
constexpr int STEPS = BP + kR - 1;

constexpr int gcd_(int a, int b) { return b == 0 ? a : gcd_(b, a % b); }
constexpr int UNROLL = NS / gcd_(NS, PF) * PF;  // lcm(NS, PF); even, so also a multiple of NR

static_assert(PF >= 2 && WAVES <= 16 && UNROLL % NR == 0, "bad configuration");
constexpr int STREAM_UNITS = NR * RING_ROW_UNITS + 2 * OUT_ROW_BYTES / 16;
constexpr int FILTER_UNITS = kIgrad ? GB * 8 * kR * kS : 0;  // staged filters (data gradient only)
constexpr int LDS_UNITS = STREAM_UNITS > FILTER_UNITS ? STREAM_UNITS : FILTER_UNITS;
static_assert(LDS_UNITS * 16 <= 160 * 1024, "LDS overflow");

constexpr int pmod(int a, int m) { return ((a % m) + m) % m; }

// Source rows shared with the neighbouring row blocks (the first and last R-1
// steps) can be served from L2 when the neighbour runs on the same XCD;
// SPIO_HALO_CACHED = 1 loads those with the default policy and only the
// interior rows with the non-temporal hint.
#ifndef SPIO_HALO_CACHED
#define SPIO_HALO_CACHED 0
#endif
SPIO_DEVICE spio_uint4 load_row(const spio_uint4* p, int step) {
    if (SPIO_HALO_CACHED && (step < kR - 1 || step >= BP)) return *p;
    return load_stream(p);
}

}  // namespace

extern "C" __global__ void SPIO_LAUNCH_BOUNDS(THREADS)
SPIO_KERNEL_NAME(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                 const spio_half* __restrict__ weights, const float* __restrict__ bias) {
    // One LDS block: the source-row ring, then the two output-stage rows.  The data-gradient
    // mode first uses the same block to stage the filters of the workgroup's groups.
    __shared__ spio_uint4 lds[LDS_UNITS];
    spio_uint4* const ring = lds;
    unsigned char* const ostage = reinterpret_cast<unsigned char*>(lds + NR * RING_ROW_UNITS);

    const int tid = thread_id();
    const int lane = tid & 63;
    // the wave index as a scalar: conditions on it become scalar branches, so that no MFMA
    // (which ignores the lane mask) is ever issued under an empty mask
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = wave % GB;  // group within the workgroup
    const int ws = wave / GB;  // tile split index

    // Workgroup -> (image block, channel block, row block), row block fastest.
    // Consecutive workgroup ids are dealt round-robin to the 8 XCDs; remap so
    // that each XCD works on a contiguous range of tiles (neighbouring row
    // blocks share halo rows through that XCD's L2).
    int b = block_id();
    if (NUM_BLOCKS % 8 == 0) b = (b & 7) * (NUM_BLOCKS / 8) + (b >> 3);
    const int pb = b % PBLKS;
    const int cb = (b / PBLKS) % GBLKS;
    const int nb = b / (PBLKS * GBLKS);
    const int p0 = pb * BP;
    const int n0 = nb * NB;
    const int gglob = cb * GB + wg;
    const bool wave_active = gglob < kGroups;

    // ---- loop-invariant addressing of the cooperative row load ----
    // Every thread issues the same number of loads on every step, without branches, so that the
    // compiler can count outstanding loads exactly and wait only for the row it needs (a load
    // under a branch makes it wait for all of them).  Cells that hold no source data (halo
    // columns, missing images or groups) load a valid dummy address and are zeroed when the row
    // is written to LDS.
    int in_off[LPT];   // 16-byte units from src; row term excluded
    bool in_ok[LPT];   // the cell carries source data
    int in_lds[LPT];   // 16-byte unit inside a ring row; -1 = no cell
    const int dummy_off = n0 * SH * SW * kGroups;  // first unit of the workgroup's first image
#pragma unroll
    for (int l = 0; l < LPT; ++l) {
        const int cell = tid + THREADS * l;
        in_off[l] = dummy_off;
        in_ok[l] = false;
        in_lds[l] = -1;
        if (cell < IN_CELLS) {
            const int g = cell % GB;
            const int f = cell / GB;
            const int img = f / WPI;
            const int col = f % WPI - EPX;
            in_lds[l] = g * GS + f;
            if (col >= 0 && col < SW && n0 + img < kN && cb * GB + g < kGroups) {
                in_off[l] = ((n0 + img) * SH * SW + col) * kGroups + cb * GB + g;
                in_ok[l] = true;
            }
        }
    }
    const long long row_units = (long long)SW * kGroups;  // 16-byte units per source row
    const long long dst_row_units = (long long)DW * kGroups;

    // ---- rows 0..PF-1 into registers, first of all: their latency covers the filter set-up ----
    spio_uint4 pre[PF][LPT];
#pragma unroll
    for (int t = 0; t < PF; ++t) {
        // rows outside the image are loaded from the nearest real row and never used
        const int h = imin(imax(p0 + t - EPY, 0), SH - 1);
#pragma unroll
        for (int l = 0; l < LPT; ++l) pre[t][l] = load_row(src + in_off[l] + h * row_units, t);
    }

    // ---- loop-invariant addressing of the cooperative row store ----
    int out_off[SPT];  // 16-byte units from dst; row term excluded; -1 = nothing to store
    int out_lds[SPT];  // byte offset inside an output-stage row
#pragma unroll
    for (int s = 0; s < SPT; ++s) {
        const int cell = tid + THREADS * s;
        out_off[s] = -1;
        out_lds[s] = 0;
        if (cell < OUT_CELLS) {
            const int g = cell % GB;
            const int q = (cell / GB) % DW;
            const int img = cell / (GB * DW);
            out_lds[s] = (img * WPI + q) * OSTRIDE + g * 16;
            if (n0 + img < kN && cb * GB + g < kGroups)
                out_off[s] = ((n0 + img) * DH * DW + q) * kGroups + cb * GB + g;
        }
    }

    // ---- filter fragments: wfrag[d][u], d = (phase - 2*acc) mod NS ----
    // Lane (m = lane%16, kb = lane/16): row slot j = m/8, channel m%8, column tap 4u+kb;
    // the filter row of slot j at distance d is r = (d - j) mod NS (none if r >= R).
    spio_half8 wfrag[NS][KB];
    if (!kIgrad) {
        // A[m = out channel ch][c] = w[8g+ch][r][s][c]: 16 contiguous bytes per lane.
        const int m = lane & 15;
        const int kb = lane >> 4;
        const int j = m >> 3;
        const int ch = m & 7;
#pragma unroll
        for (int d = 0; d < NS; ++d) {
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const int r = (d - j + NS) % NS;
                const int s = 4 * u + kb;
                Pack16 v;
                v.u = spio_uint4{0u, 0u, 0u, 0u};
                if (wave_active && r < kR && s < kS)
                    v.u = *reinterpret_cast<const spio_uint4*>(
                        weights + (((long long)(8 * gglob + ch) * kR + r) * kS + s) * 8);
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
        spio_uint4* wlds = lds;  // ring and output stage are not in use yet
        for (int i = tid; i < WUNITS; i += THREADS) {
            const int g = i / (8 * kR * kS);
            const int rem = i % (8 * kR * kS);
            spio_uint4 v = spio_uint4{0u, 0u, 0u, 0u};
            if (cb * GB + g < kGroups)
                v = reinterpret_cast<const spio_uint4*>(weights)[(long long)(cb * GB + g) * (8 * kR * kS) + rem];
            wlds[i] = v;
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
                const unsigned char* base = reinterpret_cast<const unsigned char*>(wlds) +
                                            ((((wg * 8 + jr) * kR + rr) * kS + ss) * 16) + (t4 & 1) * 8;
                union {
                    spio_short4 q[2];
                    spio_half8 h;
                } v;
                v.q[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)base);
                v.q[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(base + 4 * kR * kS * 16));
                if (!(wave_active && r_mine < kR && s < kS)) v.h = spio_half8{0, 0, 0, 0, 0, 0, 0, 0};
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

    // ---- zero the ring once: halo and slack cells are never written again ----
    for (int i = tid; i < NR * RING_ROW_UNITS; i += THREADS) ring[i] = spio_uint4{0u, 0u, 0u, 0u};


    // ---- row 0 into the ring ----
    block_sync();  // ring zeroed
    {
        const int h = p0 - EPY;
        if (h >= 0 && h < SH) {
#pragma unroll
            for (int l = 0; l < LPT; ++l)
                if (in_lds[l] >= 0) ring[in_lds[l]] = in_ok[l] ? pre[0][l] : spio_uint4{0u, 0u, 0u, 0u};
        }
    }
    block_sync();

    // Coalesced store of the output row staged at step `ts` (in stage buffer `obuf`): the row
    // that received its last tap at that step.  Called one step later, after the barrier.
    auto store_output_row = [&](int ts, int obuf) {
        const int p = p0 + ts - (kR - 1);
        if (ts >= kR - 1 && p < DH) {
#pragma unroll
            for (int s = 0; s < SPT; ++s) {
                if (out_off[s] >= 0) {
                    const spio_uint4 v =
                        *reinterpret_cast<const spio_uint4*>(ostage + obuf * OUT_ROW_BYTES + out_lds[s]);
                    store_stream(v, dst + out_off[s] + p * dst_row_units);
                }
            }
        }
    };

    for (int tb = 0; tb < STEPS; tb += UNROLL) {
#pragma unroll
        for (int uu = 0; uu < UNROLL; ++uu) {
            const int t = tb + uu;
            if (t >= STEPS) break;
            constexpr int kDummy = 0;
            (void)kDummy;
            const int ph = uu % NS;        // compile-time after unrolling
            const int rbuf = uu % NR;      // ring row holding source row t
            const int obuf = uu & 1;       // output stage buffer of this step
            const int pbuf = uu % PF;      // register buffer that held row t

            // 1. prefetch source row t+PF (its register buffer is free: row t is in LDS)
            {
                const int tt = t + PF;
                if (PF < STEPS) {  // compile-time: with PF >= STEPS the prologue loaded every row
                    // past the last row the loads repeat it (cache hits) and are never used
                    const int h = imin(imax(p0 + imin(tt, STEPS - 1) - EPY, 0), SH - 1);
#pragma unroll
                    for (int l = 0; l < LPT; ++l) pre[pbuf][l] = load_row(src + in_off[l] + h * row_units, tt);
                }
            }

            // 2. multiply source row t into the live output rows.  The fragment reads are issued
            //    first; the previous step's output row is stored while they are in flight.
            const int hcur = p0 + t - EPY;
            const bool row_live = wave_active && hcur >= 0 && hcur < SH;
            spio_half8 bfrag[TPW][KB];
            if (row_live) {
                const spio_uint4* rrow = ring + rbuf * RING_ROW_UNITS + wg * GS + (lane & 15) + (lane >> 4);
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    const int tile = ws + TS * i;
                    if (TS == 1 || tile < WT) {
#pragma unroll
                        for (int u = 0; u < KB; ++u) {
                            Pack16 v;
                            v.u = rrow[16 * tile + 4 * u];
                            bfrag[i][u] = v.h;
                        }
                    }
                }
            }
            store_output_row(t - 1, (uu + 1) & 1);
            if (row_live) {
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    const int tile = ws + TS * i;
                    if (TS == 1 || tile < WT) {
#pragma unroll
                        for (int a = 0; a < NACC; ++a) {
                            const int d = pmod(ph - 2 * a, NS);
#pragma unroll
                            for (int u = 0; u < KB; ++u)
                                acc[i][a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                    wfrag[d][u], bfrag[i][u], acc[i][a], 0, 0, 0);
                        }
                    }
                }
            }

            // 3. the row that received its last tap: stage it, reset its slot
            {
                const int slot = pmod(ph - (kR - 1), NS);
                const int a = slot >> 1;
                const int j = slot & 1;
                const bool emit = t >= kR - 1;
                if (wave_active && out_j == j) {
#pragma unroll
                    for (int i = 0; i < TPW; ++i) {
                        const int tile = ws + TS * i;
                        if (TS == 1 || tile < WT) {
                            if (emit) {
                                Pack8 o;
#pragma unroll
                                for (int e = 0; e < 4; ++e) o.h[e] = (spio_half)acc[i][a][e];
                                *reinterpret_cast<spio_uint2*>(ostage + obuf * OUT_ROW_BYTES +
                                                               (16 * tile + out_n) * OSTRIDE +
                                                               wg * 16 + out_kh * 8) = o.u;
                            }
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[i][a][e] = bias_reg[e];
                        }
                    }
                }
            }

            // 4. source row t+1 (loaded earlier) into the other ring row
            {
                const int hn = p0 + t + 1 - EPY;
                if (t + 1 < STEPS && hn >= 0 && hn < SH) {
#pragma unroll
                    for (int l = 0; l < LPT; ++l)
                        if (in_lds[l] >= 0)
                            ring[((uu + 1) % NR) * RING_ROW_UNITS + in_lds[l]] =
                                in_ok[l] ? pre[(uu + 1) % PF][l] : spio_uint4{0u, 0u, 0u, 0u};
                }
            }

            block_sync();

        }
    }
    store_output_row(STEPS - 1, (STEPS - 1) & 1);  // the last row
}
