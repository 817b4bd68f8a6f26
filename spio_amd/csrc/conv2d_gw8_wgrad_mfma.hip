// Row-streaming MFMA kernel for the conv2d_gw8 weight gradient (gfx950).
//
// Contract (reference kernel: spio/src/conv2d_gw8_wgrad.cu:10-226):
//   dw[k,r,s,c] += sum_{n,p,q} x[n,p+r-py,q+s-px,8g+c] * dy[n,p,q,k]      g = k / 8
// fp16 operands, fp32 accumulation, fp32 result added into `grad_weight`
// ([K][R][S][8] floats) with atomics, so the caller zeroes it first
// (spio/functional/conv2d_gw8_function.py:124-130).
//
// Design
//   * A workgroup owns SPIO_BH rows of dy (output rows) of SPIO_NB images side
//     by side, for SPIO_GB channel groups, and repeats that for SPIO_ITERS
//     image blocks before it publishes its sums.  Per step it stages SPIO_RB
//     (1 or 2) rows of x and of dy in LDS ([group][flattened pixel][8 ch],
//     zero halo materialised once, as in the forward kernel).
//   * One wave owns one group.  The contraction runs over pixels, so both MFMA
//     operands need "8 pixels of one channel" per lane while memory holds
//     "8 channels of one pixel"; the transposing LDS read of gfx950
//     (ds_read_b64_tr_b16) delivers exactly that from the pixel-major rows.
//   * v_mfma_f32_16x16x32_f16 per 32-pixel chunk:
//         A (16 x 32) = dy:  rows m = 8*j + k    (two dy rows j of an aligned row pair, 8 k)
//         B (32 x 16) = x:   cols n = 8*sj + c   (two column taps sj, 8 c)
//     so one MFMA yields dw for 2 filter rows x 2 filter columns.  For x row t
//     and the dy row pair (2i, 2i+1) the filter rows are r = delta - j with
//     delta = t - 2i in [0, R]; there is one accumulator per (delta, column-tap
//     pair).  Entries with r or s out of range are never read.
//   * At the end dw[k,r,s,c] = acc[delta=r] (lanes with j=0) + acc[delta=r+1]
//     (lanes with j=1); the halves are combined through LDS.  Two ways to
//     publish: SPIO_PARTIALS=0 adds into grad_weight with fp32 atomics.  Atomics
//     of different workgroups to the same 128-byte line retire one after the
//     other, so the sums are first staged in LDS in grad_weight order and then
//     added with instructions that cover 64 consecutive floats (two full
//     lines): the fewest line operations possible.  SPIO_PARTIALS=1 stores each
//     workgroup's sums into its own partial image of a workspace with plain
//     stores, and the small <name>_reduce kernel below stores the sum of the
//     partial images into grad_weight (which then needs no zero fill).  (Reducing inside the kernel by "the last workgroup of
//     a group to finish" was measured and rejected: the device-scope
//     release/acquire fences it needs write back and invalidate the L2 of an
//     XCD and cost more than the atomics they save.)
//   * With SPIO_HAS_BIAS the kernel takes a fourth pointer, grad_bias ([K]
//     fp32, accumulated into like grad_weight; null = not wanted), and sums dy
//     per channel in the same pass: one more MFMA per chunk and row pair with
//     an all-ones B operand (the reference runs a separate reduction,
//     spio/functional/conv2d_gw8_function.py:134-136).
#include "spio_conv_common.h"

using namespace spio;

#ifndef SPIO_NB
#define SPIO_NB 1
#endif
#ifndef SPIO_ITERS
#define SPIO_ITERS 1
#endif
#ifndef SPIO_PF
#define SPIO_PF 2
#endif
#ifndef SPIO_PARTIALS
#define SPIO_PARTIALS 0
#endif
#ifndef SPIO_BQ
#define SPIO_BQ 0
#endif
#ifndef SPIO_TS
#define SPIO_TS 1
#endif
#ifndef SPIO_RB
#define SPIO_RB 1
#endif
#ifndef SPIO_HAS_BIAS
#define SPIO_HAS_BIAS 0
#endif
#ifndef SPIO_PIPE
#define SPIO_PIPE 0
#endif

namespace {

constexpr int GB = SPIO_GB;        // groups (waves) per workgroup
constexpr int BH = SPIO_BH;        // dy rows per workgroup
constexpr int NB = SPIO_NB;        // images side by side
constexpr int ITERS = SPIO_ITERS;  // image blocks per workgroup
constexpr int TS = SPIO_TS;        // waves sharing the 32-pixel chunks of one group
constexpr int WAVES = GB * TS;
constexpr int THREADS = 64 * WAVES;
constexpr int PF = SPIO_PF;  // prefetch distance in steps (even)
constexpr int RB = SPIO_RB;  // x rows (and dy rows) per step: 1 or 2

constexpr int S2 = 2 * ((kS + 1) / 2);
constexpr int NBLK = S2 / 2;   // column-tap pairs
constexpr int ND = kR + 1;     // values of delta
// Column blocks (SPIO_BQ > 0): a workgroup sums over BQ columns of dy and the BQ + S - 1 columns
// of x opposite them, so rows of any width fit the rings (the reference tiles the width with a
// fixed block of 8 columns, spio/kernels/conv2d_gw8_wgrad_kernel.py:40).  0 = the whole width.
constexpr int BQ = SPIO_BQ > 0 ? SPIO_BQ : kQ;
constexpr int QBLKS = (kQ + BQ - 1) / BQ;
constexpr int WPI = BQ + kS - 1;  // x cells staged per image (block): W + 2*px for whole rows
constexpr int F = NB * WPI;
// Where the images of a staged row sit.  dy pixel q of image i lies at flattened pixel
// off(i) + q and meets, for column tap s, the x pixel at off(i) + q + s; x column c of image i
// lies at off(i) + c + px.  Between the data of two images GAP = max(px, S-1-px) zero cells are
// enough: the right halo of one image is the left halo of the next.  The contraction runs over
// 32-pixel chunks of the dy row; where a chunk holds IPC >= 1 whole images and that takes fewer
// chunks than the images laid end to end, every chunk gets its own IPC images (14x14 images
// under a 7x7 filter: two per chunk, 28 of 32 pixels, instead of four in three chunks), and the
// x row, whose pixels q + s reach S-1 cells past a chunk, is staged as chunks XCP cells apart.
#ifndef SPIO_SHARED_HALO
#define SPIO_SHARED_HALO 1
#endif
constexpr int GAP = kPadX > kS - 1 - kPadX ? kPadX : kS - 1 - kPadX;
constexpr int IP = (SPIO_BQ > 0 || !SPIO_SHARED_HALO) ? WPI : BQ + GAP;  // pitch of the images in a run
constexpr int IPC_MAX = (32 + IP - BQ) / IP;                             // whole images per 32-pixel chunk
constexpr int KC_FLAT = ((NB - 1) * IP + BQ + 31) / 32;
constexpr int KC_PACKED = IPC_MAX > 0 ? (NB + IPC_MAX - 1) / IPC_MAX : KC_FLAT;
constexpr bool kPacked = SPIO_SHARED_HALO && KC_PACKED < KC_FLAT;
constexpr int IPC = kPacked ? IPC_MAX : NB;  // images per run: a chunk, or the whole row
constexpr int KC = kPacked ? KC_PACKED : KC_FLAT;  // 32-pixel chunks
constexpr int XCP = kPacked ? 16 * ((32 + S2 - 1 + 15) / 16) : 32;  // x cells from chunk to chunk
constexpr int FPX = kPacked ? KC * XCP : 32 * KC + S2 - 1;         // x pixels the reads can touch
constexpr int GSX = FPX + ((9 - FPX % 16) + 16) % 16;  // x group stride (pixels), = 9 mod 16
constexpr int FPD = 32 * KC;
constexpr int GSD = FPD + ((9 - FPD % 16) + 16) % 16;  // dy group stride
constexpr int d_image_offset(int img) { return (img / IPC) * 32 + (img % IPC) * IP; }
constexpr int x_image_offset(int img) { return (img / IPC) * XCP + (img % IPC) * IP; }
constexpr int NRX = 2 * RB;                             // x ring rows: the step's rows and the next step's
// dy ring rows: the aligned row pairs a step multiplies (R+1 rows with one row per step, up to
// R+2 with two) plus the rows the step writes for the next one; even.  The bias sum reads the
// whole pair (t-1, t) in the step that stages row t+1, so it needs four rows even with a one-row
// filter, whose weight gradient alone gets by with two.
constexpr int NRD = ((SPIO_HAS_BIAS && kR == 1) ? 4 : 2 * ((kR + 2) / 2)) + (RB == 2 ? 2 : 0);
constexpr int XROW_UNITS = GB * GSX;
// dy ring rows are 64 bytes apart modulo the 256-byte bank period, so the two rows of a
// pair that one transposing read touches fall into different banks.
constexpr int DROW_UNITS = GB * GSD + ((4 - (GB * GSD) % 16) + 16) % 16;
constexpr int X_CELLS = F * GB;
constexpr int LPTX = (X_CELLS + THREADS - 1) / THREADS;
constexpr int D_CELLS = NB * BQ * GB;
constexpr int LPTD = (D_CELLS + THREADS - 1) / THREADS;
constexpr int GBLKS = (kGroups + GB - 1) / GB;
constexpr int PBLKS = (kP + BH - 1) / BH;
constexpr int NBLKS = (kN + NB * ITERS - 1) / (NB * ITERS);
constexpr int NUM_BLOCKS = GBLKS * PBLKS * QBLKS * NBLKS;
constexpr bool kDbias = SPIO_HAS_BIAS != 0;  // also sum grad_output per channel (grad_bias)
// x rows a workgroup streams.  The bias sum takes a grad_output row pair one step after its
// first row was staged, so a one-row filter needs one more step when the sum is wanted.
constexpr int ROWS = BH + (kDbias && kR == 1 ? 2 : kR) - 1;
constexpr int STEPS = (ROWS + RB - 1) / RB;  // barrier-separated steps of RB rows
// A workgroup that owns whole images (one row block) knows at compile time which of its x rows
// lie in the padding: the steps before the first real row would only stage dy rows, the steps
// after the last one nothing at all.  It starts at the first step with a real x row, with the dy
// rows up to that step staged in the prologue, and stops after the last.  (Not with the bias
// sum, which takes its row pairs at fixed steps.)
constexpr bool kSkipPadding = PBLKS == 1 && !kDbias;
constexpr int T_FIRST = kSkipPadding ? kPadY : 0;
constexpr int T_END = kSkipPadding && kH + kPadY < ROWS ? kH + kPadY : ROWS;
constexpr int S0 = T_FIRST / RB;               // first step
constexpr int S1 = (T_END + RB - 1) / RB;      // one past the last step
constexpr int LEAD = S0 * RB;                  // dy rows staged ahead of the first step's own
// A workgroup that owns whole images unrolls its step loop completely, up to SPIO_MAX_UNROLL
// steps (every condition on the step is then known at compile time); other loops run in chunks
// of PF steps.
#ifndef SPIO_MAX_UNROLL
#define SPIO_MAX_UNROLL 64
#endif
constexpr bool kFullUnroll = PBLKS == 1 && S1 - S0 <= SPIO_MAX_UNROLL;
constexpr int UNROLL = kFullUnroll ? (S1 - S0 + PF - 1) / PF * PF : PF;
constexpr int NPAIR = kR / 2 + 1;            // aligned dy row pairs one step can touch
constexpr int CPW = (KC + TS - 1) / TS;      // 32-pixel chunks per wave

// LDS: the two rings while streaming; at the end the same block holds the reduction scratch:
// per wave NBLK*128 floats for the row-slot halves, the sums of the other waves of a split
// group, (atomic publishing) every group's R*S*64 sums in grad_weight order, and eight
// grad_bias sums per wave.
constexpr int RING_UNITS = NRX * XROW_UNITS + NRD * DROW_UNITS;
// Filter rows whose row-slot halves are exchanged through the per-wave scratch in one go: all of
// them where that fits 96 KB of LDS for the workgroup (every exchange costs an LDS round trip
// and the waves do nothing else meanwhile), else one; one when waves share a group, whose sums
// are then added row by row.
constexpr int RCH = (TS == 1 && WAVES * kR * NBLK * 512 <= 96 * 1024) ? kR : 1;
constexpr int SCRATCH_FLOATS = RCH * NBLK * 128;  // per wave
constexpr int RED_FLOATS = GB * (TS - 1) * NBLK * 128;
constexpr int GROUP_FLOATS = kR * kS * 64;  // grad_weight values of one group
constexpr int PUBLISH_FLOATS = WAVES * SCRATCH_FLOATS + RED_FLOATS + (SPIO_PARTIALS ? 0 : GB * GROUP_FLOATS) +
                               (SPIO_HAS_BIAS ? WAVES * 8 : 0);
constexpr int LDS_UNITS = RING_UNITS > (PUBLISH_FLOATS + 3) / 4 ? RING_UNITS : (PUBLISH_FLOATS + 3) / 4;
static_assert(LDS_UNITS * 16 <= 160 * 1024, "LDS overflow");
static_assert(NRD % 2 == 0 && NRD >= kR + 1, "dy ring too small");
static_assert(PF >= 2 && PF % 2 == 0, "prefetch distance must be even");
static_assert(RB == 1 || RB == 2, "one or two rows per step");
static_assert(LEAD + RB <= NRD, "the dy rows of the prologue fit the ring");
constexpr int PART_WAVE_FLOATS = kR * NBLK * 4 * 32;  // floats one wave publishes (partial-block layout)


SPIO_DEVICE spio_half8 read_tr_pair(const unsigned char* lo, const unsigned char* hi) {
    typedef spio_short4 __attribute__((address_space(3))) * lds_ptr;
    union {
        spio_short4 s[2];
        spio_half8 h;
    } v;
    v.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)lo);
    v.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)hi);
    return v.h;
}

}  // namespace

extern "C" __global__ void SPIO_LAUNCH_BOUNDS(THREADS)
SPIO_KERNEL_NAME(float* __restrict__ grad_weight, const spio_uint4* __restrict__ x,
                 const spio_uint4* __restrict__ dy
#if SPIO_HAS_BIAS
                 , float* __restrict__ grad_bias  // [K] fp32, accumulated into; null = not wanted
#endif
) {
    // One LDS block: the x ring, then the dy ring; reused as reduction scratch at the end.
    __shared__ spio_uint4 lds[LDS_UNITS];
    spio_uint4* const xring = lds;
    spio_uint4* const dring = lds + NRX * XROW_UNITS;

    const int tid = thread_id();
    const int lane = tid & 63;
    // the wave index as a scalar: conditions on it become scalar branches, so that no MFMA
    // (which ignores the lane mask) is ever issued under an empty mask
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = wave % GB;  // group within the workgroup
    const int ws = wave / GB;  // which share of the 32-pixel chunks this wave multiplies

    int b = block_id();
    if (NUM_BLOCKS % 8 == 0) b = (b & 7) * (NUM_BLOCKS / 8) + (b >> 3);
    const int qb = b % QBLKS;  // column blocks fastest: neighbours share S - 1 columns of x
    const int q0 = qb * BQ;
    const int pb = PBLKS == 1 ? 0 : (b / QBLKS) % PBLKS;
    const int cb = (b / (QBLKS * PBLKS)) % GBLKS;
    const int nbk = b / (QBLKS * PBLKS * GBLKS);
    const int p0 = pb * BH;
    const int bh_eff = imin(BH, kP - p0);  // dy rows that exist in this block
    const int gglob = cb * GB + wg;
    const bool wave_active = gglob < kGroups;

    // lane roles inside the transposing reads: block kb = lane/16 covers pixels 8*kb..8*kb+7,
    // source lane sigma = lane%16 = 4*jr + t supplies pixel jr (+4 for the second read) of
    // unit t/2 (dy row j or column tap sj) and channel half t%2.
    const int kb = lane >> 4;
    const int jr = (lane & 15) >> 2;
    const int tt = lane & 3;
    const int sel = tt >> 1;  // j for A, sj for B
    const int xfrag_off = ((wg * GSX + 8 * kb + jr + sel) * 16) + (tt & 1) * 8;   // bytes in an x row
    const int dfrag_off = ((wg * GSD + 8 * kb + jr) * 16) + (tt & 1) * 8;         // bytes in a dy row

    spio_float4 acc[ND][NBLK];
#pragma unroll
    for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) acc[d][nb] = spio_float4{0.f, 0.f, 0.f, 0.f};

    // grad_bias rides along as one more MFMA per chunk and row pair: dy (A) times an all-ones B
    // gives, in every column, the sum of the 32 pixels for the 16 (row slot, channel) rows.
    spio_float4 accb = spio_float4{0.f, 0.f, 0.f, 0.f};
    const spio_half8 ones8 = spio_half8{1, 1, 1, 1, 1, 1, 1, 1};
    (void)ones8;
    const long long xrow_units = (long long)kW * kGroups;
    const long long drow_units = (long long)kQ * kGroups;

    for (int it = 0; it < ITERS; ++it) {
        const int n0 = (nbk * ITERS + it) * NB;
        if (n0 >= kN) break;

        // ---- loop-invariant addressing for this image block ----
        // Every thread issues the same loads on every step, without branches, so that the
        // compiler counts outstanding loads exactly and a step waits only for the rows it
        // needs (a load under a branch makes it wait for all of them, which would serialise the
        // prefetch).  Cells without data (halo columns, missing images or groups) and rows
        // outside the tensor load a valid address and become zero when written to LDS.  (Threads
        // beyond the last cell skip their LDS writes; letting them write spare cells instead, to
        // make the writes branch-free, costs 14 % at N=256, C=256, 14x14, 7x7.)
        int x_off[LPTX], x_lds[LPTX];
        bool x_ok[LPTX];
        const int x_dummy = n0 * kH * kW * kGroups;
#pragma unroll
        for (int l = 0; l < LPTX; ++l) {
            const int cell = tid + THREADS * l;
            x_off[l] = x_dummy;
            x_ok[l] = false;
            x_lds[l] = -1;
            if (cell < X_CELLS) {
                const int g = cell % GB;
                const int f = cell / GB;
                const int img = f / WPI;
                const int col = q0 + f % WPI - kPadX;
                x_lds[l] = g * GSX + x_image_offset(img) + f % WPI;
                if (col >= 0 && col < kW && n0 + img < kN && cb * GB + g < kGroups) {
                    x_off[l] = ((n0 + img) * kH * kW + col) * kGroups + cb * GB + g;
                    x_ok[l] = true;
                }
            }
        }
        int d_off[LPTD], d_lds[LPTD];
        bool d_ok[LPTD];
        const int d_dummy = n0 * kP * kQ * kGroups;
#pragma unroll
        for (int l = 0; l < LPTD; ++l) {
            const int cell = tid + THREADS * l;
            d_off[l] = d_dummy;
            d_ok[l] = false;
            d_lds[l] = -1;
            if (cell < D_CELLS) {
                const int g = cell % GB;
                const int q = (cell / GB) % BQ;
                const int img = cell / (GB * BQ);
                d_lds[l] = g * GSD + d_image_offset(img) + q;
                if (q0 + q < kQ && n0 + img < kN && cb * GB + g < kGroups) {
                    d_off[l] = ((n0 + img) * kP * kQ + q0 + q) * kGroups + cb * GB + g;
                    d_ok[l] = true;
                }
            }
        }
        const spio_uint4 zero4 = spio_uint4{0u, 0u, 0u, 0u};

        // ---- prologue: steps S0..S0+PF-1 into registers, step S0 (and the dy rows before it)
        //      into LDS ----
        spio_uint4 xpre[PF][RB][LPTX], dpre[PF][RB][LPTD];
        spio_uint4 dlead[LEAD > 0 ? LEAD : 1][LPTD];
#pragma unroll
        for (int i = 0; i < LEAD; ++i) {
            const int pr = imin(p0 + i, kP - 1);
#pragma unroll
            for (int l = 0; l < LPTD; ++l) dlead[i][l] = load_stream(dy + d_off[l] + pr * drow_units);
        }
#pragma unroll
        for (int sp = 0; sp < PF; ++sp) {
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                const int t = (S0 + sp) * RB + rr;
                const int h = imin(imax(p0 + t - kPadY, 0), kH - 1);
#pragma unroll
                for (int l = 0; l < LPTX; ++l) xpre[sp][rr][l] = load_stream(x + x_off[l] + h * xrow_units);
                const int pr = imin(p0 + t, kP - 1);
#pragma unroll
                for (int l = 0; l < LPTD; ++l) dpre[sp][rr][l] = load_stream(dy + d_off[l] + pr * drow_units);
            }
        }
        if (it == 0) {
            // zero both rings once, while the first loads are in flight: halo, gap and slack
            // cells are never written again
            for (int i = tid; i < NRX * XROW_UNITS; i += THREADS) xring[i] = zero4;
            for (int i = tid; i < NRD * DROW_UNITS; i += THREADS) dring[i] = zero4;
        }
        block_sync();  // rings zeroed / previous image block finished
#pragma unroll
        for (int i = 0; i < LEAD; ++i) {
            const bool drow_ok = i < bh_eff;
#pragma unroll
            for (int l = 0; l < LPTD; ++l)
                if (d_lds[l] >= 0) dring[(i % NRD) * DROW_UNITS + d_lds[l]] = (drow_ok && d_ok[l]) ? dlead[i][l] : zero4;
        }
#pragma unroll
        for (int rr = 0; rr < RB; ++rr) {
            const int t = S0 * RB + rr;
            const int h = p0 + t - kPadY;
            const bool xrow_ok = h >= 0 && h < kH;
#pragma unroll
            for (int l = 0; l < LPTX; ++l)
                if (x_lds[l] >= 0) xring[((S0 & 1) * RB + rr) * XROW_UNITS + x_lds[l]] = (xrow_ok && x_ok[l]) ? xpre[0][rr][l] : zero4;
            const bool drow_ok = t < bh_eff;
#pragma unroll
            for (int l = 0; l < LPTD; ++l)
                if (d_lds[l] >= 0) dring[(t % NRD) * DROW_UNITS + d_lds[l]] = (drow_ok && d_ok[l]) ? dpre[0][rr][l] : zero4;
        }
        block_sync();

        // What step `st` (of parity `sp`) multiplies: x rows t+rr against the aligned dy row pairs
        // they overlap (x row t+rr and the pair starting at row i2 meet at delta = t + rr - i2).
        // The row pair starting at tbase is complete in LDS (its second row was staged during
        // the previous step) when two rows go per step, and on odd steps otherwise; that is
        // when it is added to the bias sum, once per pair.
        struct StepPlan {
            int tbase;
            bool row_live[RB];
            bool bias_pair;
            bool do_math;
        };
        auto plan_step = [&](int st, int sp) {
            StepPlan pl;
            const int t = st * RB;  // first x row of the step, relative to the block
            pl.tbase = RB == 2 ? t : t - sp;  // even
            bool any_live = false;
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                const int hcur = p0 + t + rr - kPadY;
                pl.row_live[rr] = t + rr < ROWS && hcur >= 0 && hcur < kH;
                any_live = any_live || pl.row_live[rr];
            }
            pl.bias_pair = kDbias && (RB == 2 || sp == 1) && pl.tbase < bh_eff;
            pl.do_math = wave_active && (any_live || pl.bias_pair);
            return pl;
        };
        // A step's work comes in CPW * NPAIR groups: group (ci, m) is the products of chunk ci with
        // dy row pair m, and the share m of the chunk's fragment reads (the chunk's RB * NBLK x
        // fragments and NPAIR dy fragments dealt round-robin over its groups).
        constexpr int ITEMS = RB * NBLK + NPAIR;  // fragment reads (pairs of LDS reads) per chunk
        auto read_group = [&](const StepPlan& pl, int sp, int ci, int mslot, spio_half8(&bf)[CPW][RB][NBLK],
                              spio_half8(&af)[CPW][NPAIR]) {
            const int ch = ws + TS * ci;
            if (TS > 1 && ch >= KC) return;
#pragma unroll
            for (int j = mslot; j < ITEMS; j += NPAIR) {
                if (j < RB * NBLK) {
                    const int rr = j / NBLK, nb = j % NBLK;
                    const unsigned char* xrow =
                        reinterpret_cast<const unsigned char*>(xring + (sp * RB + rr) * XROW_UNITS) + xfrag_off;
                    const unsigned char* pb0 = xrow + (XCP * ch + 2 * nb) * 16;
                    bf[ci][rr][nb] = read_tr_pair(pb0, pb0 + 4 * 16);
                } else {
                    const int m = j - RB * NBLK;
                    const int i2 = pl.tbase - 2 * m;  // first row of the pair, relative to p0
                    if (i2 >= 0 && i2 < bh_eff) {
                        const int slot = (i2 + sel) % NRD;
                        const unsigned char* pa0 =
                            reinterpret_cast<const unsigned char*>(dring + slot * DROW_UNITS) + dfrag_off + (32 * ch) * 16;
                        af[ci][m] = read_tr_pair(pa0, pa0 + 4 * 16);
                    }
                }
            }
        };
        auto multiply_group = [&](const StepPlan& pl, int sp, int ci, int m, const spio_half8(&bf)[CPW][RB][NBLK],
                                  const spio_half8(&af)[CPW][NPAIR]) {
            const int ch = ws + TS * ci;
            if (TS > 1 && ch >= KC) return;
            const int i2 = pl.tbase - 2 * m;
            if (i2 >= 0 && i2 < bh_eff) {
#pragma unroll
                for (int rr = 0; rr < RB; ++rr) {
                    const int d = (RB == 2 ? rr : sp) + 2 * m;  // = t + rr - i2
                    if (d <= kR && pl.row_live[rr]) {
#pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb)
                            acc[d][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[ci][m], bf[ci][rr][nb], acc[d][nb],
                                                                                0, 0, 0);
                    }
                }
                if (m == 0 && pl.bias_pair) accb = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[ci][0], ones8, accb, 0, 0, 0);
            }
        };
        // 2. prefetch step st+PF (its register buffer held step st, now in LDS); rows past the end
        //    repeat a real row and are never used
        auto prefetch_rows = [&](int st, int uf) {
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                const int t2 = (st + PF) * RB + rr;
                const int h = imin(imax(p0 + t2 - kPadY, 0), kH - 1);
#pragma unroll
                for (int l = 0; l < LPTX; ++l) xpre[uf % PF][rr][l] = load_stream(x + x_off[l] + h * xrow_units);
                const int pr = imin(p0 + t2, kP - 1);
#pragma unroll
                for (int l = 0; l < LPTD; ++l) dpre[uf % PF][rr][l] = load_stream(dy + d_off[l] + pr * drow_units);
            }
        };
        // 3. the rows of step st+1 into LDS (dy rows past the block's last row become zero).  The
        //    ring rows written here are not read in this step, except for dy entries whose filter
        //    row is out of range and whose product is ignored.
        auto stage_x = [&](int st, int sp, int uf) {
            if (st + 1 >= S1) return;
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                const int tn = (st + 1) * RB + rr;
                const int hn = p0 + tn - kPadY;
                if (tn < ROWS && hn >= 0 && hn < kH) {
#pragma unroll
                    for (int l = 0; l < LPTX; ++l)
                        if (x_lds[l] >= 0)
                            xring[(((sp + 1) & 1) * RB + rr) * XROW_UNITS + x_lds[l]] =
                                x_ok[l] ? xpre[(uf + 1) % PF][rr][l] : zero4;
                }
            }
        };
        auto stage_dy = [&](int st, int uf) {
            if (st + 1 >= S1) return;
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                const int tn = (st + 1) * RB + rr;
                const int dslot = tn % NRD;
                const bool drow_ok = tn < bh_eff;
#pragma unroll
                for (int l = 0; l < LPTD; ++l)
                    if (d_lds[l] >= 0)
                        dring[dslot * DROW_UNITS + d_lds[l]] = (drow_ok && d_ok[l]) ? dpre[(uf + 1) % PF][rr][l] : zero4;
            }
        };

        // With SPIO_PIPE the products of a step are issued one step later, from a second set of
        // fragment registers, and the step's own LDS reads, row loads and ring writes are dealt
        // out between the groups of MFMAs: the matrix pipe takes 16 cycles per MFMA and the wave
        // issues the other instructions in the slots that leaves.  (The compiler does not move
        // the ring writes, which sit under lane masks, across the MFMAs by itself.)
        constexpr int FSETS = SPIO_PIPE ? 2 : 1;
        constexpr int GROUPS = CPW * NPAIR;
        spio_half8 bfrag[FSETS][CPW][RB][NBLK], afrag[FSETS][CPW][NPAIR];
        for (int sb = S0; sb < S1; sb += UNROLL) {
#pragma unroll
            for (int uf = 0; uf < UNROLL; ++uf) {
                const int st = sb + uf;
                if (st >= S1) break;
                // PF is even, so the parity of the step is known at compile time: it fixes the
                // x ring rows and, with one row per step, the parity of delta.
                const int sp = (S0 + uf) & 1;
                const StepPlan pl = plan_step(st, sp);
                if (SPIO_PIPE) {
                    const int fs = uf & 1;
                    const StepPlan before = plan_step(st - 1, sp ^ 1);
#pragma unroll
                    for (int g = 0; g < GROUPS; ++g) {
                        const int ci = g / NPAIR, m = g % NPAIR;
                        if (pl.do_math) read_group(pl, sp, ci, m, bfrag[fs], afrag[fs]);
                        if (g == 0) prefetch_rows(st, uf);
                        if (g == (GROUPS > 1 ? 1 : 0)) stage_x(st, sp, uf);
                        if (g == (GROUPS > 2 ? 2 : GROUPS - 1)) stage_dy(st, uf);
                        if (st > S0 && before.do_math) multiply_group(before, sp ^ 1, ci, m, bfrag[fs ^ 1], afrag[fs ^ 1]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    // all LDS reads first, so that their latency overlaps the loads and ring writes
                    if (pl.do_math) {
#pragma unroll
                        for (int g = 0; g < GROUPS; ++g) read_group(pl, sp, g / NPAIR, g % NPAIR, bfrag[0], afrag[0]);
                    }
                    prefetch_rows(st, uf);
                    stage_x(st, sp, uf);
                    stage_dy(st, uf);
                    if (pl.do_math) {
#pragma unroll
                        for (int g = 0; g < GROUPS; ++g) multiply_group(pl, sp, g / NPAIR, g % NPAIR, bfrag[0], afrag[0]);
                    }
                }
                block_sync();
            }
        }
        if (SPIO_PIPE) {
            constexpr int LAST = S1 - 1;
            const StepPlan pl = plan_step(LAST, LAST & 1);
            if (pl.do_math) {
#pragma unroll
                for (int g = 0; g < GROUPS; ++g)
                    multiply_group(pl, LAST & 1, g / NPAIR, g % NPAIR, bfrag[(LAST - S0) & 1], afrag[(LAST - S0) & 1]);
            }
        }
    }

    // ---- publish ----
    // dw[k,r,s,c] = acc[delta = r] (lanes 0-31: j = 0) + acc[delta = r+1] (lanes 32-63: j = 1).
    // The j = 1 halves travel through a 512-byte per-wave LDS scratch (LDS operations of one
    // wave execute in order, so no barrier is needed inside the wave).  With TS > 1 the waves of
    // one group then add their sums through LDS so that only one wave per group publishes:
    // fp32 atomics into grad_weight, or plain stores into this workgroup's partial image when a
    // second kernel does the reduction.
    block_sync();  // every wave is done with the rings; reuse them as scratch
    {
        float* scratch = reinterpret_cast<float*>(lds) + wave * SCRATCH_FLOATS;
        float* red = reinterpret_cast<float*>(lds) + WAVES * SCRATCH_FLOATS;  // [group][ts-1][nb][e][32 lanes]
        // this group's sums in grad_weight order [k][r][s][c] (atomic publishing only)
        float* gstage = reinterpret_cast<float*>(lds) + WAVES * SCRATCH_FLOATS + RED_FLOATS + wg * GROUP_FLOATS;
        (void)gstage;
        const int k4 = 4 * ((lane >> 4) & 1);
        const int sj = (lane & 15) >> 3;
        const int c = lane & 7;
#if SPIO_PARTIALS
        // this wave's slice of the workgroup's partial block: [r][tap pair][e][32 lanes], so that
        // every store instruction writes 128 contiguous bytes
        float* out = grad_weight + (((long long)((nbk * PBLKS + pb) * QBLKS + qb) * GBLKS + cb) * GB + wg) * PART_WAVE_FLOATS;
#else
        float* out = grad_weight;
#endif
        if (RCH > 1) {
            // All filter rows at once: lanes 32-63 leave their halves in the scratch as float4s,
            // one wave-level sync, lanes 0-31 add them.  LDS operations of a wave execute in order,
            // so the scratch can be rewritten right after it has been read.
            spio_float4* half4 = reinterpret_cast<spio_float4*>(scratch);
            if (lane >= 32) {
#pragma unroll
                for (int r = 0; r < kR; ++r)
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb) half4[(r * NBLK + nb) * 32 + (lane - 32)] = acc[r + 1][nb];
            }
            wave_sync();  // lanes 32-63 stored, lanes 0-31 load
            spio_float4 total[kR][NBLK];
#pragma unroll
            for (int r = 0; r < kR; ++r)
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    total[r][nb] = spio_float4{0.f, 0.f, 0.f, 0.f};
                    if (lane < 32) total[r][nb] = acc[r][nb] + half4[(r * NBLK + nb) * 32 + lane];
                }
            wave_sync();  // the halves are read; the scratch becomes the staging area
#if SPIO_PARTIALS
            // through the scratch once more, in the partial block's order [r][tap pair][e][32
            // lanes], so that all 64 lanes store 16 contiguous bytes each
            if (wave_active) {
                if (lane < 32) {
#pragma unroll
                    for (int r = 0; r < kR; ++r)
#pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb)
#pragma unroll
                            for (int e = 0; e < 4; ++e) scratch[((r * NBLK + nb) * 4 + e) * 32 + lane] = total[r][nb][e];
                }
                wave_sync();  // lanes 0-31 staged, all lanes load
                const spio_float4* stage4 = reinterpret_cast<const spio_float4*>(scratch);
                spio_float4* out4 = reinterpret_cast<spio_float4*>(out);
#pragma unroll
                for (int i = lane; i < kR * NBLK * 32; i += 64) __builtin_nontemporal_store(stage4[i], out4 + i);
            }
#else
            if (wave_active && lane < 32) {
#pragma unroll
                for (int r = 0; r < kR; ++r)
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb) {
                        const int s = 2 * nb + sj;
                        if (s < kS) {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                gstage[(((k4 + e) * kR + r) * kS + s) * 8 + c] = total[r][nb][e];
                        }
                    }
            }
#endif
        } else {
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                float total[NBLK][4];
    #pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    if (lane >= 32) {
    #pragma unroll
                        for (int e = 0; e < 4; ++e) scratch[e * 32 + (lane - 32)] = acc[r + 1][nb][e];
                    }
                    wave_sync();  // lanes 32-63 stored, lanes 0-31 load
    #pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        total[nb][e] = 0.f;
                        if (lane < 32) total[nb][e] = acc[r][nb][e] + scratch[e * 32 + lane];
                    }
                    wave_sync();  // the scratch is free for the next tap pair
                }
                if (TS > 1) {
                    if (ws > 0 && lane < 32) {
    #pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb)
    #pragma unroll
                            for (int e = 0; e < 4; ++e)
                                red[(((wg * (TS - 1) + ws - 1) * NBLK + nb) * 4 + e) * 32 + lane] = total[nb][e];
                    }
                    block_sync();
                    if (ws == 0 && lane < 32) {
    #pragma unroll
                        for (int w2 = 0; w2 < TS - 1; ++w2)
    #pragma unroll
                            for (int nb = 0; nb < NBLK; ++nb)
    #pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    total[nb][e] += red[(((wg * (TS - 1) + w2) * NBLK + nb) * 4 + e) * 32 + lane];
                    }
                }
    #if SPIO_PARTIALS
                // through the wave's LDS scratch once more so that all 64 lanes store 16 bytes each
                if (wave_active && ws == 0) {
                    float* stage = scratch;  // NBLK * 128 floats: [tap pair][e][32 lanes]
                    if (lane < 32) {
    #pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb)
    #pragma unroll
                            for (int e = 0; e < 4; ++e) stage[(nb * 4 + e) * 32 + lane] = total[nb][e];
                    }
                    wave_sync();  // lanes 0-31 staged, all lanes load
                    const spio_float4* stage4 = reinterpret_cast<const spio_float4*>(stage);
                    spio_float4* out4 = reinterpret_cast<spio_float4*>(out) + r * NBLK * 32;
    #pragma unroll
                    for (int i = lane; i < NBLK * 32; i += 64) __builtin_nontemporal_store(stage4[i], out4 + i);
                    wave_sync();  // the scratch is free for the next filter row
                }
    #else
                if (wave_active && ws == 0 && lane < 32) {
    #pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb) {
                        const int s = 2 * nb + sj;
                        if (s < kS) {
    #pragma unroll
                            for (int e = 0; e < 4; ++e)
                                gstage[(((k4 + e) * kR + r) * kS + s) * 8 + c] = total[nb][e];
                        }
                    }
                }
    #endif
                if (TS > 1) block_sync();  // the scratch is rewritten for the next filter row
            }
}
#if !SPIO_PARTIALS
        // One wave per group adds the group's R*S*64 sums into grad_weight: every atomic
        // instruction covers 64 consecutive floats (two full 128-byte lines), which the memory
        // system retires several times faster than the scattered half-lines of the accumulator
        // layout.  The wave reads back what it wrote itself, so a wave-level sync is enough.
        if (wave_active && ws == 0) {
            float* gout = out + (long long)gglob * GROUP_FLOATS;
            wave_sync();  // lanes 0-31 staged the sums, all lanes read them
#pragma unroll
            for (int i = 0; i < kR * kS; ++i) atomic_add_f32(gout + 64 * i + lane, gstage[64 * i + lane]);
        }
#endif
#if SPIO_HAS_BIAS
        // grad_bias[8g + k] = accb of row slot 0 (lanes 0-31) + row slot 1 (lanes 32-63); every
        // column holds the same sum, so lanes 0 and 16 carry channels 0-3 and 4-7.  All waves
        // leave their eight sums in LDS and one wave adds the workgroup's GB*8 consecutive
        // values with a single atomic instruction: atomics of different workgroups to the same
        // 128-byte line retire one after the other, so their number per line is what counts.
        {
            wave_sync();
            if (lane >= 32) {
#pragma unroll
                for (int e = 0; e < 4; ++e) scratch[e * 32 + (lane - 32)] = accb[e];
            }
            wave_sync();
            float* bslots = reinterpret_cast<float*>(lds) + WAVES * SCRATCH_FLOATS + RED_FLOATS +
                            (SPIO_PARTIALS ? 0 : GB * GROUP_FLOATS);  // [wave][8]
            if ((lane & 47) == 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    bslots[wave * 8 + k4 + e] = wave_active ? accb[e] + scratch[e * 32 + lane] : 0.f;
            }
            block_sync();
            if (wave == 0 && grad_bias != nullptr) {
                for (int i = lane; i < GB * 8; i += 64) {
                    float v = 0.f;
#pragma unroll
                    for (int w2 = 0; w2 < TS; ++w2) v += bslots[(w2 * GB + i / 8) * 8 + (i & 7)];
                    if (cb * GB + i / 8 < kGroups) atomic_add_f32(grad_bias + 8 * cb * GB + i, v);
                }
            }
        }
#endif
    }

}

#if SPIO_PARTIALS
// Second stage: grad_weight = sum over the partial blocks (stored whole: a caller that runs the
// two-stage kernel need not zero grad_weight first).  A workgroup owns 32 float4 columns
// of one channel block (512 contiguous bytes of every partial block: half a wave per load
// instruction); its 8 slices each add the blocks p = slice, slice + 8, ... with 4 loads in
// flight, the slices are added through LDS and slice 0 adds the total onto grad_weight.  (With 8
// columns and 32 slices per workgroup, 3584 workgroups of 128-byte rows for a 7x7 filter on 256
// channels, the stage took 5.9 us for 14.7 MB; now 5.1 us, of which about 2.2 us are what any
// kernel costs in a stream.)  Every element of grad_weight has exactly one
// owner, so no atomics are needed and the sum does not depend on timing.  A column is four
// consecutive lanes of the publishing wave, i.e. four consecutive channels c of one (k, r, s).
#define SPIO_CONCAT2(a, b) a##b
#define SPIO_CONCAT(a, b) SPIO_CONCAT2(a, b)
extern "C" __global__ void SPIO_LAUNCH_BOUNDS(256)
SPIO_CONCAT(SPIO_KERNEL_NAME, _reduce)(float* __restrict__ grad_weight, const spio_float4* __restrict__ partials) {
    constexpr int BLOCK_F4 = GB * PART_WAVE_FLOATS / 4;  // float4 columns of one partial block
    constexpr int NPART = NBLKS * PBLKS * QBLKS;
    constexpr int COLS = 32;
    constexpr int SLICES = 256 / COLS;
    constexpr int UN = 4;
    static_assert(BLOCK_F4 % COLS == 0, "a workgroup's columns lie in one channel block");
    __shared__ spio_float4 red[SLICES][COLS];
    const int tid = thread_id();
    const int cl = tid % COLS;
    const int slice = tid / COLS;
    const int col = (block_id() % (BLOCK_F4 / COLS)) * COLS + cl;
    const int cb = block_id() / (BLOCK_F4 / COLS);
    spio_float4 sum = spio_float4{0.f, 0.f, 0.f, 0.f};
    for (int base = slice; base < NPART; base += SLICES * UN) {
        spio_float4 v[UN];
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const int p = base + i * SLICES;
            v[i] = spio_float4{0.f, 0.f, 0.f, 0.f};
            if (p < NPART) v[i] = partials[((long long)p * GBLKS + cb) * BLOCK_F4 + col];
        }
#pragma unroll
        for (int i = 0; i < UN; ++i) sum += v[i];
    }
    red[slice][cl] = sum;
    block_sync();
    if (slice == 0) {
#pragma unroll 4
        for (int i = 1; i < SLICES; ++i) sum += red[i][cl];
        // float index inside the block -> (group, r, tap pair, e, lane)
        const int f = 4 * col;
        const int l32 = f & 31;
        const int e = (f >> 5) & 3;
        const int rn = (f >> 7) % (kR * NBLK);
        const int g = (f >> 7) / (kR * NBLK);
        const int r = rn / NBLK;
        const int s = 2 * (rn % NBLK) + ((l32 & 15) >> 3);
        const int k = 8 * (cb * GB + g) + 4 * (l32 >> 4) + e;
        if (cb * GB + g < kGroups && s < kS) {
            spio_float4* dst =
                reinterpret_cast<spio_float4*>(grad_weight + (((long long)k * kR + r) * kS + s) * 8 + (l32 & 7));
            *dst = sum;
        }
    }
}
#endif
