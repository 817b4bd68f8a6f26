// Fused backward kernel for conv2d_gw8 (gfx950): data gradient and weight gradient (and,
// optionally, the bias gradient) in one pass.
//
// Contract (reference kernels: spio/src/conv2d_gw8.cu:10-225 in its data-gradient mode and
// spio/src/conv2d_gw8_wgrad.cu:10-226; the reference launches them one after the other,
// spio/functional/conv2d_gw8_function.py:119-146):
//   dx[n,h,w,8g+c] = rn16(sum_{j,r,s} dy[n,h-r+py,w-s+px,8g+j] * w[8g+j,r,s,c])
//   dw[k,r,s,c]   += sum_{n,p,q} x[n,p+r-py,q+s-px,8g+c] * dy[n,p,q,k]            (fp32, atomics)
//   db[k]         += sum_{n,p,q} dy[n,p,q,k]                                      (with a bias)
//
// Why fuse: both gradients stream grad_output.  Run separately they move
// 2*|dy| + |x| + |dx| bytes through HBM; fused, dy is read once: 25 % less traffic for the
// backward step of an HBM-bound operator, and one launch instead of two.
//
// Scope: every filter size and padding the operator takes.  The kernel computes a "same"
// convolution (P = H and Q = W; padding PT rows above and PB below, PL columns left and PR right,
// PT + PB = R-1, PL + PR = S-1): then one copy of a dy row in LDS serves both gradients, and the dx
// row that completes at a step has the index of the x row of that step.  Any other padding is
// that convolution on a larger domain, DH x DW, in which x and dy sit at offsets that reproduce
// the problem's padding, with zeros around them: only the global addressing knows the tensors'
// real extents (domain rows and columns outside a tensor load zeros and store nothing), and below
// "row" and "column" are the domain's.
// A workgroup owns SPIO_BH rows (of dx, and of dy for the weight gradient) of SPIO_NB images
// side by side for SPIO_GB channel groups, repeated for SPIO_ITERS image blocks.  It streams the
// rows p0-PB .. p0+BH-1+PT of dy and p0-PT .. p0+BH-1+PB of x: step t stages dy row p0-PB+t and
// x row p0-(R-1)+t (an x row can only be multiplied once the dy rows up to PT below it are
// there).  The halo rows of dy above and below the block feed the
// data gradient only; the weight gradient masks them out of its dy fragments, so every dy row
// is counted by exactly one workgroup.  With SPIO_BH = DH a workgroup owns whole images and
// there is no halo.  Everything else is the separate kernels' design:
//   * rows of x and dy staged in LDS as [group][flattened pixel][8 ch], zero halo materialised
//     once, branch-free global loads SPIO_PF steps ahead;
//   * weight gradient: A = dy row pair, B = x (two column taps), one accumulator per (delta,
//     tap pair), transposing LDS reads (see conv2d_gw8_wgrad_mfma.hip);
//   * data gradient: A = flipped, group-transposed filter, B = dy (pixel n + tap kb is the
//     16 bytes lane (n, kb) reads), rotating accumulator row slots (see conv2d_gw8_mfma.hip);
//     a dy pixel (image i, column q) sits at flattened pixel i*WPI + q + PR, which is both its
//     place as a source pixel of the data gradient and, shifted by PR, its place opposite x
//     (column c at i*WPI + c + PL) in the weight gradient;
//   * publishing of dw (and db) as in the weight-gradient kernel: sums staged in LDS in
//     grad_weight order, atomics of 64 consecutive floats;
//   * global memory through buffer instructions with the hardware bounds check as predicate
//     (lanes without data: out-of-range offset; rows the block does not need: empty descriptor;
//     such loads return zeros, such stores are dropped) and a fully unrolled step loop, so that
//     no memory instruction sits under a branch and the compiler's count of outstanding loads and
//     stores is exact (see conv2d_gw8_mfma.hip).
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
#ifndef SPIO_BQ
#define SPIO_BQ 0
#endif
#ifndef SPIO_PARTIALS
#define SPIO_PARTIALS 0
#endif
#ifndef SPIO_TS
#define SPIO_TS 1
#endif
#ifndef SPIO_HAS_BIAS
#define SPIO_HAS_BIAS 0
#endif
#ifndef SPIO_XCD_CHUNK
#define SPIO_XCD_CHUNK 0
#endif
#ifndef SPIO_HALO_CACHED
#define SPIO_HALO_CACHED 1
#endif
#ifndef SPIO_MAX_UNROLL
#define SPIO_MAX_UNROLL 40  // a step of this kernel is long: beyond this the unroller gives up
#endif

namespace {

// The kernel works on a size-preserving convolution of DH x DW images whose padding is PT rows
// above, PB below, PL columns left and PR right (PT + PB = R-1, PL + PR = S-1; equal halves for odd
// filter sizes, the larger half above and left for even ones).  x (and dx) and dy sit inside that
// domain at the offsets (XOY, XOX) and (DOY, DOX), one of each pair being 0, such that the
// problem's own padding comes out (DOY - XOY = PT - py), and count as zero around their real extent.
constexpr int PT = kR / 2, PB = kR - 1 - PT;
constexpr int PL = kS / 2, PR = kS - 1 - PL;
constexpr int DOY = PT > kPadY ? PT - kPadY : 0, XOY = PT > kPadY ? 0 : kPadY - PT;
constexpr int DOX = PL > kPadX ? PL - kPadX : 0, XOX = PL > kPadX ? 0 : kPadX - PL;
constexpr int DH = XOY + kH > DOY + kP ? XOY + kH : DOY + kP;
constexpr int DW = XOX + kW > DOX + kQ ? XOX + kW : DOX + kQ;

constexpr int GB = SPIO_GB;        // groups per workgroup
constexpr int BH = SPIO_BH;        // rows per workgroup
constexpr int NB = SPIO_NB;        // images side by side
constexpr int ITERS = SPIO_ITERS;  // image blocks per workgroup
constexpr int TS = SPIO_TS;        // waves per group: they split the 32-pixel chunks and the 16-pixel tiles
constexpr int PF = SPIO_PF;        // prefetch distance in rows (even)
constexpr int WAVES = GB * TS;
constexpr int THREADS = 64 * WAVES;
constexpr bool kDbias = SPIO_HAS_BIAS != 0;

// ---- weight gradient ----
constexpr int S2 = 2 * ((kS + 1) / 2);
constexpr int NBLK = S2 / 2;          // column-tap pairs
constexpr int ND = kR + 1;            // values of delta
constexpr int NPAIR = kR / 2 + 1;     // aligned dy row pairs one x row meets
// Column blocks (SPIO_BQ > 0): a workgroup owns BQ columns (of dx, and of dy for the weight
// gradient) and stages BQ + S - 1 columns of x and of dy: the extra columns hold the neighbouring
// blocks' pixels (the data gradient of the block's edge columns needs the neighbours' dy, the
// weight gradient the neighbours' x), or zeros at the image's edges.  The weight gradient reads dy
// in 32-pixel chunks from the block's first column on, so BQ is a multiple of 32: a chunk that
// reached into the right-hand extra columns would count the neighbour's dy a second time.
// 0 = the whole width.
constexpr bool kColBlocks = SPIO_BQ > 0;
constexpr int BQ = kColBlocks ? SPIO_BQ : DW;
constexpr int QBLKS = (DW + BQ - 1) / BQ;
static_assert(!kColBlocks || (NB == 1 && BQ % 32 == 0), "column blocks: one image per row, a multiple of 32 columns");
constexpr int WPI = BQ + kS - 1;      // padded width of one image (block)
constexpr int F = NB * WPI;           // flattened pixels of a staged row
constexpr int KSPAN = (NB - 1) * WPI + BQ;
constexpr int KC = (KSPAN + 31) / 32;     // 32-pixel chunks
constexpr int CPW = (KC + TS - 1) / TS;   // chunks per wave
// ---- data gradient ----
constexpr int NS = 2 * ((kR + 1) / 2);   // accumulator row slots
constexpr int NACC = NS / 2;
constexpr int KB = (kS + 3) / 4;         // MFMA K-steps per dy row (4 column taps each)
constexpr int WT = (F - kS + 1 + 15) / 16;   // 16-pixel tiles of a dx row
constexpr int TPW = (WT + TS - 1) / TS;      // tiles per wave
// ---- LDS geometry ----
constexpr int FPX = 32 * KC + S2 - 1;  // x pixels a weight-gradient read can touch
constexpr int GSX = FPX + ((9 - FPX % 16) + 16) % 16;  // x group stride (pixels), = 9 mod 16
constexpr int FPD_W = PR + 32 * KC;                    // dy pixels: weight-gradient reads
constexpr int FPD_D = 16 * WT + 4 * KB - 1;            // dy pixels: data-gradient reads
constexpr int FPD = FPD_W > FPD_D ? FPD_W : FPD_D;
constexpr int GSD = FPD + ((9 - FPD % 16) + 16) % 16;  // dy group stride, = 9 mod 16
constexpr int NRX = 2;                                 // x ring rows
// dy ring rows: even, >= R+1; and at least 4 when the bias is summed, because that sum reads the
// whole row pair (t-1, t) in the step that stages row t+1 (with a one-row filter the weight
// gradient itself needs only two rows)
constexpr int NRD = (SPIO_HAS_BIAS && kR == 1) ? 4 : 2 * ((kR + 2) / 2);
// ring rows carry one spare unit behind the last group: the cell that threads without a source
// cell write their (zero) load result to
constexpr int XROW_UNITS = GB * GSX + 1;
constexpr int DROW_UNITS = GB * GSD + 1 + ((4 - (GB * GSD + 1) % 16) + 16) % 16;
constexpr int XDUMP = GB * GSX;
constexpr int DDUMP = GB * GSD;
constexpr int OSTRIDE = GB * 16 + 16;        // bytes per pixel in the dx output stage
constexpr int OUT_ROW_BYTES = 16 * WT * OSTRIDE;
constexpr int X_CELLS = F * GB;
constexpr int LPTX = (X_CELLS + THREADS - 1) / THREADS;
// dy cells a workgroup loads per row: the real columns of whole rows (the halo stays zero), all
// BQ + S - 1 columns of a column block
constexpr int D_CELLS = kColBlocks ? F * GB : NB * DW * GB;
constexpr int LPTD = (D_CELLS + THREADS - 1) / THREADS;  // dy loads per thread per row
constexpr int O_CELLS = NB * BQ * GB;
constexpr int LPTO = (O_CELLS + THREADS - 1) / THREADS;  // dx stores per thread per row
constexpr int GBLKS = (kGroups + GB - 1) / GB;
constexpr int NBLKS = (kN + NB * ITERS - 1) / (NB * ITERS);
constexpr int PBLKS = (DH + BH - 1) / BH;
constexpr int NUM_BLOCKS = GBLKS * PBLKS * QBLKS * NBLKS;
// steps: dy rows p0-PB .. p0+BH-1+PT, then PB more for the last x rows.  The bias sum takes a dy
// row pair one step after its first row was staged, so a one-row filter needs one more step
// when the sum is wanted.
constexpr int ROWS = BH + PB + kR - 1 + (SPIO_HAS_BIAS && kR == 1 ? 1 : 0);

constexpr int gcd_(int a, int b) { return b == 0 ? a : gcd_(b, a % b); }
constexpr int LCM = NS / gcd_(NS, PF) * PF;  // lcm(NS, PF): even
// up to SPIO_MAX_UNROLL steps the step loop is unrolled completely, longer ones run in chunks
constexpr bool kFullUnroll = ROWS <= SPIO_MAX_UNROLL;
constexpr int UNROLL = kFullUnroll ? (ROWS + LCM - 1) / LCM * LCM : LCM;
constexpr int pmod(int a, int m) { return ((a % m) + m) % m; }

constexpr int RING_UNITS = NRX * XROW_UNITS + NRD * DROW_UNITS;
constexpr int STREAM_UNITS = RING_UNITS + 2 * OUT_ROW_BYTES / 16;
constexpr int FILTER_UNITS = GB * 8 * kR * kS;  // filters staged once at the start
// Filter rows whose row-slot halves are exchanged through the per-wave scratch in one go: all of
// them where that fits 96 KB of LDS for the workgroup (every exchange costs an LDS round trip),
// else one; one when waves share a group, whose sums are then added row by row.
constexpr int RCH = (TS == 1 && WAVES * kR * NBLK * 512 <= 96 * 1024) ? kR : 1;
constexpr int SCRATCH_FLOATS = RCH * NBLK * 128;  // per wave: row-slot halves
constexpr int RED_FLOATS = GB * (TS - 1) * NBLK * 128;
constexpr int GROUP_FLOATS = kR * kS * 64;
// Two-stage publishing (SPIO_PARTIALS = 1): every workgroup stores its sums, in grad_weight order
// (and its GB * 8 bias sums behind them), into its own block of a workspace that takes the place
// of the grad_weight argument; the <name>_reduce kernel at the end of this file stores the sum of
// the blocks into grad_weight (and grad_bias).  No atomics: with one-round grids all workgroups
// reach the publish together and their atomic additions to the same lines retire one after the
// other (14 ns each: 3.6 us for 256 workgroups at N=128, C=64, 56x56); nothing to zero first.
constexpr int PART_FLOATS = GB * GROUP_FLOATS + (SPIO_HAS_BIAS ? GB * 8 : 0);  // one workgroup's block
constexpr int NPART = NBLKS * PBLKS * QBLKS;  // blocks per channel block
constexpr int PUBLISH_FLOATS =
    WAVES * SCRATCH_FLOATS + RED_FLOATS + GB * GROUP_FLOATS + (SPIO_HAS_BIAS ? WAVES * 8 : 0);
constexpr int max3(int a, int b, int c) { return a > b ? (a > c ? a : c) : (b > c ? b : c); }
constexpr int LDS_UNITS = max3(STREAM_UNITS, FILTER_UNITS, (PUBLISH_FLOATS + 3) / 4);
static_assert(LDS_UNITS * 16 <= 160 * 1024, "LDS overflow");
static_assert(PF >= 2 && PF % 2 == 0 && WAVES <= 16, "bad configuration");

constexpr long long X_IMAGE_BYTES = (long long)kH * kW * kC * 2;  // of x and dx
constexpr long long D_IMAGE_BYTES = (long long)kP * kQ * kC * 2;  // of dy
static_assert(NB * X_IMAGE_BYTES < (1ll << 31) && NB * D_IMAGE_BYTES < (1ll << 31),
              "an image block must stay below 2 GiB (32-bit buffer offsets)");
constexpr int X_ROW_BYTES = kW * kC * 2;
constexpr int D_ROW_BYTES = kQ * kC * 2;
constexpr unsigned OOB = 0x80000000u;  // offset of a lane without data: beyond every descriptor
constexpr int AUX_NT = SPIO_NT ? 2 : 0;

typedef __amdgpu_buffer_rsrc_t rsrc_t;
SPIO_DEVICE rsrc_t make_rsrc(const void* base, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

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
SPIO_KERNEL_NAME(spio_uint4* __restrict__ grad_input, float* __restrict__ grad_weight,
                 const spio_uint4* __restrict__ x, const spio_uint4* __restrict__ dy,
                 const spio_half* __restrict__ weights
#if SPIO_HAS_BIAS
                 , float* __restrict__ grad_bias  // [K] fp32, accumulated into; null = not wanted
#endif
) {
    // One LDS block: x ring, dy ring, two dx output-stage rows.  Before the first row it holds
    // the staged filters, after the last one the reduction scratch.
    __shared__ spio_uint4 lds[LDS_UNITS];
    spio_uint4* const xring = lds;
    spio_uint4* const dring = lds + NRX * XROW_UNITS;
    unsigned char* const ostage = reinterpret_cast<unsigned char*>(lds + RING_UNITS);

    const int tid = thread_id();
    const int lane = tid & 63;
    // scalar wave index: conditions on it become scalar branches, so no MFMA (which ignores the
    // lane mask) is issued under an empty mask
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = wave % GB;
    const int ws = wave / GB;

    // Workgroup ids are dealt round-robin to the 8 XCDs: runs of SPIO_XCD_CHUNK consecutive tiles
    // go to one XCD (row blocks share halo rows through its L2) while the tiles in flight on the
    // device form one compact range of addresses; 0 = one contiguous range of tiles per XCD.
    int b = block_id();
    {
        constexpr int CH = SPIO_XCD_CHUNK;
        if (CH == 0) {
            if (NUM_BLOCKS % 8 == 0) b = (b & 7) * (NUM_BLOCKS / 8) + (b >> 3);
        } else if (CH > 1 && NUM_BLOCKS % (8 * CH) == 0) {
            const int x8 = b & 7;
            const int k = b >> 3;
            b = (k / CH) * (8 * CH) + x8 * CH + k % CH;
        }
    }
    // Tile order: row blocks fastest, so that neighbours in a run share halo rows.  Where a
    // workgroup covers only part of a pixel's 128-byte lines (GB * 16 bytes per pixel), the channel
    // blocks that share those lines go fastest instead: dealt to different XCDs, every one of
    // them would fetch the whole lines from memory (measured: twice the algorithmic reads).
    constexpr bool kSplitLines = GBLKS > 1 && (GB * 16) % 128 != 0;
    // Column blocks go before the row blocks: neighbours share S - 1 columns of every row.
    constexpr int TILES = QBLKS * PBLKS;
    const int tile = kSplitLines ? (b / GBLKS) % TILES : b % TILES;
    const int cb = kSplitLines ? b % GBLKS : (b / TILES) % GBLKS;
    const int nbk = b / (TILES * GBLKS);
    const int pb = tile / QBLKS;
    const int q0 = (tile % QBLKS) * BQ;
    const int p0 = pb * BH;
    const int bh_eff = imin(BH, DH - p0);  // rows this block owns
    // first and last row (of the domain) the block needs: of x for the weight gradient of its dy
    // rows, of dy for its dx rows (which include the weight gradient's)
    const int xrow_lo = p0 - PT, xrow_hi = p0 + bh_eff - 1 + PB;
    const int drow_lo = p0 - PB, drow_hi = p0 + bh_eff - 1 + PT;
    const int gglob = cb * GB + wg;
    const bool wave_active = gglob < kGroups;

    // ---- data-gradient filter fragments: wfrag[d][u], d = (phase - 2*acc) mod NS ----
    // A[m = dx channel ch][jj] = w[8g+jj][R-1-r][S-1-s][ch].  The workgroup copies its groups'
    // filters to LDS as they lie in memory and every wave reads its fragments with the
    // transposing LDS read (same scheme as the data-gradient mode of conv2d_gw8_mfma.hip).
    // The filter loads are issued here, the loads of the first rows right behind them, and only
    // then does anything wait: the fragments are built while the rows are on their way.
    constexpr int FLT = (FILTER_UNITS + THREADS - 1) / THREADS;
    spio_uint4 fpre[FLT];
    {
        const int valid_groups = imin(GB, kGroups - cb * GB);
        const rsrc_t rs_w = make_rsrc(reinterpret_cast<const unsigned char*>(weights) +
                                          (long long)cb * GB * (8 * kR * kS * 16),
                                      valid_groups * (8 * kR * kS * 16));
#pragma unroll
        for (int l = 0; l < FLT; ++l) {
            Pack16 v;  // units past the workgroup's groups lie beyond the descriptor: zeros
            v.i = __builtin_amdgcn_raw_buffer_load_b128(rs_w, (tid + THREADS * l) * 16, 0, 0);
            fpre[l] = v.u;
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the filter loads ahead of the row loads
    spio_half8 wfrag[NS][KB];

    // ---- lane roles ----
    // weight gradient (transposing reads): block kb = lane/16 covers pixels 8*kb..8*kb+7, source
    // lane 4*jr + t supplies pixel jr (+4 for the second read) of unit t/2 (dy row j or column
    // tap sj) and channel half t%2.
    const int kb = lane >> 4;
    const int jr = (lane & 15) >> 2;
    const int tt = lane & 3;
    const int sel = tt >> 1;
    const int xfrag_off = ((wg * GSX + 8 * kb + jr + sel) * 16) + (tt & 1) * 8;
    const int dfrag_off = ((wg * GSD + PR + 8 * kb + jr) * 16) + (tt & 1) * 8;
    // data gradient: D[m = 4*(lane/16)+i][n = lane%16]: pixel n, row slot lane/32, channels
    // 4*((lane/16)&1) + i
    const int out_j = lane >> 5;
    const int out_kh = (lane >> 4) & 1;
    const int out_n = lane & 15;

    spio_float4 acc[ND][NBLK];  // weight gradient
#pragma unroll
    for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) acc[d][nb] = spio_float4{0.f, 0.f, 0.f, 0.f};
    spio_float4 accb = spio_float4{0.f, 0.f, 0.f, 0.f};  // bias gradient
    const spio_half8 ones8 = spio_half8{1, 1, 1, 1, 1, 1, 1, 1};
    (void)ones8;

    const spio_uint4 zero4 = spio_uint4{0u, 0u, 0u, 0u};
    const rsrc_t rs_none = make_rsrc(x, 0);  // nothing is in range: loads give zeros, stores vanish

    for (int it = 0; it < ITERS; ++it) {
        const int n0 = (nbk * ITERS + it) * NB;
        if (n0 >= kN) break;

        // ---- buffer descriptors of this image block; images past the end of the batch lie
        //      beyond their size ----
        const int images = imin(NB, kN - n0);
        const rsrc_t rs_x = make_rsrc(reinterpret_cast<const unsigned char*>(x) + n0 * X_IMAGE_BYTES,
                                      (int)(images * X_IMAGE_BYTES));
        const rsrc_t rs_dy = make_rsrc(reinterpret_cast<const unsigned char*>(dy) + n0 * D_IMAGE_BYTES,
                                       (int)(images * D_IMAGE_BYTES));
        const rsrc_t rs_dx = make_rsrc(reinterpret_cast<const unsigned char*>(grad_input) + n0 * X_IMAGE_BYTES,
                                       (int)(images * X_IMAGE_BYTES));

        // ---- loop-invariant addressing (cells without data carry the out-of-range offset: they
        //      load zeros, which is what halo and gap cells must hold) ----
        unsigned x_voff[LPTX];
        int x_lds[LPTX];
#pragma unroll
        for (int l = 0; l < LPTX; ++l) {
            const int cell = tid + THREADS * l;
            x_voff[l] = OOB;
            x_lds[l] = XDUMP;
            if (cell < X_CELLS) {
                const int g = cell % GB;
                const int f = cell / GB;
                const int img = f / WPI;
                const int col = q0 + f % WPI - PL - XOX;  // column of x
                x_lds[l] = g * GSX + f;
                if (col >= 0 && col < kW && cb * GB + g < kGroups)
                    x_voff[l] = (unsigned)(((img * kH * kW + col) * kGroups + cb * GB + g) * 16);
            }
        }
        // dy cells, and the dx cells of the same (image, domain column, group): where dy and x have
        // the same size, the same offset
        unsigned d_voff[LPTD], o_voff[LPTO];
        int d_lds[LPTD], o_lds[LPTO];
#pragma unroll
        for (int l = 0; l < LPTD; ++l) {
            const int cell = tid + THREADS * l;
            d_voff[l] = OOB;
            d_lds[l] = DDUMP;
            if (cell < D_CELLS) {
                const int g = cell % GB;
                // whole rows: the cells are the real columns; column blocks: every staged column
                const int q = kColBlocks ? q0 + (cell / GB) % WPI - PR : (cell / GB) % DW;  // domain column
                const int img = kColBlocks ? 0 : cell / (GB * DW);
                d_lds[l] = g * GSD + (kColBlocks ? cell / GB : img * WPI + q + PR);
                const int qd = q - DOX;  // column of dy
                if (qd >= 0 && qd < kQ && cb * GB + g < kGroups)
                    d_voff[l] = (unsigned)(((img * kP * kQ + qd) * kGroups + cb * GB + g) * 16);
            }
        }
#pragma unroll
        for (int l = 0; l < LPTO; ++l) {
            const int cell = tid + THREADS * l;
            o_voff[l] = OOB;
            o_lds[l] = 0;
            if (cell < O_CELLS) {
                const int g = cell % GB;
                const int q = (cell / GB) % BQ;
                const int img = cell / (GB * BQ);
                o_lds[l] = (img * WPI + q) * OSTRIDE + g * 16;
                const int wx = q0 + q - XOX;  // column of dx
                if (q0 + q < DW && wx >= 0 && wx < kW && cb * GB + g < kGroups)
                    o_voff[l] = (unsigned)(((img * kH * kW + wx) * kGroups + cb * GB + g) * 16);
            }
        }

        // Rows `t` of x (domain row p0-(R-1)+t) and of dy (p0-PB+t) for every cell of the thread.
        // Rows the block does not need, and domain rows outside the tensor, read through the empty
        // descriptor (zeros, no traffic).
        auto load_rows = [&](spio_uint4(&xr)[LPTX], spio_uint4(&dr)[LPTD], int t) {
            const int h = p0 - (kR - 1) + t;
            const rsrc_t rx = (h >= xrow_lo && h <= xrow_hi && h >= XOY && h < XOY + kH) ? rs_x : rs_none;
            const int sx = __builtin_amdgcn_readfirstlane(imin(imax(h - XOY, 0), kH - 1) * X_ROW_BYTES);
            const bool xhalo = h < p0 || h >= p0 + bh_eff;
#pragma unroll
            for (int l = 0; l < LPTX; ++l) {
                Pack16 v;
                v.i = (SPIO_HALO_CACHED && xhalo) ? __builtin_amdgcn_raw_buffer_load_b128(rx, (int)x_voff[l], sx, 0)
                                                  : __builtin_amdgcn_raw_buffer_load_b128(rx, (int)x_voff[l], sx, AUX_NT);
                xr[l] = v.u;
            }
            const int pr = p0 - PB + t;
            const rsrc_t rd = (pr >= drow_lo && pr <= drow_hi && pr >= DOY && pr < DOY + kP) ? rs_dy : rs_none;
            const int sd = __builtin_amdgcn_readfirstlane(imin(imax(pr - DOY, 0), kP - 1) * D_ROW_BYTES);
            const bool dhalo = pr < p0 || pr >= p0 + bh_eff;
#pragma unroll
            for (int l = 0; l < LPTD; ++l) {
                Pack16 v;
                v.i = (SPIO_HALO_CACHED && dhalo) ? __builtin_amdgcn_raw_buffer_load_b128(rd, (int)d_voff[l], sd, 0)
                                                  : __builtin_amdgcn_raw_buffer_load_b128(rd, (int)d_voff[l], sd, AUX_NT);
                dr[l] = v.u;
            }
        };

        // ---- prologue: rows 0..PF-1 into registers ----
        spio_uint4 xpre[PF][LPTX], dpre[PF][LPTD];
#pragma unroll
        for (int t = 0; t < PF; ++t) load_rows(xpre[t], dpre[t], t);
        __builtin_amdgcn_sched_barrier(0);  // the first loads are on their way before anything waits
        if (it == 0) {
            // while the first loads are in flight: the filter fragments, through the LDS block
            // the rings will use ...
#pragma unroll
            for (int l = 0; l < FLT; ++l)
                if (tid + THREADS * l < FILTER_UNITS) lds[tid + THREADS * l] = fpre[l];
            block_sync();
            const int fkb = lane >> 4;
            const int fjr = (lane & 15) >> 2;
            const int ft4 = lane & 3;
            const int src_slot = ft4 >> 1;
            const int my_slot = (lane & 15) >> 3;
            typedef spio_short4 __attribute__((address_space(3))) * lds_ptr;
#pragma unroll
            for (int d = 0; d < NS; ++d) {
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    const int s = 4 * u + fkb;
                    const int r_src = (d - src_slot + NS) % NS;
                    const int r_mine = (d - my_slot + NS) % NS;
                    const int rr = r_src < kR ? kR - 1 - r_src : 0;  // dead taps: any valid address
                    const int ss = s < kS ? kS - 1 - s : 0;
                    const unsigned char* base = reinterpret_cast<const unsigned char*>(lds) +
                                                ((((wg * 8 + fjr) * kR + rr) * kS + ss) * 16) + (ft4 & 1) * 8;
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
            block_sync();  // everyone has its fragments before the rings are zero-filled
            // ... and both rings zeroed once: the slack cells behind each group's pixels are
            // never written
            for (int i = tid; i < RING_UNITS; i += THREADS) lds[i] = zero4;
        }
        block_sync();  // rings zeroed / previous image block finished
#pragma unroll
        for (int l = 0; l < LPTX; ++l) xring[x_lds[l]] = xpre[0][l];
#pragma unroll
        for (int l = 0; l < LPTD; ++l) dring[d_lds[l]] = dpre[0][l];
        block_sync();

        spio_float4 dacc[TPW][NACC];  // data gradient: rotating row slots
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int a = 0; a < NACC; ++a) dacc[i][a] = spio_float4{0.f, 0.f, 0.f, 0.f};

        // Coalesced store of the dx row staged at step `ts` (domain row p0 - (R-1) + ts), one step
        // later.  Steps that finish no row of the block, or a domain row outside dx, store through
        // the empty descriptor: the
        // instructions are issued all the same and the hardware drops them.
        auto store_dx_row = [&](int ts, int obuf) {
            const int h = p0 - (kR - 1) + ts;
            const bool real = ts >= kR - 1 && ts < kR - 1 + bh_eff && h >= XOY && h < XOY + kH;
            const rsrc_t rs = real ? rs_dx : rs_none;
            // The row offset is added to the per-lane offset; the scalar-offset operand stays the
            // constant 0.  A 16-byte buffer store reads its data registers for a few cycles after
            // it issues, and only for the constant form does the compiler keep the next
            // instructions from writing them: with the row offset in a scalar register a result
            // moved into the first data register right behind the store was stored in its place
            // (seen on gfx950 as stray values in the first two channels of some pixels).
            const unsigned row_off = (unsigned)(imin(imax(h - XOY, 0), kH - 1) * X_ROW_BYTES);
#pragma unroll
            for (int l = 0; l < LPTO; ++l) {
                Pack16 v;
                v.u = *reinterpret_cast<const spio_uint4*>(ostage + obuf * OUT_ROW_BYTES + o_lds[l]);
                __builtin_amdgcn_raw_buffer_store_b128(v.i, rs, (int)(o_voff[l] + row_off), 0, AUX_NT);
            }
            store_group_end();
        };

        for (int tb = 0; tb < ROWS; tb += UNROLL) {
#pragma unroll
            for (int uu = 0; uu < UNROLL; ++uu) {
                const int t = tb + uu;
                if (t >= ROWS) break;
                const int sp = uu & 1;                   // parity of t: x ring row, parity of delta
                const int pbuf = uu % PF;                // register buffer that held row t
                const int ph = uu % NS;                  // data-gradient phase: t mod NS
                const int obuf = uu & 1;

                // 1. fragment reads: x row p0-(R-1)+t, the dy row pairs it meets (dy rows are named
                //    by the step that staged them: row p0-PB+tau at step tau; the block owns
                //    tau in [PB, PB+bh_eff)), and dy row p0-PB+t as the data gradient's source row
                const int hcur = p0 - (kR - 1) + t;
                const bool x_live = t >= PB && hcur >= XOY && hcur < XOY + kH;
                const int dcur = p0 - PB + t;
                const bool d_live = t < bh_eff + kR - 1 && dcur >= DOY && dcur < DOY + kP;
                const int tbase = t - sp;
                const int own_lo = PB, own_hi = PB + bh_eff;  // owned dy rows: [own_lo, own_hi)
                const bool bias_pair = kDbias && sp == 1 && tbase + 1 >= own_lo && tbase < own_hi;
                const bool do_w = wave_active && (x_live || bias_pair);
                spio_half8 bfrag[CPW][NBLK], afrag[CPW][NPAIR];
                if (do_w) {
#pragma unroll
                    for (int ci = 0; ci < CPW; ++ci) {
                        const int ch = ws + TS * ci;
                        if (TS > 1 && ch >= KC) break;
                        const unsigned char* xrow =
                            reinterpret_cast<const unsigned char*>(xring + sp * XROW_UNITS) + xfrag_off;
#pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb) {
                            const unsigned char* pb0 = xrow + (32 * ch + 2 * nb) * 16;
                            bfrag[ci][nb] = read_tr_pair(pb0, pb0 + 4 * 16);
                        }
#pragma unroll
                        for (int m = 0; m < NPAIR; ++m) {
                            const int i2 = tbase - 2 * m;  // first row of the pair (step numbering)
                            if (i2 + 1 >= own_lo && i2 < own_hi) {
                                const int slot = (i2 + sel + NRD) % NRD;
                                const unsigned char* pa0 =
                                    reinterpret_cast<const unsigned char*>(dring + slot * DROW_UNITS) +
                                    dfrag_off + (32 * ch) * 16;
                                spio_half8 a = read_tr_pair(pa0, pa0 + 4 * 16);
                                // a halo row in the pair belongs to the neighbouring block; the
                                // transposed fragment holds row j = (lane % 16) / 8 of the pair
                                const int row = i2 + ((lane & 15) >> 3);
                                if (row < own_lo || row >= own_hi) a = spio_half8{0, 0, 0, 0, 0, 0, 0, 0};
                                afrag[ci][m] = a;
                            }
                        }
                    }
                }
                const bool do_d = wave_active && d_live;
                spio_half8 sfrag[TPW][KB];
                if (do_d) {
                    const spio_uint4* rrow =
                        dring + (t % NRD) * DROW_UNITS + wg * GSD + (lane & 15) + (lane >> 4);
#pragma unroll
                    for (int i = 0; i < TPW; ++i) {
                        const int tile = ws + TS * i;
                        if (TS == 1 || tile < WT) {
#pragma unroll
                            for (int u = 0; u < KB; ++u) {
                                Pack16 v;
                                v.u = rrow[16 * tile + 4 * u];
                                sfrag[i][u] = v.h;
                            }
                        }
                    }
                }

                // 2. prefetch rows t+PF.  Rows past the end read through the empty descriptor in the
                //    chunked loop (every step then issues the same loads); the unrolled loop leaves
                //    them out.
                if (!kFullUnroll || t + PF < ROWS) load_rows(xpre[pbuf], dpre[pbuf], t + PF);

                // 3. the dx row finished in the previous step goes out
                if (!kFullUnroll || t - 1 >= kR - 1) store_dx_row(t - 1, (uu + 1) & 1);

                // 4. rows t+1 into LDS (dy rows past the last one become zero).  The ring rows
                //    written here are not read in this step, except for dy entries of the weight
                //    gradient whose filter row is out of range and whose product is ignored.
                if (t + 1 < ROWS) {
#pragma unroll
                    for (int l = 0; l < LPTX; ++l)
                        xring[((sp + 1) & 1) * XROW_UNITS + x_lds[l]] = xpre[(uu + 1) % PF][l];
                    const int dslot = (t + 1) % NRD;
#pragma unroll
                    for (int l = 0; l < LPTD; ++l) dring[dslot * DROW_UNITS + d_lds[l]] = dpre[(uu + 1) % PF][l];
                }

                // 5. multiply: weight gradient ...
                if (do_w) {
#pragma unroll
                    for (int ci = 0; ci < CPW; ++ci) {
                        const int ch = ws + TS * ci;
                        if (TS > 1 && ch >= KC) break;
#pragma unroll
                        for (int m = 0; m < NPAIR; ++m) {
                            const int i2 = tbase - 2 * m;
                            if (i2 + 1 >= own_lo && i2 < own_hi) {
                                const int d = sp + 2 * m;  // = t - i2
                                if (d <= kR && x_live) {
#pragma unroll
                                    for (int nb = 0; nb < NBLK; ++nb)
                                        acc[d][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                            afrag[ci][m], bfrag[ci][nb], acc[d][nb], 0, 0, 0);
                                }
                                if (m == 0 && bias_pair)
                                    accb = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[ci][0], ones8, accb, 0, 0, 0);
                            }
                        }
                    }
                }
                //    ... and data gradient: dy row t into the live dx rows
                if (do_d) {
#pragma unroll
                    for (int i = 0; i < TPW; ++i) {
                        const int tile = ws + TS * i;
                        if (TS == 1 || tile < WT) {
#pragma unroll
                            for (int a = 0; a < NACC; ++a) {
                                const int d = pmod(ph - 2 * a, NS);
#pragma unroll
                                for (int u = 0; u < KB; ++u)
                                    dacc[i][a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                        wfrag[d][u], sfrag[i][u], dacc[i][a], 0, 0, 0);
                            }
                        }
                    }
                }

                // 6. the dx row that received its last tap (row p0-(R-1)+t): stage it if the block
                //    owns it, reset its slot
                {
                    const int slot = pmod(ph - (kR - 1), NS);
                    const int a = slot >> 1;
                    const int j = slot & 1;
                    const bool emit = t >= kR - 1 && t < kR - 1 + bh_eff;
                    if (wave_active && out_j == j) {
#pragma unroll
                        for (int i = 0; i < TPW; ++i) {
                            const int tile = ws + TS * i;
                            if (TS == 1 || tile < WT) {
                                if (emit) {
                                    Pack8 o;
#pragma unroll
                                    for (int e = 0; e < 4; ++e) o.h[e] = (spio_half)dacc[i][a][e];
                                    *reinterpret_cast<spio_uint2*>(ostage + obuf * OUT_ROW_BYTES +
                                                                   (16 * tile + out_n) * OSTRIDE + wg * 16 +
                                                                   out_kh * 8) = o.u;
                                }
#pragma unroll
                                for (int e = 0; e < 4; ++e) dacc[i][a][e] = 0.f;
                            }
                        }
                    }
                }
                block_sync();
            }
        }
        store_dx_row(ROWS - 1, (ROWS - 1) & 1);  // the last staged row (if it is a real one)
    }

    // ---- publish grad_weight (and grad_bias): as in conv2d_gw8_wgrad_mfma.hip ----
    // dw[k,r,s,c] = acc[delta = r] (lanes 0-31: j = 0) + acc[delta = r+1] (lanes 32-63: j = 1);
    // the halves meet in a per-wave LDS scratch, the waves of a split group add their sums
    // through LDS, the group's R*S*64 sums are staged in grad_weight order and added with
    // atomics of 64 consecutive floats.
    block_sync();  // every wave is done with the rings and the output stage
    {
        float* scratch = reinterpret_cast<float*>(lds) + wave * SCRATCH_FLOATS;
        float* red = reinterpret_cast<float*>(lds) + WAVES * SCRATCH_FLOATS;
        float* gstage = reinterpret_cast<float*>(lds) + WAVES * SCRATCH_FLOATS + RED_FLOATS + wg * GROUP_FLOATS;
        const int k4 = 4 * ((lane >> 4) & 1);
        const int sj = (lane & 15) >> 3;
        const int c = lane & 7;
        if (RCH > 1) {
            // all filter rows at once: lanes 32-63 leave their halves in the scratch as float4s, one
            // wave-level sync, lanes 0-31 add them and stage the sums in grad_weight order
            spio_float4* half4 = reinterpret_cast<spio_float4*>(scratch);
            if (lane >= 32) {
#pragma unroll
                for (int r = 0; r < kR; ++r)
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb) half4[(r * NBLK + nb) * 32 + (lane - 32)] = acc[r + 1][nb];
            }
            wave_sync();  // lanes 32-63 stored, lanes 0-31 load
            if (wave_active && lane < 32) {
#pragma unroll
                for (int r = 0; r < kR; ++r)
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb) {
                        const spio_float4 total = acc[r][nb] + half4[(r * NBLK + nb) * 32 + lane];
                        const int s = 2 * nb + sj;
                        if (s < kS) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) gstage[(((k4 + e) * kR + r) * kS + s) * 8 + c] = total[e];
                        }
                    }
            }
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
                if (wave_active && ws == 0 && lane < 32) {
    #pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb) {
                        const int s = 2 * nb + sj;
                        if (s < kS) {
    #pragma unroll
                            for (int e = 0; e < 4; ++e) gstage[(((k4 + e) * kR + r) * kS + s) * 8 + c] = total[nb][e];
                        }
                    }
                }
                if (TS > 1) block_sync();  // the scratch is rewritten for the next filter row
            }
}
#if SPIO_PARTIALS
        // this workgroup's block of the workspace: [group][k][r][s][c], then [group][k] bias sums
        float* const pblock = grad_weight + ((long long)cb * NPART + (nbk * PBLKS + pb) * QBLKS + q0 / BQ) * PART_FLOATS;
        if (ws == 0) {  // groups past the last one store their zeros: the block is read whole
            float* gout = pblock + wg * GROUP_FLOATS;
            wave_sync();  // lanes 0-31 staged the sums, all lanes read them
#pragma unroll
            for (int i = 0; i < kR * kS; ++i)
                __builtin_nontemporal_store(wave_active ? gstage[64 * i + lane] : 0.f, gout + 64 * i + lane);
        }
#else
        if (wave_active && ws == 0) {
            float* gout = grad_weight + (long long)gglob * GROUP_FLOATS;
            wave_sync();  // lanes 0-31 staged the sums, all lanes read them
#pragma unroll
            for (int i = 0; i < kR * kS; ++i) atomic_add_f32(gout + 64 * i + lane, gstage[64 * i + lane]);
        }
#endif
#if SPIO_HAS_BIAS
        {
            wave_sync();
            if (lane >= 32) {
#pragma unroll
                for (int e = 0; e < 4; ++e) scratch[e * 32 + (lane - 32)] = accb[e];
            }
            wave_sync();
            float* bslots = reinterpret_cast<float*>(lds) + WAVES * SCRATCH_FLOATS + RED_FLOATS +
                            GB * GROUP_FLOATS;  // [wave][8]
            if ((lane & 47) == 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    bslots[wave * 8 + k4 + e] = wave_active ? accb[e] + scratch[e * 32 + lane] : 0.f;
            }
            block_sync();
#if SPIO_PARTIALS
            if (wave == 0) {
                for (int i = lane; i < GB * 8; i += 64) {
                    float v = 0.f;
#pragma unroll
                    for (int w2 = 0; w2 < TS; ++w2) v += bslots[(w2 * GB + i / 8) * 8 + (i & 7)];
                    pblock[GB * GROUP_FLOATS + i] = v;
                }
            }
#else
            if (wave == 0 && grad_bias != nullptr) {
                for (int i = lane; i < GB * 8; i += 64) {
                    float v = 0.f;
#pragma unroll
                    for (int w2 = 0; w2 < TS; ++w2) v += bslots[(w2 * GB + i / 8) * 8 + (i & 7)];
                    if (cb * GB + i / 8 < kGroups) atomic_add_f32(grad_bias + 8 * cb * GB + i, v);
                }
            }
#endif
        }
#endif
    }
}

#if SPIO_PARTIALS
// Second stage: grad_weight (and grad_bias) = sum over the workgroups' blocks.  A workgroup of
// 256 threads owns 8 float4 columns of one channel block (128 contiguous bytes of every block);
// its 32 slices each add the blocks p = slice, slice + 32, ... with up to 8 loads in flight, the
// slices are added through LDS and slice 0 stores the totals.  A block is laid out like the
// channel block's part of grad_weight, so column `col` of channel block `cb` is the float4 at
// grad_weight[cb * GB * GROUP_FLOATS + 4 * col]; the columns behind it are the bias sums.
#define SPIO_CONCAT2(a, b) a##b
#define SPIO_CONCAT(a, b) SPIO_CONCAT2(a, b)
extern "C" __global__ void SPIO_LAUNCH_BOUNDS(256)
SPIO_CONCAT(SPIO_KERNEL_NAME, _reduce)(float* __restrict__ grad_weight, const spio_float4* __restrict__ partials,
                                       float* __restrict__ grad_bias) {
    constexpr int BLOCK_F4 = PART_FLOATS / 4;  // float4 columns of one block
    constexpr int COLS = 8;
    constexpr int SLICES = 256 / COLS;
    constexpr int UN = 8;
    constexpr int WGS_PER_CB = (BLOCK_F4 + COLS - 1) / COLS;
    __shared__ spio_float4 red[SLICES][COLS];
    const int tid = thread_id();
    const int cl = tid % COLS;
    const int slice = tid / COLS;
    const int cb = block_id() / WGS_PER_CB;
    const int col = (block_id() % WGS_PER_CB) * COLS + cl;
    const bool live = col < BLOCK_F4;
    const spio_float4* base = partials + (long long)cb * NPART * BLOCK_F4 + (live ? col : 0);
    spio_float4 sum = spio_float4{0.f, 0.f, 0.f, 0.f};
    for (int p0 = slice; p0 < NPART; p0 += SLICES * UN) {
        spio_float4 v[UN];
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const int p = p0 + i * SLICES;
            v[i] = spio_float4{0.f, 0.f, 0.f, 0.f};
            if (p < NPART) v[i] = __builtin_nontemporal_load(base + (long long)p * BLOCK_F4);
        }
#pragma unroll
        for (int i = 0; i < UN; ++i) sum += v[i];
    }
    red[slice][cl] = sum;
    block_sync();
    if (slice == 0 && live) {
#pragma unroll 4
        for (int i = 1; i < SLICES; ++i) sum += red[i][cl];
        const int f = 4 * col;  // float index inside the block
        if (f < GB * GROUP_FLOATS) {
            if (cb * GB + f / GROUP_FLOATS < kGroups)
                *reinterpret_cast<spio_float4*>(grad_weight + (long long)cb * GB * GROUP_FLOATS + f) = sum;
        } else if (grad_bias != nullptr) {
            const int k = cb * GB * 8 + (f - GB * GROUP_FLOATS);
            if (k < kC) *reinterpret_cast<spio_float4*>(grad_bias + k) = sum;
        }
    }
}
#endif
