// Weight-streaming kernels for skinny M: the decode-shaped linear layer.  Three kernels:
// skinny_kernel (up to 64 rows of X per launch, W's rows split over one workgroup per CU;
// as skinny_ksplit_kernel the same code with K split over workgroups as well, for 33 to 64
// rows of X against long K), skinny_stream_kernel (very many rows of W: workgroups that
// stay on their CU) and skinny_basic_kernel (K that is not a whole number of 128-byte
// tiles).
//
// The job is HBM-bound: every byte of W (N x K/2) is read exactly once and the arithmetic
// (v_mfma_i32_16x16x64_i8 after the same 16x nibble widening as the big int8 kernel:
// (w << 4) & 0xF0F0F0F0 and w & 0xF0F0F0F0, C = acc >> 8) is free next to it.  What decides
// the speed is the shape of the global reads and what a launch spends before its first load
// and after its last byte.  Measured on MI355X for a 28 MiB weight matrix: a wave
// instruction whose eight-lane groups each read one whole 128-byte line streams as fast as
// a plain linear read, while the natural MFMA pattern (sixteen rows, 64 bytes of each) is
// 25 % slower.  So W is not loaded in MFMA layout.  Each load
// instruction moves eight rows x 128 bytes straight into LDS (global_load_lds_dwordx4,
// non-temporal), and the MFMA operands are read back from LDS in fragment layout; a
// 16-byte XOR swizzle of the slot index (applied by permuting which global chunk a lane
// fetches, since the LDS position of a lane's data is fixed) keeps those reads free of
// bank conflicts.  A lone wave issues an instruction only every five to seven cycles, so
// every instruction between the wave's start and its first load, and between its last byte
// and its store, is time nothing overlaps: 128 scalar instructions in front of the loads of
// a bare streaming kernel cost 0.45 us per launch.  Hence the first loads go out after some
// thirty instructions, the kernel arguments they need arrive preloaded in scalar registers
// (the compile option -amdgpu-kernarg-preload-count), and the plain store path is a dozen
// instructions.
//
// The rows of W are split evenly over the CUs in steps of eight; a workgroup holds its
// rows as R groups of 16 (the last one possibly half empty) over the whole of K.  Its S
// wavefronts split K into S slices of T tiles of 256 nibbles; a wave issues every load
// of its slices before it waits for anything, multiplies each row group as soon as it has
// landed (loads complete in issue order, so that is a wait for a known number of younger
// loads) and adds its share to the group's block of sums in LDS without waiting for
// anything; the waves meet once, at the end, and store the blocks side by side.  Each wave
// fetches its own slice of X once and reuses it for its R row groups, so larger R cuts the
// (L2-resident, but hot-line) X traffic.  No workspace (the form split over K apart), no
// atomic operations on data, and the result does not depend on timing (integer additions
// commute).
#include "kernels.h"

#include <utility>

namespace int4linear {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

#define I4L_LDS(p) ((__attribute__((address_space(3))) void *)(p))

constexpr int kTileK = 256;                 // nibbles of K per tile
constexpr int kTileRowBytes = kTileK / 2;   // one 128-byte line per row
constexpr int kTileBytes = 16 * kTileRowBytes;  // 16 rows: 2 KiB
constexpr int kMaxLds = 160 * 1024;

// Loads address memory as a wave-uniform base (scalar registers) plus a per-lane 32-bit
// byte offset plus the compile-time constant IMM (0 .. 4095): one vector register per
// distinct lane pattern, whatever the number of loads made with it.
//
// 16 bytes per lane straight into LDS at lds_addr + 16*lane.  NT marks the weight stream
// as read-once.  The hardware adds the instruction's constant to the LDS address as well
// as to the memory address, so it is taken off the LDS base here.
template <bool NT, int IMM>
__device__ __forceinline__ void dma16(const void *base, unsigned lane_off, unsigned lds_addr)
{
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    lds_addr -= IMM;
    if (NT)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3 nt"
                     :
                     : "v"(lane_off), "s"(base), "s"(lds_addr), "n"(IMM)
                     : "memory");
    else
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                     :
                     : "v"(lane_off), "s"(base), "s"(lds_addr), "n"(IMM)
                     : "memory");
}

// The same with the LDS address given as a wave-uniform base plus the constant LDS_OFF: one
// scalar addition straight into M0 instead of a precomputed address per load.
template <bool NT, int IMM, int LDS_OFF>
__device__ __forceinline__ void dma16_at(const void *base, unsigned lane_off, unsigned lds_base)
{
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    static_assert(LDS_OFF - IMM >= 0, "the LDS base must not go below zero");
    if (NT)
        asm volatile("s_add_u32 m0, %2, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3 nt"
                     :
                     : "v"(lane_off), "s"(base), "s"(lds_base), "n"(IMM), "n"(LDS_OFF - IMM)
                     : "memory", "scc");
    else
        asm volatile("s_add_u32 m0, %2, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                     :
                     : "v"(lane_off), "s"(base), "s"(lds_base), "n"(IMM), "n"(LDS_OFF - IMM)
                     : "memory", "scc");
}

// A wave-uniform value the compiler may have chosen to compute on the vector side: back into
// scalar registers (the "s" operands of the load instructions need that).
__device__ __forceinline__ unsigned uniform(unsigned v) { return (unsigned)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ const uint8_t *uniform(const uint8_t *p)
{
    const unsigned long long v = (unsigned long long)p;
    return (const uint8_t *)((unsigned long long)uniform((unsigned)v) | ((unsigned long long)uniform((unsigned)(v >> 32)) << 32));
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    [&]<int... I>(std::integer_sequence<int, I...>) {
        (f(std::integral_constant<int, I>{}), ...);
    }(std::make_integer_sequence<int, N>{});
}

// LDS slot (16 bytes) of chunk c of tile row r: c ^ ((r >> 1) & MASK).  Rows are 128 B apart,
// so the sixteen lanes that read one chunk of rows 0..15 hit sixteen different 16-byte
// bank groups of the 256-byte bank window.  Which mask leaves a 16-byte read per lane free of
// bank conflicts depends on which chunks the four 16-lane groups of a wave read together
// (measured with a loop of such reads, cycles per read against 57 for a linear one): four
// neighbouring chunks of one tile (the plain fragment order) want mask 7 (57; mask 3: 61),
// chunks j and 4 + j of two tiles (the order that goes with the transposed X loads) want
// mask 3 (57; mask 7: 61).
template <int MASK = 7>
__device__ __forceinline__ int slot_swizzle(int r) { return (r >> 1) & MASK; }

// Waits until at most n of this wave's vector-memory operations are outstanding
// (they complete in issue order).  n is a compile-time constant at every call site after
// unrolling; s_waitcnt needs it as an immediate: vmcnt[3:0] in bits 3:0, vmcnt[5:4] in
// bits 15:14, the other counters left at "no wait".
template <int N>
__device__ __forceinline__ void wait_vm_imm()
{
    static_assert(N >= 0 && N <= 63, "vmcnt is six bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | (((N >> 4) & 0x3) << 14));
}

// 16 bytes per lane from global memory into registers, invisible to the compiler's own
// wait-count bookkeeping (which would otherwise wait for the younger weight loads too).
// The value is only valid after a wait_vm_imm that covers it and a settle().
template <int IMM>
__device__ __forceinline__ void load16_untracked(v4i &dst, const void *base, unsigned lane_off)
{
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(lane_off), "s"(base), "n"(IMM) : "memory");
}
__device__ __forceinline__ void settle(v4i &v) { asm volatile("" : "+v"(v)); }

// Transposes a 4 x 4 arrangement of 16-byte values inside every quad of lanes: on return
// r[t] of lane j (j = lane % 4) holds what r[j] of lane t of the same quad held.  Two
// exchange steps (lane distance 2, then 1), each a quad permutation and a select.
__device__ __forceinline__ void quad_transpose(v4i &r0, v4i &r1, v4i &r2, v4i &r3, int lane)
{
    const bool up2 = (lane & 2) != 0, up1 = (lane & 1) != 0;
    auto exchange = [](v4i &a, v4i &b, bool upper, auto ctrl) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int fa = __builtin_amdgcn_mov_dpp(a[c], decltype(ctrl)::value, 0xF, 0xF, true);
            const int fb = __builtin_amdgcn_mov_dpp(b[c], decltype(ctrl)::value, 0xF, 0xF, true);
            a[c] = upper ? fb : a[c];
            b[c] = upper ? b[c] : fa;
        }
    };
    exchange(r0, r2, up2, std::integral_constant<int, 0x4E>{});  // quad_perm [2,3,0,1]
    exchange(r1, r3, up2, std::integral_constant<int, 0x4E>{});
    exchange(r0, r1, up1, std::integral_constant<int, 0xB1>{});  // quad_perm [1,0,3,2]
    exchange(r2, r3, up1, std::integral_constant<int, 0xB1>{});
}

// Largest workgroup a variant is launched with.  The register-X variant with many
// fragments (2 * T * FMX of 16 bytes) and accumulators (R * FMX of 16 bytes) per lane
// needs the 256-register budget of at most eight waves per workgroup.
constexpr int max_threads(int t, int r, int fmx, bool xdma)
{
    return (!xdma && (t * fmx > 4 || (t * fmx == 4 && r * fmx >= 8))) ? 512 : 1024;
}

// LDS in front of the waves' tiles: one 16 x 16 block of sums (1 KiB) per pair (row group
// of W, row group of X).
constexpr int head_bytes(int r, int fmx) { return r * fmx * 1024; }

// T tiles per wave, R row groups per workgroup, FMX 16-row groups of X (M <= 16*FMX).
// XDMA: X tiles go through LDS like W; otherwise they are loaded into registers in
// fragment layout (for K so long that X tiles do not fit in LDS next to the W staging).
//
// A workgroup owns rows [blockIdx.x * rows_blk, + rows_blk) of W, rows_blk a multiple of 8
// and at most 16*R.  Every wave issues all its loads up front in the order first tile of W,
// X, rest of W; since loads complete in order, "row group rg, tile t has landed" is a wait
// for a fixed number of younger loads.  Each row group is multiplied and added to the
// group's sums as soon as it has landed, while the later groups are still in flight, so
// only the last group's share, the meeting and the stores are exposed after the last byte
// arrives.
//
// KSPLIT: the grid is (row blocks) x (2 or 4 slices of K, four as launched today); workgroup b takes row block
// b / slices and slice b % slices of K (an even split into whole tiles; workgroup ids go round
// the XCDs, so an XCD's workgroups share one or two slices of X), leaves its partial sums
// in `partial` and counts itself in at `arrivals`; the last of a row block's workgroups to
// arrive adds them up and stores (see the end of the function).
template <int T, int R, int FMX, bool XDMA, bool RAGGED, bool KSPLIT>
__device__ __forceinline__ void skinny_body(const uint8_t *X, const uint8_t *W, int32_t *Y, v4i dims, const Epilogue &ep_all,
                                            int *partial, unsigned *arrivals)
{
    static_assert(!(KSPLIT && RAGGED), "slices of K are whole numbers of tiles");
    // dims: { M | passes << 8 | S << 16 | plain << 24 | log2(slices of K) << 25, N, K, rows_blk } --
    // one argument instead of seven: the host's cost of a launch grows with the number of
    // arguments (0.1 us each), and these launches are short enough for that to show.  `plain`
    // says that ep_all is all zero, which the storing wave then knows without loading it.
    int M = dims[0] & 0xFF, passes = (dims[0] >> 8) & 0xFF;
    const int waves = (dims[0] >> 16) & 0xFF;
    const bool plain = (dims[0] >> 24) & 1;
    const int N = dims[1], K = dims[2], rows_blk = dims[3];
    const int kslices_log2 = KSPLIT ? (dims[0] >> 25) & 3 : 0;
    const int kslices = 1 << kslices_log2;
    const int kslice = KSPLIT ? (int)blockIdx.x & (kslices - 1) : 0;
    const int row_block = (int)blockIdx.x >> kslices_log2;
    // first tile of this workgroup's slice of K
    const int slice_tile0 = KSPLIT ? kslice * (K / kTileK / kslices) : 0;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int kWaveTiles = T * (R + (XDMA ? FMX : 0));
    constexpr int kHead = head_bytes(R, FMX);
    constexpr int kSwMask = (!XDMA && T % 2 == 0) ? 3 : 7;  // the slot swizzle that suits the form's fragment reads
    // Row groups of W whose loads are in flight ahead of the one being multiplied.  With one
    // row group of X a wave issues everything at once.  With more, a wave has X (16 * FMX
    // rows of its K slice) to fetch as well, the CU's queue of outstanding loads fills up, a
    // wave then sits in the issue of its later loads while its first row groups are waiting
    // in LDS, and all waves reach the ends of their chains of row groups together and late:
    // there the later groups are issued one at a time, each when the group before it has been
    // multiplied (64 x 14336 x 4096: 11.3 -> 10.7 us, with the rotation below 9.9 us).
    constexpr int kAhead = (FMX >= 2 && R > 1) ? 1 : R - 1;

    // ---- first of all, the wave's first two loads (tile 0 of row group 0, first pass).
    //      Nothing overlaps the time before a wave's first load, so these go out after as few
    //      instructions as it takes; the values everything else is computed from pass through
    //      an empty asm statement afterwards, which keeps the compiler from moving that work
    //      up here.
    int lane = threadIdx.x & 63;
    int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned rowbytes = (unsigned)K >> 1;
    int n0 = row_block * rows_blk;
    int rows_here = min(rows_blk, N - n0);  // >= 1
    const unsigned lds_base = (unsigned)(size_t)I4L_LDS(lds);
    {
        // Lane p of a direct-to-LDS instruction lands at 16*p: tile row p/8 (+8 for the second
        // instruction of a tile), slot p%8, so it fetches chunk slot ^ swizzle.
        const unsigned lrow = (unsigned)lane >> 3, c8 = (unsigned)lane & 7;
        const unsigned g0 = 16u * (wave & (R - 1));  // the wave's first row group (see `rot`)
        const unsigned lim = (unsigned)(rows_here - 1);
        const int skip0 = RAGGED ? max(0, (wave + 1) * T - K / kTileK) : 0;
        const uint8_t *base = W + (size_t)n0 * rowbytes + (size_t)(slice_tile0 + wave * T - skip0) * kTileRowBytes;
        const unsigned first_lds = lds_base + kHead + wave * kWaveTiles * kTileBytes;
        dma16_at<true, 0, 0>(base, (unsigned)__umul24(min(g0 + lrow, lim), rowbytes) + ((c8 ^ ((lrow >> 1) & kSwMask)) << 4), first_lds);
        dma16_at<true, 0, 1024>(base, (unsigned)__umul24(min(g0 + lrow + 8, lim), rowbytes) + ((c8 ^ ((4 + (lrow >> 1)) & kSwMask)) << 4),
                                first_lds);
    }
    asm volatile("" : "+v"(lane), "+s"(wave), "+s"(rowbytes), "+s"(n0), "+s"(rows_here), "+s"(M), "+s"(passes));

    const unsigned my_lds = uniform(lds_base + kHead + wave * kWaveTiles * kTileBytes);
    // Waves take the row groups in different orders: wave w keeps group (i + w) mod R in its
    // i-th tiles (measured: nothing at up to 16 rows of X, 3 % with more).
    const int rot = wave & (R - 1);
    const int himask = (int)0xF0F0F0F0u;
    const uint8_t *mine = lds + kHead + wave * kWaveTiles * kTileBytes;
    int *const sums = (int *)lds;

    // Fragment layout: lane l supplies row l%16 and, in step s of a tile, chunk
    // 4*s + l/16 (32 nibbles: even ones feed one MFMA, odd ones the next).
    const int fr = lane & 15;
    const int fg = lane >> 4;
    const int sw = slot_swizzle<kSwMask>(fr);

    // With X in registers and an even T the X loads are made in a form the memory pipeline
    // takes at full rate (every quad of lanes reads 64 contiguous bytes of one row; the
    // fragment form, in which neighbouring lanes read different rows, is served at less
    // than a third of that) and turned into fragments by a transposition inside the quads.
    // Over a pair of tiles (256 bytes of a row, chunks 0..15) register j of the pair then
    // holds, for lane (fr, fg), chunk 4 * fg + j of row fr, and W is read from LDS to match.
    constexpr bool kPairX = !XDMA && T % 2 == 0;
    v4i xg[XDMA ? 1 : T][2][FMX];

    // K longer than S * T tiles is covered in several passes: pass c takes the c-th run of
    // S * T tiles, each wave refills its own LDS tiles (nobody else reads them, and its own
    // reads of the previous pass have been consumed).
    int skip = 0;
#pragma unroll 1
    for (int pass = 0; pass < passes; ++pass) {
    {
    // ---- loads.  Rows past the workgroup's (or the matrix's) end re-read the last valid
    //      row: every wave issues the same number of loads, which the waits below rely on,
    //      and nothing is read out of bounds.
    // (The offsets are derived anew in every pass from a copy of the lane number that the
    // compiler cannot see through: kept across the multiplication they would cost registers
    // there.)
    int lane_here = lane;
    asm volatile("" : "+v"(lane_here));
    const unsigned lrow = (unsigned)lane_here >> 3;
    const unsigned c8 = (unsigned)lane_here & 7;
    const unsigned chunk[2] = {(c8 ^ ((lrow >> 1) & kSwMask)) << 4, (c8 ^ ((4 + (lrow >> 1)) & kSwMask)) << 4};
    // This wave's slice of every row: T tiles from tile (pass * S + wave) * T on.  When
    // K's tiles do not fill the last slices, a slice that would run past the end is
    // moved back to end with the last tile, and its first `skip` tiles (someone else's,
    // or all T of them) are loaded like the others but not multiplied.
    const int first_tile = slice_tile0 + (pass * waves + wave) * T;
    if (RAGGED)
        skip = max(0, first_tile + T - K / kTileK);
    const size_t kbyte0 = (size_t)(first_tile - skip) * kTileRowBytes;
    const uint8_t *wbase = uniform(W + (size_t)n0 * rowbytes + kbyte0);
    unsigned w_off[R][2];
#pragma unroll
    for (int rg = 0; rg < R; ++rg)
#pragma unroll
        for (int u = 0; u < 2; ++u)
            w_off[rg][u] = (unsigned)__umul24(min(16 * ((rg + rot) & (R - 1)) + lrow + 8 * u, (unsigned)(rows_here - 1)), rowbytes) + chunk[u];
    auto issue_w = [&](auto rgc, auto first, auto count) {  // tiles first .. first + count - 1 of the rg-th group
        constexpr int rg = decltype(rgc)::value;
        static_for<count()>([&](auto i) {
            constexpr int t = first() + i();
            dma16_at<true, t * kTileRowBytes, (rg * T + t) * kTileBytes>(wbase, w_off[rg][0], my_lds);
            dma16_at<true, t * kTileRowBytes, (rg * T + t) * kTileBytes + 1024>(wbase, w_off[rg][1], my_lds);
        });
    };
    constexpr std::integral_constant<int, 0> kZero{};
    constexpr std::integral_constant<int, 1> kOne{};
    constexpr std::integral_constant<int, T - 1> kRestOfGroup{};
    constexpr std::integral_constant<int, T> kAllTiles{};
    // Issue order: the first tile of W (in the first pass it is on its way already), X, the
    // rest of W.
    if (pass > 0)
        issue_w(kZero, kZero, kOne);
    // With the first loads on their way: the sums start at zero, which everybody has to have
    // seen before anybody adds to them.  (Meeting here, where every wave is about to wait for
    // memory anyway, measured better than meeting in front of the first addition.)
    if (pass == 0) {
        for (int i = threadIdx.x; i < R * FMX * 256; i += waves * 64)
            sums[i] = 0;
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
    // X: through LDS like W (two loads per tile); as fragments (row fr, 64 bytes of a tile
    // per load); or in the paired form, where load j of a tile pair has quad q read row
    // 4 * (q % 4) + j, bytes 64 * (q / 4) .. + 64 of the pair.
    {
        const uint8_t *xbase = uniform(X + kbyte0);
        constexpr int kXPatterns = XDMA ? 2 : kPairX ? 4 : 1;
#pragma unroll
        for (int f = 0; f < FMX; ++f) {
            unsigned x_off[kXPatterns];
#pragma unroll
            for (int j = 0; j < kXPatterns; ++j) {
                const unsigned q = (unsigned)lane_here >> 2;
                const unsigned xr = f * 16 + (XDMA ? lrow + 8 * j : kPairX ? 4 * (q & 3) + j : ((unsigned)lane_here & 15));
                const unsigned within = XDMA ? chunk[j & 1] : kPairX ? 64 * (q >> 2) + 16 * ((unsigned)lane_here & 3)
                                                                     : ((unsigned)lane_here >> 4) * 16;
                x_off[j] = (unsigned)__umul24(min(xr, (unsigned)(M - 1)), rowbytes) + within;
            }
            if constexpr (XDMA) {
                static_for<T>([&](auto t) {
                    dma16_at<false, t() * kTileRowBytes, (R * T + t()) * kTileBytes>(xbase, x_off[0], my_lds + f * T * kTileBytes);
                    dma16_at<false, t() * kTileRowBytes, (R * T + t()) * kTileBytes + 1024>(xbase, x_off[1],
                                                                                              my_lds + f * T * kTileBytes);
                });
            } else if constexpr (kPairX) {
                static_for<2 * T>([&](auto j) {
                    load16_untracked<(j() >> 2) * 2 * kTileRowBytes>(xg[XDMA ? 0 : j() >> 1][j() & 1][f], xbase, x_off[j() & 3]);
                });
            } else {
                static_for<2 * T>([&](auto j) {  // tile j / 2, step j % 2
                    load16_untracked<(j() >> 1) * kTileRowBytes + (j() & 1) * 64>(xg[XDMA ? 0 : j() >> 1][j() & 1][f], xbase, x_off[0]);
                });
            }
        }
    }
    if constexpr (T > 1)
        issue_w(kZero, kOne, kRestOfGroup);
    static_for<kAhead>([&](auto g) { issue_w(std::integral_constant<int, decltype(g)::value + 1>{}, kZero, kAllTiles); });
    }

    // Waits until tile t of the wave's i-th row group has landed: loads complete in issue
    // order, so that is a wait for a fixed number of younger loads (the rest of this group and
    // the groups issued ahead of it), which s_waitcnt takes as a constant: hence the switch.
    // X sits right behind the first tile of W, so that tile's wait covers X too.  (A store of
    // this wave that is still on its way counts like a load: the wait then lasts one load
    // longer than needed.)
    auto wait_tile = [&](int i, auto tc) {
        constexpr int kRest = (T - 1 - decltype(tc)::value) * 2;  // of the tile's own group
        switch (min(kAhead, R - 1 - i)) {  // younger groups in flight
        case 3:
            wait_vm_imm<(kAhead >= 3 ? 3 : 0) * T * 2 + kRest>();
            break;
        case 2:
            wait_vm_imm<(kAhead >= 2 ? 2 : 0) * T * 2 + kRest>();
            break;
        case 1:
            wait_vm_imm<(kAhead >= 1 ? 1 : 0) * T * 2 + kRest>();
            break;
        default:
            wait_vm_imm<kRest>();
            break;
        }
    };
    // All tiles of the wave's i-th row group, i wave-uniform but not a constant.
    auto issue_w_dyn = [&](int i) {
        int lane_here = lane;
        asm volatile("" : "+v"(lane_here));
        const unsigned lrow = (unsigned)lane_here >> 3;
        const unsigned c8 = (unsigned)lane_here & 7;
        const int first_tile = slice_tile0 + (pass * waves + wave) * T;
        const uint8_t *wbase = uniform(W + (size_t)n0 * rowbytes + (size_t)(first_tile - skip) * kTileRowBytes);
        const unsigned g = 16 * ((i + rot) & (R - 1));
        const unsigned off0 = (unsigned)__umul24(min(g + lrow, (unsigned)(rows_here - 1)), rowbytes) + ((c8 ^ ((lrow >> 1) & kSwMask)) << 4);
        const unsigned off1 = (unsigned)__umul24(min(g + lrow + 8, (unsigned)(rows_here - 1)), rowbytes) +
                              ((c8 ^ ((4 + (lrow >> 1)) & kSwMask)) << 4);
        const unsigned grp_lds = uniform(my_lds + i * T * kTileBytes);
        static_for<T>([&](auto t) {
            dma16_at<true, t() * kTileRowBytes, t() * kTileBytes>(wbase, off0, grp_lds);
            dma16_at<true, t() * kTileRowBytes, t() * kTileBytes + 1024>(wbase, off1, grp_lds);
        });
    };

    if constexpr (!XDMA) {
        // X has landed when the first tile of W has: the fragments are formed
        wait_tile(0, std::integral_constant<int, 0>{});
#pragma unroll
        for (int f = 0; f < FMX; ++f)
#pragma unroll
            for (int tp = 0; tp < (XDMA ? 1 : T) / (kPairX ? 2 : 1); ++tp) {
                constexpr int kTilesHere = kPairX ? 2 : 1;
#pragma unroll
                for (int h = 0; h < 2 * kTilesHere; ++h)
                    settle(xg[kTilesHere * tp + (h >> 1)][h & 1][f]);
                if constexpr (kPairX)
                    quad_transpose(xg[XDMA ? 0 : 2 * tp][0][f], xg[XDMA ? 0 : 2 * tp][1][f],
                                   xg[XDMA ? 0 : 2 * tp + 1][0][f], xg[XDMA ? 0 : 2 * tp + 1][1][f], lane);
            }
    }

    // With several row groups of W and of X, X is widened once per pass where the registers
    // allow it (16 per tile and row group of X) instead of once per row group of W.
    constexpr bool kWideX = R > 1 && FMX > 1 && (T * FMX <= 4 || (max_threads(T, R, FMX, XDMA) == 512 && T * FMX <= 8));
    v4i xw[kWideX ? T : 1][2][kWideX ? FMX : 1][2];
    if constexpr (kWideX) {
        if constexpr (XDMA)
            wait_tile(0, std::integral_constant<int, 0>{});  // X sits right behind the first tile of W
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                for (int f = 0; f < FMX; ++f) {
                    const int frag = fr * kTileRowBytes + (((4 * s2 + fg) ^ sw) * 16);
                    const v4i x = XDMA ? *(const v4i *)(mine + ((R + f) * T + t) * kTileBytes + frag) : xg[XDMA ? 0 : t][s2][f];
                    xw[t][s2][f][0] = (x << 4) & himask;
                    xw[t][s2][f][1] = x & himask;
                }
    }

    // ---- one row group at a time, in a loop (not unrolled): every group after the first runs
    //      code that is already in the instruction cache, which matters for the last one --
    //      nothing overlaps it.
#pragma unroll 1
    for (int slot = 0; slot < R; ++slot) {
        const int rg = (slot + rot) & (R - 1);  // the row group in the wave's slot-th tiles
        if constexpr (kAhead < R - 1)
            if (slot >= 1 && slot + kAhead < R)
                issue_w_dyn(slot + kAhead);
        v4i acc[FMX];
#pragma unroll
        for (int f = 0; f < FMX; ++f)
            acc[f] = (v4i){0, 0, 0, 0};
        const uint8_t *group = mine + slot * T * kTileBytes;
        static_for<T>([&](auto tc) {
            constexpr int t = decltype(tc)::value;
            wait_tile(slot, tc);
            // In the paired form a pair of tiles is multiplied when its second tile has
            // landed: step s of tile t is register j = 2 * (t % 2) + s of the pair, whose
            // chunk 4 * fg + j lies in tile fg / 2 of the pair.
            if constexpr (!(kPairX && t % 2 == 0)) {
#pragma unroll
                for (int tq = (kPairX ? t - 1 : t); tq <= t; ++tq)
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        // Tiles before `skip` are not this wave's.  In the paired form every
                        // register spans both tiles of the pair (lanes with fg < 2 hold the
                        // first one): the pair is left out if its second tile is, and only
                        // the first tile's lanes are blanked if just that one is.
                        if (RAGGED && (kPairX ? t : tq) < skip)
                            continue;
                        const bool blank_first = RAGGED && kPairX && t - 1 < skip;
                        const int j = 2 * (tq & 1) + s;
                        const int frag = fr * kTileRowBytes + (((4 * s + fg) ^ sw) * 16);
                        const int off = kPairX ? ((t - 1) + (fg >> 1)) * kTileBytes + fr * kTileRowBytes +
                                                     (((4 * (fg & 1) + j) ^ sw) * 16)
                                               : t * kTileBytes + frag;
                        v4i w = *(const v4i *)(group + off);
                        if (blank_first && fg < 2)
                            w = (v4i){0, 0, 0, 0};
                        const v4i wlo = (w << 4) & himask;
                        const v4i whi = w & himask;
#pragma unroll
                        for (int f = 0; f < FMX; ++f) {
                            if constexpr (kWideX) {
                                acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, xw[tq][s][f][0], acc[f], 0, 0, 0);
                                acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, xw[tq][s][f][1], acc[f], 0, 0, 0);
                            } else {
                                const v4i x = XDMA ? *(const v4i *)(mine + ((R + f) * T + t) * kTileBytes + frag)
                                                   : xg[XDMA ? 0 : tq][s][f];
                                acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, (x << 4) & himask, acc[f], 0, 0, 0);
                                acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, x & himask, acc[f], 0, 0, 0);
                            }
                        }
                    }
            }
        });

        // Lane (fr, fg) holds Y[m = fr][n = 4 * fg ..+4) of each of the group's FMX blocks; its
        // element q is added to word 64 * q + lane of the block in LDS, so neither these
        // additions nor the reads of the storing wave meet a bank conflict.  Both operands
        // carried a factor 16, so every product, and with it every wave's share, is a multiple
        // of 256: the shift happens here, where all waves do it side by side, not in the
        // storing wave.
        int *const block = sums + rg * FMX * 256 + lane;
#pragma unroll
        for (int f = 0; f < FMX; ++f)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                __hip_atomic_fetch_add(block + f * 256 + q * 64, acc[f][q] >> 8, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    }  // passes

    // ---- everybody's shares are in after one meeting; the R * FMX blocks are then stored by
    //      as many waves, side by side.  (An arrival counter per row group, ds_append returning
    //      its old value, with the last wave to arrive storing the group while the others were
    //      still multiplying, was 4 % slower with several row groups and no faster with one:
    //      every wave then waits for the counter's old value after every group.)
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const int om = lane >> 2, oj = lane & 3;  // this lane stores Y[om][4 * oj ..+4) of a block
    // A wave's blocks are j = wave, wave + waves, ...; `sum_of(i, j)` is the i-th of them,
    // complete.  Unsplit: read from LDS.  Split over K: read back from all slices' slabs.
    constexpr int kBlocks = R * FMX;
    constexpr int kMine = KSPLIT ? (kBlocks + 3) / 4 : 1;  // blocks per wave when split (at least four waves: the host checks)
    v4i gathered[kMine];
    if constexpr (KSPLIT) {
        // The exchange.  Slab (row block, slice) of `partial` holds the workgroup's kBlocks
        // blocks of 256 sums, a lane's four as two 64-bit words at 64 * h + lane of the block.
        // The stores and the loads are relaxed atomic operations at device scope, which on
        // this device are plain accesses that go through to (come from) the level all
        // workgroups share; the stores have been acknowledged before the wave counts itself
        // in, so whoever sees the last increment of a counter finds every slice's slab.  The
        // counter is that of (row block, wave): the waves with one number hold the same blocks
        // in every slice's workgroup, so the last of them to arrive adds those blocks up and
        // stores them, and puts the counter back to zero for the next launch.  Nobody waits
        // for anybody; integer sums do not depend on who arrives when.  All of a wave's
        // operations of a kind go out together: a trip to memory costs far more than they do.
        // (Release and acquire fences at device scope in place of the wait would say the same
        // in the language's terms, but on this device they write back and invalidate the whole
        // L2 of the XCD: measured 28 instead of 13 us for 64 x 4096 x 14336.)
        typedef unsigned long long u64;
        u64 *const slabs = (u64 *)partial + (size_t)row_block * kslices * kBlocks * 128 + lane;
        u64 *const mine_at = slabs + (size_t)kslice * kBlocks * 128;
#pragma unroll
        for (int i = 0; i < kMine; ++i) {
            const int j = wave + i * waves;
            if (j < kBlocks) {
                const int *mine_of = sums + j * 256 + 16 * oj + om;
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    __hip_atomic_store(mine_at + j * 128 + 64 * h,
                                       (u64)(unsigned)mine_of[128 * h] | ((u64)(unsigned)mine_of[128 * h + 64] << 32), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        unsigned *const counter = arrivals + row_block * waves + wave;
        unsigned before = 0;
        if (lane == 0)
            before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        before = uniform(before);
        if (before != (unsigned)(kslices - 1))
            return;
        if (lane == 0)
            __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        u64 got[kMine][4][2];
#pragma unroll
        for (int i = 0; i < kMine; ++i)
#pragma unroll
            for (int p = 0; p < 4; ++p)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int j = wave + i * waves;
                    got[i][p][h] = (j < kBlocks && p < kslices)
                                       ? __hip_atomic_load(slabs + ((size_t)p * kBlocks + j) * 128 + 64 * h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                       : 0ull;
                }
#pragma unroll
        for (int i = 0; i < kMine; ++i) {
            gathered[i] = (v4i){0, 0, 0, 0};
#pragma unroll
            for (int p = 0; p < 4; ++p)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    gathered[i][2 * h] += (int)(unsigned)got[i][p][h];
                    gathered[i][2 * h + 1] += (int)(unsigned)(got[i][p][h] >> 32);
                }
        }
    }
    auto sum_of = [&](int i, int j) -> v4i {
        if constexpr (KSPLIT) {
            return gathered[i];
        } else {
            const int *mine_of = sums + j * 256 + 16 * oj + om;
            return (v4i){mine_of[0], mine_of[64], mine_of[128], mine_of[192]};
        }
    };
    // f(i, j) for each of the wave's blocks; unrolled when split (the sums are in registers).
    auto for_my_blocks = [&](auto &&f) {
        if constexpr (KSPLIT) {
#pragma unroll
            for (int i = 0; i < kMine; ++i)
                if (wave + i * waves < kBlocks)
                    f(i, wave + i * waves);
        } else {
#pragma unroll 1
            for (int j = wave; j < kBlocks; j += waves)
                f(0, j);
        }
    };
    if (plain && ((N | rows_here) & 3) == 0) {
        // Nothing to load or to convert, and a lane's four outputs exist together or not at
        // all: the path that ends the kernel in the common case, kept to a few instructions.
        for_my_blocks([&](int i, int j) {  // block j: row group j / FMX of W, j % FMX of X
            const int rg = j / FMX, f = j % FMX;
            const v4i sum = sum_of(i, j);
            if (f * 16 + om < M && rg * 16 + 4 * oj < rows_here)
                *(v4i *)(Y + (size_t)(f * 16 + om) * N + n0 + rg * 16 + 4 * oj) = sum;
        });
        return;
    }
    // (the epilogue's operands are first looked at here, not ahead of the loads)
    Epilogue ep = ep_all;
    asm volatile("" : "+s"(ep.bias), "+s"(ep.row_scale), "+s"(ep.col_scale), "+s"(ep.out));
    for_my_blocks([&](int i, int j) {
        const int rg = j / FMX, f = j % FMX;
        v4i sum = sum_of(i, j);
        const int m = f * 16 + om;
        const int nb = rg * 16 + 4 * oj;  // within the workgroup's rows
        if (m < M) {
            const float rs = ep.row_scale ? ep.row_scale[m] : 1.f;
            by_output_width(ep, [&](auto half) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nn = n0 + (nb + q < rows_here ? nb + q : rows_here - 1);
                    sum[q] = epilogue_value_of<half()>(ep, sum[q], ep.bias ? ep.bias[nn] : 0, rs, ep.col_scale ? ep.col_scale[nn] : 1.f);
                }
                store_out4<half()>(Y, (size_t)m * N + n0 + nb, sum, rows_here - nb, nb + 3 < rows_here && ((N | n0) & 3) == 0);
            });
        }
    });
}

template <int T, int R, int FMX, bool XDMA, bool RAGGED>
__global__ __launch_bounds__(max_threads(T, R, FMX, XDMA)) void skinny_kernel(const uint8_t *X, const uint8_t *W, int32_t *Y,
                                                                              v4i dims, Epilogue ep_all)
{
    skinny_body<T, R, FMX, XDMA, RAGGED, false>(X, W, Y, dims, ep_all, nullptr, nullptr);
}

template <int T, int R, int FMX, bool XDMA>
__global__ __launch_bounds__(max_threads(T, R, FMX, XDMA)) void skinny_ksplit_kernel(const uint8_t *X, const uint8_t *W, int32_t *Y,
                                                                                     v4i dims, Epilogue ep_all, int *partial,
                                                                                     unsigned *arrivals)
{
    skinny_body<T, R, FMX, XDMA, false, true>(X, W, Y, dims, ep_all, partial, arrivals);
}

// ---- long-W form: many 16-row groups of W per CU, FMX 16-row groups of X.
//
// One workgroup per CU stays there and walks its groups.  Wave w owns the k range of tiles
// [w * TW, (w + 1) * TW) of every row: its slice of X sits in registers for the whole
// kernel, and its tiles of W pass through a ring of NBUF wave-private LDS tiles, so the
// waves need no barrier to stream (a tile is refilled by the wave that has just consumed
// it) and the stream never stops between groups.  A step is one tile of one group: wait
// for it (loads complete in order: NBUF - 2 younger steps stay in flight), read its two
// fragments, issue the load of step + NBUF - 1 into the tile consumed one step earlier,
// multiply.  After the last tile of a group a wave adds its share to the group's block of
// sums in LDS and goes on; the waves meet once per epoch of four groups, and the epoch's
// blocks are then stored and cleared by as many waves as there are blocks (they take
// turns) while the others go on.  (One meeting per group, with one wave adding up
// everybody's partial sums, cost a tenth of the kernel at 128256 rows of W, and more with
// several row groups of X: 64 x 128256 x 4096 68 -> 60 us.)  The loads stop with the last
// tile; the waits of the last NBUF - 2 steps count down accordingly.  (Reloading the last
// group into tiles nobody reads, which keeps every wait count the same, cost 3 % to 6 %:
// with seven groups per CU those reloads are a fifth of all loads.)
constexpr int kStreamEpoch = 4;  // groups between two meetings of the waves
constexpr int stream_head_bytes(int fmx) { return 2 * kStreamEpoch * fmx * 1024; }

template <int TW, int NBUF, int FMX>
__global__ __launch_bounds__(FMX == 1 ? 1024 : 512) void skinny_stream_kernel(const uint8_t *__restrict__ X,
                                                            const uint8_t *__restrict__ W,
                                                            int32_t *__restrict__ Y, int M, int N, int K,
                                                            int groups_per_block, Epilogue ep)
{
    static_assert(NBUF >= 3 && (NBUF & (NBUF - 1)) == 0, "ring positions wrap by masking");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int rowbytes = K >> 1;
    const int groups_total = (N + 15) >> 4;
    const int g_begin = blockIdx.x * groups_per_block;  // < groups_total by the grid's size
    const int g_end = min(groups_total, g_begin + groups_per_block);
    const int fr = lane & 15, fg = lane >> 4, sw = slot_swizzle(fr);
    const int himask = (int)0xF0F0F0F0u;
    // LDS: two sets (for alternate epochs) of one 16 x 16 block of sums per (group of the
    // epoch, row group of X), then the waves' rings.
    constexpr int kHead = stream_head_bytes(FMX);
    const unsigned ring_lds = (unsigned)(size_t)I4L_LDS(lds) + kHead + wave * NBUF * kTileBytes;
    const uint8_t *ring = lds + kHead + wave * NBUF * kTileBytes;
    int *const sums = (int *)lds;

    // X fragments: packed as loaded and widened at every use, or, where the 256 registers of
    // the eight-wave form have room for it, widened once (several row groups of X make the
    // widening the bottleneck otherwise).
    constexpr bool kKeepWide = FMX > 1 && TW * FMX <= 8;
    v4i xg[TW][2][FMX];
    v4i xw[kKeepWide ? TW : 1][2][kKeepWide ? FMX : 1][2];

    // W: step (group, tile c) lands in ring position `pos`.
    const uint8_t *wbase = W + (size_t)wave * TW * kTileRowBytes;
    const int lrow = lane >> 3;
    unsigned chunk[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
        chunk[u] = ((lane & 7) ^ slot_swizzle(lrow + 8 * u)) * 16;
    auto issue = [&](int g, auto c, unsigned pos) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int row = min(16 * g + lrow + 8 * u, N - 1);
            // (the tile's offset goes into the scalar base, not into the instruction: the ring
            // position is unrelated to it, and the LDS base must not go below zero)
            dma16<true, 0>(wbase + c() * kTileRowBytes, (unsigned)row * rowbytes + chunk[u], ring_lds + pos * kTileBytes + u * 1024);
        }
    };
    // The first step of W goes out ahead of X, so that the weight stream starts at once; the
    // first wait of the loop (all but NBUF - 2 steps landed) then covers X as well.
    int left = (g_end - g_begin) * TW - 1;  // steps after the current one
    static_for<NBUF - 1>([&](auto j) {
        if (j() <= left)
            issue(g_begin + j() / TW, std::integral_constant<int, j() % TW>{}, (unsigned)j());
        if constexpr (j() == 0) {
            // X: fragment form, once.
            const uint8_t *xbase = X + (size_t)wave * TW * kTileRowBytes;
#pragma unroll
            for (int f = 0; f < FMX; ++f) {
                const int xr = 16 * f + fr;
                const unsigned x_off = (unsigned)(xr < M ? xr : M - 1) * rowbytes + fg * 16;
                static_for<2 * TW>([&](auto q) {
                    load16_untracked<(q() >> 1) * kTileRowBytes + (q() & 1) * 64>(xg[q() >> 1][q() & 1][f], xbase, x_off);
                });
            }
        }
    });

    // With the first loads on their way: the sums start at zero, which everybody has to have
    // seen before anybody adds to them.
    for (int i = threadIdx.x; i < 2 * kStreamEpoch * FMX * 256; i += waves * 64)
        sums[i] = 0;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    v4i acc[FMX];
#pragma unroll
    for (int f = 0; f < FMX; ++f)
        acc[f] = (v4i){0, 0, 0, 0};
    unsigned pos = 0;  // ring position of the current step
    int turn = 0;      // the wave that takes the first block of the current epoch
#pragma unroll 1
    for (int g = g_begin; g < g_end; ++g) {
        // (the shift count and mask are hidden from the optimiser in every group: widened
        // once outside the loop, X would take three times the registers)
        int shift = 4, mask = himask;
        asm volatile("" : "+s"(shift), "+s"(mask));
        static_for<TW>([&](auto c) {
            // all but the younger steps in flight have landed: NBUF - 2 of them, fewer at the end
            if (left >= NBUF - 2) {
                wait_vm_imm<2 * (NBUF - 2)>();
            } else {
                switch (left) {
                case 0:
                    wait_vm_imm<0>();
                    break;
                case 1:
                    wait_vm_imm<2>();
                    break;
                case 2:
                    wait_vm_imm<NBUF >= 5 ? 4 : 0>();
                    break;
                case 3:
                    wait_vm_imm<NBUF >= 6 ? 6 : 0>();
                    break;
                case 4:
                    wait_vm_imm<NBUF >= 7 ? 8 : 0>();
                    break;
                default:
                    wait_vm_imm<NBUF >= 8 ? 10 : 0>();
                    break;
                }
            }
            if constexpr (c() == 0) {
                // (needed once, after the first wait; it costs nothing to say it per group)
#pragma unroll
                for (int cc = 0; cc < TW; ++cc)
#pragma unroll
                    for (int s = 0; s < 2; ++s)
#pragma unroll
                        for (int f = 0; f < FMX; ++f)
                            settle(xg[cc][s][f]);
                if constexpr (kKeepWide) {
                    if (g == g_begin) {
#pragma unroll
                        for (int cc = 0; cc < TW; ++cc)
#pragma unroll
                            for (int s = 0; s < 2; ++s)
#pragma unroll
                                for (int f = 0; f < FMX; ++f) {
                                    xw[cc][s][f][0] = (xg[cc][s][f] << 4) & himask;
                                    xw[cc][s][f][1] = xg[cc][s][f] & himask;
                                }
                    }
                }
            }
            v4i w[2];
#pragma unroll
            for (int s = 0; s < 2; ++s)
                w[s] = *(const v4i *)(ring + pos * kTileBytes + fr * kTileRowBytes + (((4 * s + fg) ^ sw) * 16));
            constexpr int ahead = c() + NBUF - 1;
            if (left >= NBUF - 1)
                issue(g + ahead / TW, std::integral_constant<int, ahead % TW>{}, (pos + NBUF - 1) & (NBUF - 1));
            --left;
            pos = (pos + 1) & (NBUF - 1);
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const v4i wlo = (w[s] << 4) & himask, whi = w[s] & himask;
#pragma unroll
                for (int f = 0; f < FMX; ++f) {
                    if constexpr (kKeepWide) {
                        acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, xw[c()][s][f][0], acc[f], 0, 0, 0);
                        acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, xw[c()][s][f][1], acc[f], 0, 0, 0);
                    } else {
                        const v4i x = xg[c()][s][f];
                        acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, (x << shift) & mask, acc[f], 0, 0, 0);
                        acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, x & mask, acc[f], 0, 0, 0);
                    }
                }
            }
        });
        // The wave adds its share to the group's blocks of sums (every product carries the
        // factor 256, so the shift happens here; element q of a lane at word 64 * q + lane: no
        // bank conflicts) and goes on without waiting.  Once per epoch of kStreamEpoch groups
        // the waves meet; the epoch's blocks are complete then and are stored and cleared by
        // as many waves as there are blocks, side by side, while the stream goes on.  The next
        // epoch adds into the other set of blocks, so a set is used again only after the
        // meeting that follows its clearing.
        const int e = (g - g_begin) & (kStreamEpoch - 1);
        const int set = ((g - g_begin) / kStreamEpoch) & 1;
        int *const epoch_blocks = sums + set * kStreamEpoch * FMX * 256;
        int *const block = epoch_blocks + e * FMX * 256;
#pragma unroll
        for (int f = 0; f < FMX; ++f) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                __hip_atomic_fetch_add(block + f * 256 + q * 64 + lane, acc[f][q] >> 8, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_WORKGROUP);
            acc[f] = (v4i){0, 0, 0, 0};
        }
        if (e == kStreamEpoch - 1 || g + 1 == g_end) {
            __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const int om = lane >> 2, oj = lane & 3;  // this lane stores Y[om][4 * oj ..+4) of a block
            // block j of the epoch: group g - e + j / FMX, row group j % FMX of X; the waves take
            // them in turn, starting with a different wave every epoch
            int first = wave - turn;
            if (first < 0)
                first += waves;
#pragma unroll 1
            for (int j = first; j < (e + 1) * FMX; j += waves) {
                const int f = j % FMX, gj = g - e + j / FMX;
                int *const mine_of = epoch_blocks + j * 256 + 16 * oj + om;
                v4i sum = {mine_of[0], mine_of[64], mine_of[128], mine_of[192]};
                mine_of[0] = 0;
                mine_of[64] = 0;
                mine_of[128] = 0;
                mine_of[192] = 0;
                const int m = 16 * f + om, n = 16 * gj + 4 * oj;
                if (m < M) {
                    const float rs = ep.row_scale ? ep.row_scale[m] : 1.f;
                    by_output_width(ep, [&](auto half) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int nn = n + q < N ? n + q : N - 1;
                            sum[q] = epilogue_value_of<half()>(ep, sum[q], ep.bias ? ep.bias[nn] : 0, rs,
                                                               ep.col_scale ? ep.col_scale[nn] : 1.f);
                        }
                        store_out4<half()>(Y, (size_t)m * N + n, sum, N - n, n + 3 < N && (N & 3) == 0);
                    });
                }
            }
            turn = (turn + kStreamEpoch * FMX) % waves;
        }
    }
}

// ---- fallback for K that is a multiple of 128 but does not split into tiles: the
//      straightforward version (fragment-layout global loads, 128 nibbles per step).
template <int FMX, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void skinny_basic_kernel(
    const uint8_t *__restrict__ X, const uint8_t *__restrict__ W, int32_t *__restrict__ Y,
    int M, int N, int K, Epilogue ep)
{
    __shared__ v4i partial[WAVES][FMX][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int fr = lane & 15;
    const int fg = lane >> 4;
    const int rowbytes = K >> 1;
    const int KT = K / 128;
    const int n0 = blockIdx.x * 16;
    const int wrow = (n0 + fr < N) ? n0 + fr : N - 1;
    const uint8_t *wp = W + (size_t)wrow * rowbytes + fg * 16;
    const uint8_t *xp[FMX];
#pragma unroll
    for (int f = 0; f < FMX; ++f) {
        const int xrow = (f * 16 + fr < M) ? f * 16 + fr : M - 1;
        xp[f] = X + (size_t)xrow * rowbytes + fg * 16;
    }
    const int himask = (int)0xF0F0F0F0u;
    v4i acc[FMX];
#pragma unroll
    for (int f = 0; f < FMX; ++f)
        acc[f] = (v4i){0, 0, 0, 0};
    for (int ks = wave; ks < KT; ks += WAVES) {
        const size_t off = (size_t)ks * 64;
        const v4i w = __builtin_nontemporal_load((const v4i *)(wp + off));
        const v4i wlo = (w << 4) & himask;
        const v4i whi = w & himask;
#pragma unroll
        for (int f = 0; f < FMX; ++f) {
            const v4i x = *(const v4i *)(xp[f] + off);
            acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, (x << 4) & himask, acc[f], 0, 0, 0);
            acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, x & himask, acc[f], 0, 0, 0);
        }
    }
#pragma unroll
    for (int f = 0; f < FMX; ++f)
        partial[wave][f][lane] = acc[f];
    __syncthreads();
    for (int e = threadIdx.x; e < FMX * 64; e += WAVES * 64) {
        const int f = e >> 6, l = e & 63;
        v4i s = partial[0][f][l];
#pragma unroll
        for (int wv = 1; wv < WAVES; ++wv)
            s += partial[wv][f][l];
        s = s >> 8;
        const int m = f * 16 + (l & 15);
        const int n = n0 + 4 * (l >> 4);
        if (m < M) {
            const float rs = ep.row_scale ? ep.row_scale[m] : 1.f;
            by_output_width(ep, [&](auto half) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nn = n + q < N ? n + q : N - 1;
                    s[q] = epilogue_value_of<half()>(ep, s[q], ep.bias ? ep.bias[nn] : 0, rs,
                                                     ep.col_scale ? ep.col_scale[nn] : 1.f);
                }
                store_out4<half()>(Y, (size_t)m * N + n, s, N - n, n + 3 < N && (N & 3) == 0);
            });
        }
    }
}

template <int FMX>
hipError_t launch_basic(const void *a, const void *b, void *c, int m, int n, int k,
                        const Epilogue &ep, hipStream_t stream)
{
    const unsigned grid = (unsigned)((n + 15) / 16);
    const int steps = k / 128;
    if (steps >= 8)
        skinny_basic_kernel<FMX, 8><<<grid, 512, 0, stream>>>((const uint8_t *)a, (const uint8_t *)b,
                                                              (int32_t *)c, m, n, k, ep);
    else
        skinny_basic_kernel<FMX, 2><<<grid, 128, 0, stream>>>((const uint8_t *)a, (const uint8_t *)b,
                                                              (int32_t *)c, m, n, k, ep);
    return hipGetLastError();
}

constexpr int kMaxRows = 1024;  // of X: runs of 64 rows, each a pass over the workgroup's rows of W

struct Plan {
    int t = 0, s = 0, r = 0, fmx = 0;
    int rows_blk = 0;  // rows of W per workgroup: a multiple of 8, <= 16 * r
    int passes = 1;    // K = passes * s * t tiles
    bool xdma = true;
    bool ragged = false;  // S * T * passes > K's tiles: the last slices are partly or wholly empty
    int lds = 0;
};

// Which (T, R, FMX, XDMA) combinations exist as kernels: the register-X variant holds
// 2 * T * FMX 16-byte fragments per lane, which bounds T * FMX; the other bounds keep the
// number of instantiations down (shapes outside them have a plan with another T or R).
constexpr bool variant_exists(int t, int r, int fmx, bool xdma)
{
    if (xdma)
        return r == 1 || fmx <= 2 * t;
    return fmx <= 2 * t && t * fmx <= 8;
}

// Splits K over the waves and picks the X path for r row groups per workgroup: a single
// pass if any T <= 4 allows it (smallest T first: most waves, S = tiles / T <= 16), else
// the fewest passes; X through LDS if possible.  `ragged` admits splits whose last slices
// are partly or wholly empty (S * T * passes > tiles).  Returns false if nothing fits.
bool fit(int tiles, int fmx, int r, bool ragged, Plan &p)
{
    for (int passes = 1; passes <= 8; ++passes)
        for (int t = 1; t <= 4; ++t) {
            const int s = (tiles + t * passes - 1) / (t * passes);
            if (s > 16 || t > tiles || (!ragged && s * t * passes != tiles))
                continue;
            for (int xd = 1; xd >= 0; --xd) {
                const int lds = head_bytes(r, fmx) + s * t * (r + (xd ? fmx : 0)) * kTileBytes;
                if (variant_exists(t, r, fmx, xd != 0) && lds <= kMaxLds &&
                    s * 64 <= max_threads(t, r, fmx, xd != 0)) {
                    p.t = t;
                    p.s = s;
                    p.r = r;
                    p.fmx = fmx;
                    p.xdma = xd != 0;
                    p.ragged = s * t * passes != tiles;
                    p.lds = lds;
                    p.passes = passes;
                    return true;
                }
            }
        }
    return false;
}

// Rows per workgroup: the matrix split evenly over the CUs, in as few rounds as the
// largest feasible R allows, rounded up to a multiple of 8; R is then the number of
// 16-row groups that takes (a power of two).
bool make_plan(int m, int n, int k, int cu_count, bool ragged, Plan &p)
{
    if (k % kTileK != 0)
        return false;
    const int tiles = k / kTileK;
    const int fmx = m > 64 ? 4 : (m + 15) / 16;
    int rmax = 0;
    for (int r = 4; r >= 1 && rmax == 0; r >>= 1)
        if (fit(tiles, fmx, r, ragged, p))
            rmax = r;
    if (rmax == 0)
        return false;
    const long cus = cu_count > 0 ? cu_count : 1;
    const long rounds = (n + cus * 16 * rmax - 1) / (cus * 16 * rmax);
    const long per_block = (n + cus * rounds - 1) / (cus * rounds);
    const int rows_blk = (int)((per_block + 7) / 8 * 8);
    int r = 1;
    while (16 * r < rows_blk)
        r <<= 1;
    if (!fit(tiles, fmx, r, ragged, p))  // r <= rmax, so this succeeds
        return false;
    p.rows_blk = rows_blk;
    return true;
}

// An even split of K's tiles if there is one (every slice full), else a ragged one.
bool make_plan(int m, int n, int k, int cu_count, Plan &p)
{
    return make_plan(m, n, k, cu_count, false, p) || make_plan(m, n, k, cu_count, true, p);
}

// The split over K across workgroups exists for more than 32 rows of X and several row groups
// of W per workgroup (the shapes it is for; every instantiation costs build time).
constexpr bool ksplit_variant_exists(int t, int r, int fmx, bool xdma)
{
    return variant_exists(t, r, fmx, xdma) && fmx >= 3 && r >= 2;
}

// Where a launch that is split over K keeps its partial sums and counts its arrivals.
struct KSplit {
    int slices = 1;
    int *partial = nullptr;
    unsigned *arrivals = nullptr;
};

template <int T, int R, int FMX, bool XDMA>
hipError_t launch_plan(const Plan &p, const void *a, const void *b, void *c, int m, int n, int k,
                       const Epilogue &ep, hipStream_t stream, const KSplit &split = KSplit{})
{
    if constexpr (!variant_exists(T, R, FMX, XDMA)) {
        return p.s == 0 ? hipSuccess : hipErrorInvalidConfiguration;  // never planned
    } else {
    if constexpr (ksplit_variant_exists(T, R, FMX, XDMA)) {
        auto kern = skinny_ksplit_kernel<T, R, FMX, XDMA>;
        if (p.s == 0) {  // set-up call, for both forms
            const hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
            if (e != hipSuccess)
                return e;
        } else if (split.slices > 1) {
            const unsigned row_blocks = (unsigned)((n + p.rows_blk - 1) / p.rows_blk);
            const int plain = !ep.bias && !ep.row_scale && !ep.col_scale && !ep.out;
            kern<<<row_blocks * split.slices, p.s * 64, p.lds, stream>>>(
                (const uint8_t *)a, (const uint8_t *)b, (int32_t *)c,
                (v4i){m | (p.passes << 8) | (p.s << 16) | (plain << 24) | ((split.slices == 4 ? 2 : 1) << 25), n, k, p.rows_blk}, ep, split.partial,
                split.arrivals);
            return hipGetLastError();
        }
    } else if (split.slices > 1) {
        return hipErrorInvalidConfiguration;
    }
    auto kern = p.ragged ? skinny_kernel<T, R, FMX, XDMA, true> : skinny_kernel<T, R, FMX, XDMA, false>;
    if (p.s == 0)  // set-up call: raise the dynamic-LDS limit of this instantiation
        return hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    const unsigned grid = (unsigned)((n + p.rows_blk - 1) / p.rows_blk);
    const int plain = !ep.bias && !ep.row_scale && !ep.col_scale && !ep.out;
    // More than 16 * FMX rows of X go out in runs of that many, one launch each (the rows of
    // W are then streamed again, through the caches they were just pulled through).
    for (int m0 = 0; m0 < m; m0 += 16 * FMX) {
        Epilogue run_ep = ep;
        if (run_ep.row_scale)
            run_ep.row_scale += m0;
        const int rows = m - m0 < 16 * FMX ? m - m0 : 16 * FMX;
        kern<<<grid, p.s * 64, p.lds, stream>>>((const uint8_t *)a + (size_t)m0 * (size_t)(k >> 1), (const uint8_t *)b,
                                                (int32_t *)((uint8_t *)c + (size_t)m0 * (size_t)n * (ep.out >= kOutF16 ? 2u : 4u)),
                                                (v4i){rows | (p.passes << 8) | (p.s << 16) | (plain << 24), n, k, p.rows_blk}, run_ep);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return e;
    }
    return hipSuccess;
    }
}

template <int T, bool XDMA>
hipError_t dispatch_rf(const Plan &p, const void *a, const void *b, void *c, int m, int n, int k,
                       const Epilogue &ep, hipStream_t stream, const KSplit &split)
{
#define I4L_CASE(R_, F_)                                                      \
    if (p.r == R_ && p.fmx == F_)                                             \
        return launch_plan<T, R_, F_, XDMA>(p, a, b, c, m, n, k, ep, stream, split);
    I4L_CASE(4, 1) I4L_CASE(2, 1) I4L_CASE(1, 1)
    I4L_CASE(4, 2) I4L_CASE(2, 2) I4L_CASE(1, 2)
    I4L_CASE(4, 3) I4L_CASE(2, 3) I4L_CASE(1, 3)
    I4L_CASE(4, 4) I4L_CASE(2, 4) I4L_CASE(1, 4)
#undef I4L_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace

namespace {

template <bool XDMA>
hipError_t dispatch_t(const Plan &p, const void *a, const void *b, void *c, int m, int n, int k,
                      const Epilogue &ep, hipStream_t stream, const KSplit &split = KSplit{})
{
    switch (p.t) {
    case 1:
        return dispatch_rf<1, XDMA>(p, a, b, c, m, n, k, ep, stream, split);
    case 2:
        return dispatch_rf<2, XDMA>(p, a, b, c, m, n, k, ep, stream, split);
    case 3:
        return dispatch_rf<3, XDMA>(p, a, b, c, m, n, k, ep, stream, split);
    case 4:
        return dispatch_rf<4, XDMA>(p, a, b, c, m, n, k, ep, stream, split);
    default:
        return hipErrorInvalidConfiguration;
    }
}

}  // namespace

namespace {

// The long-W form: K in whole tiles that split evenly over the waves with 2 to 8 tiles each
// (with one tile the waves meet after every step), W below 4 GiB (32-bit lane offsets), and
// enough 16-row groups per CU that a workgroup which stays on its CU beats one workgroup
// per 64 rows.  At most 16 rows of X: 7 to 16 waves, most waves first (with fewer the stream
// does not keep going: K up to 3072 is faster in the other form).  17 to 64 rows: 7 or 8
// waves (256 registers each for the X fragments, TW * FMX <= 16 of them per step parity)
// and an eight-tile ring.
constexpr int kStreamMinGroupsPerCu = 5;       // measured crossover at up to 16 rows of X on eight waves (K = 4096)
constexpr int kStreamMinGroupsPerCuFull = 3;   // ... on fourteen to sixteen waves (K = 8192: 16 x 12288 x 8192 11.9 -> 10.5 us)
constexpr int kStreamMinGroupsPerCuWide = 10;  // ... with more rows of X and more than two tiles per wave

struct StreamPlan {
    int tw = 0, s = 0, fmx = 1, bufs = 4, groups_per_block = 0, grid = 0, lds = 0;
};

bool make_stream_plan(int m, int n, int k, int cu_count, StreamPlan &p)
{
    if (m > 64 || k % kTileK != 0 || cu_count <= 0 || (unsigned long long)n * (unsigned long long)(k >> 1) >= (1ull << 32))
        return false;
    const int tiles = k / kTileK;
    const int fmx = (m + 15) / 16;
    int s = 0;
    for (int cand = fmx == 1 ? 16 : 8; cand >= 7 && s == 0; --cand)
        if (tiles % cand == 0 && tiles / cand <= 8 && tiles / cand >= 2 && (fmx == 1 || tiles / cand * fmx <= 16))
            s = cand;
    if (s == 0)
        return false;
    const int groups = (n + 15) / 16;
    const int min_groups = fmx == 1 ? (s >= 14 ? kStreamMinGroupsPerCuFull : kStreamMinGroupsPerCu)
                                    : (tiles / s <= 2 ? kStreamMinGroupsPerCu : kStreamMinGroupsPerCuWide);
    if (groups < min_groups * cu_count)
        return false;
    p.tw = tiles / s;
    p.s = s;
    p.fmx = fmx;
    p.groups_per_block = (groups + cu_count - 1) / cu_count;
    p.grid = (groups + p.groups_per_block - 1) / p.groups_per_block;
    p.bufs = s <= 8 ? 8 : 4;  // up to eight waves: a deeper ring keeps as many bytes in flight
    p.lds = stream_head_bytes(fmx) + s * p.bufs * kTileBytes;
    return p.lds <= kMaxLds;
}

template <int TW, int FMX>
hipError_t launch_stream(const StreamPlan &p, const void *a, const void *b, void *c, int m, int n, int k,
                         const Epilogue &ep, hipStream_t stream)
{
    if constexpr (FMX > 1 && TW * FMX > 16) {
        return p.s == 0 ? hipSuccess : hipErrorInvalidConfiguration;  // never planned
    } else {
        auto kern = (FMX == 1 && p.bufs == 4) ? skinny_stream_kernel<TW, 4, FMX> : skinny_stream_kernel<TW, 8, FMX>;
        if (p.s == 0)  // set-up call
            return hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
        kern<<<p.grid, p.s * 64, p.lds, stream>>>((const uint8_t *)a, (const uint8_t *)b, (int32_t *)c, m, n, k,
                                                   p.groups_per_block, ep);
        return hipGetLastError();
    }
}

template <int TW>
hipError_t dispatch_stream_f(const StreamPlan &p, const void *a, const void *b, void *c, int m, int n, int k,
                             const Epilogue &ep, hipStream_t stream)
{
    switch (p.fmx) {
    case 1: return launch_stream<TW, 1>(p, a, b, c, m, n, k, ep, stream);
    case 2: return launch_stream<TW, 2>(p, a, b, c, m, n, k, ep, stream);
    case 3: return launch_stream<TW, 3>(p, a, b, c, m, n, k, ep, stream);
    case 4: return launch_stream<TW, 4>(p, a, b, c, m, n, k, ep, stream);
    default: return hipErrorInvalidConfiguration;
    }
}

hipError_t dispatch_stream(const StreamPlan &p, const void *a, const void *b, void *c, int m, int n, int k,
                           const Epilogue &ep, hipStream_t stream)
{
    switch (p.tw) {
    case 2: return dispatch_stream_f<2>(p, a, b, c, m, n, k, ep, stream);
    case 3: return dispatch_stream_f<3>(p, a, b, c, m, n, k, ep, stream);
    case 4: return dispatch_stream_f<4>(p, a, b, c, m, n, k, ep, stream);
    case 5: return dispatch_stream_f<5>(p, a, b, c, m, n, k, ep, stream);
    case 6: return dispatch_stream_f<6>(p, a, b, c, m, n, k, ep, stream);
    case 7: return dispatch_stream_f<7>(p, a, b, c, m, n, k, ep, stream);
    case 8: return dispatch_stream_f<8>(p, a, b, c, m, n, k, ep, stream);
    default: return hipErrorInvalidConfiguration;
    }
}

}  // namespace

hipError_t skinny_init(const DeviceInfo &)
{
    for (int tw = 2; tw <= 8; ++tw) {
        for (int fmx = 1; fmx <= 4; ++fmx)
            for (int bufs = 4; bufs <= 8; bufs += 4) {
                StreamPlan sp;  // s == 0: set-up call
                sp.tw = tw;
                sp.fmx = fmx;
                sp.bufs = bufs;
                const hipError_t e = dispatch_stream(sp, nullptr, nullptr, nullptr, 0, 0, 0, Epilogue{}, nullptr);
                if (e != hipSuccess)
                    return e;
            }
    }
    // Every instantiation may use up to the full LDS of a CU (a plan with s == 0 is the
    // set-up call of launch_plan).
    for (int t = 1; t <= 4; ++t)
        for (int r = 1; r <= 4; r <<= 1)
            for (int fmx = 1; fmx <= 4; ++fmx) {
                Plan p;
                p.s = 0;
                p.t = t;
                p.r = r;
                p.fmx = fmx;
                for (int ragged = 0; ragged < 2; ++ragged) {
                    p.ragged = ragged != 0;
                    hipError_t e = dispatch_t<true>(p, nullptr, nullptr, nullptr, 0, 0, 0, Epilogue{}, nullptr);
                    if (e == hipSuccess)
                        e = dispatch_t<false>(p, nullptr, nullptr, nullptr, 0, 0, 0, Epilogue{}, nullptr);
                    if (e != hipSuccess)
                        return e;
                }
            }
    return hipSuccess;
}

// More than 64 rows of X need the tiled kernel (which takes them in runs of 64); the
// fallback does not loop.
bool skinny_supports(int m, int n, int k)
{
    if (!(m >= 1 && n >= 1 && k >= 128 && k % 128 == 0 && k <= 131071 - 127))
        return false;
    if (m <= 64)
        return true;
    Plan p;
    return m <= kMaxRows && make_plan(m, n, k, 1, p);
}

// Where the kernel is the fastest one: up to 64 rows of X.  With more rows it takes X in runs
// of 64 and streams W again for each (128 x 14336 x 4096: 21 us), which the int8 kernel's
// small-grid forms beat from 65 rows on (17.7 us; 65 rows: 15.5 against 20 us).
bool skinny_preferred(int m, int n, int k, const DeviceInfo &)
{
    return m <= 64 && skinny_supports(m, n, k);
}

namespace {

// The split over K across workgroups.  Whole rows of W per workgroup mean that every
// workgroup pulls all of X: with N = 4096 on 256 CUs that is 16 rows of W against all M rows
// of X, four times the workgroup's share of W at M = 64, and every workgroup widens all of
// it.  A workgroup that takes four times the rows and a quarter of K pulls (and widens) a
// quarter of X for the same bytes of W.  What it costs is the exchange at the end -- partial
// sums to memory, an arrival counter, the last workgroup to arrive reading them back: three
// trips to memory that nothing overlaps, about 3 us while the other workgroups still stream
// (measured: 64 x 4096 x 14336 takes 10.3 us split four ways with the exchange left out and
// 13.3 us with it, against 14.1 us unsplit; one returning atomic addition per output
// element instead of the slabs is a single trip but is bound by the rate of the atomic
// units, 3.5 us for the same shape; up to 32 rows of X the gain is smaller than that, and
// with up to 16 rows there is none even with the exchange left out).  So: 33 to 64 rows
// of X, K in whole tiles that split evenly into four slices of at least 14 tiles
// (K >= 14336; at 8192 the exchange costs more than the split saves), at most 64 rows per
// workgroup.
bool make_ksplit_plan(int m, int n, int k, int cu_count, Plan &p, int &slices)
{
    constexpr int kSlices = 4, kMinTilesPerSlice = 14;
    if (m <= 32 || m > 64 || k % kTileK != 0 || cu_count <= 0)
        return false;
    const int tiles = k / kTileK;
    const int fmx = (m + 15) / 16;
    const long row_blocks_max = cu_count / kSlices;
    if (tiles % kSlices != 0 || tiles / kSlices < kMinTilesPerSlice || row_blocks_max < 1)
        return false;
    const long per_block = (n + row_blocks_max - 1) / row_blocks_max;
    const int rows_blk = (int)((per_block + 7) / 8 * 8);
    if (rows_blk > 64)
        return false;  // more rows than one round of workgroups holds: the unsplit form's case
    int r = 1;
    while (16 * r < rows_blk)
        r <<= 1;
    if (r < 2 || !fit(tiles / kSlices, fmx, r, false, p) || !ksplit_variant_exists(p.t, p.r, p.fmx, p.xdma))
        return false;
    const long row_blocks = (n + rows_blk - 1) / rows_blk;
    if (p.s < 4 || row_blocks * p.s > kSkinnyArrivalWords)
        return false;
    p.rows_blk = rows_blk;
    slices = kSlices;
    return true;
}

// The plans of the shape a host thread asked for last: a decode loop calls with a handful of
// shapes over and over, and next to a kernel of a few microseconds the plan search (some
// hundred candidate splits) is not free.
struct PlanCache {
    int m = -1, n = -1, k = -1, cus = -1;
    int kind = 0;  // 1: long-W form, 2: tiled form, 3: neither
    StreamPlan sp;
    Plan p;
    int slices = 1;  // > 1: the split over K across workgroups applies, with plan `split`
    Plan split;
    size_t split_bytes = 0;
};
thread_local PlanCache t_plan;

PlanCache &plans_for(int m, int n, int k, const DeviceInfo &dev)
{
    PlanCache &pc = t_plan;
    if (pc.m != m || pc.n != n || pc.k != k || pc.cus != dev.cu_count) {
        pc.kind = make_stream_plan(m, n, k, dev.cu_count, pc.sp) ? 1 : make_plan(m, n, k, dev.cu_count, pc.p) ? 2 : 3;
        pc.slices = 1;
        pc.split_bytes = 0;
        if (pc.kind == 2 && make_ksplit_plan(m, n, k, dev.cu_count, pc.split, pc.slices)) {
            const size_t row_blocks = (size_t)((n + pc.split.rows_blk - 1) / pc.split.rows_blk);
            pc.split_bytes = row_blocks * pc.slices * pc.split.r * pc.split.fmx * 1024;
        } else {
            pc.slices = 1;
        }
        pc.m = m;
        pc.n = n;
        pc.k = k;
        pc.cus = dev.cu_count;
    }
    return pc;
}

}  // namespace

size_t skinny_workspace_bytes(int m, int n, int k, const DeviceInfo &dev)
{
    if (m <= 32 || !skinny_supports(m, n, k))  // (the common decode call: not even a look at the cache)
        return 0;
    return plans_for(m, n, k, dev).split_bytes;
}

hipError_t launch_skinny_ksplit(const void *a, const void *b, void *c, int m, int n, int k, void *workspace,
                                unsigned *arrivals, const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    PlanCache &pc = plans_for(m, n, k, dev);
    if (pc.slices <= 1 || !workspace || !arrivals)
        return launch_skinny(a, b, c, m, n, k, ep, dev, stream);
    const KSplit split{pc.slices, (int *)workspace, arrivals};
    return pc.split.xdma ? dispatch_t<true>(pc.split, a, b, c, m, n, k, ep, stream, split)
                         : dispatch_t<false>(pc.split, a, b, c, m, n, k, ep, stream, split);
}

hipError_t launch_skinny(const void *a, const void *b, void *c, int m, int n, int k,
                         const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    PlanCache &pc = plans_for(m, n, k, dev);
    if (pc.kind == 1)
        return dispatch_stream(pc.sp, a, b, c, m, n, k, ep, stream);
    if (pc.kind == 2)
        return pc.p.xdma ? dispatch_t<true>(pc.p, a, b, c, m, n, k, ep, stream)
                         : dispatch_t<false>(pc.p, a, b, c, m, n, k, ep, stream);
    if (m > 64)
        return hipErrorInvalidConfiguration;  // skinny_supports() says no
    switch ((m + 15) / 16) {
    case 1:
        return launch_basic<1>(a, b, c, m, n, k, ep, stream);
    case 2:
        return launch_basic<2>(a, b, c, m, n, k, ep, stream);
    case 3:
        return launch_basic<3>(a, b, c, m, n, k, ep, stream);
    default:
        return launch_basic<4>(a, b, c, m, n, k, ep, stream);
    }
}

}  // namespace int4linear
