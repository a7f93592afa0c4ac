// LDS-pipelined int8-MFMA GEMM over packed signed-int4 operands for gfx950 (CDNA4).
//
// gfx950 has no 4-bit integer MFMA, so nibbles are widened to int8 in registers and fed
// to v_mfma_i32_32x32x32_i8.  The widening keeps each nibble in the HIGH half of its
// byte: for a packed word w,  (w << 4) & 0xF0F0F0F0  holds the even-k nibbles and
// w & 0xF0F0F0F0 the odd-k nibbles, each as the signed byte 16*value (the nibble's own
// sign bit lands in bit 7, so no sign-extension step exists).  Both operands carry the
// factor 16, every product carries 256, and C = acc >> 8 exactly.  |acc| <= K * 2^14, so
// int32 holds it for K <= 131071; the launcher refuses larger K.
//
// A dot product does not care in which order k is visited as long as both operands
// visit it in the same order, so even and odd nibbles are never re-interleaved and a
// lane simply owns whatever 32 nibbles its 16-byte LDS read returns.
//
// Data movement per workgroup (tile BM x BN of C, K consumed 128 nibbles per stage):
//   HBM/L2 --global_load_lds_dwordx4 (16 B per lane, straight into LDS)--> NSTAGE-deep ring
//   LDS    --ds_read_b128 (bank-conflict-free through a 16-byte-chunk XOR swizzle)--> VGPRs
//   VGPRs  --3 VALU ops per packed dword--> int8 operands --MFMA--> int32 accumulators
//   accumulators --buffer_store_dword (X is the MFMA A operand, so the 32 lanes of a
//                 half-wave hold 32 consecutive n: every store writes whole 128-byte
//                 row segments), non-temporal--> C
// Two wavefronts share each SIMD: while one widens nibbles on the VALU the other keeps
// the matrix pipe busy.  The kernel is persistent: gridDim.x workgroups walk a list of
// tiles, and the load ring runs NSTAGE-1 stages ahead of the math ACROSS tile
// boundaries, so the next tile's first stages are in flight while this tile stores C.
//
// Grids of few tiles run in a second form (mfma_pair_kernel, mfma_pair64_kernel: one
// 128 x 128 or 64 x 64 tile per workgroup, eight waves of which the two on a SIMD split
// every stage's K), described where it is defined; shapes with few tiles and long K are
// split over K into slabs of partial sums that a second kernel adds up.
#include "kernels.h"

#include <type_traits>
#include <utility>

namespace int4linear {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

#define I4L_LDS(p) ((__attribute__((address_space(3))) void *)(p))

// s_waitcnt immediate for gfx9: vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14,
// expcnt (bits 6:4) and lgkmcnt (bits 11:8) left at "no wait".
#define I4L_VMCNT(n) ((0x0F70) | ((n) & 0xF) | ((((n) >> 4) & 0x3) << 14))

// 16 bytes per lane from global memory straight into LDS: lane l's data lands at LDS
// byte lds_addr + 16*l.  Global address = wave-uniform base (SGPR pair) + per-lane
// 32-bit offset.  M0 carries the LDS address; one wait state separates its write from
// the load that reads it.  The compiler does not count this load in its own vmcnt
// bookkeeping, which only makes the waits it inserts for its own accesses stricter.
// The LDS address is the sum of two scalars (a fixed place inside a stage buffer and the
// buffer's offset in the ring), added on the way into M0.
__device__ __forceinline__ void dma16(const void *sbase, unsigned voff, unsigned lds_place, unsigned lds_ring)
{
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(lds_place), "s"(lds_ring)
                 : "memory", "scc");
}

// Hides a value's origin from the optimiser so that work derived from it stays where
// it is written instead of being hoisted out of the stage loop into live registers.
__device__ __forceinline__ int opaque(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// Marks a value as used (and possibly changed) at this point of the program.
__device__ __forceinline__ void keep(v4i &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void keep(const v16i &v) { asm volatile("" ::"v"(v)); }

constexpr int kStoreAux = 2;  // nt: C is written once and not read back by this kernel

constexpr int kStageK = 128;                 // nibbles of K per pipeline stage
constexpr int kRowBytes = kStageK / 2;       // bytes per LDS row (64)
constexpr int kChunkRows = 16;               // rows moved by one 64-lane 16-byte load
constexpr int kChunkBytes = kChunkRows * kRowBytes;  // 1 KiB
constexpr int kFrag = 32;                    // rows of an MFMA 32x32x32 operand

// Tile configuration.  A workgroup is WAVES_M x WAVES_N wavefronts; each owns
// FM x FN MFMA tiles of 32x32, i.e. a (FM*32) x (FN*32) patch of C.
template <int WAVES_M_, int WAVES_N_, int FM_, int FN_, int NSTAGE_, int OCC_>
struct TileConfig {
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int FM = FM_, FN = FN_;
    static constexpr int NSTAGE = NSTAGE_;
    static constexpr int OCC = OCC_;  // workgroups per CU
    static constexpr int NWAVES = WAVES_M * WAVES_N;
    static constexpr int THREADS = NWAVES * 64;
    static constexpr int BM = WAVES_M * FM * kFrag;
    static constexpr int BN = WAVES_N * FN * kFrag;
    static constexpr int X_CHUNKS = BM / kChunkRows;
    static constexpr int W_CHUNKS = BN / kChunkRows;
    static constexpr int CH = (X_CHUNKS + W_CHUNKS) / NWAVES;  // loads per wave per stage
    static constexpr int X_CH = X_CHUNKS / NWAVES;             // of which from X
    static constexpr int STAGE_BYTES = (BM + BN) * kRowBytes;
    static constexpr int LDS_BYTES = STAGE_BYTES * NSTAGE;
    static constexpr int STORES = FM * FN * 16;  // dword stores per lane per tile
    static_assert(X_CHUNKS % NWAVES == 0 && W_CHUNKS % NWAVES == 0, "chunks must split evenly");
    static_assert(NSTAGE >= 4 && CH <= 63, "vmcnt is six bits");
};

// Which 16-byte slot of its 64-byte LDS row holds logical chunk c of row r:  c ^ swz(r),
// a function of r mod 16 (the rows one 64-lane load moves).
// With rows 64 B apart, sixteen lanes reading the same c of sixteen consecutive rows
// touch sixteen different 16-byte bank groups of a 256-byte window, and any aligned
// eight of them touch eight different groups of a 128-byte window.
__device__ __forceinline__ int swz(int r) { r &= 15; return ((r >> 1) + (r >> 3)) & 3; }

// Tile order.  Workgroup ids go round-robin over the 8 XCDs, each with a private L2, so
// the tiles that run together on one XCD (ids congruent mod 8, consecutive quotients)
// are given consecutive positions of a grouped order: 8 tile-rows tall, column-major
// inside the group.  32 consecutive positions are then an 8x4 patch sharing rows of A
// and B in that L2.
__device__ __forceinline__ void tile_coords(int v, int total, int tiles_m, int tiles_n,
                                            int &tm, int &tn)
{
    constexpr int kXcd = 8, kGroup = 8;
    const int x = v % kXcd, j = v / kXcd;
    const int cnt = total / kXcd, rem = total % kXcd;
    const int q = x * cnt + (x < rem ? x : rem) + j;
    const int per_group = kGroup * tiles_n;
    const int group = q / per_group;
    const int first_m = group * kGroup;
    const int gsz = (tiles_m - first_m < kGroup) ? (tiles_m - first_m) : kGroup;
    const int in_group = q % per_group;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

// What mfma_gemm_kernel is put together from.  The library builds WholeInt8Kernel and nothing
// else; tests/host/int8_ablation.cpp, which compiles this file again, passes variations of
// its own (derived from this one, with single members changed) to time what each part costs.
struct WholeInt8Kernel {
    static constexpr bool kStores = true;    // a finished tile is stored
    static constexpr bool kLoads = true;     // global -> LDS loads go on after the prologue
    static constexpr bool kLdsReads = true;  // LDS -> register reads go on after the prologue
    static constexpr bool kWiden = true;     // nibbles are widened to bytes between the MFMAs (false: the first operands stay)
    static constexpr bool kStagger = true;   // workgroups of an XCD start in groups
    // Called by lane 0 of wave 0 when the workgroup starts and after its last tile.
    __device__ static void stamp(int /* workgroup */, int /* 0: start, 1: end */) {}
};

template <class C, class Parts = WholeInt8Kernel>
__global__ __launch_bounds__(C::THREADS, C::OCC) void mfma_gemm_kernel(
    const uint8_t *__restrict__ X, const uint8_t *__restrict__ W, int32_t *__restrict__ Y,
    int M, int N, int K, int tiles_m, int tiles_n, int ksplit, Epilogue ep)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / C::WAVES_N;
    const int wn = wave % C::WAVES_N;
    const int rowbytes = K >> 1;
    // With ksplit > 1 a work item is one K-slice of one tile: item v is slice v % ksplit of
    // tile v / ksplit, covers KT stages, and stores its plain partial sums into slab
    // v % ksplit of Y (M * N int32 each), which a second kernel adds up.
    const int KT = K / kStageK / ksplit;
    const int total_tiles = tiles_m * tiles_n * ksplit;  // work items
    const int nblk = gridDim.x;
    const int bid = blockIdx.x;
    const bool ep_plain = ksplit > 1 || (!ep.bias && !ep.row_scale && !ep.col_scale && !ep.out);
    if (bid >= total_tiles)
        return;
    const int my_tiles = (total_tiles - bid + nblk - 1) / nblk;
    const int total_stages = my_tiles * KT;
    if (threadIdx.x == 0)
        Parts::stamp(bid, 0);
    // Workgroups that start together reach every tile end together, and the stores of all
    // tiles then queue for the same path to memory while no CU computes.  With 256 x 256
    // tiles and two or more of them per workgroup, the workgroups of an XCD (ids congruent
    // mod 8) start in eight groups 0.8 us apart instead (measured: 4096 x 8192 x 1024 runs
    // 20 % faster, 8192^3 2 %; with the 128 x 128 tiles the spread costs more than it saves).
    if constexpr (C::BM == 256 && C::BN == 256) {
        if (Parts::kStagger && total_tiles >= 2 * nblk) {
            const int grp = (bid >> 3) & 7;
            const unsigned long long until = wall_clock64() + (unsigned long long)(grp * 80);  // 10-ns ticks
            while (wall_clock64() < until)
                __builtin_amdgcn_s_sleep(2);
        }
    }

    // ---- load side -------------------------------------------------------------------
    // Lane p of a chunk lands at LDS byte p*16 of that chunk: row p/4, slot p%4.
    const int ld_row = lane >> 2;
    const int ld_c = (lane & 3) ^ swz(ld_row);
    unsigned voff[C::CH];                // per-chunk byte offset of this lane from the tile base
    const uint8_t *xptr = X, *wptr = W;  // wave-uniform: tile base + k offset
    int ld_it = 0, ld_k = 0, issued = 0;
    const unsigned lds_base = (unsigned)(size_t)I4L_LDS(lds);

    auto ld_setup_tile = [&](int it) {
        int tm, tn;
        const int item = bid + it * nblk;
        tile_coords(item / ksplit, total_tiles / ksplit, tiles_m, tiles_n, tm, tn);
        const int m0 = tm * C::BM, n0 = tn * C::BN;
        const int row = opaque(ld_row);
#pragma unroll
        for (int c = 0; c < C::CH; ++c) {
            const bool is_x = c < C::X_CH;
            const int ci = (is_x ? c : c - C::X_CH) * C::NWAVES + wave;
            const int r = ci * kChunkRows + row;
            const int lim = is_x ? (M - 1 - m0) : (N - 1 - n0);  // last valid row, tile-relative
            const int rc = r < lim ? r : lim;
            voff[c] = (unsigned)rc * (unsigned)rowbytes + (unsigned)ld_c * 16u;
        }
        const size_t k_off = (size_t)(item % ksplit) * KT * kRowBytes;
        xptr = X + (size_t)m0 * rowbytes + k_off;
        wptr = W + (size_t)n0 * rowbytes + k_off;
    };

    // One stage = CH loads per wave (ld_chunk) followed by the cursor advance.  Chunk c of
    // this wave always lands at the same place of a stage buffer; wr_ring is the offset of
    // the buffer being filled (ring position issued % NSTAGE).
    unsigned chunk_place[C::CH];
#pragma unroll
    for (int c = 0; c < C::CH; ++c) {
        const bool is_x = c < C::X_CH;
        const int ci = (is_x ? c : c - C::X_CH) * C::NWAVES + wave;
        chunk_place[c] = lds_base + (is_x ? 0 : C::BM * kRowBytes) + ci * kChunkBytes;
    }
    unsigned wr_ring = 0;
    auto ld_chunk = [&](int c) {
        dma16(c < C::X_CH ? xptr : wptr, voff[c], chunk_place[c], wr_ring);
    };
    // Past the last stage the cursor stays where it is: the loads go on, as refills of
    // buffers already consumed with data nobody reads, so that every iteration of the
    // stage loop issues the same loads and the wait counts are constants.
    auto ld_advance = [&]() {
        ++issued;
        wr_ring = wr_ring + C::STAGE_BYTES == C::LDS_BYTES ? 0u : wr_ring + C::STAGE_BYTES;
        if (issued < total_stages) {
            ++ld_k;
            xptr += kRowBytes;
            wptr += kRowBytes;
            if (ld_k == KT) {
                ld_k = 0;
                ++ld_it;
                ld_setup_tile(ld_it);
            }
        }
    };
    auto ld_issue = [&]() {
#pragma unroll
        for (int c = 0; c < C::CH; ++c)
            ld_chunk(c);
        ld_advance();
    };

    ld_setup_tile(0);
#pragma unroll 1
    for (int s = 0; s < C::NSTAGE - 1; ++s)
        ld_issue();

    // ---- math side -------------------------------------------------------------------
    // Lane l of a 32x32x32 MFMA supplies row l%32 and 16 of the 32 k values of both
    // operands.  A 16-byte LDS read holds 32 nibbles: the even ones feed one MFMA, the odd
    // ones the next.  Half h of a stage is the two 16-byte chunks 2h and 2h+1 of a row,
    // one per 32-lane group.
    const int fr = lane & 31;
    const int fg = lane >> 5;
    const int fsw = swz(fr);
    unsigned rd_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
        rd_off[h] = (unsigned)fr * kRowBytes + (unsigned)(((2 * h + fg) ^ fsw) * 16);
    const unsigned x_rd = (unsigned)(wm * C::FM * kFrag * kRowBytes);
    const unsigned w_rd = (unsigned)(C::BM * kRowBytes + wn * C::FN * kFrag * kRowBytes);
    int himask;  // kept in a scalar register: a VALU source operand that costs nothing
    asm volatile("s_mov_b32 %0, 0xf0f0f0f0" : "=s"(himask));

    // The math is software-pipelined in units of half a stage.  Unit u = (stage, half h)
    // owns FN W fragments and FM X fragments; step j of a unit issues the 2*FN MFMAs of X
    // fragment j.  Two wavefronts share a SIMD and run in lockstep between barriers, so a
    // wave that widened all its nibbles first and multiplied afterwards would leave the
    // matrix pipe idle while BOTH waves widen.  Instead every MFMA is followed by a few
    // of the VALU ops that prepare later operands:
    //   step (u, j) widens X fragment j+1 (or fragment 0 of unit u+1) and, for j >= 1,
    //   a third of unit u+1's W fragments; step (u, 0) issues the LDS reads of unit u+1.
    // __builtin_amdgcn_sched_barrier(0) after each slot pins that order.
    v16i acc[C::FN][C::FM];
    v4i pk_w[2][C::FN], pk_x[2][C::FM];  // packed fragments, by unit parity (= half)
    v4i wlo[2][C::FN], whi[2][C::FN];    // widened W, by unit parity
    v4i xlo[2], xhi[2];                  // widened X fragment, by step parity
    int cur_it = 0, kk = 0;
    static_assert(C::FM % 2 == 0, "step parity must line up across units");

    // One 16-byte LDS read per fragment of half h of stage st.  A unit's reads come in
    // kReadParts parts so that they can be spread over several steps: part 0 is the W
    // fragments, the others split the X fragments evenly.
    constexpr int kReadParts = 3;
    constexpr int kXPerPart = C::FM / (kReadParts - 1);
    static_assert(kXPerPart * (kReadParts - 1) == C::FM, "X fragments must split evenly");
    auto read_part = [&](unsigned ring, int h, int part, v4i (&w)[C::FN], v4i (&x)[C::FM]) {
        const uint8_t *stage = lds + ring;  // the stage's buffer
        if (part == 0) {
#pragma unroll
            for (int i = 0; i < C::FN; ++i)
                w[i] = *(const v4i *)(stage + w_rd + rd_off[h] + i * kFrag * kRowBytes);
        } else {
#pragma unroll
            for (int j = (part - 1) * kXPerPart; j < part * kXPerPart; ++j)
                x[j] = *(const v4i *)(stage + x_rd + rd_off[h] + j * kFrag * kRowBytes);
        }
    };

    // Op k (0..11) of widening one packed fragment: the four shifts first, then the masks of
    // the shifted words (even-k nibbles), then the masks of the unshifted words (odd-k
    // nibbles), so that no op directly follows the one it depends on.
    auto widen_op = [&](int k, const v4i &p, v4i &lo, v4i &hi) {
        const int d = k % 4;
        switch (k / 4) {
        case 0:
            lo[d] = p[d] << 4;
            break;
        case 1:
            lo[d] = lo[d] & himask;
            break;
        default:
            hi[d] = p[d] & himask;
            break;
        }
    };

    constexpr int kSlots = 2 * C::FN;             // MFMAs per step
    constexpr int kWOps = 12 * C::FN;             // VALU ops to widen one unit's W
    constexpr int kWPerStep = (kWOps + C::FM - 2) / (C::FM - 1);  // spread over steps 1..FM-1

    // Step j of the unit with parity h.  `next_x` is the packed X fragment widened during
    // this step into step parity (j+1)%2.  `hook(j, slot)` is housekeeping placed behind
    // the MFMA of that slot; it may branch, so the slot's VALU results are pinned first.
    auto step = [&](auto h_tag, auto j_tag, const v4i &next_x, auto &&hook) {
        constexpr int h = decltype(h_tag)::value;
        constexpr int j = decltype(j_tag)::value;
        constexpr int w_begin = j == 0 ? 0 : (j - 1) * kWPerStep;
        constexpr int w_end = j == 0 ? 0 : (j * kWPerStep < kWOps ? j * kWPerStep : kWOps);
        constexpr int n_ops = 12 + (w_end - w_begin);
        [&]<int... SLOT>(std::integer_sequence<int, SLOT...>) {
            ([&] {
                constexpr int slot = SLOT;
                constexpr int i = slot % C::FN;
                if (slot < C::FN)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xlo[j % 2], wlo[h][i], acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xhi[j % 2], whi[h][i], acc[i][j], 0, 0, 0);
                constexpr int op0 = slot * n_ops / kSlots, op1 = (slot + 1) * n_ops / kSlots;
#pragma unroll
                for (int op = op0; op < (Parts::kWiden ? op1 : op0); ++op) {
                    if (op < 12) {
                        widen_op(op, next_x, xlo[(j + 1) % 2], xhi[(j + 1) % 2]);
                    } else {
                        const int wop = w_begin + op - 12;
                        widen_op(wop % 12, pk_w[1 - h][wop / 12], wlo[1 - h][wop / 12], whi[1 - h][wop / 12]);
                    }
                }
                keep(xlo[(j + 1) % 2]);
                keep(xhi[(j + 1) % 2]);
                __builtin_amdgcn_sched_barrier(0);
                hook(j_tag, std::integral_constant<int, slot>{});
                __builtin_amdgcn_sched_barrier(0);
            }(), ...);
        }(std::make_integer_sequence<int, kSlots>{});
    };

    // All steps of the unit with parity h, then the pins that keep the operands widened
    // for the next unit inside this unit's MFMA shadow.
    auto unit = [&](auto h_tag, auto &&hook) {
        constexpr int h = decltype(h_tag)::value;
        [&]<int... J>(std::integer_sequence<int, J...>) {
            ((step(h_tag, std::integral_constant<int, J>{},
                   J + 1 < C::FM ? pk_x[h][(J + 1) % C::FM] : pk_x[1 - h][0], hook)), ...);
        }(std::make_integer_sequence<int, C::FM>{});
#pragma unroll
        for (int i = 0; i < C::FN; ++i) {
            keep(wlo[1 - h][i]);
            keep(whi[1 - h][i]);
        }
    };

    // Stage 0 must have landed before the first read.
    __builtin_amdgcn_s_waitcnt(I4L_VMCNT((C::NSTAGE - 2) * C::CH));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // Pipeline fill: unit (0, 0) read, its W and its X fragment 0 widened.
#pragma unroll
    for (int part = 0; part < kReadParts; ++part)
        read_part(0u, 0, part, pk_w[0], pk_x[0]);
#pragma unroll
    for (int i = 0; i < C::FN; ++i)
#pragma unroll
        for (int op = 0; op < 12; ++op)
            widen_op(op, pk_w[0][i], wlo[0][i], whi[0][i]);
#pragma unroll
    for (int op = 0; op < 12; ++op)
        widen_op(op, pk_x[0][0], xlo[0], xhi[0]);

    // Housekeeping is spread thinly behind the MFMAs, for two reasons.  A wave must not
    // go long without issuing an MFMA: its SIMD partner runs the same code at the same
    // time, so whatever sits between two MFMAs is matrix-pipe idle time once it exceeds
    // one MFMA.  And the eight waves of a workgroup run in step between barriers, so work
    // that all of them issue at the same point (32 direct-to-LDS loads, 48 LDS reads)
    // queues up in the memory pipeline and blocks the waves behind it.  Hence:
    //   * the LDS reads of the next unit go out in kReadParts parts, evenly spaced over
    //     the unit's FM * kSlots slot positions;
    //   * the CH loads of stage gs+3 are split between the second half of iteration gs
    //     (loads 0..CH/2-1) and the first half of iteration gs+1 (the rest); inside a half
    //     they are evenly spaced and odd waves go one place after even waves, so at any
    //     position at most half the waves issue one load;
    //   * the load cursor advances at the last position of the first half.
    // All loads of stage gs+3 are still issued between the barriers of iterations gs and
    // gs+1, in order, which is all the wait counts below rely on.
    constexpr int kPositions = C::FM * kSlots;       // slot positions per unit
    constexpr int kDmaStride = kPositions / C::CH;   // CH/2 loads x 2 wave parities per half
    static_assert(C::CH % 2 == 0 && kDmaStride >= 1 && kDmaStride * C::CH == kPositions,
                  "load spreading needs CH places per half");
    // X fragment 0 of the next unit is read with part 1 and widened during this unit's last
    // step, so part 1 must go out before that step begins.
    static_assert(kPositions / kReadParts + 1 < (C::FM - 1) * kSlots, "part 1 of the LDS reads comes too late");
    const int wave_par = wave & 1;
    // Housekeeping common to both halves at position (j, slot): `read_ring`/`read_h` name the
    // unit whose fragments are read, `half_pos` is 0 in the second half of an iteration,
    // `do_load` is false only in the first half of the very first iteration (nothing begun).
    auto spread = [&](auto j_tag, auto slot_tag, unsigned read_ring, int read_h, int half_pos, bool do_load) {
        constexpr int pos = decltype(j_tag)::value * kSlots + decltype(slot_tag)::value;
#pragma unroll
        for (int part = 0; part < kReadParts; ++part)
            if (Parts::kLdsReads && pos == part * kPositions / kReadParts + 1)
                read_part(read_ring, read_h, part, pk_w[read_h], pk_x[read_h]);
        constexpr int off = kDmaStride / 2;
        if constexpr (pos >= off && (pos - off) % kDmaStride == 0) {
            constexpr int idx = (pos - off) / kDmaStride;  // 0 .. CH-1
            if (Parts::kLoads && do_load && wave_par == idx % 2)
                ld_chunk(half_pos * (C::CH / 2) + idx / 2);
        }
    };

    unsigned rd_cur = 0, rd_next = C::STAGE_BYTES;  // ring offsets of stages gs and gs+1
#pragma unroll 1
    for (int gs = 0; gs < total_stages; ++gs) {
        if (kk == 0) {
#pragma unroll
            for (int i = 0; i < C::FN; ++i)
#pragma unroll
                for (int j = 0; j < C::FM; ++j)
#pragma unroll
                    for (int t = 0; t < 16; ++t)
                        acc[i][j][t] = 0;
        }

        // ---- first half: reads the second half of this stage, finishes the loads begun
        //      in the previous iteration
        const bool begun = gs > 0;
        unit(std::integral_constant<int, 0>{}, [&](auto j_tag, auto slot_tag) {
            constexpr int j = decltype(j_tag)::value;
            constexpr int slot = decltype(slot_tag)::value;
            spread(j_tag, slot_tag, rd_cur, 1, 1, begun);
            if constexpr (slot == kSlots - 1 && j == C::FM - 1) {
                if (begun)
                    ld_advance();
            }
        });

        // ---- second half: makes stage gs+1 readable, reads its first half, begins the
        //      loads of stage gs+NSTAGE-1 into the buffer of stage gs-1
        unit(std::integral_constant<int, 1>{}, [&](auto j_tag, auto slot_tag) {
            constexpr int j = decltype(j_tag)::value;
            constexpr int slot = decltype(slot_tag)::value;
            if constexpr (slot == 0 && j == 0) {
                // This wave's loads of stage gs+1 must have landed, then every wave's.
                // Outstanding VMEM ops complete in order; NSTAGE - 3 younger stages are in
                // flight behind them, and the C stores of a finished tile as well while the
                // stage waited for was issued wholly before those stores, i.e. for the first
                // NSTAGE - 3 stages of the next tile (after that the loads waited for were
                // themselves issued after the stores).  The counter holds at most 63: a larger
                // allowance becomes 63, which only waits longer.
                constexpr int plain = (C::NSTAGE - 3) * C::CH, with_stores = plain + C::STORES;
                if (cur_it > 0 && kk < C::NSTAGE - 3)
                    __builtin_amdgcn_s_waitcnt(I4L_VMCNT(with_stores < 63 ? with_stores : 63));
                else
                    __builtin_amdgcn_s_waitcnt(I4L_VMCNT(plain < 63 ? plain : 63));
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                // Every wave is past its reads of stage gs-1: that buffer may be refilled.
            }
            // (past the last stage the reads fetch a stale buffer whose contents never reach
            // a stored tile; unconditional reads keep the LDS wait counts exact)
            spread(j_tag, slot_tag, rd_next, 0, 0, true);
        });
        rd_cur = rd_next;
        rd_next = rd_next + C::STAGE_BYTES == C::LDS_BYTES ? 0u : rd_next + C::STAGE_BYTES;

        ++kk;
        if (kk == KT) {
            // ---- store the tile
            int tm, tn;
            const int item = bid + cur_it * nblk;
            tile_coords(item / ksplit, total_tiles / ksplit, tiles_m, tiles_n, tm, tn);
            const int m0 = tm * C::BM, n0 = tn * C::BN;
            const int rows_left = M - m0;  // > 0
            const int cols_left = N - n0;  // > 0
            int32_t *ybase = Y + (size_t)(item % ksplit) * ((size_t)M * N) + (size_t)m0 * N + n0;
            // Byte extent of this tile's slab of C, measured from ybase.
            const size_t slab_rows = rows_left < C::BM ? rows_left : C::BM;
            const size_t extent = ((slab_rows - 1) * (size_t)N + (size_t)(cols_left < C::BN ? cols_left : C::BN)) * 4u;
            __amdgpu_buffer_rsrc_t rsrc =
                __builtin_amdgcn_make_buffer_rsrc(ybase, 0, (int)extent, 0x00020000);
            // X is the MFMA A operand: accumulator t of tile (i, j) belongs to
            //   m = 32*j + 8*(t/4) + 4*(lane/32) + t%4,  n = 32*i + lane%32,
            // so one dword store writes two rows of 32 consecutive n (128 B each).
            // Offsets are split into a row part and a column part; a lane outside the
            // matrix gets a part so large that the sum falls outside the descriptor's
            // range and the hardware drops the store.
            const int lm = opaque(wm * C::FM * kFrag + fg * 4);
            const int ln = opaque(wn * C::FN * kFrag + fr);
            const unsigned lm_off = (unsigned)lm * (unsigned)N * 4u;
            unsigned col_off[C::FN];
#pragma unroll
            for (int i = 0; i < C::FN; ++i) {
                const int ncol = ln + i * kFrag;
                col_off[i] = ncol < cols_left ? (unsigned)ncol * 4u : 0x40000000u;
            }
            if constexpr (!Parts::kStores) {
#pragma unroll
                for (int i = 0; i < C::FN; ++i)
#pragma unroll
                    for (int j = 0; j < C::FM; ++j)
                        keep(acc[i][j]);  // (every accumulator counts as used: no MFMA may be dropped)
            } else if (ep_plain) {
#pragma unroll
                for (int j = 0; j < C::FM; ++j) {
#pragma unroll
                    for (int t = 0; t < 16; ++t) {
                        const int dm = j * kFrag + 8 * (t / 4) + (t % 4);  // uniform
                        const unsigned row_off = lm + dm < rows_left ? lm_off + (unsigned)dm * (unsigned)N * 4u : 0x80000000u;
#pragma unroll
                        for (int i = 0; i < C::FN; ++i) {
                            const int v = acc[i][j][t] >> 8;
                            __builtin_amdgcn_raw_buffer_store_b32((unsigned)v, rsrc, row_off + col_off[i], 0, kStoreAux);
                        }
                    }
                }
            } else {
                // Epilogue operands of this lane's columns and rows (clamped inside the
                // matrix).  These ordinary loads make the compiler wait for everything in
                // flight, prefetched stages included: the price of an epilogue, kept out of
                // the plain path above.
                int bias_v[C::FN];
                float cs_v[C::FN];
#pragma unroll
                for (int i = 0; i < C::FN; ++i) {
                    const int ncol = ln + i * kFrag;
                    const int nn = n0 + (ncol < cols_left ? ncol : cols_left - 1);
                    bias_v[i] = ep.bias ? ep.bias[nn] : 0;
                    cs_v[i] = ep.col_scale ? ep.col_scale[nn] : 1.f;
                }
                if (!out_is_half_width(ep)) {
#pragma unroll
                    for (int j = 0; j < C::FM; ++j) {
                        float rs[16];
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int dm = j * kFrag + 8 * (t / 4) + (t % 4);
                            rs[t] = ep.row_scale ? ep.row_scale[m0 + (lm + dm < rows_left ? lm + dm : rows_left - 1)] : 1.f;
                        }
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int dm = j * kFrag + 8 * (t / 4) + (t % 4);  // uniform
                            const unsigned row_off = lm + dm < rows_left ? lm_off + (unsigned)dm * (unsigned)N * 4u : 0x80000000u;
#pragma unroll
                            for (int i = 0; i < C::FN; ++i) {
                                const int v = epilogue_value32(ep, acc[i][j][t] >> 8, bias_v[i], rs[t], cs_v[i]);
                                __builtin_amdgcn_raw_buffer_store_b32((unsigned)v, rsrc, row_off + col_off[i], 0, kStoreAux);
                            }
                        }
                    }
                } else {
                    // The half-width kinds: a descriptor over the same tile of an output of
                    // two-byte elements, every offset halved (no K-slices here: an epilogue
                    // goes with ksplit == 1, Y is the output's base).
                    __amdgpu_buffer_rsrc_t rsrc16 = __builtin_amdgcn_make_buffer_rsrc(
                        (uint8_t *)Y + ((size_t)m0 * N + n0) * 2u, 0, (int)(extent / 2u), 0x00020000);
#pragma unroll
                    for (int j = 0; j < C::FM; ++j) {
                        float rs[16];
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int dm = j * kFrag + 8 * (t / 4) + (t % 4);
                            rs[t] = ep.row_scale ? ep.row_scale[m0 + (lm + dm < rows_left ? lm + dm : rows_left - 1)] : 1.f;
                        }
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int dm = j * kFrag + 8 * (t / 4) + (t % 4);  // uniform
                            const unsigned row_off = lm + dm < rows_left ? (lm_off + (unsigned)dm * (unsigned)N * 4u) / 2u : 0x80000000u;
#pragma unroll
                            for (int i = 0; i < C::FN; ++i) {
                                const int v = epilogue_value16(ep, acc[i][j][t] >> 8, bias_v[i], rs[t], cs_v[i]);
                                __builtin_amdgcn_raw_buffer_store_b16((unsigned short)v, rsrc16,
                                                                      row_off + (col_off[i] == 0x40000000u ? col_off[i] : col_off[i] / 2u), 0, kStoreAux);
                            }
                        }
                    }
                }
            }
            kk = 0;
            ++cur_it;
        }
    }
    // The refills issued past the last stage must have landed before the workgroup's LDS
    // is handed to another one.
    __builtin_amdgcn_s_waitcnt(I4L_VMCNT(0));
    if (threadIdx.x == 0)
        Parts::stamp(bid, 1);
}

// ---- the form for grids of a few tiles per CU -----------------------------------------
//
// With one 128 x 128 tile per CU the kernel above has a single wave per SIMD (two with two
// tiles), and a single wave cannot issue the nibble widening and the MFMAs fast enough to
// keep the matrix pipe busy (about 90 cycles per 32-cycle MFMA).  Here the tile has eight waves: wave w owns the
// 64 x 64 quadrant w % 4 of C together with wave w ^ 4, and the two (they share a SIMD)
// split every stage's K between them: group w / 4 takes half w / 4 of the stage's 128 k (the
// 16-byte chunks 2h and 2h + 1 of a row).  Each wave thus widens the same four fragments per
// eight MFMAs as before but has half of everything to issue, and the pipe is fed by two
// instruction streams.  At the tile's end the upper group hands its accumulators to the
// lower one through LDS.  One tile per workgroup, a four-stage ring of 16 KiB stages, two
// direct-to-LDS loads per wave and stage, one barrier per stage.
constexpr int kPairTile = 128;
constexpr int kPairStages = 4;
constexpr int kPairStageBytes = 2 * kPairTile * kRowBytes;    // 16 KiB: X rows, then W rows
constexpr int kPairLdsBytes = kPairStages * kPairStageBytes;  // 64 KiB, also the merge area
constexpr int kPairRounds = 2;  // used up to this many tiles per CU (two workgroups fit a CU); measured: beyond, the 256 x 256 tiles win

//
// DEEP: the widening of a stage is interleaved with the MFMAs of the stage before it, from a
// second set of widened operands (187 registers: one workgroup per CU); otherwise it follows
// them (110 registers: two workgroups fit a CU, and their waves fill each other's gaps).
// HALF_OUT: the build for the two output kinds of 16-bit elements (a build of its own, so
// that the one for 32-bit elements carries none of its code or registers).
template <bool DEEP, bool HALF_OUT = false>
__global__ __launch_bounds__(512, DEEP ? 2 : 4) void mfma_pair_kernel(const uint8_t *__restrict__ X,
                                                        const uint8_t *__restrict__ W,
                                                        int32_t *__restrict__ Y, int M, int N, int K,
                                                        int tiles_m, int tiles_n, int ksplit, Epilogue ep)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = wave >> 2;  // which half of every stage's K
    const int quad = wave & 3;
    const int wm = quad >> 1, wn = quad & 1;
    const int rowbytes = K >> 1;
    // With ksplit > 1 workgroup v is K-slice v / tiles of tile v % tiles: it covers KT of the
    // stages and stores plain partial sums into slab v / tiles of Y (M * N int32 each).
    const int tiles = tiles_m * tiles_n;
    const int slice = blockIdx.x / tiles;
    const int KT = K / kStageK / ksplit;
    int tm, tn;
    tile_coords(blockIdx.x - slice * tiles, tiles, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * kPairTile, n0 = tn * kPairTile;
    Y += (size_t)slice * (size_t)M * (size_t)N;

    // ---- loads: wave w moves the 16-row chunk w of the X rows and of the W rows of every
    //      stage.  Lane p lands at byte 16 p of the chunk: row p / 4, slot p % 4, and fetches
    //      the row's chunk slot ^ swz(row).  Rows past the matrix re-read its last row.
    const int ld_row = lane >> 2;
    const int ld_c = (lane & 3) ^ swz(ld_row);
    const int xr = min(wave * kChunkRows + ld_row, M - 1 - m0);
    const int wr = min(wave * kChunkRows + ld_row, N - 1 - n0);
    const unsigned voff_x = (unsigned)xr * (unsigned)rowbytes + (unsigned)ld_c * 16u;
    const unsigned voff_w = (unsigned)wr * (unsigned)rowbytes + (unsigned)ld_c * 16u;
    const uint8_t *xptr = X + (size_t)m0 * rowbytes + (size_t)slice * KT * kRowBytes;
    const uint8_t *wptr = W + (size_t)n0 * rowbytes + (size_t)slice * KT * kRowBytes;
    const unsigned lds_base = (unsigned)(size_t)I4L_LDS(lds);
    const unsigned place_x = lds_base + (unsigned)(wave * kChunkBytes);
    const unsigned place_w = place_x + (unsigned)(kPairTile * kRowBytes);
    // Stage st into ring position st % 4.  Past the last stage the last one is fetched
    // again, into a buffer nobody reads any more, so that every iteration issues the same
    // number of loads and the wait below is a constant.
    auto issue = [&](int st) {
        const int src = st < KT ? st : KT - 1;
        const unsigned ring = (unsigned)((st % kPairStages) * kPairStageBytes);
        dma16(xptr + (size_t)src * kRowBytes, voff_x, place_x, ring);
        dma16(wptr + (size_t)src * kRowBytes, voff_w, place_w, ring);
    };
#pragma unroll
    for (int st = 0; st < kPairStages - 1; ++st)
        issue(st);

    // ---- math: lane (fr, fg) supplies row fr of a 32-row fragment and, of this wave's half
    //      of the stage, the 16-byte chunk fg (32 nibbles: the even ones feed one MFMA, the
    //      odd ones the next).
    const int fr = lane & 31;
    const int fg = lane >> 5;
    const unsigned rd_off = (unsigned)fr * kRowBytes + (unsigned)(((2 * half + fg) ^ swz(fr)) * 16);
    const unsigned x_rd = (unsigned)(wm * 64 * kRowBytes) + rd_off;
    const unsigned w_rd = (unsigned)((kPairTile + wn * 64) * kRowBytes) + rd_off;
    const int himask = (int)0xF0F0F0F0u;
    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int t = 0; t < 16; ++t)
                acc[i][j][t] = 0;

    if constexpr (DEEP) {
        // The MFMAs of a stage are issued one iteration late, between the LDS reads of the next
        // stage and, slot by slot, the 48 vector operations that widen that stage's fragments:
        // a wave issues in order, so widening done after the eight MFMAs would start only when the
        // last of them has been issued, i.e. when the matrix pipe has nearly run dry.  The
        // widened operands alternate between two register sets by the stage's parity; the four
        // accumulators get their even-nibble MFMAs first, then the odd-nibble ones, so that no
        // MFMA follows the one it depends on.
        v4i xlo[2][2], xhi[2][2], wlo[2][2], whi[2][2];  // [parity of the stage][fragment]
        auto arrive = [&](int st, v4i (&px)[2], v4i (&pw)[2]) {
            // Stage st has landed once this wave's two loads of it have (the loads of the two
            // younger stages may still be in flight) and every wave has said the same; by then
            // every wave has also finished reading stage st - 1, whose buffer the loads of
            // stage st + 3 now refill.
            __builtin_amdgcn_s_waitcnt(I4L_VMCNT(2 * (kPairStages - 2)));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue(st + kPairStages - 1);
            const uint8_t *stage = lds + (st % kPairStages) * kPairStageBytes;
    #pragma unroll
            for (int j = 0; j < 2; ++j)
                px[j] = *(const v4i *)(stage + x_rd + j * kFrag * kRowBytes);
    #pragma unroll
            for (int i = 0; i < 2; ++i)
                pw[i] = *(const v4i *)(stage + w_rd + i * kFrag * kRowBytes);
        };
        // Operation op (0..47) of widening the four fragments of a stage into register set P:
        // fragment op / 12 (X 0, X 1, W 0, W 1); within a fragment the four shifts, then the
        // four masks of the shifted words, then the four masks of the unshifted words.
        auto widen_op = [&](auto par_tag, int op, const v4i (&px)[2], const v4i (&pw)[2]) {
            constexpr int P = decltype(par_tag)::value;
            const int f = op / 12, k = op % 12, d = k % 4;
            const v4i &src = f < 2 ? px[f] : pw[f - 2];
            v4i &lo = f < 2 ? xlo[P][f] : wlo[P][f - 2];
            v4i &hi = f < 2 ? xhi[P][f] : whi[P][f - 2];
            if (k < 4)
                lo[d] = src[d] << 4;
            else if (k < 8)
                lo[d] = lo[d] & himask;
            else
                hi[d] = src[d] & himask;
        };
        // MFMA `slot` (0..7) of the stage whose operands are in register set P.
        auto mfma_slot = [&](auto par_tag, int slot) {
            constexpr int P = decltype(par_tag)::value;
            const int j = (slot >> 1) & 1, i = slot & 1;
            if (slot < 4)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xlo[P][j], wlo[P][i], acc[i][j], 0, 0, 0);
            else
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xhi[P][j], whi[P][i], acc[i][j], 0, 0, 0);
        };
        // Stage st (parity P) arrives and is widened while stage st - 1 is multiplied.  The first
        // two MFMAs go out bare (the LDS reads are still under way), the other six are each
        // followed by eight of the widening operations.
        auto body = [&](auto par_tag, int st) {
            constexpr int P = decltype(par_tag)::value;
            v4i px[2], pw[2];
            arrive(st, px, pw);
    #pragma unroll
            for (int slot = 0; slot < 8; ++slot) {
                mfma_slot(std::integral_constant<int, 1 - P>{}, slot);
                if (slot >= 2) {
    #pragma unroll
                    for (int op = (slot - 2) * 8; op < (slot - 1) * 8; ++op)
                        widen_op(par_tag, op, px, pw);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        {
            v4i px[2], pw[2];
            arrive(0, px, pw);
    #pragma unroll
            for (int op = 0; op < 48; ++op)
                widen_op(std::integral_constant<int, 0>{}, op, px, pw);
        }
    #pragma unroll 1
        for (int st = 1; st < KT; st += 2) {
            body(std::integral_constant<int, 1>{}, st);
            if (st + 1 < KT)
                body(std::integral_constant<int, 0>{}, st + 1);
        }
        // the last stage
        if ((KT - 1) & 1) {
    #pragma unroll
            for (int slot = 0; slot < 8; ++slot)
                mfma_slot(std::integral_constant<int, 1>{}, slot);
        } else {
    #pragma unroll
            for (int slot = 0; slot < 8; ++slot)
                mfma_slot(std::integral_constant<int, 0>{}, slot);
        }
    } else {
        // The MFMAs of a stage are issued one iteration late, behind the LDS reads of the next
        // stage, so that those reads (and the widening that waits for them) run in their shadow.
        v4i xlo[2], xhi[2], wlo[2], whi[2];
        auto multiply = [&]() {
    #pragma unroll
            for (int j = 0; j < 2; ++j)
    #pragma unroll
                for (int i = 0; i < 2; ++i) {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xlo[j], wlo[i], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xhi[j], whi[i], acc[i][j], 0, 0, 0);
                }
        };
    #pragma unroll 1
        for (int st = 0; st < KT; ++st) {
            // Stage st has landed once this wave's two loads of it have (the loads of the two
            // younger stages may still be in flight) and every wave has said the same; by then
            // every wave has also finished reading stage st - 1, whose buffer the loads of
            // stage st + 3 now refill.
            __builtin_amdgcn_s_waitcnt(I4L_VMCNT(2 * (kPairStages - 2)));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue(st + kPairStages - 1);
            const uint8_t *stage = lds + (st % kPairStages) * kPairStageBytes;
            v4i px[2], pw[2];
    #pragma unroll
            for (int j = 0; j < 2; ++j)
                px[j] = *(const v4i *)(stage + x_rd + j * kFrag * kRowBytes);
    #pragma unroll
            for (int i = 0; i < 2; ++i)
                pw[i] = *(const v4i *)(stage + w_rd + i * kFrag * kRowBytes);
            if (st > 0)
                multiply();  // stage st - 1
    #pragma unroll
            for (int j = 0; j < 2; ++j) {
                xlo[j] = (px[j] << 4) & himask;
                xhi[j] = px[j] & himask;
                wlo[j] = (pw[j] << 4) & himask;
                whi[j] = pw[j] & himask;
            }
        }
        multiply();  // the last stage
    }

    // ---- the upper group's sums go through LDS to the lower group, which stores the tile.
    //      Register r of lane l of quadrant q sits at word (q * 64 + r) * 64 + l.
    __builtin_amdgcn_s_waitcnt(I4L_VMCNT(0));  // the loads past the end have landed too
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    int *merge = (int *)lds + (size_t)quad * 64 * 64 + lane;
    if (half == 1) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < 16; ++t)
                    merge[((i * 2 + j) * 16 + t) * 64] = acc[i][j][t];
    }
    __syncthreads();
    if (half == 1)
        return;
    // X is the MFMA A operand: accumulator t of fragment (i, j) is
    //   m = 32 j + 8 (t / 4) + 4 (lane / 32) + t % 4,  n = 32 i + lane % 32.
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int t = 0; t < 16; ++t)
                acc[i][j][t] = (acc[i][j][t] + merge[((i * 2 + j) * 16 + t) * 64]) >> 8;  // both operands carried a factor 16 (exact per slice: every product is a multiple of 256)
            if constexpr (HALF_OUT) {  // the sums stay here: moved down to their uses, all 64 reads ahead of them do not fit the registers of this build
#pragma unroll
                for (int t = 0; t < 16; ++t)
                    acc[i][j][t] = opaque(acc[i][j][t]);
            }
        }
    const int mw = m0 + wm * 64 + 4 * (lane >> 5);
    const int nw = n0 + wn * 64 + (lane & 31);
    int32_t *out = Y + (size_t)mw * N + nw;
    // a half-width output as a whole (launch_mfma sends at most a few hundred tiles here)
    __amdgpu_buffer_rsrc_t rsrc16 = __builtin_amdgcn_make_buffer_rsrc(Y, 0, (int)((unsigned)M * (unsigned)N * 2u), 0x00020000);
    if (!HALF_OUT && (ksplit > 1 || (!ep.bias && !ep.row_scale && !ep.col_scale && !ep.out))) {
        // nothing to load: the stores follow one another without a wait
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int dm = 32 * j + 8 * (t / 4) + (t % 4);
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    if (mw + dm < M && nw + 32 * i < N)
                        out[(size_t)dm * N + 32 * i] = acc[i][j][t];
            }
        return;
    }
    // The epilogue's operands of this lane's columns and rows (clamped inside the matrix)
    // are fetched before the first store, so that no store waits for a load behind it.
    int bias_v[2];
    float cs_v[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int nn = min(nw + 32 * i, N - 1);
        bias_v[i] = ep.bias ? ep.bias[nn] : 0;
        cs_v[i] = ep.col_scale ? ep.col_scale[nn] : 1.f;
    }
    constexpr bool half_width = HALF_OUT;  // (no K-slices there: Y is the output's base)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        float rs[16];
#pragma unroll
        for (int t = 0; t < 16; ++t)
            rs[t] = ep.row_scale ? ep.row_scale[min(mw + 32 * j + 8 * (t / 4) + (t % 4), M - 1)] : 1.f;
        if constexpr (!half_width) {
            // The values first (opaque: they stay here), then the stores, each behind nothing
            // but its bounds test: a value computed behind the test makes every store wait
            // for the one before it.
            int v[2][16];
#pragma unroll
            for (int t = 0; t < 16; ++t)
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    v[i][t] = opaque(epilogue_value32(ep, acc[i][j][t], bias_v[i], rs[t], cs_v[i]));
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int dm = 32 * j + 8 * (t / 4) + (t % 4);
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    if (mw + dm < M && nw + 32 * i < N)
                        out[(size_t)dm * N + 32 * i] = v[i][t];
            }
        } else {
            // Stores through a descriptor over the whole output (this form only runs where
            // it is a few MiB): an element outside the matrix gets an offset beyond it and the
            // hardware drops the store, so there is no branch and no 64-bit address per store.
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int dm = 32 * j + 8 * (t / 4) + (t % 4);
                const unsigned row_off = mw + dm < M ? (unsigned)(mw + dm) * (unsigned)N * 2u : 0x80000000u;
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const unsigned col_off = nw + 32 * i < N ? (unsigned)(nw + 32 * i) * 2u : 0x40000000u;
                    __builtin_amdgcn_raw_buffer_store_b16(
                        (unsigned short)epilogue_value16(ep, acc[i][j][t], bias_v[i], rs[t], cs_v[i]), rsrc16,
                        row_off + col_off, 0, 0);
                }
            }
        }
    }
}

// The same form with a 64 x 64 tile, for grids so small that 128 x 128 tiles would leave
// most CUs without one: wave w and wave w ^ 4 own the 32 x 32 quadrant w % 4 (one
// accumulator fragment) and split every stage's K; a stage is 8 KiB, moved by one load per
// wave (waves 0..3 the four chunks of X rows, waves 4..7 those of W rows).
constexpr int kTinyTile = 64;
constexpr int kTinyStageBytes = 2 * kTinyTile * kRowBytes;    // 8 KiB
constexpr int kTinyLdsBytes = kPairStages * kTinyStageBytes;  // 32 KiB; the merge takes 16 KiB of it

template <bool HALF_OUT = false>
__global__ __launch_bounds__(512) void mfma_pair64_kernel(const uint8_t *__restrict__ X,
                                                          const uint8_t *__restrict__ W,
                                                          int32_t *__restrict__ Y, int M, int N, int K,
                                                          int tiles_m, int tiles_n, int ksplit, Epilogue ep)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = wave >> 2;  // which half of every stage's K; also: 0 loads X, 1 loads W
    const int quad = wave & 3;
    const int wm = quad >> 1, wn = quad & 1;
    const int rowbytes = K >> 1;
    // ksplit > 1: workgroup v is K-slice v / tiles of tile v % tiles, as in the larger form
    const int tiles = tiles_m * tiles_n;
    const int slice = blockIdx.x / tiles;
    const int KT = K / kStageK / ksplit;
    int tm, tn;
    tile_coords(blockIdx.x - slice * tiles, tiles, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * kTinyTile, n0 = tn * kTinyTile;
    Y += (size_t)slice * (size_t)M * (size_t)N;

    // ---- loads: lane p of a chunk lands at byte 16 p: row p / 4, slot p % 4, and fetches the
    //      row's chunk slot ^ swz(row).  Rows past the matrix re-read its last row.
    const int ld_row = lane >> 2;
    const int ld_c = (lane & 3) ^ swz(ld_row);
    const int row_here = quad * kChunkRows + ld_row;
    const int row = half ? min(row_here, N - 1 - n0) : min(row_here, M - 1 - m0);
    const unsigned voff = (unsigned)row * (unsigned)rowbytes + (unsigned)ld_c * 16u;
    const uint8_t *src_base = (half ? W + (size_t)n0 * rowbytes : X + (size_t)m0 * rowbytes) + (size_t)slice * KT * kRowBytes;
    const unsigned lds_base = (unsigned)(size_t)I4L_LDS(lds);
    const unsigned place = lds_base + (unsigned)(half * kTinyTile * kRowBytes + quad * kChunkBytes);
    auto issue = [&](int st) {  // past the last stage the last one again, into a buffer nobody reads
        const int src = st < KT ? st : KT - 1;
        dma16(src_base + (size_t)src * kRowBytes, voff, place, (unsigned)((st % kPairStages) * kTinyStageBytes));
    };
#pragma unroll
    for (int st = 0; st < kPairStages - 1; ++st)
        issue(st);

    const int fr = lane & 31;
    const int fg = lane >> 5;
    const unsigned rd_off = (unsigned)fr * kRowBytes + (unsigned)(((2 * half + fg) ^ swz(fr)) * 16);
    const unsigned x_rd = (unsigned)(wm * kFrag * kRowBytes) + rd_off;
    const unsigned w_rd = (unsigned)((kTinyTile + wn * kFrag) * kRowBytes) + rd_off;
    const int himask = (int)0xF0F0F0F0u;
    v16i acc;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        acc[t] = 0;
    v4i xlo, xhi, wlo, whi;
#pragma unroll 1
    for (int st = 0; st < KT; ++st) {
        // this wave's load of stage st has landed (two younger ones may be in flight), and
        // after the barrier everybody's; the buffer of stage st - 1 is free for stage st + 3
        __builtin_amdgcn_s_waitcnt(I4L_VMCNT(kPairStages - 2));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue(st + kPairStages - 1);
        const uint8_t *stage = lds + (st % kPairStages) * kTinyStageBytes;
        const v4i px = *(const v4i *)(stage + x_rd);
        const v4i pw = *(const v4i *)(stage + w_rd);
        if (st > 0) {  // stage st - 1, behind the reads of stage st
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xlo, wlo, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xhi, whi, acc, 0, 0, 0);
        }
        xlo = (px << 4) & himask;
        xhi = px & himask;
        wlo = (pw << 4) & himask;
        whi = pw & himask;
    }
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xlo, wlo, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xhi, whi, acc, 0, 0, 0);

    // ---- the upper group's sums go through LDS to the lower group, which stores the tile
    __builtin_amdgcn_s_waitcnt(I4L_VMCNT(0));  // the loads past the end have landed too
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    int *merge = (int *)lds + (size_t)quad * 16 * 64 + lane;
    if (half == 1) {
#pragma unroll
        for (int t = 0; t < 16; ++t)
            merge[t * 64] = acc[t];
    }
    __syncthreads();
    if (half == 1)
        return;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        acc[t] = (acc[t] + merge[t * 64]) >> 8;  // both operands carried a factor 16
    // accumulator t is  m = 8 (t / 4) + 4 (lane / 32) + t % 4,  n = lane % 32  of the quadrant
    const int mw = m0 + wm * kFrag + 4 * (lane >> 5);
    const int nw = n0 + wn * kFrag + (lane & 31);
    int32_t *out = Y + (size_t)mw * N + nw;
    // a half-width output as a whole (launch_mfma sends at most a few hundred tiles here)
    __amdgpu_buffer_rsrc_t rsrc16 = __builtin_amdgcn_make_buffer_rsrc(Y, 0, (int)((unsigned)M * (unsigned)N * 2u), 0x00020000);
    if (!HALF_OUT && (ksplit > 1 || (!ep.bias && !ep.row_scale && !ep.col_scale && !ep.out))) {
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int dm = 8 * (t / 4) + (t % 4);
            if (mw + dm < M && nw < N)
                out[(size_t)dm * N] = acc[t];
        }
        return;
    }
    const int nn = min(nw, N - 1);
    const int bias_v = ep.bias ? ep.bias[nn] : 0;
    const float cs_v = ep.col_scale ? ep.col_scale[nn] : 1.f;
    float rs[16];
#pragma unroll
    for (int t = 0; t < 16; ++t)
        rs[t] = ep.row_scale ? ep.row_scale[min(mw + 8 * (t / 4) + (t % 4), M - 1)] : 1.f;
    constexpr bool half_width = HALF_OUT;  // (no K-slices there: Y is the output's base)
    if constexpr (!half_width) {
        int v[16];  // the values first (opaque: they stay here), then the stores, each behind nothing but its bounds test
#pragma unroll
        for (int t = 0; t < 16; ++t)
            v[t] = opaque(epilogue_value32(ep, acc[t], bias_v, rs[t], cs_v));
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int dm = 8 * (t / 4) + (t % 4);
            if (mw + dm < M && nw < N)
                out[(size_t)dm * N] = v[t];
        }
    } else {
        // (stores through a descriptor over the whole output, as in mfma_pair_kernel)
        const unsigned col_off = nw < N ? (unsigned)nw * 2u : 0x40000000u;
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int dm = 8 * (t / 4) + (t % 4);
            const unsigned row_off = mw + dm < M ? (unsigned)(mw + dm) * (unsigned)N * 2u : 0x80000000u;
            __builtin_amdgcn_raw_buffer_store_b16((unsigned short)epilogue_value16(ep, acc[t], bias_v, rs[t], cs_v),
                                                  rsrc16, row_off + col_off, 0, 0);
        }
    }
}

// 256 x 256 tile, eight wavefronts of 128 (m) x 64 (n), one workgroup per CU, two
// wavefronts per SIMD: the large-shape configuration.
using CfgLarge = TileConfig<2, 4, 4, 2, 4, 1>;
// 128 x 128 tile, four wavefronts of 64 x 64, two workgroups per CU: mid-sized shapes
// whose 256 x 256 tile count would leave CUs idle.
using CfgMedium = TileConfig<2, 2, 2, 2, 4, 2>;

template <class C>
hipError_t set_lds_limit()
{
    return hipFuncSetAttribute((const void *)mfma_gemm_kernel<C>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
}

template <class C>
hipError_t launch_cfg(const void *a, const void *b, void *c, int m, int n, int k,
                      const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream, int ksplit = 1)
{
    const int tiles_m = (m + C::BM - 1) / C::BM;
    const int tiles_n = (n + C::BN - 1) / C::BN;
    const long total = (long)tiles_m * tiles_n * ksplit;
    if (total > 0x7fffffffL)
        return hipErrorInvalidValue;
    long grid = (long)dev.cu_count * C::OCC;
    if (grid > total)
        grid = total;
    // The epilogue addresses a tile's slab of C with 32-bit byte offsets below 2^30.
    if ((size_t)C::BM * (size_t)n * 4u > 0x40000000ull)
        return hipErrorInvalidValue;
    mfma_gemm_kernel<C><<<(unsigned)grid, C::THREADS, C::LDS_BYTES, stream>>>(
        (const uint8_t *)a, (const uint8_t *)b, (int32_t *)c, m, n, k, tiles_m, tiles_n, ksplit, ep);
    return hipGetLastError();
}

}  // namespace

bool mfma_supports(int m, int n, int k)
{
    // K <= 131071 keeps 256 * (sum of products) inside int32; one LDS row per stage is
    // 128 nibbles.
    // The store addresses a tile's rows of C (at most 256) with byte offsets below 2^30.
    return m >= 1 && n >= 1 && n <= (1 << 20) && k >= kStageK && k % kStageK == 0 && k <= 131071 - 127;
}

hipError_t mfma_init(const DeviceInfo &dev)
{
    if (dev.lds_per_cu < CfgLarge::LDS_BYTES)
        return hipErrorInvalidConfiguration;
    hipError_t e = set_lds_limit<CfgLarge>();
    if (e != hipSuccess)
        return e;
    return set_lds_limit<CfgMedium>();
}

hipError_t launch_mfma_tile(const void *a, const void *b, void *c, int m, int n, int k, int tile,
                            const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    if (tile == 256)
        return launch_cfg<CfgLarge>(a, b, c, m, n, k, ep, dev, stream);
    if (tile == 128)
        return launch_cfg<CfgMedium>(a, b, c, m, n, k, ep, dev, stream);
    return hipErrorInvalidValue;
}

// K-slices per tile for shapes with few tiles and long K: at most half as many 128 x 128
// tiles as CUs at K >= 12288, or a sixteenth at K >= 8192 (measured against the unsplit
// 64 x 64 form, which wins everywhere else: e.g. 160 x 4096 x 4096 9.6 against 16 us,
// 1024 x 512 x 8192 16 against 20 us, but 128 x 4096 x 14336 26 against 19.5 us and
// 512 x 4096 x 14336 52 against 41 us): the largest
// divisor of the stage count
// that keeps at least eight stages per slice, at most eight slices, and at most half a
// work item per slot.
int mfma_ksplit(int m, int n, int k, const DeviceInfo &dev)
{
    if (!mfma_supports(m, n, k))
        return 1;
    const long tiles = (long)((m + CfgMedium::BM - 1) / CfgMedium::BM) * ((n + CfgMedium::BN - 1) / CfgMedium::BN);
    const long slots = (long)dev.cu_count * CfgMedium::OCC;
    const int stages = k / kStageK;
    const bool few_tiles = tiles * 16 <= dev.cu_count && stages >= 64;
    const bool long_k = tiles * 2 <= dev.cu_count && stages >= 96;
    if (!few_tiles && !long_k)
        return 1;
    long limit = slots / (2 * tiles);
    if (limit > 8)
        limit = 8;
    int best = 1;
    for (int d = 2; d <= limit; ++d)
        if (stages % d == 0 && stages / d >= 8)
            best = d;
    return best;
}

size_t mfma_workspace_bytes(int m, int n, int k, const DeviceInfo &dev)
{
    const int d = mfma_ksplit(m, n, k, dev);
    return d > 1 ? (size_t)d * (size_t)m * (size_t)n * 4u : 0;
}

hipError_t launch_mfma_splitk(const void *a, const void *b, void *c, int m, int n, int k, void *workspace,
                              const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    const int d = mfma_ksplit(m, n, k, dev);
    if (d <= 1 || !workspace)
        return launch_mfma(a, b, c, m, n, k, ep, dev, stream);
    // the K-slices run as work items of the small-grid form
    const int pair_m = (m + kPairTile - 1) / kPairTile, pair_n = (n + kPairTile - 1) / kPairTile;
    // With very few tiles (a sixteenth as many as CUs) the slices are 64 x 64 tiles, as many
    // slices as leave at most two work items per CU (200 x 136 x 16384: 15.3 -> 11.6 us; with
    // more tiles the 128 x 128 slices are as fast or faster).
    if ((long)pair_m * pair_n * 16 <= dev.cu_count) {
        const int tiny_m = (m + kTinyTile - 1) / kTinyTile, tiny_n = (n + kTinyTile - 1) / kTinyTile;
        const int stages = k / kStageK;
        int dt = 1;  // at most d: the slabs have room for d slices
        for (int q = 2; q <= d; ++q)
            if (stages % q == 0 && (long)tiny_m * tiny_n * q <= (long)dev.cu_count * 2)
                dt = q;
        mfma_pair64_kernel<false><<<(unsigned)(tiny_m * tiny_n * dt), 512, kTinyLdsBytes, stream>>>(
            (const uint8_t *)a, (const uint8_t *)b, (int32_t *)workspace, m, n, k, tiny_m, tiny_n, dt, Epilogue{});
        const hipError_t e2 = hipGetLastError();
        if (e2 != hipSuccess)
            return e2;
        return launch_splitk_reduce(workspace, c, (size_t)m * (size_t)n, dt, n, ep, stream);
    }
    if ((long)pair_m * pair_n * d <= dev.cu_count)
        mfma_pair_kernel<true><<<(unsigned)(pair_m * pair_n * d), 512, kPairLdsBytes, stream>>>(
            (const uint8_t *)a, (const uint8_t *)b, (int32_t *)workspace, m, n, k, pair_m, pair_n, d, Epilogue{});
    else
        mfma_pair_kernel<false><<<(unsigned)(pair_m * pair_n * d), 512, kPairLdsBytes, stream>>>(
            (const uint8_t *)a, (const uint8_t *)b, (int32_t *)workspace, m, n, k, pair_m, pair_n, d, Epilogue{});
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return e;
    return launch_splitk_reduce(workspace, c, (size_t)m * (size_t)n, d, n, ep, stream);
}

hipError_t launch_mfma(const void *a, const void *b, void *c, int m, int n, int k,
                       const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    const long tiles_large = (long)((m + CfgLarge::BM - 1) / CfgLarge::BM) *
                             ((n + CfgLarge::BN - 1) / CfgLarge::BN);
    // Few 128 x 128 tiles per CU: the form whose two waves per SIMD split K.
    const int pair_m = (m + kPairTile - 1) / kPairTile, pair_n = (n + kPairTile - 1) / kPairTile;
    // ... and so few that they would leave half of the CUs idle or more: 64 x 64 tiles
    // (measured: 512 x 4096 x 4096 17 -> 14.5 us, 1024 x 1024 x 2048 10.8 -> 7.8 us; with more
    // than cu_count / 2 tiles of 128 x 128 the larger tile wins).
    if ((long)pair_m * pair_n * 2 <= dev.cu_count) {
        const int tiny_m = (m + kTinyTile - 1) / kTinyTile, tiny_n = (n + kTinyTile - 1) / kTinyTile;
        if (ep.out >= kOutF16)
            mfma_pair64_kernel<true><<<(unsigned)(tiny_m * tiny_n), 512, kTinyLdsBytes, stream>>>(
                (const uint8_t *)a, (const uint8_t *)b, (int32_t *)c, m, n, k, tiny_m, tiny_n, 1, ep);
        else
            mfma_pair64_kernel<false><<<(unsigned)(tiny_m * tiny_n), 512, kTinyLdsBytes, stream>>>(
                (const uint8_t *)a, (const uint8_t *)b, (int32_t *)c, m, n, k, tiny_m, tiny_n, 1, ep);
        return hipGetLastError();
    }
    if ((long)pair_m * pair_n <= (long)dev.cu_count * kPairRounds) {
        const bool deep = (long)pair_m * pair_n <= dev.cu_count, half_out = ep.out >= kOutF16;
        auto *kern = deep ? (half_out ? mfma_pair_kernel<true, true> : mfma_pair_kernel<true, false>)
                          : (half_out ? mfma_pair_kernel<false, true> : mfma_pair_kernel<false, false>);
        kern<<<(unsigned)(pair_m * pair_n), 512, kPairLdsBytes, stream>>>(
            (const uint8_t *)a, (const uint8_t *)b, (int32_t *)c, m, n, k, pair_m, pair_n, 1, ep);
        return hipGetLastError();
    }
    // Use the big tile once it alone can occupy every CU.
    if (tiles_large >= dev.cu_count)
        return launch_cfg<CfgLarge>(a, b, c, m, n, k, ep, dev, stream);
    return launch_cfg<CfgMedium>(a, b, c, m, n, k, ep, dev, stream);
}

}  // namespace int4linear
