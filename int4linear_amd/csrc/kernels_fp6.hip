// FP6-MFMA GEMM over signed-int4 operands for gfx950 (CDNA4), exact in int32.
//
// CDNA4's matrix cores run the 6-bit float format E2M3 at twice the int8 rate
// (v_mfma_scale_f32_32x32x64_f8f6f4: 32x32x64 per instruction in the time the int8
// instruction does 32x32x32), and E2M3 holds every signed 4-bit integer exactly:
// sign, two exponent bits and three mantissa bits encode n/8 for n = -15..15 as the plain
// sign-magnitude integer |n| with the sign in bit 5 (subnormals 0..7 are |n| itself, 8 is
// exponent 1 with mantissa 0).  The instruction is used without block scales (both scale
// arguments zero select the unscaled opcode, one instruction where the scaled one is a
// pair), so a product is n*m/64, the fp32 accumulator holds multiples of 1/64, which fp32
// represents exactly while |sum of n*m| < 2^24, i.e. for K * 64 < 2^24, and the store
// multiplies by 64 (exact) before the conversion to int32.  The launcher refuses larger K;
// the result is bit-identical to integer arithmetic (the tests compare it against the CPU
// oracle).
//
// Two kernels:
//   * fp6_convert_kernel rewrites packed s4 operands (rows x K/2 bytes) into FP6
//     "fragment-major" form in a workspace: for every block of 32 rows x 64 k the 24
//     bytes each of the 64 MFMA lanes feeds to the instruction, stored as 64 x 16 B
//     followed by 64 x 8 B.  Rows are padded with zeros to a multiple of the 256-row
//     tile.  One launch converts both operands.  HBM-bound: 0.5 B read and 0.75 B
//     written per element.
//   * fp6_gemm_kernel is a persistent, LDS-pipelined GEMM over those fragments.  Because
//     the workspace is already in the order lanes consume it, global->LDS is a linear
//     direct-to-LDS copy, LDS->VGPR is one 16-byte and one 8-byte read per lane per
//     fragment at consecutive addresses (no swizzle, no bank conflicts), and the main loop
//     contains no VALU work at all.  With few output tiles and long K its work items are
//     K-slices of tiles, which store partial sums into slabs of the workspace.
//     (launch_splitk_reduce adds those slabs up and applies the epilogue).
//
// Order of k inside a fragment is whatever the converter produces; it only has to be the
// same for both operands, which it is because both go through the same converter.
#include "kernels.h"

#include <type_traits>
#include <utility>

namespace int4linear {

namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define I4L_LDS(p) ((__attribute__((address_space(3))) void *)(p))
// s_waitcnt immediate for gfx9: vmcnt[3:0] bits 3:0, vmcnt[5:4] bits 15:14, expcnt bits
// 6:4, lgkmcnt bits 11:8.  VM only leaves the others at "no wait".
#define I4L_WAIT_VM(n) ((0x0F70) | ((n) & 0xF) | ((((n) >> 4) & 0x3) << 14))
#define I4L_WAIT_LGKM0 0xC07F

constexpr int kTileRows = 256;                        // rows of either operand per tile
constexpr int kFragRows = 32;                         // rows of one MFMA operand
constexpr int kFragK = 64;                            // k of one MFMA
constexpr int kFragBytes = 64 * 24;                   // 64 lanes x 192 bits
constexpr int kFragLoBytes = 64 * 16;                 // the 16-byte parts come first
constexpr int kStageK = 128;                          // k per pipeline stage
constexpr int kFragsK = kStageK / kFragK;             // 2
constexpr int kFragsRows = kTileRows / kFragRows;     // 8
constexpr int kOperandStageBytes = kFragsK * kFragsRows * kFragBytes;  // 24 KiB
constexpr int kStageBytes = 2 * kOperandStageBytes;                    // 48 KiB
constexpr int kStages = 3;
constexpr int kLdsBytes = kStages * kStageBytes;                       // 144 KiB
constexpr int kStaggerGroups = 8;                     // start groups within an XCD (power of two)
constexpr int kStaggerTicks = 120;                    // delay between groups, in 10-ns ticks of the constant clock
constexpr int kStaggerMinRounds = 2;                  // tiles per workgroup from which the start is staggered
constexpr float kUnscale = 64.f;                      // the codes are n/8: a product is n*m/64

// ---- converter --------------------------------------------------------------------------

// Four nibble values (one per byte of x, 0..15 meaning 0..7,-8..-1) -> four E2M3 codes
// (sign << 5 | magnitude), one per byte.
__device__ __forceinline__ unsigned fp6_codes(unsigned x)
{
    const unsigned s = x & 0x08080808u;   // sign bits
    const unsigned t = s >> 3;            // 1 in negative bytes
    const unsigned m = t * 15u;           // 0x0F in negative bytes
    const unsigned mag = (x ^ m) + t;     // 16 - x for negatives, x otherwise
    return mag | (s << 2);
}

// Four 6-bit codes, one per byte -> 24 contiguous bits.
__device__ __forceinline__ unsigned pack_codes(unsigned c)
{
    const unsigned t = (c & 0x003F003Fu) | ((c >> 2) & 0x0FC00FC0u);  // 12 bits per half
    return (t & 0x00000FFFu) | ((t >> 4) & 0x00FFF000u);
}

// One packed dword (8 nibbles) -> 48 bits of FP6 codes.
__device__ __forceinline__ unsigned long long fp6_from_dword(unsigned w)
{
    const unsigned even = pack_codes(fp6_codes(w & 0x0F0F0F0Fu));
    const unsigned odd = pack_codes(fp6_codes((w >> 4) & 0x0F0F0F0Fu));
    return (unsigned long long)even | ((unsigned long long)odd << 24);
}

// Workspace index of the fragment (tile, stage, k-fragment, row-fragment).
__device__ __forceinline__ size_t frag_offset(int tile, int stage, int kf, int rf, int stages)
{
    return ((((size_t)tile * stages + stage) * kFragsK + kf) * kFragsRows + rf) * (size_t)kFragBytes;
}

// One operand of a conversion launch.
struct ConvertJob {
    const uint8_t *src;   // packed s4, rows x k/2 bytes
    uint8_t *dst;         // fragment-major FP6
    int rows;             // real rows; rows up to the next multiple of 256 are written as zeros
    int row_blocks;       // 32-row blocks including the padding
};

constexpr int kConvK = 512;                          // k per converter workgroup
constexpr int kConvFrags = kConvK / kFragK;          // 8 fragments out
constexpr int kConvChunks = kConvK / 32;             // 16-byte input chunks per row
// LDS stride of a fragment being assembled: 64 bytes more than its size, so that the eight
// lanes of a wave that write the same lane slot of different fragments hit different banks.
constexpr int kConvFragLds = kFragBytes + 64;

// One workgroup converts 32 rows x 512 k of one operand: thread t reads the 16-byte chunks
// t%8 and t%8 + 8 of row t/8 (eight neighbouring lanes fetch a whole 128-byte line), the
// FP6 fragments are assembled in LDS, and the eight finished fragments (1536 contiguous
// bytes each) leave with full-line 16-byte stores.  blockIdx.y selects the operand and the
// 32-row block, so one launch converts both A and B.
// k is the operand's real K (a multiple of 8; the row stride is k/2 bytes), k_pad the next
// multiple of 128: k positions from k up to k_pad are written as zeros.  ALIGNED16: k is a
// multiple of 32, so every 16-byte chunk of a row is aligned and entirely inside the row.
template <bool ALIGNED16>
__global__ __launch_bounds__(256) void fp6_convert_kernel(ConvertJob ja, ConvertJob jb, int k, int k_pad)
{
    __shared__ __attribute__((aligned(16))) uint8_t out[kConvFrags * kConvFragLds];
    const bool second = (int)blockIdx.y >= ja.row_blocks;
    const ConvertJob job = second ? jb : ja;
    const int rb = second ? blockIdx.y - ja.row_blocks : blockIdx.y;
    const int r = threadIdx.x >> 3;
    const int c = threadIdx.x & 7;
    const int row = rb * kFragRows + r;
    const int stages = k_pad / kStageK;
    const int kchunk0 = blockIdx.x * kConvChunks;
    const int chunks_here = min(kConvChunks, (k_pad >> 5) - kchunk0);   // k_pad % 512 may be 128..384

    v4i w[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int kc = c + 8 * h;
        w[h] = (v4i){0, 0, 0, 0};
        const int k0 = (kchunk0 + kc) * 32;  // first k of the chunk
        const uint8_t *src = job.src + (size_t)row * (k >> 1) + (size_t)(kchunk0 + kc) * 16;
        if (ALIGNED16) {
            if (row < job.rows && k0 < k)
                w[h] = __builtin_nontemporal_load((const v4i *)src);
        } else {
#pragma unroll
            for (int d = 0; d < 4; ++d)
                if (row < job.rows && k0 + 8 * d < k)
                    w[h][d] = *(const int *)(src + 4 * d);
        }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const unsigned long long q0 = fp6_from_dword((unsigned)w[h][0]);
        const unsigned long long q1 = fp6_from_dword((unsigned)w[h][1]);
        const unsigned long long q2 = fp6_from_dword((unsigned)w[h][2]);
        const unsigned long long q3 = fp6_from_dword((unsigned)w[h][3]);
        const unsigned long long o0 = q0 | (q1 << 48);
        const unsigned long long o1 = (q1 >> 16) | (q2 << 32);
        const unsigned long long o2 = (q2 >> 32) | (q3 << 16);
        const int kc = c + 8 * h;
        const int lane = (kc & 1) * 32 + r;
        uint8_t *frag = out + (kc >> 1) * kConvFragLds;
        *(v4i *)(frag + lane * 16) = (v4i){(int)o0, (int)(o0 >> 32), (int)o1, (int)(o1 >> 32)};
        *(v2i *)(frag + kFragLoBytes + lane * 8) = (v2i){(int)o2, (int)(o2 >> 32)};
    }
    __syncthreads();

    // Fragment f of this workgroup is k-fragment kfrag0 + f of the row block.
    const int tile = row / kTileRows;                 // uniform in the workgroup
    const int rf = rb % kFragsRows;
    const int kfrag0 = kchunk0 >> 1;
    const int frags_here = chunks_here >> 1;
    constexpr int kVecPerFrag = kFragBytes / 16;      // 96
    for (int i = threadIdx.x; i < frags_here * kVecPerFrag; i += 256) {
        const int f = i / kVecPerFrag, v = i % kVecPerFrag;
        const int kfrag = kfrag0 + f;
        uint8_t *dst = job.dst + frag_offset(tile, kfrag / kFragsK, kfrag % kFragsK, rf, stages);
        *(v4i *)(dst + v * 16) = *(const v4i *)(out + f * kConvFragLds + v * 16);
    }
}

// ---- GEMM ---------------------------------------------------------------------------------

// 16 bytes per lane from sbase + voff + IMM straight into LDS at place + ring + IMM + 16 * lane
// (the hardware adds the instruction's constant on both sides, which is what a linear copy
// wants; the two scalar summands of the LDS address are added on the way into M0).
template <int IMM>
__device__ __forceinline__ void dma16(const void *sbase, unsigned voff, unsigned place, unsigned ring)
{
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate");
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%4"
                 :
                 : "v"(voff), "s"(sbase), "s"(place), "s"(ring), "n"(IMM)
                 : "memory", "scc");
}

// Marks a value as used at this point of the program without generating code.
__device__ __forceinline__ void pin(const v16f &v) { asm volatile("" ::"v"(v)); }

__device__ __forceinline__ int opaque(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// Same XCD-aware grouped tile order as the int8 kernel: workgroup ids go round-robin
// over 8 XCDs; ids congruent mod 8 get consecutive positions of an 8-tile-row-tall,
// column-major grouped order so that concurrent tiles of one XCD share operand rows in L2.
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

// WAVES_M x WAVES_N wavefronts per workgroup; each owns FM x FN MFMA tiles of 32x32.
template <int WAVES_M_, int WAVES_N_, int OCC_>
struct Fp6Config {
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, OCC = OCC_;
    static constexpr int NWAVES = WAVES_M * WAVES_N;
    static constexpr int THREADS = NWAVES * 64;
    static constexpr int FM = kTileRows / kFragRows / WAVES_M;
    static constexpr int FN = kTileRows / kFragRows / WAVES_N;
    static constexpr int CHUNKS = kStageBytes / 1024;  // 1-KiB direct-to-LDS loads per stage
    static constexpr int CH = CHUNKS / NWAVES;         // per wave
    static constexpr int STORES = FM * FN * 16;        // dword stores per lane per tile
    static constexpr int SLOTS = FM * FN;              // MFMAs per unit (one k-fragment)
    static_assert(CHUNKS % NWAVES == 0 && CH % 2 == 0 && CH <= 63, "loads must split evenly");
};

// What the GEMM kernel is put together from.  The library builds WholeKernel and nothing else;
// tests/host/fp6_ablation.cpp, which compiles this file again, passes variations of its own
// (derived from this one, with single members changed) to time what each part costs.
struct WholeKernel {
    static constexpr bool kStores = true;    // a finished tile is stored
    static constexpr bool kLoads = true;     // global -> LDS loads go on after the prologue
    static constexpr bool kLdsReads = true;  // LDS -> register reads go on after the prologue
    static constexpr bool kOwnTile = true;   // a tile reads its own operands (false: those of tile (0, 0), L2-resident)
    static constexpr bool kStagger = true;   // workgroups of an XCD start in groups (see the kernel)
    static constexpr bool kFences = true;    // every MFMA and its share of the housekeeping are fenced off from the scheduler
    // Called by lane 0 of wave 0 when the workgroup starts and after its last tile.
    __device__ static void stamp(const Epilogue &, int /* workgroup */, int /* 0: start, 1: end */) {}
};

// HALF_OUT: the build for the two output kinds of 16-bit elements (its own build, so that the
// one for 32-bit elements carries none of its code).
template <class C, bool HALF_OUT = false, class Parts = WholeKernel>
__global__ __launch_bounds__(C::THREADS, C::OCC) void fp6_gemm_kernel(
    const uint8_t *__restrict__ XW, const uint8_t *__restrict__ WW, int32_t *__restrict__ Y,
    int M, int N, int K, int tiles_m, int tiles_n, int ksplit, Epilogue ep)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / C::WAVES_N;
    const int wn = wave % C::WAVES_N;
    // With ksplit > 1 a work item is one K-slice of one tile: item v is slice v / tiles of
    // tile v % tiles (so the items of one slice are laid out like the tiles of an unsplit
    // launch), covers KT of the KT_all stages, and stores its plain partial sums into slab
    // `slice` of Y (M * N int32 each), which a second kernel adds up.
    const int KT_all = K / kStageK;
    const int KT = KT_all / ksplit;
    const int tiles = tiles_m * tiles_n;
    const int total_tiles = tiles * ksplit;  // work items
    const int nblk = gridDim.x;
    const int bid = blockIdx.x;
    const bool ep_plain = !HALF_OUT && (ksplit > 1 || (!ep.bias && !ep.row_scale && !ep.col_scale && !ep.out));
    if (bid >= total_tiles)
        return;
    const int my_tiles = (total_tiles - bid + nblk - 1) / nblk;
    // ---- load side: stage = 24 KiB of X fragments then 24 KiB of W fragments, copied
    //      linearly; wave w moves CH/2 consecutive 1-KiB chunks of either half, so that the
    //      chunks of a half differ only in the instruction's constant.
    const uint8_t *xptr = XW, *wptr = WW;  // wave-uniform: this tile's current stage
    int ld_it = 0, ld_k = 0;
    const unsigned lds_base = (unsigned)(size_t)I4L_LDS(lds);
    const unsigned lane16 = (unsigned)lane * 16u;
    constexpr int kHalfChunks = C::CH / 2;
    static_assert(kHalfChunks * 1024 <= 4096, "a wave's chunks of one half must be within reach of the constant");
    const unsigned ld_voff = lane16 + (unsigned)(wave * kHalfChunks * 1024);
    const unsigned place_x = lds_base + (unsigned)(wave * kHalfChunks * 1024);
    const unsigned place_w = place_x + (unsigned)kOperandStageBytes;
    unsigned wr_ring = 0;  // the prologue's: offset of the stage buffer being filled

    auto ld_setup_tile = [&](int it) {
        int tm, tn;
        const int item = bid + it * nblk;
        const int slice = item / tiles;
        tile_coords(item - slice * tiles, tiles, tiles_m, tiles_n, tm, tn);
        if constexpr (!Parts::kOwnTile)
            tm = tn = 0;
        xptr = XW + ((size_t)tm * KT_all + (size_t)slice * KT) * kOperandStageBytes;
        wptr = WW + ((size_t)tn * KT_all + (size_t)slice * KT) * kOperandStageBytes;
    };
    auto ld_chunk = [&](auto c, unsigned ring) {  // c < CH/2: X half, else W half; ring: the buffer's offset
        constexpr int cc = decltype(c)::value;
        if constexpr (cc < kHalfChunks)
            dma16<cc * 1024>(xptr, ld_voff, place_x, ring);
        else
            dma16<(cc - kHalfChunks) * 1024>(wptr, ld_voff, place_w, ring);
    };
    auto ld_advance = [&]() {
        wr_ring = wr_ring + kStageBytes == kLdsBytes ? 0u : wr_ring + kStageBytes;
        ++ld_k;
        xptr += kOperandStageBytes;
        wptr += kOperandStageBytes;
        if (ld_k == KT) {
            if (ld_it + 1 < my_tiles) {
                ld_k = 0;
                ++ld_it;
                ld_setup_tile(ld_it);
            } else {
                // Past the last stage the cursor stays on it: the loop keeps issuing loads
                // unconditionally, and these re-read valid data into buffers nobody reads.
                ld_k = KT - 1;
                xptr -= kOperandStageBytes;
                wptr -= kOperandStageBytes;
            }
        }
    };

    // Prologue: stages 0 and 1 in full and the first half of stage 2's loads.  From then on
    // every iteration gs finishes stage gs+2 in its first unit and begins stage gs+3 in its
    // second, so the loop body needs no branch around a load.
    ld_setup_tile(0);
    auto ld_chunks = [&]<int... CC>(std::integer_sequence<int, CC...>) {
        (ld_chunk(std::integral_constant<int, CC>{}, wr_ring), ...);
    };
#pragma unroll
    for (int s = 0; s < kStages - 1; ++s) {
        ld_chunks(std::make_integer_sequence<int, C::CH>{});
        ld_advance();
    }
    ld_chunks(std::make_integer_sequence<int, C::CH / 2>{});

    // ---- math side.  Unit u = (stage, k-fragment kf); its operands are FM X fragments
    //      and FN W fragments, each 6 VGPRs read as 16 + 8 bytes.  While the MFMAs of unit
    //      u run, the fragments of unit u+1 are read into the other register set.
    const unsigned x_rd = (unsigned)(wm * C::FM * kFragBytes) + lane16;
    const unsigned w_rd = (unsigned)(kOperandStageBytes + wn * C::FN * kFragBytes) + lane16;
    const unsigned hi_delta = (unsigned)kFragLoBytes - (unsigned)lane * 8u;  // from the 16-B to the 8-B part

    v16f acc[C::FN][C::FM];
    v4i xlo[2][C::FM], wlo[2][C::FN];  // first 128 bits of each fragment's 192
    v2i xhi[2][C::FM], whi[2][C::FN];  // last 64 bits
    int cur_it = 0, kk = 0;

    // Read instruction r (0 .. 2*(FM+FN)-1) of unit (st, kf) into register set p:
    // fragment r/2, 16-byte part for even r, 8-byte part for odd r; X fragments first.
    auto read_op = [&](unsigned ring, int kf, int p, int r) {  // ring: offset of the stage's buffer
        const uint8_t *base = lds + ring + kf * kFragsRows * kFragBytes;
        const int f = r >> 1;
        const bool is_x = f < C::FM;
        const int idx = is_x ? f : f - C::FM;
        const uint8_t *a = base + (is_x ? x_rd : w_rd) + idx * kFragBytes;
        if ((r & 1) == 0)
            (is_x ? xlo[p][idx] : wlo[p][idx]) = *(const v4i *)a;
        else
            (is_x ? xhi[p][idx] : whi[p][idx]) = *(const v2i *)(a + hi_delta);
    };
    auto frag = [](const v4i &lo, const v2i &hi) {
        return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], 0, 0};
    };
    constexpr int kReads = 2 * (C::FM + C::FN);

    // The MFMAs of the unit held in register set p; `hook(slot)` is housekeeping placed
    // behind the MFMA of that slot.
    auto unit = [&](auto p_tag, auto &&hook) {
        constexpr int p = decltype(p_tag)::value;
        [&]<int... SLOT>(std::integer_sequence<int, SLOT...>) {
            ([&] {
                constexpr int j = SLOT / C::FN, i = SLOT % C::FN;
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    frag(xlo[p][j], xhi[p][j]), frag(wlo[p][i], whi[p][i]), acc[i][j], 2, 2, 0, 0, 0,
                    0);
                // An MFMA has no side effect, so nothing stops the optimiser from moving it
                // down to its next use, past the housekeeping meant to run in its shadow;
                // this empty statement "uses" the result here and keeps the MFMA in place.
                pin(acc[i][j]);
                if constexpr (Parts::kFences)
                    __builtin_amdgcn_sched_barrier(0);
                hook(std::integral_constant<int, SLOT>{});
                if constexpr (Parts::kFences)
                    __builtin_amdgcn_sched_barrier(0);
            }(), ...);
        }(std::make_integer_sequence<int, C::SLOTS>{});
    };

    // Housekeeping positions inside a unit of SLOTS slots: the kReads LDS reads of the
    // next unit go two per slot from slot 0 (so they have landed well before the unit
    // ends), the CH/2 direct-to-LDS loads one per slot from slot SLOTS/2.
    constexpr int kReadsPerSlot = 2;
    constexpr int kDmaFirstSlot = C::SLOTS / 2;
    static_assert(kReads <= kReadsPerSlot * C::SLOTS, "not enough slots for the LDS reads");
    static_assert(kDmaFirstSlot + C::CH / 2 <= C::SLOTS, "not enough slots for the loads");
    auto spread = [&](auto slot_tag, unsigned read_ring, int read_kf, int read_p, auto half_pos, unsigned load_ring) {
        constexpr int slot = decltype(slot_tag)::value;
        if constexpr (Parts::kLdsReads) {
#pragma unroll
            for (int r = slot * kReadsPerSlot; r < (slot + 1) * kReadsPerSlot && r < kReads; ++r)
                read_op(read_ring, read_kf, read_p, r);
        }
        if constexpr (Parts::kLoads && slot >= kDmaFirstSlot && slot < kDmaFirstSlot + C::CH / 2) {
            ld_chunk(std::integral_constant<int, decltype(half_pos)::value * (C::CH / 2) + slot - kDmaFirstSlot>{}, load_ring);
        }
    };

    // Workgroups that start together reach every tile end together, and the stores of all
    // tiles then queue for the same path to memory while no CU computes.  With two or
    // more tiles per workgroup the 32 workgroups of an XCD (ids congruent mod 8) therefore
    // start in eight groups about a microsecond apart: their tile ends stay that
    // far apart for the rest of the launch, which costs the spread once at the end and
    // saves most of the wait at every tile end before.  (The wait sits behind the first loads,
    // which travel meanwhile.)
    if (threadIdx.x == 0)
        Parts::stamp(ep, bid, 0);
    if (Parts::kStagger && total_tiles >= kStaggerMinRounds * nblk) {
        const int grp = (bid >> 3) & (kStaggerGroups - 1);
        const unsigned long long until = wall_clock64() + (unsigned long long)(grp * kStaggerTicks);
        while (wall_clock64() < until)
            __builtin_amdgcn_s_sleep(2);
    }

    // Stage 0 must have landed before the first read; stage 1 and half of stage 2 are
    // in flight behind it.
    __builtin_amdgcn_s_waitcnt(I4L_WAIT_VM(C::CH + C::CH / 2));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < kReads; ++r)
        read_op(0u, 0, 0, r);
    if constexpr (!Parts::kLdsReads) {
#pragma unroll
        for (int r = 0; r < kReads; ++r)
            read_op(0u, 1, 1, r);
    }

    int stores_behind = 0;  // a tile has just been stored: its stores sit behind the loads waited for next
    // One iteration of the stage loop, for the stage whose buffer is ring position RING.  The
    // loop below is unrolled over the three positions, so that every LDS address is a
    // loop-invariant register plus a constant and every buffer offset a constant.
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < C::FN; ++i)
#pragma unroll
            for (int j = 0; j < C::FM; ++j)
#pragma unroll
                for (int t = 0; t < 16; ++t)
                    acc[i][j][t] = 0.f;
    };
    clear_acc();
    // Returns true after the block's last tile.  Whatever a stage does only at a tile's end
    // (store, clear the accumulators, test for the end) sits behind the one branch on kk.
    auto iteration = [&](auto ring_tag) -> bool {
        constexpr unsigned rd_cur = decltype(ring_tag)::value * kStageBytes;              // stage gs
        constexpr unsigned rd_next = (decltype(ring_tag)::value + 1) % kStages * kStageBytes;  // stage gs+1
        constexpr unsigned wr_first = (decltype(ring_tag)::value + 2) % kStages * kStageBytes; // stage gs+2
        constexpr unsigned wr_second = rd_cur;                                            // stage gs+3
        // ---- unit (gs, 0): reads unit (gs, 1); finishes the loads of stage gs+2
        unit(std::integral_constant<int, 0>{}, [&](auto slot_tag) {
            spread(slot_tag, rd_cur, 1, 1, std::integral_constant<int, 1>{}, wr_first);
            if constexpr (decltype(slot_tag)::value == C::SLOTS - 1)
                ld_advance();
        });

        // ---- between the units: every LDS read of stage gs has been issued; once they
        //      have returned (lgkmcnt 0) and every wave is here, the buffer of stage gs is
        //      free for stage gs+3.  Stage gs+1 must have landed: memory operations complete
        //      in order and normally one younger stage (gs+2) is in flight behind it.  In
        //      the first stage after a tile end that tile's C stores sit behind it as well:
        //      they are more than the counter can hold (63), so their issue has already
        //      waited for everything older, and no wait is wanted (one for CH would stall
        //      until the stores have drained).  The common case falls through the branch.
        {
            static_assert(C::STORES >= 64, "the stores of a tile must saturate the counter");
            asm volatile("s_cmp_lg_u32 %0, 0\n\t"
                         "s_cbranch_scc1 1f\n\t"
                         "s_waitcnt vmcnt(%1)\n"
                         "1:"
                         :
                         : "s"(stores_behind), "n"(C::CH)
                         : "scc", "memory");
            stores_behind = 0;
            __builtin_amdgcn_s_waitcnt(I4L_WAIT_LGKM0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }

        // ---- unit (gs, 1): reads unit (gs+1, 0) (a stale buffer past the last stage, never
        //      multiplied into a stored tile); begins the loads of stage gs+3 into the
        //      buffer of stage gs
        unit(std::integral_constant<int, 1>{}, [&](auto slot_tag) {
            spread(slot_tag, rd_next, 0, 0, std::integral_constant<int, 0>{}, wr_second);
        });
        ++kk;
        if (kk != KT)
            return false;
        {
            // ---- store the tile.  X is the MFMA A operand: accumulator t of tile (i, j) is
            //   m = 32*j + 8*(t/4) + 4*(lane/32) + t%4,  n = 32*i + lane%32,
            // so one dword store writes two rows of 32 consecutive n (128 B each).
            int tm, tn;
            const int item = bid + cur_it * nblk;
            const int slice = item / tiles;
            tile_coords(item - slice * tiles, tiles, tiles_m, tiles_n, tm, tn);
            const int m0 = tm * kTileRows, n0 = tn * kTileRows;
            const int rows_left = M - m0;  // > 0
            const int cols_left = N - n0;  // > 0
            int32_t *ybase = Y + (size_t)slice * (size_t)M * (size_t)N + (size_t)m0 * N + n0;
            const size_t slab_rows = rows_left < kTileRows ? rows_left : kTileRows;
            const size_t extent = ((slab_rows - 1) * (size_t)N + (size_t)(cols_left < kTileRows ? cols_left : kTileRows)) * 4u;
            __amdgpu_buffer_rsrc_t rsrc =
                __builtin_amdgcn_make_buffer_rsrc(ybase, 0, (int)extent, 0x00020000);
            // A lane outside the matrix gets an offset part so large that the sum falls
            // outside the descriptor's range and the hardware drops the store.
            const int lm = opaque(wm * C::FM * kFragRows + (lane >> 5) * 4);
            const int ln = opaque(wn * C::FN * kFragRows + (lane & 31));
            const unsigned lm_off = (unsigned)lm * (unsigned)N * 4u;
            unsigned col_off[C::FN];
#pragma unroll
            for (int i = 0; i < C::FN; ++i) {
                const int ncol = ln + i * kFragRows;
                col_off[i] = ncol < cols_left ? (unsigned)ncol * 4u : 0x40000000u;
            }
            if constexpr (!Parts::kStores) {
                pin(acc[0][0]);
            } else if (ep_plain) {
#pragma unroll
                for (int j = 0; j < C::FM; ++j) {
#pragma unroll
                    for (int t = 0; t < 16; ++t) {
                        const int dm = j * kFragRows + 8 * (t / 4) + (t % 4);  // uniform
                        const unsigned row_off = lm + dm < rows_left ? lm_off + (unsigned)dm * (unsigned)N * 4u : 0x80000000u;
#pragma unroll
                        for (int i = 0; i < C::FN; ++i) {
                            const int v = (int)(acc[i][j][t] * kUnscale);
                            __builtin_amdgcn_raw_buffer_store_b32((unsigned)v, rsrc, row_off + col_off[i], 0, 2 /* nt */);
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
                    const int ncol = ln + i * kFragRows;
                    const int nn = n0 + (ncol < cols_left ? ncol : cols_left - 1);
                    bias_v[i] = ep.bias ? ep.bias[nn] : 0;
                    cs_v[i] = ep.col_scale ? ep.col_scale[nn] : 1.f;
                }
                if constexpr (!HALF_OUT) {
#pragma unroll
                    for (int j = 0; j < C::FM; ++j) {
                        float rs[16];
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int dm = j * kFragRows + 8 * (t / 4) + (t % 4);
                            rs[t] = ep.row_scale ? ep.row_scale[m0 + (lm + dm < rows_left ? lm + dm : rows_left - 1)] : 1.f;
                        }
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int dm = j * kFragRows + 8 * (t / 4) + (t % 4);  // uniform
                            const unsigned row_off = lm + dm < rows_left ? lm_off + (unsigned)dm * (unsigned)N * 4u : 0x80000000u;
#pragma unroll
                            for (int i = 0; i < C::FN; ++i) {
                                const int v = epilogue_value32(ep, (int)(acc[i][j][t] * kUnscale), bias_v[i], rs[t], cs_v[i]);
                                __builtin_amdgcn_raw_buffer_store_b32((unsigned)v, rsrc, row_off + col_off[i], 0, 2 /* nt */);
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
                            const int dm = j * kFragRows + 8 * (t / 4) + (t % 4);
                            rs[t] = ep.row_scale ? ep.row_scale[m0 + (lm + dm < rows_left ? lm + dm : rows_left - 1)] : 1.f;
                        }
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int dm = j * kFragRows + 8 * (t / 4) + (t % 4);  // uniform
                            const unsigned row_off = lm + dm < rows_left ? (lm_off + (unsigned)dm * (unsigned)N * 4u) / 2u : 0x80000000u;
#pragma unroll
                            for (int i = 0; i < C::FN; ++i) {
                                const int v = epilogue_value16(ep, (int)(acc[i][j][t] * kUnscale), bias_v[i], rs[t], cs_v[i]);
                                __builtin_amdgcn_raw_buffer_store_b16((unsigned short)v, rsrc16,
                                                                      row_off + (col_off[i] == 0x40000000u ? col_off[i] : col_off[i] / 2u), 0, 2 /* nt */);
                            }
                        }
                    }
                }
            }
            kk = 0;
            ++cur_it;
            stores_behind = 1;
            clear_acc();
        }
        return cur_it == my_tiles;
    };
    for (;;) {
        if (iteration(std::integral_constant<int, 0>{}))
            break;
        if (iteration(std::integral_constant<int, 1>{}))
            break;
        if (iteration(std::integral_constant<int, 2>{}))
            break;
    }
    if (threadIdx.x == 0)
        Parts::stamp(ep, bid, 1);
}

// Eight wavefronts of 64 (m) x 128 (n), two per SIMD, one workgroup per CU.  (With four
// fragments along n a wave's stores of one accumulator row cover 512 contiguous bytes of a
// row of C; measured 0-2 % faster than 128 (m) x 64 (n) on every large shape tried.)
using Fp6Cfg = Fp6Config<4, 2, 1>;

size_t operand_ws_bytes(int rows, int k)
{
    const size_t tiles = (size_t)(rows + kTileRows - 1) / kTileRows;
    return tiles * (size_t)((k + kStageK - 1) / kStageK) * (size_t)kOperandStageBytes;
}

}  // namespace

bool fp6_supports(int m, int n, int k)
{
    // fp32 accumulation of products bounded by 64 stays exact while K * 64 < 2^24.  The
    // converter pads K to a multiple of 128 with zeros, so any K % 8 == 0 is fine.
    // Rows: the converter's grid (one y block per 32 rows of either operand) ends at 65535
    // and the store addresses a tile's 256 rows of C with byte offsets below 2^30.
    constexpr int kMaxRows = (1 << 20) - kTileRows;
    return m >= 1 && n >= 1 && m <= kMaxRows && n <= kMaxRows && k >= 8 && k % 8 == 0 && k <= (1 << 18) - kStageK;
}

int fp6_ksplit(int m, int n, int k, const DeviceInfo &dev)
{
    const long tiles = (long)((m + kTileRows - 1) / kTileRows) * ((n + kTileRows - 1) / kTileRows);
    const int stages = (k + kStageK - 1) / kStageK;
    // Measured: two slices of 128 tiles gain nothing over 128 unsplit tiles (the second kernel
    // and the slabs cost what the idle half of the device did); four of 64 tiles gain 9-16 %.
    if (dev.cu_count <= 0 || tiles * 4 > dev.cu_count)
        return 1;
    // The most slices that still leave a workgroup per CU, 2048 k per slice and equal slices.
    for (int ks : {8, 7, 6, 5, 4, 3, 2})
        if (tiles * ks <= dev.cu_count && stages % ks == 0 && stages / ks >= 16)
            return ks;
    return 1;
}

size_t fp6_workspace_bytes(int m, int n, int k, const DeviceInfo &dev)
{
    const int ks = fp6_ksplit(m, n, k, dev);
    return operand_ws_bytes(m, k) + operand_ws_bytes(n, k) + (ks > 1 ? (size_t)ks * (size_t)m * (size_t)n * 4u : 0);
}

hipError_t fp6_init(const DeviceInfo &dev)
{
    if (dev.lds_per_cu < kLdsBytes)
        return hipErrorInvalidConfiguration;
    hipError_t e = hipFuncSetAttribute((const void *)fp6_gemm_kernel<Fp6Cfg>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess)
        return e;
    return hipFuncSetAttribute((const void *)fp6_gemm_kernel<Fp6Cfg, true>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
}

size_t fp6_operand_bytes(int rows, int k) { return operand_ws_bytes(rows, k); }

namespace {

ConvertJob make_job(const void *src, void *dst, int rows)
{
    const int tiles = (rows + kTileRows - 1) / kTileRows;
    return ConvertJob{(const uint8_t *)src, (uint8_t *)dst, rows, tiles * kFragsRows};
}

int padded_k(int k) { return (k + kStageK - 1) / kStageK * kStageK; }

hipError_t launch_convert_jobs(const ConvertJob &ja, const ConvertJob &jb, int k, hipStream_t stream)
{
    const int yblocks = ja.row_blocks + jb.row_blocks;
    if (yblocks > 65535)
        return hipErrorInvalidValue;
    if (yblocks == 0)
        return hipSuccess;
    const int k_pad = padded_k(k);
    const dim3 grid((k_pad + kConvK - 1) / kConvK, yblocks);
    if (k % 32 == 0)
        fp6_convert_kernel<true><<<grid, 256, 0, stream>>>(ja, jb, k, k_pad);
    else
        fp6_convert_kernel<false><<<grid, 256, 0, stream>>>(ja, jb, k, k_pad);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_fp6_convert(const void *src, void *dst, int rows, int k, hipStream_t stream)
{
    return launch_convert_jobs(make_job(src, dst, rows), ConvertJob{nullptr, nullptr, 0, 0}, k, stream);
}

namespace {

// ksplit > 1: `c` is ksplit slabs of m * n partial sums and `ep` must be empty.
hipError_t launch_gemm_items(const void *a_conv, const void *b_conv, void *c, int m, int n, int k, int ksplit,
                             const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    using C = Fp6Cfg;
    const int tiles_m = (m + kTileRows - 1) / kTileRows;
    const int tiles_n = (n + kTileRows - 1) / kTileRows;
    const long total = (long)tiles_m * tiles_n * ksplit;
    if (total > 0x7fffffffL || (size_t)kTileRows * (size_t)n * 4u > 0x40000000ull)
        return hipErrorInvalidValue;
    long grid = (long)dev.cu_count * C::OCC;
    if (grid > total)
        grid = total;
    if (ep.out >= kOutF16) {
        if (ksplit != 1)
            return hipErrorInvalidValue;
        fp6_gemm_kernel<C, true><<<(unsigned)grid, C::THREADS, kLdsBytes, stream>>>(
            (const uint8_t *)a_conv, (const uint8_t *)b_conv, (int32_t *)c, m, n, padded_k(k), tiles_m, tiles_n, ksplit, ep);
    } else {
        fp6_gemm_kernel<C><<<(unsigned)grid, C::THREADS, kLdsBytes, stream>>>(
            (const uint8_t *)a_conv, (const uint8_t *)b_conv, (int32_t *)c, m, n, padded_k(k), tiles_m, tiles_n, ksplit, ep);
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_fp6_gemm(const void *a_conv, const void *b_conv, void *c, int m, int n, int k,
                           const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    return launch_gemm_items(a_conv, b_conv, c, m, n, k, 1, ep, dev, stream);
}

hipError_t launch_fp6(const void *a, const void *b, void *c, int m, int n, int k, void *workspace,
                      const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream)
{
    uint8_t *xws = (uint8_t *)workspace;
    uint8_t *wws = xws + operand_ws_bytes(m, k);
    hipError_t e = launch_convert_jobs(make_job(a, xws, m), make_job(b, wws, n), k, stream);
    if (e != hipSuccess)
        return e;
    // Few tiles and long K: K-slices of every tile on their own CUs, partial sums in slabs
    // behind the operands, a second kernel for the sum and the epilogue.
    const int ks = fp6_ksplit(m, n, k, dev);
    if (ks == 1)
        return launch_gemm_items(xws, wws, c, m, n, k, 1, ep, dev, stream);
    int32_t *slabs = (int32_t *)(wws + operand_ws_bytes(n, k));
    e = launch_gemm_items(xws, wws, slabs, m, n, k, ks, Epilogue{}, dev, stream);
    if (e != hipSuccess)
        return e;
    return launch_splitk_reduce(slabs, c, (size_t)m * (size_t)n, ks, n, ep, stream);
}

}  // namespace int4linear
