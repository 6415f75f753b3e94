// Stage 3 on the matrix cores: the same +-1 dot products as the XNOR/popcount kernel, as an
// implicit GEMM in FP4 (E2M1 holds +1, -1 and 0 exactly; products are accumulated in FP32,
// which is exact for |sum| < 2^24, so every accumulator equals 2*popc - n as an integer).
// Semantics: reference src/default/bcast_convolution_default.cpp:60-105.
//
// Why FP4 MFMA rather than v_xnor/v_bcnt: one v_mfma_f32_32x32x64_f8f6f4 does 65536
// multiply-accumulates in ~32 cycles per SIMD, the XNOR/popcount pair does 2048 in 8; the
// measured ceilings on MI355X are 8.1 POP/s against 1.1 POP/s.  Out-of-bounds taps read a
// row of FP4 zeros, which contributes nothing, so "skip the tap" needs no predication.
//
// Shape of the GEMM: C[oc][pixel] = sum over (tap, channel) W[oc][tap, channel] *
// X[pixel shifted by tap][channel].  Filters are the A operand (rows), pixels the B
// operand (columns): in the 32x32 accumulator layout a register then holds 32 consecutive
// pixels of one filter, i.e. 128 contiguous bytes of the NCHW output.
//
// Workgroup = 32*PS consecutive output pixels x 256 filters; wave w owns filters
// 64w .. 64w+63 for all pixels of the tile (2 x PS accumulator blocks of 32x32).
//   * X: the packed sign bits of every input pixel the tile touches are expanded to FP4
//     once and kept in LDS, one row per input pixel (channel-major, 16 spare bytes per row
//     so that the rows a fragment load touches spread over all banks).  A tap is a row
//     offset; invalid taps point at a zero row.  All four waves read the same rows.
//   * W: pre-packed on the weight stage in fragment order (1 KB per 32 filters x 64
//     channels), loaded straight into registers ahead of use.  A wave's two fragments
//     per step feed 2*PS matrix instructions: with PS >= 3 the weight stream stays well
//     below what the vector memory path of a compute unit delivers (with 2 x 2 blocking it
//     ran at 80% of it and set the pace).
//   * PS (1 to 4) is chosen per problem so that the waves divide evenly over the SIMDs:
//     for 43264 pixels, PS = 3 gives 1.76 waves per SIMD (2 in the busiest), PS = 4 gives
//     1.32 (also 2, but each a third longer).
#include <atomic>
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "plan.hpp"

namespace xnor_hip {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int NT = 256;       // filters per workgroup (4 waves x 64)
constexpr int ROW_PAD = 16;   // spare bytes per LDS row
constexpr int TABLE_BYTES = 1024;
constexpr int ALPHA_BYTES = NT * 4;
constexpr int TURN_ROW = 36;  // floats per pixel row of the NHWC turn-around buffer (32 + 4)
constexpr int LDS_LIMIT = 160 * 1024;    // a gfx950 workgroup may take the whole LDS of its CU
constexpr int LDS_DEFAULT = 64 * 1024;   // above this the kernel has to ask for it
constexpr int LDS_TWO_PER_CU = 80 * 1024;
constexpr int MAX_DEVICES = 64;
// Cache policy of the output stores: 0 = write-back through L2 and the Infinity Cache, 2 = the
// "nt" bit, streaming.  Streaming stores keep an output that will not be read soon from
// pushing the next input out of the 256 MB Infinity Cache (and from sitting there as dirty
// lines that the next kernel's reads have to wait for): ResNet 3x3 56x56 MB 64, 205 MB in and
// 205 MB out, 130 -> 105 us per forward pass (the binarize kernel of the next pass 56 -> 31 us,
// this kernel 64.5 -> 66.4 us).  Where input and output fit the cache together, write-back is
// faster (AlexNet conv4 MB 256: this kernel 23.6 us against 28.8 us streaming).
constexpr int STORE_WRITE_BACK = 0, STORE_STREAMING = 2;

__device__ __forceinline__ v16f mfma_fp4(const v4i a, const v4i b, const v16f c) {
    const v8i a8 = {a.x, a.y, a.z, a.w, 0, 0, 0, 0};
    const v8i b8 = {b.x, b.y, b.z, b.w, 0, 0, 0, 0};
    // cbsz = blgp = 4: both operands FP4 (E2M1).  Scale operands of zero select the plain
    // v_mfma_f32_32x32x64_f8f6f4, which multiplies the operands as they are; a scale of 2^0
    // passed in registers gives the same products through v_mfma_scale_..., which costs a
    // v_mfma_ld_scale_b32 and a scale register read per matrix instruction.
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c, 4, 4, 0, 0, 0, 0);
}

// Operand traffic is issued by hand.  Left to itself the compiler hoists the global loads of
// the next weight fragments to the top of the current group and then waits for them before
// the first matrix instruction, and it sinks every LDS read to just ahead of its first use,
// where the matrix pipe then idles for the whole LDS latency.
//   * load_frag_async / fetch_rows_after only start loads; the destination registers hold
//     data once a later wait has run.
//   * Every wait is an "s_waitcnt" that carries the accumulator blocks as read-write
//     operands.  That data dependence orders it behind the matrix instructions issued
//     before it and ahead of those that follow, which are the ones that consume the
//     awaited registers.  The awaited registers themselves are deliberately not operands
//     of the wait: a read-write operand lets the compiler copy the register on the way in,
//     and a copy of a register whose load is still in flight copies stale data.
//   * fetch_rows_after first waits for the LDS reads of the previous call (the operands of
//     the matrix instructions that follow it) and then starts the reads for the step after,
//     which the 2*PS matrix instructions of the current step cover.
//   * Weight fragments are asked for one group (HS steps) ahead, two per step, and awaited
//     by count: vector memory returns in order, so "at most 2*HS loads outstanding" at step
//     hs means the two fragments of step hs, asked for 2*HS loads ago, have arrived.
//   * A register must stay named by the program for as long as a load into it is on the
//     way: the compiler takes the load for an ordinary definition and hands a register it
//     thinks dead to the next computation, which the late data then overwrites.  Inside
//     the loops both fragment sets are live by construction; after them they are named once
//     more behind the final wait.  tests/test_isa_hazards.py checks the machine code of
//     every variant for this.
template <int... I, class F>
__device__ __forceinline__ void static_for_each(std::integer_sequence<int, I...>, F &&f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) { // f(integral_constant<int, 0>) ... <N-1>
    static_for_each(std::make_integer_sequence<int, N>{}, f);
}

// Fragment loads are buffer loads: the lane's byte offset is one VGPR that never changes, the
// fragment is a scalar offset plus an immediate, so a load costs no vector instruction for
// its address.
template <int IMM>
__device__ __forceinline__ void load_frag_async(v4i &dst, const v4i desc, const uint32_t voff,
        const uint32_t soff) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4"
            : "=v"(dst) : "v"(voff), "s"(desc), "s"(soff), "n"(IMM));
}
#define XNOR_ACC1 "+v"(acc[0][0]), "+v"(acc[1][0])
#define XNOR_ACC2 "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[1][0]), "+v"(acc[1][1])
#define XNOR_ACC3 "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[0][2]), "+v"(acc[1][0]), \
        "+v"(acc[1][1]), "+v"(acc[1][2])
#define XNOR_ACC4 "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[0][2]), "+v"(acc[0][3]), \
        "+v"(acc[1][0]), "+v"(acc[1][1]), "+v"(acc[1][2]), "+v"(acc[1][3])
template <int PS>
__device__ __forceinline__ void wait_all_after(v16f (&acc)[2][PS]) {
    if constexpr (PS == 1) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : XNOR_ACC1);
    else if constexpr (PS == 2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : XNOR_ACC2);
    else if constexpr (PS == 3) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : XNOR_ACC3);
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : XNOR_ACC4);
}
template <int PS, int VM>
__device__ __forceinline__ void fetch_rows_after(v4i (&bn)[PS], const uint32_t (&a)[PS],
        v16f (&acc)[2][PS]) {
    if constexpr (PS == 1)
        asm volatile("s_waitcnt vmcnt(%[vm]) lgkmcnt(0)\n\tds_read_b128 %[b0], %[a0]"
                : [b0] "=&v"(bn[0]), XNOR_ACC1
                : [a0] "v"(a[0]), [vm] "n"(VM));
    else if constexpr (PS == 2)
        asm volatile("s_waitcnt vmcnt(%[vm]) lgkmcnt(0)\n\tds_read_b128 %[b0], %[a0]\n\t"
                     "ds_read_b128 %[b1], %[a1]"
                : [b0] "=&v"(bn[0]), [b1] "=&v"(bn[1]), XNOR_ACC2
                : [a0] "v"(a[0]), [a1] "v"(a[1]), [vm] "n"(VM));
    else if constexpr (PS == 3)
        asm volatile("s_waitcnt vmcnt(%[vm]) lgkmcnt(0)\n\tds_read_b128 %[b0], %[a0]\n\t"
                     "ds_read_b128 %[b1], %[a1]\n\tds_read_b128 %[b2], %[a2]"
                : [b0] "=&v"(bn[0]), [b1] "=&v"(bn[1]), [b2] "=&v"(bn[2]), XNOR_ACC3
                : [a0] "v"(a[0]), [a1] "v"(a[1]), [a2] "v"(a[2]), [vm] "n"(VM));
    else
        asm volatile("s_waitcnt vmcnt(%[vm]) lgkmcnt(0)\n\tds_read_b128 %[b0], %[a0]\n\t"
                     "ds_read_b128 %[b1], %[a1]\n\tds_read_b128 %[b2], %[a2]\n\t"
                     "ds_read_b128 %[b3], %[a3]"
                : [b0] "=&v"(bn[0]), [b1] "=&v"(bn[1]), [b2] "=&v"(bn[2]), [b3] "=&v"(bn[3]),
                  XNOR_ACC4
                : [a0] "v"(a[0]), [a1] "v"(a[1]), [a2] "v"(a[2]), [a3] "v"(a[3]), [vm] "n"(VM));
}
#undef XNOR_ACC1
#undef XNOR_ACC2
#undef XNOR_ACC3
#undef XNOR_ACC4

// FP4 codes of eight channels from one byte of packed sign bits (bit 7 = first channel,
// set = sign bit clear = +1): nibble i = channel i, +1 -> 0x2, -1 -> 0xA.
__device__ __forceinline__ uint32_t fp4_of_byte(uint32_t byte) {
    uint32_t out = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
        out |= (((byte >> (7 - i)) & 1u) ? 0x2u : 0xAu) << (4 * i);
    return out;
}

// What a persistent workgroup carries from one tile to the next (conv_tile with PERSIST).
// The packed input words of a tile (and mean|x| of its input pixels) are copied into one of two
// LDS staging areas while the tile before it is multiplied, so that a tile's staging phase
// reads LDS only and waits for no global load.
struct TileTurn {
    bool first;          // the workgroup's first tile: table, zero row, alphas are not in LDS yet
    uint32_t parity;     // which staging area holds this tile's words
    uint32_t next_first, next_end; // output pixels of the workgroup's next tile; 0, 0: none
};

// Starts a copy of n dwords from global memory to LDS that does not pass through registers
// (LDS-direct loads: lane l of a wave writes the dword it fetches to M0 + 4*l): dword i of src
// goes to byte 4*i of the LDS area at lds_addr.  Counts in vmcnt like any load; nothing waits
// here.  The compiler emits no instruction of its own that uses M0 in these kernels; the
// s_nop is the wait state the hardware asks for between a write of M0 and an LDS-direct load
// (the compiler inserts it for its own code, not inside an asm statement).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void copy_to_lds_async(const void *src, const int n,
        const uint32_t lds_addr, const int tid, const int wave) {
    for (int base = 0; base < n; base += 256) {
        const int i = base + tid;
        const uint32_t m0 = lds_addr + (uint32_t)(base + wave * 64) * 4u; // wave-uniform
        if (i < n)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                    : : "s"(m0), "v"((uint32_t)i * 4u), "s"(src) : "memory", "m0");
    }
}
#pragma clang diagnostic pop

// KS = 64-channel steps per tap (ceil(IC/64), rounded up to even above 4 and to 12 or 16
// above 8), PS = 32-pixel
// blocks per workgroup tile.
// DEEP (more than 1024 channels): the channels of a pixel are cut into ic_parts parts of
// 64*KS, and every (tap, part) is walked like a tap of its own whose rows start
// 32*KS bytes further into the same LDS rows.
// One tile: the output pixels [p_first, min(p_first + 32*PS, p_limit)) x the 256 filters of
// filter chunk `chunk`.
// With 128 filters or fewer (g.mfma_groups = 2 or 4) the waves that would have no filters take
// further pixels instead: the tile is 32*PS*groups pixels, wave w multiplies the filters of
// wave w % (4/groups) with the pixel blocks of group w / (4/groups), and everything the
// workgroup does together (staging, the K sums, the alphas) covers the whole tile.
// PERSIST: the caller loops over tiles (see conv_mfma_fp4_persistent_kernel); `turn` says what
// is already in LDS and which tile to prefetch.  The LDS layout then has room for four pixel
// blocks whatever PS is, so that tiles of two sizes can follow each other.
template <int KS, int PS, bool RAW, bool PAIR, bool DEEP, bool PERSIST = false>
__device__ __forceinline__
void conv_tile(const uint32_t *__restrict__ xbits, const v4i *__restrict__ wfrag,
        const float *__restrict__ alpha, const float *__restrict__ kplane,
        float *__restrict__ dst, int32_t *__restrict__ popc,
        const Geometry &g, const int max_rows, const FastDiv &div_xw,
        const float *__restrict__ a_plane, float *__restrict__ k_out, const float inv_khw,
        const int ic_parts, const uint32_t wfrag_bytes, const uint32_t p_first,
        const uint32_t p_limit, const int chunk, const TileTurn turn = TileTurn{}) {
    static_assert(!PERSIST || (!RAW && !DEEP), "persistent tiles: scaled output, one channel part");
    extern __shared__ unsigned char smem[];
    uint32_t *table = reinterpret_cast<uint32_t *>(smem);
    float *alpha_lds = reinterpret_cast<float *>(smem + TABLE_BYTES);
    // PERSIST: two staging areas of max_rows * xw packed words, then two of max_rows + 1
    // floats (mean|x|; the last slot holds zero), ahead of the rows: the LDS-direct loads
    // that fill them take a 16-bit LDS offset
    const int stage_words = max_rows * g.xw;
    const int stage_at = TABLE_BYTES + ALPHA_BYTES;
    const int stage_bytes = PERSIST ? (2 * stage_words * 4 + 2 * (max_rows + 1) * 4 + 15) & ~15 : 0;
    unsigned char *rows = smem + stage_at + stage_bytes; // row 0 is zero, then the tile
    // PAIR (an odd number KS of 32-channel words per pixel): two taps share KS steps, so no
    // step is half empty; the rows then hold exactly KS words (16*KS bytes is 4 mod 8 dwords,
    // which keeps the fragment reads conflict-free without padding).
    const int ROW_BYTES = DEEP ? ic_parts * KS * 32 + ROW_PAD
                               : PAIR ? KS * 16 : KS * 32 + ROW_PAD;
    // mean|x| of the tile's input pixels, when the K plane is computed here (after the rows;
    // PERSIST: read from the staging area instead, a_lds is pointed there below)
    float *a_lds = reinterpret_cast<float *>(rows + (size_t)(1 + max_rows) * ROW_BYTES);
    float *k_lds = reinterpret_cast<float *>(rows + (size_t)(1 + max_rows) * ROW_BYTES)
        + max_rows + 1; // K of the tile's pixels, same case
    // NHWC output: per wave 32 pixel rows of TURN_ROW floats to turn a block around in
    // (an offset from smem, not a rounded pointer: the compiler has to see an LDS address)
    constexpr int PSL = PERSIST ? 4 : PS; // pixel blocks the layout has room for
    const int groups = PERSIST ? 1 : g.mfma_groups; // pixel groups: 1, 2 or 4 (uniform)
    float *turn_lds = reinterpret_cast<float *>(smem + ((stage_at + stage_bytes
            + (1 + max_rows) * ROW_BYTES + (max_rows + 1 + 32 * PSL * groups) * 4 + 15) & ~15));
    constexpr int MT = 32 * PS;
    // Weight fragments are fetched in groups of HS steps, one group ahead: a whole tap where
    // the registers allow it (8 VGPRs per step on top of 32 per pixel block), half a tap
    // otherwise.  The longer lead hides more of the L2 latency of the fragment stream
    // (conv4 MB 256: main loop 11.9 -> 10.9 us per wave).
    // Above 8 steps per tap (more than 512 channels) a group is a quarter of a tap.
    constexpr int HS = PAIR ? KS : (KS > 8 || (KS == 8 && PS == 4)) ? KS / 4
        : (KS % 2 == 0 && KS >= 4 && (PS > 3 || 40 * PS + 16 * KS > 216)) ? KS / 2 : KS;
    constexpr int GROUPS_PER_TAP = KS / HS; // 1, 2 or 4

    int thread = threadIdx.x;
    // PERSIST: a value the compiler cannot see through, so that nothing computed from it
    // counts as invariant of the loop over tiles: what is hoisted out of that loop stays in
    // registers through the main loop, where there are none to spare
    if constexpr (PERSIST) asm volatile("" : "+v"(thread));
    const int tid = thread;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // this wave's filters are those of wave `fw` of a full workgroup, its pixels those of
    // pixel group `pg` (fw = wave, pg = 0 with one group)
    const int nfw = 4 / groups, fw = wave & (nfw - 1), pg = wave / nfw;
    const uint32_t p_wave = p_first + (uint32_t)(pg * MT);
    // "taps" below are the units the main loop walks over: kernel taps, or pairs of them
    const int taps = PAIR ? (g.kh * g.kw + 1) / 2 : DEEP ? g.kh * g.kw * ic_parts : g.kh * g.kw;

    // ---- which input pixels does the tile touch ------------------------------------------
    int lo, hi;
    tile_span(g, p_first, min(p_first + (uint32_t)(MT * groups), p_limit), lo, hi);
    const int nrows = min(hi - lo + 1, max_rows);

    // ---- the 32*PS output pixels of the tile, one per lane and 32-pixel block -----------------
    bool live[PS];
    // Per pixel: LDS address of the row of tap (0,0), and which kernel rows / columns fall
    // inside the image (bit kh of rowmask, bit kw of colmask; no bits for a dead pixel).
    uint32_t base_addr[PS], rowmask[PS], colmask[PS];
    int in0[PS]; // input pixel of tap (0,0), relative to the first staged row
    uint32_t pix[PS], img[PS], rem[PS];
#pragma unroll
    for (int ps = 0; ps < PS; ps++) {
        pix[ps] = p_wave + ps * 32 + (lane & 31);
        live[ps] = pix[ps] < p_limit;
        const uint32_t pc = live[ps] ? pix[ps] : p_limit - 1;
        img[ps] = g.div_ohw.div(pc);
        rem[ps] = pc - img[ps] * g.ohw;
        const int oh = (int)g.div_ow.div(rem[ps]);
        const int ow = (int)rem[ps] - oh * g.ow;
        const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw; // input pixel of tap (0,0)
        in0[ps] = (int)(img[ps] * g.ihw) + ih0 * g.iw + iw0 - lo;
        base_addr[ps] = (uint32_t)(size_t)rows + (uint32_t)((1 + in0[ps]) * ROW_BYTES)
            + (PAIR ? 0 : (lane >> 5) * 16);
        // kernel rows kh with 0 <= ih0 + kh < ih, as a run of bits (kh < 32)
        auto run_of_bits = [](int first, int last) -> uint32_t { // bits first..last, clipped
            if (first < 0) first = 0;
            if (last > 31) last = 31;
            if (last < first) return 0u;
            return (0xFFFFFFFFu >> (31 - last)) & (0xFFFFFFFFu << first);
        };
        rowmask[ps] = live[ps] ? run_of_bits(-ih0, g.ih - 1 - ih0) : 0u;
        colmask[ps] = run_of_bits(-iw0, g.iw - 1 - iw0);
    }
    const uint32_t zero_addr = (uint32_t)(size_t)rows + (PAIR ? 0 : (lane >> 5) * 16);

    // ---- LDS: lookup table, zero row, this workgroup's alphas, FP4 rows ----------------------
    // The rows of the tile are contiguous in the packed input: item i is word i of that
    // run.  The first EARLY loads of every thread are in flight while the table is built.
    // Words past ceil(IC/32) of a row are left as they are: the matching weights are FP4
    // zeros and FP4 has no NaN or infinity, so whatever LDS holds there contributes nothing.
    const int nitems = nrows * g.xw;
    const uint32_t *run = xbits + (size_t)lo * g.xw;
    constexpr int EARLY = PERSIST ? 1 : 8;
    uint32_t early[EARLY];
    // PERSIST: always with mean|x| (a K plane to read would be loads the compiler waits for
    // with vmcnt(0) in the middle of the staging phase, which would also wait for the copy
    // of the next tile's words that has just been started)
    const bool fuse_k = PERSIST || (!RAW && a_plane != nullptr); // uniform
    float alpha_early = 0.f;
    const uint32_t *stage = nullptr; // PERSIST: this tile's packed words in LDS
    if constexpr (PERSIST) {
        stage = reinterpret_cast<const uint32_t *>(smem + stage_at) + turn.parity * stage_words;
        float *a_stage = reinterpret_cast<float *>(smem + stage_at + 2 * stage_words * 4);
        a_lds = a_stage + turn.parity * (max_rows + 1);
        if (turn.first) { // what stays in LDS for all tiles of this workgroup
            table[tid] = fp4_of_byte(tid);
            for (int i = tid; i < ROW_BYTES / 4; i += 256)
                reinterpret_cast<uint32_t *>(rows)[i] = 0;
            alpha_lds[tid] = chunk * NT + tid < g.oc ? alpha[chunk * NT + tid] : 0.f;
            if (tid < 2) a_stage[tid * (max_rows + 1) + max_rows] = 0.f;
            // the words of the first tile: the kernel started their copy before its loop
            asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        }
        // All waves have finished with the rows, alphas and K of the tile before, and every
        // wave has waited for its share of this tile's words (ahead of its main loop: the
        // waits there let no older load pass) before it arrives here.
        __syncthreads();
        if (turn.next_end != 0) { // the next tile's words go to the other area meanwhile
            int nlo, nhi;
            tile_span(g, turn.next_first, turn.next_end, nlo, nhi);
            const int nn = min(nhi - nlo + 1, max_rows);
            const uint32_t other = turn.parity ^ 1u;
            copy_to_lds_async(xbits + (size_t)nlo * g.xw, nn * g.xw,
                    (uint32_t)(size_t)smem + stage_at + other * stage_words * 4, tid, wave);
            copy_to_lds_async(a_plane + nlo, nn, (uint32_t)(size_t)smem + stage_at
                        + 2 * stage_words * 4 + other * (max_rows + 1) * 4, tid, wave);
        }
    } else {
#pragma unroll
    for (int u = 0; u < EARLY; u++) {
        const int i = u * 256 + tid;
        early[u] = i < nitems ? run[i] : 0u;
    }
    float a_early = 0.f;
    if (fuse_k && tid < nrows) a_early = a_plane[lo + tid];
    table[tid] = fp4_of_byte(tid);
    for (int i = tid; i < ROW_BYTES / 4; i += 256) reinterpret_cast<uint32_t *>(rows)[i] = 0;
    // asked for now, put into LDS after the expansion: nothing needs it before the epilogue,
    // and the first barrier does not have to wait for it
    // (the raw-accumulator variant takes a table that need not hold alpha at all)
    alpha_early = !RAW && chunk * NT + tid < g.oc ? alpha[chunk * NT + tid] : 0.f;
    if (fuse_k) { // mean|x| of the staged input pixels, plus one slot that holds zero
        if (tid < nrows) a_lds[tid] = a_early;
        if (tid == 0) a_lds[max_rows] = 0.f;
        for (int i = 256 + tid; i < nrows; i += 256) a_lds[i] = a_plane[lo + i];
    }
    __syncthreads();
    }
    auto expand = [&](int i, uint32_t word) { // item i of the run -> 32 FP4 codes of its row
        const int r = (int)div_xw.div((uint32_t)i), j = i - r * g.xw; // row, 32-channel word
        v4i q;
        q.x = table[word >> 24];
        q.y = table[(word >> 16) & 0xFF];
        q.z = table[(word >> 8) & 0xFF];
        q.w = table[word & 0xFF];
        *reinterpret_cast<v4i *>(rows + (size_t)(1 + r) * ROW_BYTES + j * 16) = q;
    };
    if constexpr (!PERSIST) {
#pragma unroll
        for (int u = 0; u < EARLY; u++) {
            const int i = u * 256 + tid;
            if (i < nitems) expand(i, early[u]);
        }
    }
    // K of the tile's pixels, when it is not read from the K plane: wave ps (of the waves
    // that share a pixel group) sums the block of 32 pixels ps exactly as the box filter does (in-bounds taps in row-major order, each
    // product rounded, then added: reference src/bcast_calculate_k.cpp:69-85), leaves it in
    // LDS for the epilogue of all waves and stores it to the K plane.
    if (fuse_k) {
#pragma unroll
        for (int ps = 0; ps < PS; ps++) {
            if ((ps & (nfw - 1)) != fw) continue; // uniform
            float sum = 0.f;
            // Four taps per round, all reads of a round issued before its first addition.  A
            // tap outside the image (or past the kernel row) reads the slot that holds zero
            // and so contributes +0, which leaves the sum of non-negative terms unchanged
            // bit for bit; reading unconditionally keeps the reads free of branches.
            for (int kh = 0; kh < g.kh; kh++)
                for (int kw0 = 0; kw0 < g.kw; kw0 += 4) {
                    float term[4];
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const int kw = kw0 + u;
                        const int kwc = kw < g.kw ? kw : 0;
                        const bool ok = kw < g.kw
                            && ((rowmask[ps] >> kh) & (colmask[ps] >> kwc) & 1u);
                        term[u] = __fmul_rn(
                                a_lds[ok ? in0[ps] + kh * g.iw + kw : max_rows], inv_khw);
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++) sum = __fadd_rn(sum, term[u]);
                }
            if (lane < 32) {
                k_lds[(pg * PS + ps) * 32 + lane] = sum;
                if (chunk == 0 && live[ps]) k_out[pix[ps]] = sum;
            }
        }
    }
    for (int base = PERSIST ? 0 : EARLY * 256; base < nitems; base += 4 * 256) {
        uint32_t w[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = base + u * 256 + tid;
            if constexpr (PERSIST) w[u] = i < nitems ? stage[i] : 0u;
            else w[u] = i < nitems ? run[i] : 0u;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = base + u * 256 + tid;
            if (i < nitems) expand(i, w[u]);
        }
    }

    if constexpr (!PERSIST) alpha_lds[tid] = alpha_early;

    // ---- this wave: 64 filters x 32*PS pixels --------------------------------------------------
    const int oc_sub0 = chunk * (NT / 32) + fw * 2; // first 32-filter block
    const bool wave_has_filters = oc_sub0 * 32 < g.oc; // wave-uniform

    v16f acc[2][PS];
#pragma unroll
    for (int os = 0; os < 2; os++)
#pragma unroll
        for (int ps = 0; ps < PS; ps++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[os][ps][i] = 0.f;

    // Weight fragments: [32-filter block][tap][step][lane], two register sets of HS steps
    // used in turn (a "group" is HS steps of one tap).  Group n+1 is requested before group
    // n is multiplied and awaited after its 2*PS*HS matrix instructions.
    const uint64_t wfrag_at = reinterpret_cast<uint64_t>(wfrag);
    const v4i wdesc = {(int)(uint32_t)wfrag_at, (int)(uint32_t)((wfrag_at >> 32) & 0xFFFFu),
                       (int)wfrag_bytes, 0x00020000};
    const uint32_t wvoff = (uint32_t)lane * 16u;
    uint32_t wbase[2]; // byte offset of this wave's two 32-filter blocks
#pragma unroll
    for (int os = 0; os < 2; os++)
        wbase[os] = (uint32_t)(oc_sub0 + os) * (uint32_t)(taps * KS) * 1024u;
    // the two fragments of step hs of a group (group = tap * GROUPS_PER_TAP + part)
    auto request_step = [&](int group, auto step, v4i (&w)[HS][2]) {
        constexpr int hs = decltype(step)::value;
#pragma unroll
        for (int os = 0; os < 2; os++)
            load_frag_async<(hs & 3) * 1024>(w[hs][os], wdesc, wvoff,
                    wbase[os] + (uint32_t)(group * HS + (hs & ~3)) * 1024u);
    };
    // LDS address of each pixel's row for tap (kh, kw): a fixed offset from the row of tap
    // (0,0), or the zero row when the tap falls outside the image.  Every in-bounds tap of a
    // tile lies inside the span of rows the tile has staged (tile_span).
    int npart = 0; // DEEP: channel part of the tap that nkh, nkw (below) name
    auto tap_rows = [&](int kh, int kw, uint32_t (&out)[PS]) {
        const uint32_t shift = (uint32_t)((kh * g.iw + kw) * ROW_BYTES)
            + (DEEP ? (uint32_t)(npart * KS * 32) : 0u);
#pragma unroll
        for (int ps = 0; ps < PS; ps++) {
            const uint32_t ok = (rowmask[ps] >> kh) & (colmask[ps] >> kw) & 1u;
            out[ps] = ok ? base_addr[ps] + shift : zero_addr;
        }
    };
    int nkh = 0, nkw = 0; // the tap after the one being multiplied (the last tap repeats)
    bool ntap_valid = true; // PAIR: false once the walk has run past the last tap
    auto advance_tap = [&]() {
        if constexpr (DEEP) {
            if (npart + 1 < ic_parts) { npart++; return; }
        }
        if (nkw + 1 < g.kw) { nkw++; npart = 0; }
        else if (nkh + 1 < g.kh) { nkw = 0; nkh++; npart = 0; }
        else ntap_valid = false;
    };
    // PAIR: rows of the two taps of a pair (index 0 and 1); a missing second tap (odd number
    // of taps, or the repeated last pair) reads the zero row.
    auto pair_rows = [&](uint32_t (&out)[2][PS]) {
        tap_rows(nkh, nkw, out[0]);
        if (!ntap_valid) {
#pragma unroll
            for (int ps = 0; ps < PS; ps++) out[0][ps] = zero_addr;
        }
        advance_tap();
        tap_rows(nkh, nkw, out[1]);
        if (!ntap_valid) {
#pragma unroll
            for (int ps = 0; ps < PS; ps++) out[1][ps] = zero_addr;
        }
        advance_tap();
    };
    // PAIR: address of step hs for this lane: lanes 0..31 take word 2*hs, lanes 32..63 word
    // 2*hs + 1 of the 2*KS words of the pair (first tap's KS words, then the second's)
    const bool lane_hi_half = lane >= 32;
    auto pair_addr = [&](int hs, const uint32_t (&r)[2][PS], uint32_t (&out)[PS]) {
        const int c_lo = 2 * hs, c_hi = 2 * hs + 1;
#pragma unroll
        for (int ps = 0; ps < PS; ps++) {
            const uint32_t lo = c_lo < KS ? r[0][ps] + c_lo * 16 : r[1][ps] + (c_lo - KS) * 16;
            const uint32_t hi = c_hi < KS ? r[0][ps] + c_hi * 16 : r[1][ps] + (c_hi - KS) * 16;
            out[ps] = lane_hi_half ? hi : lo;
        }
    };
    auto mma = [&](const v4i (&w)[2], const v4i (&b)[PS]) {
#pragma unroll
        for (int os = 0; os < 2; os++)
#pragma unroll
            for (int ps = 0; ps < PS; ps++)
                acc[os][ps] = mfma_fp4(w[os], b[ps], acc[os][ps]);
    };

    const int last_group = taps * GROUPS_PER_TAP - 1;
    uint32_t rowaddr[PS];                    // rows of the current group's tap
    uint32_t pairaddr[PAIR ? 2 : 1][PAIR ? PS : 1]; // PAIR: rows of both taps of the pair
    v4i b0[PS], b1[PS];   // pixel fragments of the current and the following step, in turn
    // One group with the fragments in wc, while those of the next group arrive in wn.
    // P0: which of b0/b1 holds the group's first step; OFF / NOFF: byte offset within a row of
    // this group's and of the next group's first step.  In the loops the group after the
    // last one is the last one again: loaded, awaited after the loops and never multiplied.
    // MORE = false (the single group after the paired loop) asks for nothing.
    auto run_group = [&](auto more, auto newtap, auto p0, auto off, auto noff, int n,
                         const v4i (&wc)[HS][2], v4i (&wn)[HS][2]) {
        constexpr bool MORE = decltype(more)::value, NEWTAP = decltype(newtap)::value;
        constexpr int P0 = decltype(p0)::value, OFF = decltype(off)::value,
                      NOFF = decltype(noff)::value;
        uint32_t nextaddr[PS];
        uint32_t nextpair[PAIR ? 2 : 1][PAIR ? PS : 1];
        const int next_group = min(n + 1, last_group);
        if constexpr (MORE) {
            if constexpr (PAIR) {
                pair_rows(nextpair);
            } else if constexpr (NEWTAP) { // the next group starts the next tap
                tap_rows(nkh, nkw, nextaddr);
                advance_tap();
            } else {
#pragma unroll
                for (int ps = 0; ps < PS; ps++) nextaddr[ps] = rowaddr[ps];
            }
        }
        // Step hs first asks for the two fragments of step hs of the next group, then waits
        // until its own two have arrived: they were asked for one group ago, and the 2*HS
        // loads started since (vector memory returns in order) may still be under way.
        constexpr int VM = MORE ? 2 * HS : 0;
        static_for<HS>([&](auto step) {
            constexpr int hs = decltype(step)::value;
            if constexpr (MORE) request_step(next_group, step, wn);
            if constexpr (hs + 1 < HS || MORE) {
                uint32_t a[PS];
                if constexpr (PAIR) {
                    if constexpr (hs + 1 < HS) pair_addr(hs + 1, pairaddr, a);
                    else pair_addr(0, nextpair, a);
                } else {
#pragma unroll
                    for (int ps = 0; ps < PS; ps++)
                        a[ps] = hs + 1 < HS ? rowaddr[ps] + OFF + (hs + 1) * 32
                                            : nextaddr[ps] + NOFF;
                }
                if constexpr (((P0 + hs) & 1) == 0) fetch_rows_after<PS, VM>(b1, a, acc);
                else fetch_rows_after<PS, VM>(b0, a, acc);
            } else {
                wait_all_after<PS>(acc); // the last fragments of the kernel are in
            }
            if constexpr (((P0 + hs) & 1) == 0) mma(wc[hs], b0);
            else mma(wc[hs], b1);
        });
        if constexpr (MORE) {
            if constexpr (PAIR) {
#pragma unroll
                for (int ps = 0; ps < PS; ps++) {
                    pairaddr[0][ps] = nextpair[0][ps];
                    pairaddr[1][ps] = nextpair[1][ps];
                }
            } else {
#pragma unroll
                for (int ps = 0; ps < PS; ps++) rowaddr[ps] = nextaddr[ps];
            }
        }
    };

    v4i wa[HS][2], wb[HS][2];
    // A wave without filters (fewer than 256 of them in this chunk) leaves here, through a
    // barrier of its own: the barrier counts arrivals, whichever instruction they come from.
    // One test of the condition, ahead of the first hand-issued load, so that no path (of the
    // hardware, or of the walk in tests/test_isa_hazards.py, which knows nothing of branch
    // conditions) mixes "has asked for fragments" with "skips the waits of the main loop".
    if (!wave_has_filters) {
        __syncthreads();
        // PERSIST: this wave's share of the next tile's words has to be in LDS before it
        // meets the others at the next tile's first barrier (the others wait for theirs
        // ahead of their main loops: the waits there let no older load pass)
        if constexpr (PERSIST) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        return;
    }
    static_for<HS>([&](auto step) { request_step(0, step, wa); });
    if constexpr (PAIR) {
        pair_rows(pairaddr);
    } else {
        tap_rows(0, 0, rowaddr);
        advance_tap();
    }
    __syncthreads(); // FP4 rows are in place
    float kv[PS]; // K of this wave's pixels
#pragma unroll
    for (int ps = 0; ps < PS; ps++) kv[ps] = 0.f;
    if (!RAW) { // two branches: one select of an LDS and a global pointer would be a flat load
        if (fuse_k) {
#pragma unroll
            for (int ps = 0; ps < PS; ps++) kv[ps] = k_lds[(pg * PS + ps) * 32 + (lane & 31)];
        } else {
#pragma unroll
            for (int ps = 0; ps < PS; ps++) kv[ps] = kplane[live[ps] ? pix[ps] : 0];
        }
    }
    {
        if constexpr (PAIR) {
            uint32_t a0[PS];
            pair_addr(0, pairaddr, a0);
            fetch_rows_after<PS, 0>(b0, a0, acc);
        } else {
            fetch_rows_after<PS, 0>(b0, rowaddr, acc);
        }
        wait_all_after<PS>(acc);
        constexpr int P1 = HS & 1, OFF1 = GROUPS_PER_TAP == 2 ? HS * 32 : 0;
        using std::integral_constant;
        int n = 0;
        if constexpr (GROUPS_PER_TAP == 4) { // the four quarters of a tap, wa and wb in turn
            for (; n + 3 <= last_group; n += 4) {
                run_group(std::true_type{}, std::false_type{}, integral_constant<int, 0>{},
                        integral_constant<int, 0>{}, integral_constant<int, HS * 32>{}, n, wa, wb);
                run_group(std::true_type{}, std::false_type{}, integral_constant<int, P1>{},
                        integral_constant<int, HS * 32>{}, integral_constant<int, 2 * HS * 32>{},
                        n + 1, wb, wa);
                run_group(std::true_type{}, std::false_type{}, integral_constant<int, 0>{},
                        integral_constant<int, 2 * HS * 32>{},
                        integral_constant<int, 3 * HS * 32>{}, n + 2, wa, wb);
                run_group(std::true_type{}, std::true_type{}, integral_constant<int, P1>{},
                        integral_constant<int, 3 * HS * 32>{}, integral_constant<int, 0>{},
                        n + 3, wb, wa);
            }
        }
        for (; n + 1 <= last_group; n += 2) {
            run_group(std::true_type{}, integral_constant<bool, GROUPS_PER_TAP == 1>{},
                    integral_constant<int, 0>{}, integral_constant<int, 0>{},
                    integral_constant<int, OFF1>{}, n, wa, wb);
            run_group(std::true_type{}, std::true_type{}, integral_constant<int, P1>{},
                    integral_constant<int, OFF1>{}, integral_constant<int, 0>{}, n + 1, wb, wa);
        }
        if (n <= last_group) // odd number of groups (only with one group per tap)
            run_group(std::false_type{}, std::false_type{}, integral_constant<int, 0>{},
                    integral_constant<int, 0>{}, integral_constant<int, 0>{}, n, wa, wb);
        // The last group of the loops has asked for fragments that nothing multiplies.  They
        // are awaited here, and both register sets are named as inputs after the wait: a
        // register that is dead after the loop would otherwise be handed to the epilogue's
        // address arithmetic while its load is still on the way.
        // The same holds for the pixel fragments: the last step has started LDS reads for a
        // step that does not exist.
        wait_all_after<PS>(acc);
        static_for<HS>([&](auto step) {
            constexpr int hs = decltype(step)::value;
            const v4i a0 = wa[hs][0], a1 = wa[hs][1], c0 = wb[hs][0], c1 = wb[hs][1];
            asm volatile("" : : "v"(a0), "v"(a1), "v"(c0), "v"(c1));
        });
        static_for<PS>([&](auto block) {
            constexpr int ps = decltype(block)::value;
            const v4i p0 = b0[ps], p1 = b1[ps];
            asm volatile("" : : "v"(p0), "v"(p1));
        });
    }

    // ---- epilogue: register i of a 32x32 block holds filter 8*(i/4) + 4*(lane/32) + i%4,
    //      pixel lane%32.  Values are scaled in that layout.  For NCHW output
    //      v_permlane32_swap then joins two pixel blocks, so that a register holds 64
    //      consecutive pixels of ONE filter and a store instruction writes one 256-byte run
    //      (the odd block of PS = 3 keeps the 2 x 128-byte form); the runs of one filter are
    //      stored back to back so that the cache lines they share fill up in L2 before they
    //      can leave it.  Stores are raw buffer stores: the lane's pixel offset is one VGPR
    //      computed once, the filter is a scalar offset, and a dead pixel or a filter past
    //      OC gets an offset beyond the buffer, which the hardware drops; no 64-bit address
    //      arithmetic and no branches per store. ------------------------------------------------
    const int lane_hi = lane >> 5;
    constexpr uint32_t DROP = 0xFFFFFFF0u; // >= the buffer size: the store is discarded
    const __amdgpu_buffer_rsrc_t outbuf = __builtin_amdgcn_make_buffer_rsrc(
            RAW ? static_cast<void *>(popc) : static_cast<void *>(dst), 0,
            (int)((uint32_t)g.npix_out * (uint32_t)g.oc * 4u), 0x00020000);
    const bool nchw = RAW || g.dst_fmt == xnor_nn_data_format_nchw;
    const uint32_t fstep = nchw ? (uint32_t)g.ohw * 4u : 4u; // bytes from a filter to the next
    int n[PS];
    const uint32_t kh_bits = 0xFFFFFFFFu >> (32 - g.kh), kw_bits = 0xFFFFFFFFu >> (32 - g.kw);
    uint32_t off1[PS]; // one block: lanes 0..31 filter f, lanes 32..63 filter f + 4
#pragma unroll
    for (int ps = 0; ps < PS; ps++) {
        // operation count of the pixel (reference src/bcast_binarize_weights.cpp:126-142):
        // channels times the taps inside the image, from the same masks the main loop used
        n[ps] = RAW ? g.ic * __popc(rowmask[ps] & kh_bits) * __popc(colmask[ps] & kw_bits) : 0;
        const uint32_t at = nchw ? (img[ps] * (uint32_t)g.oc * (uint32_t)g.ohw + rem[ps]) * 4u
                                 : pix[ps] * (uint32_t)g.oc * 4u;
        off1[ps] = live[ps] ? at + (uint32_t)lane_hi * 4u * fstep : DROP;
    }
    uint32_t off2[PS / 2 > 0 ? PS / 2 : 1]; // joined pair q: pixels 64q + lane of one filter
#pragma unroll
    for (int q = 0; q < PS / 2; q++) {
        const uint32_t p64 = p_wave + q * 64 + lane;
        const uint32_t pc = p64 < p_limit ? p64 : p_limit - 1;
        const uint32_t im = g.div_ohw.div(pc);
        off2[q] = p64 < p_limit
            ? (im * (uint32_t)g.oc * (uint32_t)g.ohw + (pc - im * g.ohw)) * 4u : DROP;
    }
    // 16-byte stores need filter runs that start on a 16-byte boundary
    const bool vec4_ok = !nchw && (g.oc & 3) == 0
        && ((size_t)(RAW ? static_cast<void *>(popc) : static_cast<void *>(dst)) & 15) == 0;
    auto store_tile = [&](auto check_filters, auto planar, auto policy) {
        constexpr bool CHECK = decltype(check_filters)::value, NCHW = decltype(planar)::value;
        constexpr int STORE_AUX = decltype(policy)::value;
#pragma unroll
        for (int os = 0; os < 2; os++) {
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                // alphas of the four filters 8*i4 + 4*lane_hi + 0..3 of this 32-filter block
                const int ocl4 = (fw * 2 + os) * 32 + 8 * i4 + lane_hi * 4;
                const v4f al = *reinterpret_cast<const v4f *>(alpha_lds + ocl4);
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    const int i = 4 * i4 + ii;
                    const int f = chunk * NT + (fw * 2 + os) * 32 + 8 * i4 + ii; // lanes 0..31
                    const uint32_t soff = (uint32_t)f * fstep; // uniform
                    uint32_t v[PS]; // bit patterns of the results in the accumulator layout
#pragma unroll
                    for (int ps = 0; ps < PS; ps++) {
                        const float d = acc[os][ps][i]; // = 2*popc - n, exactly
                        if constexpr (RAW)
                            v[ps] = (uint32_t)(((int)d + n[ps]) / 2);
                        else // dst = fl(fl((float)(2*popc - n) * alpha) * k), rounded per product
                            v[ps] = __float_as_uint(__fmul_rn(__fmul_rn(d, al[ii]), kv[ps]));
                    }
                    if constexpr (NCHW) {
#pragma unroll
                        for (int q = 0; q < PS / 2; q++) {
                            const auto r = __builtin_amdgcn_permlane32_swap(v[2 * q],
                                    v[2 * q + 1], false, false);
                            // r[0]: filter f, pixels 64q + lane; r[1]: filter f + 4
                            if (!CHECK || f < g.oc)
                                __builtin_amdgcn_raw_buffer_store_b32(r[0], outbuf, off2[q], soff, STORE_AUX);
                            if (!CHECK || f + 4 < g.oc)
                                __builtin_amdgcn_raw_buffer_store_b32(r[1], outbuf, off2[q],
                                        soff + 4u * fstep, STORE_AUX);
                        }
                    }
#pragma unroll
                    for (int ps = NCHW ? (PS / 2) * 2 : 0; ps < PS; ps++) {
                        const uint32_t voff = CHECK && f + lane_hi * 4 >= g.oc ? DROP : off1[ps];
                        __builtin_amdgcn_raw_buffer_store_b32(v[ps], outbuf, voff, soff, STORE_AUX);
                    }
                }
            }
        }
    };
    // NHWC with whole cache lines: a 32-filter x 32-pixel block is scaled in the accumulator
    // layout (a lane holds 4 x 4 consecutive filters of one pixel), written to the wave's own
    // LDS rows and read back eight lanes to a pixel, so that a store instruction writes the
    // 128 contiguous bytes of 8 pixels instead of 32 bytes of 32 pixels.  Rows of 144 bytes
    // keep both sides free of bank conflicts.  A piece past OC (OC is a multiple of 4 here)
    // or a pixel past the end gets an offset outside the buffer.
    auto store_lines_nhwc = [&](auto policy) {
        constexpr int STORE_AUX = decltype(policy)::value;
        float *mine = turn_lds + wave * (32 * TURN_ROW);
        const int piece = lane & 7, prow = lane >> 3;
        const uint32_t left = p_limit > p_wave ? p_limit - p_wave : 0u; // of this wave's pixels
#pragma unroll
        for (int os = 0; os < 2; os++) {
            const uint32_t fpiece = (uint32_t)(chunk * NT + (fw * 2 + os) * 32 + 4 * piece);
            const uint32_t base = fpiece < (uint32_t)g.oc
                ? ((p_wave + (uint32_t)prow) * (uint32_t)g.oc + fpiece) * 4u : DROP;
#pragma unroll
            for (int ps = 0; ps < PS; ps++) {
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    const int ocl4 = (fw * 2 + os) * 32 + 8 * i4 + lane_hi * 4;
                    const v4f al = *reinterpret_cast<const v4f *>(alpha_lds + ocl4);
                    v4i q;
#pragma unroll
                    for (int ii = 0; ii < 4; ii++)
                        q[ii] = (int)__float_as_uint(
                                __fmul_rn(__fmul_rn(acc[os][ps][4 * i4 + ii], al[ii]), kv[ps]));
                    *reinterpret_cast<v4i *>(mine + (lane & 31) * TURN_ROW + 8 * i4 + 4 * lane_hi)
                        = q;
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4i r = *reinterpret_cast<const v4i *>(
                            mine + (8 * j + prow) * TURN_ROW + 4 * piece);
                    const uint32_t in_tile = (uint32_t)(ps * 32 + 8 * j); // + prow
                    const uint32_t voff = in_tile + (uint32_t)prow < left ? base : DROP;
                    __builtin_amdgcn_raw_buffer_store_b128(r, outbuf, voff,
                            in_tile * (uint32_t)g.oc * 4u, STORE_AUX);
                }
            }
        }
    };
    const bool all_filters = chunk * NT + (fw + 1) * 64 <= g.oc; // wave-uniform
    if constexpr (!RAW) {
        if (vec4_ok) {
            if (g.stream_dst) store_lines_nhwc(std::integral_constant<int, STORE_STREAMING>{});
            else store_lines_nhwc(std::integral_constant<int, STORE_WRITE_BACK>{});
            return;
        }
    }
    using WriteBack = std::integral_constant<int, STORE_WRITE_BACK>;
    using Streaming = std::integral_constant<int, STORE_STREAMING>;
    if (nchw) {
        if (g.stream_dst) {
            if (all_filters) store_tile(std::false_type{}, std::true_type{}, Streaming{});
            else store_tile(std::true_type{}, std::true_type{}, Streaming{});
        } else {
            if (all_filters) store_tile(std::false_type{}, std::true_type{}, WriteBack{});
            else store_tile(std::true_type{}, std::true_type{}, WriteBack{});
        }
    } else {
        if (all_filters) store_tile(std::false_type{}, std::false_type{}, WriteBack{});
        else store_tile(std::true_type{}, std::false_type{}, WriteBack{});
    }
}

// Which tile a workgroup takes.  Workgroups are dealt to the eight XCDs round-robin, so
// workgroup b runs on XCD b % 8 and is the (b / 8)-th of that XCD.
//
// PSB == 0, one tile size: unit (b % 8) * units_per_xcd + b / 8 gives each XCD one contiguous
// range of tiles, so the input rows two neighbouring tiles share and the output cache lines
// they both write into meet in one L2.  A unit is a (tile, filter chunk) pair.
//
// PSB > 0, two tile sizes: XCD x owns the pixel blocks
// [x * blocks_per_xcd, (x+1) * blocks_per_xcd); its first big_per_xcd tiles have PS blocks
// each, the following ones PSB blocks each, and workgroup n of the XCD takes tile
// n / oc_chunks with filter chunk n % oc_chunks.  The hardware starts workgroups in the
// order of their index and the matrix pipe serves the older wave of a SIMD first, so on a
// compute unit that holds two workgroups the one with the small tile is the one that
// finishes last: its epilogue, the only one nothing overlaps, is the short one.
template <int KS, int PS, int PSB, bool RAW, bool PAIR, bool DEEP>
__global__ __launch_bounds__(256, 2)
void conv_mfma_fp4_kernel(const uint32_t *__restrict__ xbits, const v4i *__restrict__ wfrag,
        const float *__restrict__ alpha, const float *__restrict__ kplane,
        float *__restrict__ dst, int32_t *__restrict__ popc,
        const Geometry g, const int max_rows, const int oc_chunks, const uint32_t units,
        const uint32_t units_per_xcd, const FastDiv div_xw, const float *__restrict__ a_plane,
        float *__restrict__ k_out, const float inv_khw, const int ic_parts,
        const uint32_t wfrag_bytes, const uint32_t big_per_xcd, const uint32_t blocks_per_xcd) {
    const uint32_t xcd = blockIdx.x & 7, nth = blockIdx.x >> 3;
    if constexpr (PSB == 0) {
        const uint32_t unit = xcd * units_per_xcd + nth;
        if (unit >= units) return;
        const uint32_t tile = oc_chunks == 1 ? unit : unit / oc_chunks;
        const int chunk = unit - tile * oc_chunks;
        conv_tile<KS, PS, RAW, PAIR, DEEP>(xbits, wfrag, alpha, kplane, dst, popc, g, max_rows,
                div_xw, a_plane, k_out, inv_khw, ic_parts, wfrag_bytes,
                tile * (32u * PS * (uint32_t)g.mfma_groups), g.npix_out, chunk);
    } else {
        const uint32_t first = xcd * blocks_per_xcd; // pixel blocks of this XCD: [first, last)
        const uint32_t p_limit = min((first + blocks_per_xcd) * 32u, g.npix_out);
        const uint32_t tile = oc_chunks == 1 ? nth : nth / oc_chunks;
        const int chunk = nth - tile * oc_chunks;
        if (tile < big_per_xcd) {
            const uint32_t p_first = (first + tile * PS) * 32u;
            if (p_first >= p_limit) return;
            conv_tile<KS, PS, RAW, PAIR, DEEP>(xbits, wfrag, alpha, kplane, dst, popc, g,
                    max_rows, div_xw, a_plane, k_out, inv_khw, ic_parts, wfrag_bytes, p_first,
                    p_limit, chunk);
        } else {
            const uint32_t p_first = (first + big_per_xcd * PS + (tile - big_per_xcd) * PSB) * 32u;
            if (p_first >= p_limit) return;
            conv_tile<KS, PSB, RAW, PAIR, DEEP>(xbits, wfrag, alpha, kplane, dst, popc, g,
                    max_rows, div_xw, a_plane, k_out, inv_khw, ic_parts, wfrag_bytes, p_first,
                    p_limit, chunk);
        }
    }
}

// The same tiles for launches with several rounds of them: two workgroups per compute unit
// that stay, each walking over its tiles.  Tiles are numbered per XCD as in the two-size
// kernel above (the first big_per_xcd have PS blocks, the rest PSB); workgroup n of an XCD
// has filter chunk n % oc_chunks and takes the tiles n / oc_chunks + j * tiles_per_round,
// j = 0, 1, ...: a round of tiles is a contiguous stretch of pixels, so neighbouring tiles
// are worked on at the same time and meet in one L2, and the host picks big_per_xcd as a
// whole number of rounds so that every workgroup gets the same sequence of sizes.
// What a workgroup gains over a fresh one per tile: the table, the zero row, the alphas and
// the kernel arguments are set up once; the packed words of the next tile (and mean|x| of its
// input pixels) are copied into LDS while the current tile is multiplied, so staging waits
// for no global load; and no dispatch has to be waited for between tiles.
template <int KS, int PS, int PSB, bool PAIR>
__global__ __launch_bounds__(256, 2)
void conv_mfma_fp4_persistent_kernel(const uint32_t *__restrict__ xbits,
        const v4i *__restrict__ wfrag, const float *__restrict__ alpha,
        const float *__restrict__ kplane, float *__restrict__ dst, const Geometry g,
        const int max_rows, const int oc_chunks, const uint32_t tiles_per_round,
        const FastDiv div_xw, const float *__restrict__ a_plane, float *__restrict__ k_out,
        const float inv_khw, const uint32_t wfrag_bytes, const uint32_t big_per_xcd,
        const uint32_t blocks_per_xcd, const uint32_t rounds, const int reverse_second,
        const uint32_t stagger) {
    extern __shared__ unsigned char smem[];
    const uint32_t xcd = blockIdx.x & 7, nth = blockIdx.x >> 3;
    const uint32_t first = xcd * blocks_per_xcd; // pixel blocks of this XCD: [first, last)
    const uint32_t p_limit = min((first + blocks_per_xcd) * 32u, g.npix_out);
    uint32_t tile = oc_chunks == 1 ? nth : nth / oc_chunks;
    const int chunk = nth - tile * oc_chunks;
    if (tile >= tiles_per_round) return; // more workgroups than a round has (tile, chunk) pairs
    // first pixel of tile t of this XCD; tiles past the XCD's pixels start at or after p_limit
    auto first_pixel = [&](uint32_t t) {
        return t < big_per_xcd ? (first + t * PS) * 32u
                               : (first + big_per_xcd * PS + (t - big_per_xcd) * PSB) * 32u;
    };
    auto end_pixel = [&](uint32_t t, uint32_t p) {
        return min(p + (t < big_per_xcd ? 32u * PS : 32u * PSB), p_limit);
    };
    if (first_pixel(tile) >= p_limit) return;
    // The two workgroups of a compute unit should not run the same phase at the same time: a
    // wave that has issued a tile's stores cannot take in the next tile's weight fragments
    // before those stores are acknowledged (one in-order counter for loads and stores), and
    // the matrix pipes should have the other workgroup's main loop to run meanwhile.  The
    // hardware places workgroups n and n + (workgroups per XCD) / 2 of an XCD on one CU; the
    // second of them walks its tiles in the opposite order (small tiles first) and may start
    // late.
    uint32_t step = tiles_per_round; // (to the next tile; the unsigned sum wraps when reversed)
    if (reverse_second != 0 && nth >= (tiles_per_round * oc_chunks) / 2) {
        uint32_t last = tile + (rounds - 1) * tiles_per_round;
        while (last != tile && first_pixel(last) >= p_limit) last -= tiles_per_round;
        tile = last;
        step = 0u - tiles_per_round;
    }
    if (nth >= (tiles_per_round * oc_chunks) / 2)
        for (uint32_t i = 0; i < stagger; i++) __builtin_amdgcn_s_sleep(16);
    uint32_t p_first = first_pixel(tile);
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    { // the first tile's words: into staging area 0 (the layout is conv_tile's)
        int lo, hi;
        tile_span(g, p_first, end_pixel(tile, p_first), lo, hi);
        const int nrows = min(hi - lo + 1, max_rows);
        const uint32_t stage = (uint32_t)(size_t)smem + TABLE_BYTES + ALPHA_BYTES;
        copy_to_lds_async(xbits + (size_t)lo * g.xw, nrows * g.xw, stage, tid, wave);
        copy_to_lds_async(a_plane + lo, nrows, stage + 2u * (uint32_t)(max_rows * g.xw) * 4u,
                tid, wave);
    }
    TileTurn turn{true, 0u, 0u, 0u};
    for (;;) {
        const uint32_t next = tile + step;
        // (walking backwards, tile numbers below the first wrap around to huge values)
        const uint32_t next_first = next < rounds * tiles_per_round ? first_pixel(next) : p_limit;
        const bool more = next_first < p_limit;
        turn.next_first = more ? next_first : 0u;
        turn.next_end = more ? end_pixel(next, next_first) : 0u;
        if (tile < big_per_xcd)
            conv_tile<KS, PS, false, PAIR, false, true>(xbits, wfrag, alpha, kplane, dst, nullptr,
                    g, max_rows, div_xw, a_plane, k_out, inv_khw, 1, wfrag_bytes, p_first,
                    p_limit, chunk, turn);
        else
            conv_tile<KS, PSB, false, PAIR, false, true>(xbits, wfrag, alpha, kplane, dst,
                    nullptr, g, max_rows, div_xw, a_plane, k_out, inv_khw, 1, wfrag_bytes,
                    p_first, p_limit, chunk, turn);
        if (!more) break;
        tile = next;
        p_first = next_first;
        turn.first = false;
        turn.parity ^= 1u;
    }
}

// Calibration only: the matrix instruction of the convolution kernel and nothing else.  Every
// wave multiplies pseudo-random +-1 fragments (the FP4 codes 0x2 and 0xA) that never leave
// its registers into eight independent accumulator blocks, `iterations` times.  What this
// reaches is what the matrix pipes deliver on this data under the chip's power management,
// with no operand traffic at all.
__global__ __launch_bounds__(256, 2)
void mfma_only_kernel(const int iterations) {
    auto signs = [](uint32_t h) { // eight FP4 codes, sign bits from h
        h *= 0x9E3779B1u;
        h ^= h >> 15;
        uint32_t spread = 0;
#pragma unroll
        for (int n = 0; n < 8; n++) spread |= ((h >> n) & 1u) << (4 * n + 3);
        return (int)(0x22222222u | spread);
    };
    const uint32_t id = blockIdx.x * 256u + threadIdx.x;
    v4i a[2], b[4];
#pragma unroll
    for (int i = 0; i < 2; i++)
        a[i] = v4i{signs(id * 24u + i * 4u), signs(id * 24u + i * 4u + 1), signs(id * 24u + i * 4u + 2),
                   signs(id * 24u + i * 4u + 3)};
#pragma unroll
    for (int i = 0; i < 4; i++)
        b[i] = v4i{signs(id * 24u + 8u + i * 4u), signs(id * 24u + 9u + i * 4u),
                   signs(id * 24u + 10u + i * 4u), signs(id * 24u + 11u + i * 4u)};
    v16f acc[2][4];
#pragma unroll
    for (int os = 0; os < 2; os++)
#pragma unroll
        for (int ps = 0; ps < 4; ps++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[os][ps][i] = 0.f;
    for (int it = 0; it < iterations; it++) {
#pragma unroll
        for (int os = 0; os < 2; os++)
#pragma unroll
            for (int ps = 0; ps < 4; ps++) acc[os][ps] = mfma_fp4(a[os], b[ps], acc[os][ps]);
    }
#pragma unroll
    for (int os = 0; os < 2; os++)
#pragma unroll
        for (int ps = 0; ps < 4; ps++) asm volatile("" : : "v"(acc[os][ps]));
}

// One thread per dword of the fragment layout [OC/32][tap][KS][lane][4 dwords]:
// lane l of a fragment holds filter (l % 32) and channels (l / 32) * 32 .. +31 of the step,
// eight channels per dword, low nibble first.  Channels >= IC and filters >= OC are FP4 zero.
// With pair set, [tap] runs over pairs of taps and the 2*KS half-steps of a pair are the KS
// 32-channel words of its first tap followed by those of its second (zero if there is none).
// With ic_parts > 1, [tap] runs over (tap, channel part) with the part innermost, and part p
// holds channels 64*KS*p onwards.
__global__ __launch_bounds__(256)
void pack_weights_fp4_kernel(const float *__restrict__ w, uint32_t *__restrict__ frag,
        const Geometry g, const int ks_n, const int oc_subs, const int pair,
        const int ic_parts) {
    const int taps = pair ? (g.kh * g.kw + 1) / 2 : g.kh * g.kw * ic_parts;
    const size_t total = (size_t)oc_subs * taps * ks_n * 64 * 4;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int dw = (int)(i & 3);
    const int lane = (int)((i >> 2) & 63);
    const size_t f = i >> 8; // fragment index
    const int ks = (int)(f % ks_n);
    int tap = (int)((f / ks_n) % taps);
    const int sub = (int)(f / ((size_t)ks_n * taps));
    const int oc = sub * 32 + (lane & 31);
    int c0 = ks * 64 + (lane >> 5) * 32 + dw * 8;
    if (ic_parts > 1) {
        c0 += (tap % ic_parts) * ks_n * 64;
        tap /= ic_parts;
    }
    if (pair) {
        const int word = 2 * ks + (lane >> 5); // of the 2*KS words of the pair
        tap = 2 * tap + (word >= ks_n ? 1 : 0);
        c0 = (word >= ks_n ? word - ks_n : word) * 32 + dw * 8;
    }
    const bool tap_exists = tap < g.kh * g.kw;
    const int kh = tap / g.kw, kw = tap % g.kw;
    uint32_t out = 0;
    for (int n = 0; n < 8; n++) {
        const int c = c0 + n;
        if (tap_exists && oc < g.oc && c < g.ic) {
            const size_t at = g.w_fmt == xnor_nn_weights_format_oihw
                ? (((size_t)oc * g.ic + c) * g.kh + kh) * g.kw + kw
                : (((size_t)kh * g.kw + kw) * g.ic + c) * g.oc + oc;
            out |= ((__float_as_uint(w[at]) >> 31) ? 0xAu : 0x2u) << (4 * n);
        }
    }
    frag[i] = out;
}

// Steps per tap as the kernel is instantiated: ceil(IC/64), odd counts above 4 rounded up,
// counts above 8 rounded up to 12 or 16 (the extra steps multiply FP4 zeros).
// Pairing two taps per KS = ceil(IC/32) steps pays when the number of 32-channel words is odd
// (otherwise every tap ends on a half-empty step) and small enough for the register file.
bool pair_taps(const Geometry &g) {
    const int taps = g.kh * g.kw;
    if ((g.xw & 1) == 0 || g.xw > 5 || taps < 2) return false;
    if (const char *e = getenv("XNOR_NN_HIP_MFMA_PAIR")) return e[0] == '1';
    return ((taps + 1) / 2) * g.xw < taps * ((g.xw + 1) / 2);
}
// More than 1024 channels: parts of 12 or 16 steps, as few padded steps as possible (the
// fewer parts on a tie).  Sets the steps per part; returns the number of parts, 1 if the
// channels fit one part.
int channel_parts(const Geometry &g, int *steps = nullptr) {
    const int ks = (g.ic + 63) / 64;
    int best_parts = 1, best_steps = 16;
    if (ks > 16) {
        best_parts = 0;
        for (int parts = 2; parts <= 6; parts++)
            for (int steps = 12; steps <= 16; steps += 4)
                if (parts * steps >= ks
                        && (best_parts == 0 || parts * steps < best_parts * best_steps)) {
                    best_parts = parts;
                    best_steps = steps;
                }
    }
    if (steps) *steps = best_steps;
    return best_parts;
}
int steps_per_tap(const Geometry &g) {
    if (pair_taps(g)) return g.xw; // per pair of taps
    const int ks = (g.ic + 63) / 64;
    if (ks > 16) {
        int steps;
        channel_parts(g, &steps);
        return steps;
    }
    if (ks > 8) return (ks + 3) / 4 * 4; // 12 or 16
    return ks > 4 && (ks & 1) ? ks + 1 : ks;
}
int oc_subblocks(const Geometry &g) { return ((g.oc + NT - 1) / NT) * (NT / 32); }

// Largest number of input pixels any tile of mt output pixels touches.  Tiles start at
// multiples of `step` pixels (their own size for a launch with one tile size, 32 for a launch
// with two); the offset of a tile within its image repeats after at most OHW starts, so that
// many (plus the last, possibly short, tile) are enough to look at.
int max_tile_rows(const Geometry &g, uint32_t mt, uint32_t step = 0) {
    if (step == 0) step = mt;
    const uint32_t starts = (g.npix_out + step - 1) / step;
    const uint32_t look = starts < (uint32_t)g.ohw + 1 ? starts : (uint32_t)g.ohw + 1;
    int most = 1;
    auto see = [&](uint32_t t) {
        int lo, hi;
        const uint32_t first = t * step;
        tile_span(g, first, first + mt < g.npix_out ? first + mt : g.npix_out, lo, hi);
        if (hi - lo + 1 > most) most = hi - lo + 1;
    };
    for (uint32_t t = 0; t < look; t++) see(t);
    see(starts - 1);
    return most;
}

// Pixel groups per tile: with 128 filters or fewer only two of a workgroup's four waves would
// have filters, with 64 or fewer only one; the others then take the same filters on further
// pixel blocks (see conv_tile).  Not with channel parts.  XNOR_NN_HIP_MFMA_GROUPS=1|2|4
// overrides (for measurements; more groups than idle waves are not taken).
int pixel_groups(const Geometry &g) {
    if (channel_parts(g) > 1) return 1;
    // two tile sizes in one launch or persistent workgroups asked for by name: one group
    if (const char *e = getenv("XNOR_NN_HIP_MFMA_MIX"))
        if (e[0] != '0') return 1;
    if (getenv("XNOR_NN_HIP_MFMA_PERSIST")) return 1;
    int groups = g.oc <= 64 ? 4 : g.oc <= 128 ? 2 : 1;
    if (const char *e = getenv("XNOR_NN_HIP_MFMA_GROUPS")) {
        const int v = atoi(e);
        if ((v == 1 || v == 2 || v == 4) && v <= groups) groups = v;
    }
    return groups;
}

size_t lds_bytes_for(const Geometry &g, size_t rows, int ps, bool persist = false) {
    const size_t row_bytes = pair_taps(g) ? g.xw * 16
        : channel_parts(g) * steps_per_tap(g) * 32 + ROW_PAD;
    // persistent workgroups: two staging areas for packed words and for mean|x| (conv_tile)
    const size_t stage = persist ? (2 * rows * g.xw * 4 + 2 * (rows + 1) * 4 + 15) & ~(size_t)15 : 0;
    const int groups = persist ? 1 : g.mfma_groups;
    size_t bytes = TABLE_BYTES + ALPHA_BYTES + stage + (1 + rows) * row_bytes
        + (rows + 1 + 32 * ps * groups) * sizeof(float);
    if (g.dst_fmt == xnor_nn_data_format_nhwc && (g.oc & 3) == 0) // turn-around rows, 4 waves
        bytes = ((bytes + 15) & ~(size_t)15) + 4 * 32 * TURN_ROW * sizeof(float);
    return bytes;
}
size_t lds_bytes(const Geometry &g, int ps) {
    return lds_bytes_for(g, (size_t)max_tile_rows(g, 32 * ps * g.mfma_groups), ps);
}

// 32-pixel blocks per tile, by a model of the kernel's time in core cycles that was fitted to
// measurements on MI355X (conv4 from MB 4 to MB 1024, ResNet 3x3 56x56 MB 1 to 64, VGG 512 MB
// 1 to 32, the conv2 shape, 64- and 128-channel layers; PS 1/2/3/4 at conv4 MB 256 = 34.7 /
// 27.0 / 26.6 / 27.5 us, at MB 32 = 8.2 / 9.4 / 11.7 / 13.8 us).
//   one wave:   staging (set-up, plus 264 cycles per 256 packed words to expand)
//               + PS x (epilogue 1700 + 64 per step of the main loop)
//               -- with one pixel block and more than one wave per SIMD a step costs as much
//               as with two: the weight stream (2 KB per wave and step whatever the tile)
//               sets its pace, not the matrix instructions;
//               Tiles of two pixel blocks pay 10 % more per step: their weight stream is
//               as wide as the vector-memory return path of the CU;
//   the kernel: one wave's time for the first wave of the busiest SIMD, 0.35 of it more for
//               every further wave that is resident with it (their phases overlap), and for
//               every wave beyond the resident ones 0.75 of it with two resident waves per
//               SIMD, 0.5 with three, 0.35 with four (small tiles of shallow inputs need at
//               most 168 or 128 registers, so a third or fourth workgroup fits a CU, and a
//               launch of many rounds of such tiles is faster than one of large tiles:
//               ResNet 3x3 56x56 MB 64 61.0 against 63.1 us, 128 filters on the same input
//               32.5 against 38.1, 64 filters 18.0 against 23.5); with few waves per SIMD the
//               busiest one counts (rounded up), with many the hardware's dynamic
//               scheduling evens the load out;
//   a tile that needs more than half the LDS runs alone on its CU: 15 % more.
// Ties go to the larger tile, which streams fewer weight bytes.
// Refitted on 56 shapes (13x13 to 112x112 images, 32 to 512 channels, 64 to 512 filters,
// 1x1 to 5x5 kernels, MB 1 to 1024) with every tile size forced in turn: the choice is the
// fastest tile on 50 of them and within 3.2 % on the rest.
// Four pixel blocks do not fit the register file with 16 steps per tap or with tap pairing
// over five words (those variants spill), and are not instantiated for channel parts.
bool tile_fits_registers(const Geometry &g, int ps) {
    if (ps < 4) return true;
    if (channel_parts(g) > 1) return false;
    return pair_taps(g) ? g.xw < 5 : steps_per_tap(g) < 16;
}

// Workgroups of a tile size that fit a compute unit together, two to four: by registers (the
// counts of the compiled variants: four pixel blocks 199 to 254, three 168 with one step per
// tap and 184 or more otherwise, two 119 with one step per tap, 135 to 167 with two to four or
// twelve steps and 188 or more otherwise, one 70 to 118 up to four steps and from twelve, 139
// or 149 with five or six, 181 with eight; a SIMD holds 512 per lane) and by LDS.
int resident_workgroups(const Geometry &g, int ps) {
    const int ks = steps_per_tap(g);
    int by_regs = 2;
    if (ps == 3) by_regs = ks == 1 ? 3 : 2;
    if (ps == 2) by_regs = ks == 1 ? 4 : (ks <= 4 || ks == 12) ? 3 : 2;
    if (ps == 1) by_regs = (ks <= 4 || ks >= 12) ? 4 : ks <= 6 ? 3 : 2;
    const int by_lds = (int)((size_t)LDS_LIMIT / lds_bytes(g, ps));
    const int fit = by_regs < by_lds ? by_regs : by_lds;
    return fit < 2 ? 2 : fit; // a tile that runs alone is priced separately
}

int pick_ps(const Geometry &g) {
    if (const char *e = getenv("XNOR_NN_HIP_MFMA_PS")) {
        const int v = atoi(e);
        if (v >= 1 && v <= 4 && lds_bytes(g, v) <= (size_t)LDS_LIMIT && tile_fits_registers(g, v))
            return v;
    }
    const int chunks = (g.oc + NT - 1) / NT;
    const double simds = (double)g.cus * 4;
    const int units = pair_taps(g) ? (g.kh * g.kw + 1) / 2 : g.kh * g.kw * channel_parts(g);
    const double steps_total = (double)units * steps_per_tap(g);
    int best = 0;
    double best_cost = 0;
    for (int ps = 4; ps >= 1; ps--) {
        if (lds_bytes(g, ps) > (size_t)LDS_LIMIT) continue;
        if (!tile_fits_registers(g, ps)) continue;
        const uint32_t mt = 32u * ps * g.mfma_groups; // pixels per tile
        const double tiles = (double)((g.npix_out + mt - 1) / mt);
        // workgroups per compute unit = waves per SIMD; a workgroup whose filters fill fewer
        // than four waves (OC below 256) still takes its slot with all four
        const double per_simd = tiles * chunks * 4 / simds;
        const double busiest = per_simd <= 1 ? 1.0
            : per_simd <= 4 ? (double)(long)(per_simd + 0.999999) : per_simd + 0.5;
        const double words = (double)max_tile_rows(g, mt) * g.xw;
        const double stream_bound = ps < 2 && per_simd > 1 ? 2.0 : (double)ps;
        const double wave = 3700.0 + 264.0 * words / 256.0 + 1700.0 * ps
            + (ps == 2 ? 70.4 : 64.0) * steps_total * stream_bound;
        const int resident = resident_workgroups(g, ps);
        const double further = resident >= 4 ? 0.35 : resident == 3 ? 0.5 : 0.75;
        const double together = busiest < resident ? busiest : (double)resident;
        const double waves = busiest < 2 ? 1.0
            : 1.0 + 0.35 * (together - 1.0) + further * (busiest - together);
        const double alone = lds_bytes(g, ps) > (size_t)LDS_TWO_PER_CU ? 1.15 : 1.0;
        const double cost = wave * waves * alone;
        if (best == 0 || cost < best_cost - 1e-9) { best = ps; best_cost = cost; }
    }
    return best;
}

template <int KS, int PS, bool PAIR, bool DEEP = false, int PSB = 0>
hipError_t launch_mfma(const Geometry &g, const uint32_t *xbits, const uint32_t *wfrag,
        const float *alpha, const float *k, float *dst, int32_t *popc,
        const float *a_or_null, float *k_out, hipStream_t s, const KernelEvents &ev) {
    const int chunks = (g.oc + NT - 1) / NT;
    const uint32_t mt = 32u * PS * (PSB > 0 ? 1u : (uint32_t)g.mfma_groups);
    const uint32_t tiles = (g.npix_out + mt - 1) / mt;
    const uint32_t units = tiles * chunks;
    uint32_t per_xcd = (units + 7) / 8; // workgroups per XCD
    uint32_t big = 0, blocks = 0;
    if constexpr (PSB > 0) { // two tile sizes: see the kernel
        blocks = g.mfma_blocks_per_xcd;
        big = g.mfma_big_per_xcd;
        const uint32_t rest = blocks > big * PS ? blocks - big * PS : 0;
        per_xcd = (big + (rest + PSB - 1) / PSB) * chunks;
    }
    const dim3 grid(per_xcd * 8), block(256);
    const int rows = g.mfma_rows;
    const size_t lds = g.mfma_lds;
    const int parts = g.mfma_parts;
    const v4i *wf = reinterpret_cast<const v4i *>(wfrag);
    if (lds > (size_t)LDS_DEFAULT) {
        // asked for once per kernel, device and size (what has been granted is remembered)
        static std::atomic<size_t> granted[2][MAX_DEVICES];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
            return hipErrorInvalidDevice;
        std::atomic<size_t> &have = granted[popc ? 1 : 0][dev];
        if (lds > have.load(std::memory_order_acquire)) {
            const void *fn = popc
                ? (const void *)conv_mfma_fp4_kernel<KS, PS, PSB, true, PAIR, DEEP>
                : (const void *)conv_mfma_fp4_kernel<KS, PS, PSB, false, PAIR, DEEP>;
            const hipError_t e = hipFuncSetAttribute(fn,
                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            have.store(lds, std::memory_order_release);
        }
    }
    if (popc)
        launch_kernel(conv_mfma_fp4_kernel<KS, PS, PSB, true, PAIR, DEEP>, grid, block, lds, s,
                ev, xbits, wf, alpha, k, dst, popc, g, rows, chunks, units, per_xcd,
                FastDiv::make((uint32_t)g.xw), a_or_null, k_out, 1.f / g.kh / g.kw, parts,
                g.mfma_wbytes, big, blocks);
    else
        launch_kernel(conv_mfma_fp4_kernel<KS, PS, PSB, false, PAIR, DEEP>, grid, block, lds, s,
                ev, xbits, wf, alpha, k, dst, popc, g, rows, chunks, units, per_xcd,
                FastDiv::make((uint32_t)g.xw), a_or_null, k_out, 1.f / g.kh / g.kw, parts,
                g.mfma_wbytes, big, blocks);
    return hipGetLastError();
}

template <int KS, bool PAIR>
hipError_t launch_mfma_persistent(const Geometry &g, const uint32_t *xbits,
        const uint32_t *wfrag, const float *alpha, const float *k, float *dst,
        const float *a_or_null, float *k_out, hipStream_t s, const KernelEvents &ev) {
    const int chunks = (g.oc + NT - 1) / NT;
    const dim3 grid(g.mfma_tiles_per_round * chunks * 8), block(256);
    const size_t lds = g.mfma_lds;
    const auto kernel = conv_mfma_fp4_persistent_kernel<KS, 4, 3, PAIR>;
    if (lds > (size_t)LDS_DEFAULT) { // asked for once per device and size
        static std::atomic<size_t> granted[MAX_DEVICES];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
            return hipErrorInvalidDevice;
        if (lds > granted[dev].load(std::memory_order_acquire)) {
            const hipError_t e = hipFuncSetAttribute((const void *)kernel,
                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            granted[dev].store(lds, std::memory_order_release);
        }
    }
    launch_kernel(kernel, grid, block, lds, s, ev, xbits, reinterpret_cast<const v4i *>(wfrag),
            alpha, k, dst, g, g.mfma_rows, chunks, g.mfma_tiles_per_round,
            FastDiv::make((uint32_t)g.xw), a_or_null, k_out, 1.f / g.kh / g.kw, g.mfma_wbytes,
            g.mfma_big_per_xcd, g.mfma_blocks_per_xcd, g.mfma_rounds, g.mfma_reverse,
            g.mfma_stagger);
    return hipGetLastError();
}

template <int KS>
hipError_t launch_mfma_deep(const Geometry &g, const uint32_t *xbits, const uint32_t *wfrag,
        const float *alpha, const float *k, float *dst, int32_t *popc,
        const float *a_or_null, float *k_out, hipStream_t s, const KernelEvents &ev) {
    switch (g.mfma_ps) {
    case 1: return launch_mfma<KS, 1, false, true>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 2: return launch_mfma<KS, 2, false, true>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 3: return launch_mfma<KS, 3, false, true>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    }
    return hipErrorInvalidValue;
}

template <int KS, bool PAIR = false>
hipError_t launch_mfma_ps(const Geometry &g, const uint32_t *xbits, const uint32_t *wfrag,
        const float *alpha, const float *k, float *dst, int32_t *popc,
        const float *a_or_null, float *k_out, hipStream_t s, const KernelEvents &ev) {
    if (g.mfma_ps_small > 0) { // two tile sizes: four blocks, and two or three
        if constexpr (KS < 16 && !(PAIR && KS >= 5)) {
            // persistent workgroups; the raw accumulators, and a pass that reads a K plane
            // instead of mean|x|, go through the same tiles with a workgroup per tile
            if (g.mfma_persist && popc == nullptr && a_or_null != nullptr)
                return launch_mfma_persistent<KS, PAIR>(g, xbits, wfrag, alpha, k, dst,
                        a_or_null, k_out, s, ev);
            if (g.mfma_ps_small == 3)
                return launch_mfma<KS, 4, PAIR, false, 3>(g, xbits, wfrag, alpha, k, dst, popc,
                        a_or_null, k_out, s, ev);
            return launch_mfma<KS, 4, PAIR, false, 2>(g, xbits, wfrag, alpha, k, dst, popc,
                    a_or_null, k_out, s, ev);
        }
        return hipErrorInvalidValue;
    }
    switch (g.mfma_ps) {
    case 1: return launch_mfma<KS, 1, PAIR>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 2: return launch_mfma<KS, 2, PAIR>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 3: return launch_mfma<KS, 3, PAIR>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 4:
        // four pixel blocks with 16 steps per tap, or with tap pairing over five words, do not
        // fit the register file (tile_fits_registers) and are not compiled
        if constexpr (KS < 16 && !(PAIR && KS >= 5))
            return launch_mfma<KS, 4, PAIR>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
        break;
    }
    return hipErrorInvalidValue;
}

} // namespace

// The matrix-core kernel covers convolutions with up to 4096 input channels whose
// tile of input rows fits the 160 KB of LDS; everything else runs the XNOR/popcount kernel.
// XNOR_NN_HIP_CONV=valu forces the latter (used to profile the two side by side).
// Returns the tile size (32-pixel blocks per workgroup, 1..4) or 0 when not applicable.
static int mfma_tile_blocks(const Geometry &g) {
    if (const char *e = getenv("XNOR_NN_HIP_CONV"))
        if (e[0] == 'v') return 0;
    if ((g.ic + 63) / 64 > 64) return 0;
    if (g.kh > 32 || g.kw > 32) return 0; // taps inside the image are kept as 32-bit masks
    if ((uint64_t)g.npix_out * g.oc * 4u >= 0xFFFFFFF0ull) return 0; // 32-bit output offsets
    if ((uint64_t)g.npix_in * g.xw > 0x7FFFFFFFull) return 0;
    if (mfma_weight_bytes(g) >= 0xFFFFFFF0ull) return 0; // 32-bit fragment offsets
    return pick_ps(g);
}

size_t mfma_weight_bytes(const Geometry &g) {
    const int units = pair_taps(g) ? (g.kh * g.kw + 1) / 2 : g.kh * g.kw * channel_parts(g);
    return (size_t)oc_subblocks(g) * units * steps_per_tap(g) * 1024;
}

void mfma_plan(Geometry &g) {
    // as many pixel groups as idle waves, fewer if even a one-block tile would not fit the LDS
    for (g.mfma_groups = pixel_groups(g); g.mfma_groups > 1; g.mfma_groups /= 2)
        if (lds_bytes(g, 1) <= (size_t)LDS_LIMIT) break;
    g.mfma_ps = mfma_tile_blocks(g);
    g.use_mfma = g.mfma_ps > 0 ? 1 : 0;
    g.mfma_steps = g.mfma_pair = g.mfma_rows = 0;
    g.mfma_ps_small = 0;
    g.mfma_big_per_xcd = g.mfma_blocks_per_xcd = 0;
    g.mfma_small = g.mfma_small_rows = 0;
    g.mfma_small_lds = 0;
    g.mfma_persist = g.mfma_reverse = 0;
    g.mfma_tiles_per_round = g.mfma_rounds = g.mfma_stagger = 0;
    g.stream_dst = 0;
    g.mfma_parts = 1;
    g.mfma_lds = g.mfma_wbytes = 0;
    if (!g.use_mfma) return;
    // Output stores stream past the caches when the input of the next forward pass and this
    // output cannot both stay in the 256 MB Infinity Cache, and the runs of one filter start
    // on 64-byte boundaries: with ragged planes (13 x 13, 27 x 27) streaming stores leave
    // partial lines behind and cost the kernel 15 to 25 %, more than the next pass gains.
    // XNOR_NN_HIP_STREAM_DST=0|1 overrides, for measurements.
    const uint64_t in_bytes = (uint64_t)g.npix_in * g.ic * 4u;
    const uint64_t out_bytes = (uint64_t)g.npix_out * g.oc * 4u;
    const uint32_t run_bytes = g.dst_fmt == xnor_nn_data_format_nchw ? (uint32_t)g.ohw * 4u
                                                                     : (uint32_t)g.oc * 4u;
    g.stream_dst = in_bytes + out_bytes > (200ull << 20) && run_bytes % 64 == 0 ? 1 : 0;
    if (const char *e = getenv("XNOR_NN_HIP_STREAM_DST")) g.stream_dst = e[0] == '1' ? 1 : 0;
    g.mfma_steps = steps_per_tap(g);
    g.mfma_pair = pair_taps(g) ? 1 : 0;
    g.mfma_parts = channel_parts(g);
    g.mfma_rows = max_tile_rows(g, 32 * g.mfma_ps * g.mfma_groups);
    g.mfma_lds = (uint32_t)lds_bytes(g, g.mfma_ps);
    g.mfma_wbytes = (uint32_t)mfma_weight_bytes(g);
    // Few tiles: the small-problem kernel takes the scaled output (the raw accumulators still
    // go through the kernel planned below).
    {
        int rows = 0;
        uint32_t lds = 0;
        if (small_kernel_applies(g, &rows, &lds)) {
            g.mfma_small = 1;
            g.mfma_small_rows = rows;
            g.mfma_small_lds = lds;
        }
    }
    // Two tile sizes in one launch (see the kernel): worth it when every compute unit gets
    // more than four and at most six pixel blocks, i.e. when equal tiles would give it two
    // workgroups of three that finish together.  Needs the four-block variant and room for
    // two workgroups in a CU's LDS.  XNOR_NN_HIP_MFMA_MIX=0|1|3 overrides the size rules (off,
    // four and two, four and three; for measurements), a forced tile size switches them off.
    const uint32_t blocks = (g.npix_out + 31) / 32, blocks_per_xcd = (blocks + 7) / 8;
    const uint32_t cus_per_xcd = (uint32_t)(g.cus + 7) / 8;
    // The same in filter chunks: `slots` workgroups per XCD and chunk when every CU holds two.
    const uint32_t chunks = (uint32_t)(g.oc + NT - 1) / NT;
    const uint32_t slots = 2 * cus_per_xcd / chunks;
    bool mix = chunks == 1 && blocks_per_xcd > 4 * cus_per_xcd && blocks_per_xcd <= 6 * cus_per_xcd;
    // Between three and four blocks per slot, equal tiles of four leave slots empty and tiles
    // of three need a second round for the last few: blocks - 3 * slots tiles of four and
    // tiles of three for the rest fill every slot exactly once (VGG 512, MB 32: 98 blocks
    // and 32 slots per XCD and chunk: 2 tiles of four, 30 of three).
    bool fill = slots > 0 && blocks_per_xcd > 3 * slots && blocks_per_xcd < 4 * slots;
    if (const char *e = getenv("XNOR_NN_HIP_MFMA_MIX")) {
        mix = e[0] == '1';
        fill = e[0] == '3';
    }
    if (getenv("XNOR_NN_HIP_MFMA_PS") || g.mfma_parts > 1 || g.mfma_steps >= 16
            || (g.mfma_pair && g.xw >= 5) || !tile_fits_registers(g, 4) || g.mfma_groups > 1)
        mix = fill = false;
    // Persistent workgroups (see the kernel): only on request, XNOR_NN_HIP_MFMA_PERSIST=N with
    // N workgroups per XCD (64 = two per compute unit).  Measured on MI355X they are slower than
    // a workgroup per tile wherever a launch has several rounds of tiles (ResNet 3x3 MB 64:
    // 68.4 against 66.0 us, conv2 shape MB 128: 41.4 against 40.7 us): the two workgroups of a
    // compute unit then run every phase at the same time, so staging (4.9 us per tile) and
    // stores (2.5 to 4.3 us) overlap no matrix instructions, where workgroups dispatched one
    // by one drift apart.  Kept because tests walk small problems in many rounds this way.
    // With `per_round` (tile, chunk) slots per XCD a workgroup gets n = ceil(blocks /
    // per_round) pixel blocks, walked as a rounds of four-block tiles and b rounds of
    // three-block tiles, 4a + 3b >= n as small as possible, a as large as possible.
    {
        uint32_t wgs_per_xcd = 0;
        if (const char *e = getenv("XNOR_NN_HIP_MFMA_PERSIST"))
            wgs_per_xcd = (uint32_t)(atoi(e) > 0 ? atoi(e) : 0);
        const uint32_t per_round = wgs_per_xcd / chunks;
        const uint32_t n = per_round ? (blocks_per_xcd + per_round - 1) / per_round : 0;
        bool persist = n >= 1;
        if (getenv("XNOR_NN_HIP_MFMA_PS") || getenv("XNOR_NN_HIP_MFMA_MIX") || g.mfma_parts > 1
                || g.mfma_steps >= 16 || (g.mfma_pair && g.xw >= 5) || !tile_fits_registers(g, 4))
            persist = false;
        if (persist) {
            const int rows = max_tile_rows(g, 32 * 4, 32);
            const size_t lds = lds_bytes_for(g, (size_t)rows, 4, true);
            if (lds <= (size_t)LDS_TWO_PER_CU) {
                uint32_t best_a = 0, best_total = 0;
                for (uint32_t a = 0; 4 * a <= n + 3; a++) {
                    const uint32_t rest = n > 4 * a ? n - 4 * a : 0, b = (rest + 2) / 3;
                    const uint32_t total = 4 * a + 3 * b;
                    if (best_total == 0 || total < best_total || (total == best_total && a > best_a)) {
                        best_a = a;
                        best_total = total;
                    }
                }
                g.mfma_persist = 1;
                g.mfma_groups = 1; // a persistent workgroup walks tiles of one pixel group
                g.mfma_tiles_per_round = per_round;
                g.mfma_rounds = best_a + (best_total - 4 * best_a) / 3;
                g.mfma_reverse = 0;
                g.mfma_stagger = 0;
                if (const char *e = getenv("XNOR_NN_HIP_MFMA_REVERSE")) g.mfma_reverse = e[0] == '1';
                if (const char *e = getenv("XNOR_NN_HIP_MFMA_STAGGER")) g.mfma_stagger = (uint32_t)atoi(e);
                g.mfma_ps = 4;
                g.mfma_ps_small = 3;
                g.mfma_big_per_xcd = best_a * per_round;
                g.mfma_blocks_per_xcd = blocks_per_xcd;
                g.mfma_rows = rows;
                g.mfma_lds = (uint32_t)lds;
                return;
            }
        }
    }
    if (mix || fill) {
        const int rows = max_tile_rows(g, 32 * 4, 32);
        const size_t lds = lds_bytes_for(g, (size_t)rows, 4);
        if (lds <= (size_t)LDS_TWO_PER_CU) {
            g.mfma_ps = 4;
            g.mfma_blocks_per_xcd = blocks_per_xcd;
            if (mix) {
                g.mfma_ps_small = 2;
                const uint32_t fit = blocks_per_xcd / 4; // whole four-block tiles in the range
                g.mfma_big_per_xcd = fit < cus_per_xcd ? fit : cus_per_xcd;
            } else {
                g.mfma_ps_small = 3;
                g.mfma_big_per_xcd = blocks_per_xcd > 3 * slots ? blocks_per_xcd - 3 * slots : 0;
                if (g.mfma_big_per_xcd > blocks_per_xcd / 4) g.mfma_big_per_xcd = blocks_per_xcd / 4;
            }
            g.mfma_rows = rows;
            g.mfma_lds = (uint32_t)lds;
        }
    }
}

hipError_t launch_mfma_only(int workgroups, int iterations, hipStream_t s) {
    hipLaunchKernelGGL(mfma_only_kernel, dim3((unsigned)workgroups), dim3(256), 0, s, iterations);
    return hipGetLastError();
}

hipError_t launch_pack_weights_fp4(const Geometry &g, const float *w, uint32_t *frag,
        hipStream_t s) {
    const size_t dwords = g.mfma_wbytes / 4;
    hipLaunchKernelGGL(pack_weights_fp4_kernel, dim3((unsigned)((dwords + 255) / 256)),
            dim3(256), 0, s, w, frag, g, g.mfma_steps, oc_subblocks(g), g.mfma_pair, g.mfma_parts);
    return hipGetLastError();
}

const char *mfma_kernel_name(const Geometry &g) {
    static thread_local char name[80];
    if (g.mfma_small)
        snprintf(name, sizeof name, "conv_mfma_fp4_small_kernel<KS=%d>", g.mfma_steps);
    else if (g.mfma_parts > 1)
        snprintf(name, sizeof name, "conv_mfma_fp4_kernel<KS=%d,PS=%d,PARTS=%d>",
                g.mfma_steps, g.mfma_ps, g.mfma_parts);
    else if (g.mfma_persist)
        snprintf(name, sizeof name, "conv_mfma_fp4_persistent_kernel<KS=%d,PS=%d+%d%s>",
                g.mfma_steps, g.mfma_ps, g.mfma_ps_small, g.mfma_pair ? ",PAIR" : "");
    else if (g.mfma_ps_small > 0)
        snprintf(name, sizeof name, "conv_mfma_fp4_kernel<KS=%d,PS=%d+%d%s>", g.mfma_steps,
                g.mfma_ps, g.mfma_ps_small, g.mfma_pair ? ",PAIR" : "");
    else if (g.mfma_groups > 1)
        snprintf(name, sizeof name, "conv_mfma_fp4_kernel<KS=%d,PS=%d%s,GROUPS=%d>", g.mfma_steps,
                g.mfma_ps, g.mfma_pair ? ",PAIR" : "", g.mfma_groups);
    else
        snprintf(name, sizeof name, "conv_mfma_fp4_kernel<KS=%d,PS=%d%s>", g.mfma_steps,
                g.mfma_ps, g.mfma_pair ? ",PAIR" : "");
    return name;
}

hipError_t launch_convolution_mfma(const Geometry &g, const uint32_t *xbits,
        const uint32_t *wfrag, const float *alpha, const float *k,
        float *dst, int32_t *popc, const float *a_or_null, float *k_out, hipStream_t s, const KernelEvents &ev) {
    if (g.mfma_small && popc == nullptr)
        return launch_convolution_small(g, xbits, wfrag, alpha, k, dst, a_or_null, k_out, s, ev);
    if (g.mfma_pair) {
        switch (g.xw) {
        case 1: return launch_mfma_ps<1, true>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
        case 3: return launch_mfma_ps<3, true>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
        case 5: return launch_mfma_ps<5, true>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
        }
        return hipErrorInvalidValue;
    }
    if (g.mfma_parts > 1) {
        if (g.mfma_steps == 12)
            return launch_mfma_deep<12>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
        return launch_mfma_deep<16>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    }
    switch (g.mfma_steps) {
    case 1: return launch_mfma_ps<1>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 2: return launch_mfma_ps<2>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 3: return launch_mfma_ps<3>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 4: return launch_mfma_ps<4>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 6: return launch_mfma_ps<6>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 8: return launch_mfma_ps<8>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 12: return launch_mfma_ps<12>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    case 16: return launch_mfma_ps<16>(g, xbits, wfrag, alpha, k, dst, popc, a_or_null, k_out, s, ev);
    }
    return hipErrorInvalidValue;
}

} // namespace xnor_hip
