// Large-M GEMM over 8-bit operands on the CDNA4 matrix cores:
//     fp8 e4m3 x fp8 e4m3 -> fp32   (v_mfma_f32_32x32x64_f8f6f4)
//     int8     x int8     -> int32  (v_mfma_i32_32x32x32_i8)
//   y[M, N] = epi( (x[M, K] . w[N, K]^T) * scale + bias[N] )
// Both operands are K-contiguous, which is the layout the MFMA wants: a lane
// supplies 32 consecutive bytes of one row.
//
// Tiling.  One workgroup of 4 wavefronts (2 x 2) owns a 256 x 256 tile of y;
// each wavefront owns 128 x 128 of it as 4 x 4 MFMA tiles of 32 x 32, i.e. 256
// fp32/int32 accumulators per lane (the AGPR half of the unified register
// file), one workgroup per CU.  A tile this large is what keeps operand traffic
// down: a stage moves 64 KiB from L2 into a CU for 2048 cycles of MFMA work.
//
// K loop.  Stages of BK = 128 bytes: x tile 256 x 128 B and w tile 256 x 128 B
// (64 KiB), double-buffered in LDS (128 of the CU's 160 KiB).  While a stage is
// being multiplied, the stage after next streams from global memory straight
// into the buffer the previous stage has just freed (global_load_lds_dwordx4, 16
// per lane per stage): no registers, no ds_write, one wait + one barrier per
// stage.
//
// What bounds the loop, measured on this GPU (8192 x 4096 x 4096 fp8, stamps of the
// cycle counter around the loop, parts switched off one at a time).  In cycles, with
// N(0,1) data: the whole stage 2610 at a clock of 1.82 GHz; without the barrier 2340;
// without the transfers 2280; MFMAs alone 2230 (2048 + the switches' own branches).
// Barrier and transfers cost little each and ~450 cycles together: right after the
// barrier all four wavefronts ask the CU's address unit for their 16 KiB at once, the
// issue blocks, and the MFMAs queue up behind it.  Neither L2 nor LDS is near a limit:
// the same transfers alone, two stages in flight, land in 1390 cycles (47 B/clk per
// CU, 26 TB/s over the chip), from one CU alone in 1030 (the 64 B/clk of the L1 path),
// and the LDS serves the stage's 128 KiB of fragment reads in 517 cycles (253 B/clk)
// while taking the transfers' writes at full rate.
// But cycles are not what the time is made of here.  A variant with four 32 KiB
// buffers that spreads each refill over a whole stage takes 2390 cycles per stage -
// and runs at 1.67 GHz instead of 1.82: 1.43 us per stage either way.  With all-zero
// or constant activations the same two kernels run at 2.24 - 2.38 GHz and the call
// takes 93 - 98 us instead of 114 - 121.  On data that toggles the multipliers the
// loop sits on the board's power limit: the governor trades every cycle saved for
// clock, so what is left to gain is energy per stage (bytes moved, instructions
// issued), not issue slots.  MFMAs alone, on random data, are held to 3.7 - 3.9
// PFLOP/s by the same limit; this loop delivers 2.4 of them.
// (All of the above was timed within milliseconds of an idle spell.  The board's power
// management needs 30 - 40 ms of load to settle, and then leaves more clock: MFMAs alone
// on random data 4.28 PFLOP/s at 2.08 GHz, a stage of this loop 1.28 us, the call 101 -
// 110 us, 2.5 - 2.7 PFLOP/s.  The proportions hold: the loop is at 78 % of what the
// matrix cores alone sustain on such data.)
//
// LDS layout.  Row-major [256][128 B] with the eight 16-byte slots of a row
// permuted by slot ^= (row >> 1) & 7.  Rows r and r + 1 then sit 128 B apart in
// different bank halves and rows two apart in different slots, so both the
// 128-bit fragment reads (32 rows x 2 slots per wavefront instruction) and the
// staging writes are conflict free.
//
// Epilogue.  The MFMA takes the weight tile as its first operand, so a lane
// ends up with one token and runs of four consecutive channels; results are
// staged per wavefront through LDS and leave as 128-bit stores covering whole
// 256/512-byte row segments of y (2-byte scattered stores cost 37 % of the
// kernel before).
//
// Workgroup order.  Hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs, each with its own L2.  Ids are first regrouped so that each XCD
// gets one contiguous run of tiles, and runs walk the tile grid in bands of 8
// row tiles, so the ~32 tiles resident on an XCD share 8 x-tiles and 4 w-tiles
// in that XCD's L2 instead of 32 + 32.
#include <type_traits>

#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

constexpr int BM = 256;  // rows of x per workgroup tile (2 wavefronts x 128)

struct Gemm8Params {
    const uint8_t* a;  // x [M][K]
    const uint8_t* b;  // w [N][K]
    void* y;
    const void* bias;
    const float* row_scale;  // int8: per-row activation scales [M]; fp8: [1]
    const float* col_scale;  // int8: per-channel weight scales [N]
    float tscale;            // fp8: the weight's per-tensor scale
    int32_t M, N, K;
    int32_t tiles_m, tiles_n;
    int32_t y_dtype, bias_dtype, epilogue;
    unsigned long long* stamps;  // a diagnostic: per workgroup, four readings of the constant 100 MHz clock, or null
    int32_t chan_vec;  // N % 4 == 0 and col_scale / bias aligned for one 16-byte (bf16 bias: 8-byte) load per 4 channels
};

__device__ __forceinline__ uint16_t f32_to_bf16(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

// BN and BK are parameters of the body for the arithmetic's sake; the tile built is 256 x 256 with
// BK = 128 (a 256 x 128, BK = 64 variant with two workgroups per CU measured slower: its stage is
// too short for a transfer to land in).
// KIND: the output type the epilogue is built for (0 fp32, 1 bf16, 2 raw int32 accumulators); one
// kernel per kind, because with all three in one function the register allocator spills.
template <bool FP8, int KIND_, int BN, int BK>
__device__ __forceinline__ void gemm8_body(const Gemm8Params& p) {
    constexpr int STAGE_BYTES = (BM + BN) * BK;
    constexpr int SLOTS = BK / 16;     // 16-byte slots per LDS row
    constexpr int SWZ = SLOTS - 1;     // slot ^= (row >> 1) & SWZ
    constexpr int WN = BN / 2;         // channels per wavefront
    constexpr int TJ = WN / 32;        // weight fragments (MFMA tiles along N) per wavefront
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const unsigned long long t_entry = wall_clock64();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform, and known to be
    const int wm = wave >> 1, wn = wave & 1;

    // ---- XCD-aware tile assignment
    const int nb = gridDim.x;
    const int bid = blockIdx.x;
    const int per = nb / 8, rem = nb % 8;
    const int xcd = bid % 8, local = bid / 8;
    const int lid = xcd * per + min(xcd, rem) + local;
    constexpr int GM = 8;
    const int band = lid / (GM * p.tiles_n);
    const int first_m = band * GM;
    const int band_rows = min(GM, p.tiles_m - first_m);
    const int in_band = lid - band * GM * p.tiles_n;
    const int tm = first_m + in_band % band_rows;
    const int tn = in_band / band_rows;
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- global -> LDS, direct (global_load_lds_dwordx4): no register round trip.  One
    // instruction fills 1 KiB of LDS, lane l at byte 16 l, i.e. 1024 / BK rows; wavefront w owns
    // a quarter of the rows of both tiles.  The slot swizzle is applied on the global side: the
    // lane that lands in physical slot s of its row fetches logical slot s ^ swz(row).
    typedef __attribute__((address_space(3))) void lptr_t;
    constexpr int DROWS = 1024 / BK;           // rows per instruction
    constexpr int DA = BM / 4 / DROWS;         // instructions per wavefront and stage, x tile
    constexpr int DB = BN / 4 / DROWS;         // ... w tile
    // addresses as a uniform 64-bit tile base (advanced by k0) plus a 32-bit per-lane offset, and
    // the LDS destination as a scalar: two instructions per transfer (set M0, issue)
    const uint8_t* const abase = p.a + (int64_t)m0 * p.K;
    const uint8_t* const bbase = p.b + (int64_t)n0 * p.K;
    uint32_t doff[DA + DB];
#pragma unroll
    for (int t = 0; t < DA; t++) {
        const int row = wave * (BM / 4) + t * DROWS + lane / SLOTS;
        const int slot = (lane % SLOTS) ^ ((row >> 1) & SWZ);
        doff[t] = (uint32_t)(min(m0 + row, p.M - 1) - m0) * (uint32_t)p.K + slot * 16;
    }
#pragma unroll
    for (int t = 0; t < DB; t++) {
        const int row = wave * (BN / 4) + t * DROWS + lane / SLOTS;
        const int slot = (lane % SLOTS) ^ ((row >> 1) & SWZ);
        doff[DA + t] = (uint32_t)(min(n0 + row, p.N - 1) - n0) * (uint32_t)p.K + slot * 16;
    }
    // transfer t (0 .. DA+DB-1) of a stage: M0 = the LDS address of the 1 KiB the instruction
    // fills (a scalar base of the buffer half plus t KiB), global address = scalar base + lane
    // offset.  Three instructions per transfer.  (M0 is a reserved register the compiler sets itself
    // right before each of its own uses, so writing it here needs no clobber; SCC does.)
    const uint32_t lds_addr0 = (uint32_t)(uintptr_t)(lptr_t*)lds;
    uint32_t dbase[2][2];  // [buffer][x tile, w tile]: this wavefront's first destination
#pragma unroll
    for (int buf = 0; buf < 2; buf++) {
        dbase[buf][0] = lds_addr0 + buf * STAGE_BYTES + wave * (BM / 4) * BK;
        dbase[buf][1] = lds_addr0 + buf * STAGE_BYTES + BM * BK + wave * (BN / 4) * BK;
    }
#define NQ_DMA(t, buf, srca, srcb)                                                                     \
    do {                                                                                               \
        if constexpr ((t) < DA)                                                                        \
            asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"           \
                         :                                                                             \
                         : "s"(dbase[buf][0]), "v"(doff[(t)]), "s"(srca), "n"((t) * 1024)              \
                         : "memory", "scc");                                                            \
        else                                                                                           \
            asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"           \
                         :                                                                             \
                         : "s"(dbase[buf][1]), "v"(doff[(t)]), "s"(srcb), "n"(((t) - DA) * 1024)       \
                         : "memory", "scc");                                                            \
    } while (0)
    const float fp8_scale = FP8 ? p.tscale * p.row_scale[0] : 0.0f;  // requested now, used in the epilogue

    typedef typename std::conditional<FP8, f32x16, i32x16>::type acc_t;
    acc_t acc[4][TJ];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // Fragment addressing.  fp8: a 64-byte k-step, this lane supplies bytes [32 h, 32 h + 32) of
    // its row (h = lane / 32), i.e. slots 4 s + 2 h and 4 s + 2 h + 1.  int8: a 32-byte k-step,
    // bytes [16 h, 16 h + 16), slot 2 s + h.  Tile bases are multiples of 32 rows, so the swizzle
    // term depends on the row within the tile only.
    const int frow = lane & 31;
    const int fh = lane >> 5;
    const int fsw = (frow >> 1) & SWZ;

    // ---- main loop, software-pipelined by hand, with the LDS reads and their waits written out.
    // Measured on this GPU: an MFMA 32x32x64 occupies the matrix core for 64 cycles and other
    // instructions of the same wavefront issue in its shadow, about seven of them; past that
    // every extra instruction delays the next MFMA.  With one wavefront per SIMD the loop is
    // therefore laid out so that no gap between two MFMAs holds more than a handful of
    // instructions, and nothing in it waits longer than it must:
    //   - the compiler's own s_waitcnt before a use of loaded data is lgkmcnt(0) here (it waits
    //     for every read in flight), so the fragment reads are inline-asm ds_read_b128 whose
    //     latency the compiler does not see, and each MFMA is preceded by s_waitcnt lgkmcnt(N)
    //     with N from a compile-time model of the issue order (Sched): "all but the N youngest
    //     reads have landed";
    //   - per stage of G = 4 SPS groups (a group = the TJ MFMAs of one x fragment): the x
    //     fragment of group g+2 is requested in group g (four register sets in rotation), the
    //     w fragments of the next sub-step in the first two groups of the current one (two
    //     sets), each after the group's first MFMA;
    //   - the stage's only barrier sits at the start of its last-but-one group, with vmcnt(0)
    //     (this wavefront's part of the next stage has landed) and lgkmcnt(0) (its reads of
    //     this stage are done: the buffer may be overwritten); the two groups after it request
    //     the next stage's first fragments and issue the global -> LDS transfers of the stage
    //     after next into the buffer just freed, two or three between consecutive MFMAs, so a
    //     transfer has a whole stage to land;
    //   - the K loop is unrolled by two stages so that buffer addresses are loop invariants.
    // __builtin_amdgcn_sched_barrier(0) pins the order against the instruction scheduler.
    constexpr int KE = FP8 ? 64 : 32;       // bytes of K one MFMA consumes
    constexpr int SPS = BK / KE;             // sub-steps (one MFMA k-extent each) per stage
    constexpr int G = 4 * SPS;               // groups per stage
    constexpr int R = FP8 ? 2 : 1;           // 128-bit reads per fragment
    constexpr int HB = TJ / 2;               // w fragments requested per group (in the groups that request any)
    static_assert(SPS % 2 == 0 && TJ == 4, "register-set rotation and transfer slots assume this tile");

    struct Sched {
        // reads requested in group g (after its first MFMA): the x fragment of group g+2, then w fragments
        static constexpr int wfrags(int g) {
            const int sub = g / 4, i = g % 4;
            return (sub < SPS - 1) ? (i < 2 ? HB : 0) : (i >= 2 ? HB : 0);
        }
        static constexpr int reads(int g) { return R * (1 + wfrags(g)); }
        static constexpr int before(int g) {  // reads requested in groups 0..g-1 of a stage
            int n = 0;
            for (int t = 0; t < g; t++) n += reads(t);
            return n;
        }
        static constexpr int total() { return before(G); }
        // position (reads since the start of the stage, negative = previous stage) of the LAST read of ...
        static constexpr int pos_a(int g) {  // ... the x fragment group g consumes
            return g >= 2 ? before(g - 2) + R - 1 : before(G + g - 2) + R - 1 - total();
        }
        static constexpr int pos_b(int sub, int j) {  // ... w fragment j of sub-step sub
            const int g = sub >= 1 ? (sub - 1) * 4 + j / HB : (SPS - 1) * 4 + 2 + j / HB;
            const int pos = before(g) + R + (j % HB) * R + R - 1;
            return sub >= 1 ? pos : pos - total();
        }
        // reads that may still be in flight when MFMA j of group g issues
        static constexpr int allow(int g, int j) {
            const int issued = before(g) + (j >= 1 ? reads(g) : 0);
            const int pa = pos_a(g), pb = pos_b(g / 4, j);
            const int n = issued - 1 - (pa > pb ? pa : pb);
            return n > 15 ? 15 : n;
        }
    };

    // LDS byte addresses (32-bit) of this lane's reads: [buffer][sub-step][half of the fragment];
    // the fragment index t is the instruction's immediate offset
    uint32_t aaddr[2][SPS][R], baddr[2][SPS][R];
#pragma unroll
    for (int buf = 0; buf < 2; buf++)
#pragma unroll
        for (int sub = 0; sub < SPS; sub++)
#pragma unroll
            for (int e = 0; e < R; e++) {
                const uint32_t so = FP8 ? (uint32_t)(((4 * sub + 2 * fh + e) ^ fsw) << 4)
                                        : (uint32_t)(((2 * sub + fh) ^ fsw) << 4);
                aaddr[buf][sub][e] = lds_addr0 + buf * STAGE_BYTES + (wm * 128 + frow) * BK + so;
                baddr[buf][sub][e] = lds_addr0 + buf * STAGE_BYTES + BM * BK + (wn * WN + frow) * BK + so;
            }

    i32x4 af[4][R], bf[2][TJ][R];
#define NQ_LDS_READ(dst, addr, imm) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm))
#define NQ_LDS_WAIT(n) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n))
    auto mma = [&](int i, int j, const i32x4(&a)[R], const i32x4(&b)[R]) {
        if constexpr (FP8) {
            const i32x8 av = {a[0][0], a[0][1], a[0][2], a[0][3], a[1][0], a[1][1], a[1][2], a[1][3]};
            const i32x8 bv = {b[0][0], b[0][1], b[0][2], b[0][3], b[1][0], b[1][1], b[1][2], b[1][3]};
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, acc[i][j], 0, 0, 0, 0, 0, 0);
        } else {
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[0], a[0], acc[i][j], 0, 0, 0);
        }
    };
    // the requests of group g of the stage in buffer BUF, in Sched's order (a request that would
    // belong to a stage past K reads stale LDS into registers nobody uses)
    auto requests = [&](auto gc, auto bufc) {
        constexpr int g = decltype(gc)::value, BUF = decltype(bufc)::value;
        auto& afr = af;  // (named outside the asm statements so that the lambda captures them)
        auto& bfr = bf;
        constexpr int sub = g / 4, i = g % 4;
        constexpr int g2 = (g + 2) % G;                       // the group whose x fragment is requested
        constexpr int abuf = (g + 2 >= G) ? BUF ^ 1 : BUF;    // ... in the next stage's buffer when it wraps
#pragma unroll
        for (int e = 0; e < R; e++) {
            const uint32_t addr = aaddr[abuf][g2 / 4][e];
            NQ_LDS_READ(afr[(g + 2) % 4][e], addr, (g2 % 4) * 32 * BK);
        }
        if constexpr (Sched::wfrags(g) > 0) {
            constexpr bool nb = sub == SPS - 1;  // the w fragments are the next stage's first sub-step
            constexpr int first = (nb ? i - 2 : i) * HB;
            constexpr int set = (sub + 1) & 1, bsub = nb ? 0 : sub + 1, bbuf = nb ? BUF ^ 1 : BUF;
#pragma unroll
            for (int f = 0; f < HB; f++)
#pragma unroll
                for (int e = 0; e < R; e++) {
                    const uint32_t addr = baddr[bbuf][bsub][e];
                    NQ_LDS_READ(bfr[set][first + f][e], addr, (first + f) * 32 * BK);
                }
        }
    };
    // transfers of the stage after next, issued from groups G-2 and G-1 in three slots each
    constexpr int ND = DA + DB, DPG = ND / 2;
    static_assert(ND == 16, "transfer slots below are written for 16 transfers per wavefront and stage");
#define NQ_DMA_SLOT(g, slot, buf, srca, srcb)                                                      \
    if constexpr ((g) >= G - 2) {                                                                  \
        if (have2) {                                                                               \
            constexpr int t0 = ((g) - (G - 2)) * DPG + (slot) * 3;                                 \
            NQ_DMA(t0, buf, srca, srcb);                                                           \
            NQ_DMA(t0 + 1, buf, srca, srcb);                                                       \
            if constexpr ((slot) < 2) NQ_DMA(t0 + 2, buf, srca, srcb);                             \
        }                                                                                          \
    }
#define NQ_GROUP(g, BUF)                                                                           \
    if constexpr ((g) < G) {                                                                       \
        constexpr int sub_ = (g) / 4, i_ = (g) % 4, set_ = sub_ & 1;                               \
        constexpr int w0_ = ((g) == G - 2) ? 0 : Sched::allow((g), 0);                             \
        if constexpr ((g) == G - 2) {                                                              \
            /* this wavefront's share of the next stage has landed and its reads of this stage */ \
            /* are done; past the barrier that holds for every wavefront */                        \
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                            \
            __builtin_amdgcn_s_barrier();                                                          \
        } else {                                                                                   \
            NQ_LDS_WAIT(w0_);                                                                      \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        mma(i_, 0, af[(g) % 4], bf[set_][0]);                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        requests(std::integral_constant<int, (g)>{}, std::integral_constant<int, BUF>{});          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        /* later MFMAs of the group wait again only where their w fragment is younger */           \
        constexpr int b1_ = w0_ + Sched::reads((g));                                               \
        constexpr int w1_ = Sched::allow((g), 1) < b1_ ? Sched::allow((g), 1) : b1_;               \
        if constexpr (w1_ < b1_) NQ_LDS_WAIT(w1_);                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        mma(i_, 1, af[(g) % 4], bf[set_][1]);                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        NQ_DMA_SLOT((g), 0, BUF, srca, srcb)                                                       \
        constexpr int w2_ = Sched::allow((g), 2) < w1_ ? Sched::allow((g), 2) : w1_;               \
        if constexpr (w2_ < w1_) NQ_LDS_WAIT(w2_);                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        mma(i_, 2, af[(g) % 4], bf[set_][2]);                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        NQ_DMA_SLOT((g), 1, BUF, srca, srcb)                                                       \
        constexpr int w3_ = Sched::allow((g), 3) < w2_ ? Sched::allow((g), 3) : w2_;               \
        if constexpr (w3_ < w2_) NQ_LDS_WAIT(w3_);                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        mma(i_, 3, af[(g) % 4], bf[set_][3]);                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        NQ_DMA_SLOT((g), 2, BUF, srca, srcb)                                                       \
    }
    // one stage, read from buffer BUF; its groups G-2 and G-1 refill BUF with stage st+2
#define NQ_STAGE(BUF)                                                                              \
    {                                                                                              \
        const bool have2 = st + 2 < KT;                                                            \
        const uint8_t* const srca = abase + (int64_t)(st + 2) * BK;                                \
        const uint8_t* const srcb = bbase + (int64_t)(st + 2) * BK;                                \
        NQ_GROUP(0, BUF) NQ_GROUP(1, BUF) NQ_GROUP(2, BUF) NQ_GROUP(3, BUF) NQ_GROUP(4, BUF)       \
        NQ_GROUP(5, BUF) NQ_GROUP(6, BUF) NQ_GROUP(7, BUF) NQ_GROUP(8, BUF) NQ_GROUP(9, BUF)       \
        NQ_GROUP(10, BUF) NQ_GROUP(11, BUF) NQ_GROUP(12, BUF) NQ_GROUP(13, BUF) NQ_GROUP(14, BUF)  \
        NQ_GROUP(15, BUF)                                                                          \
    }

    const int KT = p.K / BK;
    {
        // stage 0 now, stage 1 on its way during all of stage 0
        const bool have2 = true;
        (void)have2;
        const uint8_t* srca = abase;
        const uint8_t* srcb = bbase;
#define NQ_DMA_ALL(buf)                                                                            \
    NQ_DMA(0, buf, srca, srcb); NQ_DMA(1, buf, srca, srcb); NQ_DMA(2, buf, srca, srcb);            \
    NQ_DMA(3, buf, srca, srcb); NQ_DMA(4, buf, srca, srcb); NQ_DMA(5, buf, srca, srcb);            \
    NQ_DMA(6, buf, srca, srcb); NQ_DMA(7, buf, srca, srcb); NQ_DMA(8, buf, srca, srcb);            \
    NQ_DMA(9, buf, srca, srcb); NQ_DMA(10, buf, srca, srcb); NQ_DMA(11, buf, srca, srcb);          \
    NQ_DMA(12, buf, srca, srcb); NQ_DMA(13, buf, srca, srcb); NQ_DMA(14, buf, srca, srcb);         \
    NQ_DMA(15, buf, srca, srcb);
        NQ_DMA_ALL(0)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (KT > 1) {
            srca = abase + BK, srcb = bbase + BK;
            NQ_DMA_ALL(1)
        }
#undef NQ_DMA_ALL
    }
    const unsigned long long t_first = wall_clock64();  // stage 0 has landed
    // what groups G-2 and G-1 of a previous stage (in buffer 1) would have requested
    requests(std::integral_constant<int, G - 2>{}, std::integral_constant<int, 1>{});
    requests(std::integral_constant<int, G - 1>{}, std::integral_constant<int, 1>{});
    int st = 0;
    for (; st + 1 < KT; st++) {
        NQ_STAGE(0)
        st++;
        NQ_STAGE(1)
    }
    if (st < KT) NQ_STAGE(0)  // an odd number of stages: the last one, in buffer 0 again
    NQ_LDS_WAIT(0);  // requests past the last stage still target registers: let them land
    const unsigned long long t_loop = wall_clock64();
#undef NQ_STAGE
#undef NQ_GROUP
#undef NQ_DMA_SLOT
#undef NQ_DMA
#undef NQ_LDS_READ
#undef NQ_LDS_WAIT

    // ---- epilogue.  The MFMA was issued with the weight tile as its first operand, so in
    // acc[i][j] a lane holds ONE token m = 32 i + lane % 32 (MFMA column) and, for g = 0..3, the
    // four consecutive channels n = 32 j + 8 g + 4 (lane / 32) + 0..3 (MFMA rows, registers 4g..4g+3).
    // Per-token work is lane-local and four outputs of a row of y are adjacent.  Each wavefront
    // stages its results through its own LDS region (free now: the loop ended on a barrier) as
    // [token][channel] rows, and writes them out as 128-bit stores, 256 B (bf16) or 512 B (fp32 /
    // int32) contiguous per row of y.
    const int wm0 = m0 + wm * 128, wn0 = n0 + wn * WN;
    const int lm = lane & 31, lh = lane >> 5;
    // whole 16-byte stores wherever the tile's columns all exist and rows of y stay 16-byte aligned
    // (a tile that only M cuts short just skips the rows past M)
    const bool full_cols = (n0 + BN <= p.N) && (p.N % 8 == 0) && (((uintptr_t)p.y & 15) == 0);

    // channel scale and bias for the lane's channels of tile j, group g (needs n < N: clamped)
    auto chan = [&](int j, int g, float (&cs)[4], float (&cb)[4], bool need_scale, int zero) {
        if (p.chan_vec) {  // uniform: the lane's four channels are adjacent, one load per operand
            const int nb = min(wn0 + 32 * j + 8 * g + 4 * lh, p.N - 4) + zero;
            if (need_scale) {
                const float4 sv = *reinterpret_cast<const float4*>(p.col_scale + nb);
                cs[0] = sv.x, cs[1] = sv.y, cs[2] = sv.z, cs[3] = sv.w;
            } else {
                cs[0] = cs[1] = cs[2] = cs[3] = 1.0f;
            }
            cb[0] = cb[1] = cb[2] = cb[3] = 0.0f;
            if (p.bias) {
                if (p.bias_dtype == NQ_DT_F32) {
                    const float4 bv = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.bias) + nb);
                    cb[0] = bv.x, cb[1] = bv.y, cb[2] = bv.z, cb[3] = bv.w;
                } else {
                    const uint2 bv = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p.bias) + nb);
                    cb[0] = __uint_as_float(bv.x << 16), cb[1] = __uint_as_float(bv.x & 0xFFFF0000u);
                    cb[2] = __uint_as_float(bv.y << 16), cb[3] = __uint_as_float(bv.y & 0xFFFF0000u);
                }
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int n = min(wn0 + 32 * j + 8 * g + 4 * lh + r, p.N - 1) + zero;
            cs[r] = need_scale ? p.col_scale[n] : 1.0f;
            cb[r] = 0.0f;
            if (p.bias)
                cb[r] = (p.bias_dtype == NQ_DT_F32)
                            ? reinterpret_cast<const float*>(p.bias)[n]
                            : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n] << 16);
        }
    };

    auto emit = [&](auto kind, auto plain) {
        constexpr int KIND = decltype(kind)::value;  // 0: fp32, 1: bf16, 2: raw int32
        // MODE (uniform over the launch, so chosen once and not per channel tile: a branch around a load makes the
        // wavefront wait for that load where the branches meet).  0: one scale for the whole tensor and no bias (fp8 x
        // fp8): no channel operands at all; 1 .. 3: the lane's four channels adjacent and aligned, one load per
        // operand - no bias, fp32 bias, bf16 bias; 4: channel by channel
        constexpr int MODE = decltype(plain)::value;
        constexpr bool PLAIN = MODE == 0;
        constexpr int ES = (KIND == 1) ? 2 : 4;      // bytes per output element
        constexpr int IP = (KIND == 1) ? 2 : 1;      // token tiles (of 32) staged per pass
        constexpr int ROWB = WN * ES + 16;           // staged row: the wavefront's channels + pad (bank spread)
        uint8_t* stage = lds + wave * (32 * IP * ROWB);
#pragma unroll
        for (int ip = 0; ip < 4; ip += IP) {
            // ---- registers -> LDS (this wavefront's region only).  Channel scales and biases are
            // fetched per channel tile j; the compiler barrier keeps it from hoisting all 16 (j, g)
            // sets above the loop, which would spill.
            // (a zero the compiler cannot see through, new in every pass: the channel operands do not depend on
            // the pass, and kept across all four passes of the fp32 epilogue they cost 129 spilled registers and
            // 60 % of the call's time; they are re-read from L1 per pass instead)
            int zero = 0;
            asm volatile("" : "+v"(zero));
            float rscale[IP];
#pragma unroll
            for (int ii = 0; ii < IP; ii++) {
                rscale[ii] = 1.0f;
                if constexpr (!FP8 && KIND != 2) rscale[ii] = p.row_scale[min(wm0 + 32 * (ip + ii) + lm, p.M - 1)];
            }
            // modes 1 .. 3: the operands of channel tile j + 1 are requested before tile j is worked on
            auto fetch = [&](int j, float (&cs)[4][4], float (&cb)[4][4]) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int nb = min(wn0 + 32 * j + 8 * g + 4 * lh, p.N - 4) + zero;
                    if constexpr (!FP8) {
                        const float4 sv = *reinterpret_cast<const float4*>(p.col_scale + nb);
                        cs[g][0] = sv.x, cs[g][1] = sv.y, cs[g][2] = sv.z, cs[g][3] = sv.w;
                    } else {
                        cs[g][0] = cs[g][1] = cs[g][2] = cs[g][3] = 1.0f;
                    }
                    if constexpr (MODE == 2) {
                        const float4 bv = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.bias) + nb);
                        cb[g][0] = bv.x, cb[g][1] = bv.y, cb[g][2] = bv.z, cb[g][3] = bv.w;
                    } else if constexpr (MODE == 3) {
                        const uint2 bv = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p.bias) + nb);
                        cb[g][0] = __uint_as_float(bv.x << 16), cb[g][1] = __uint_as_float(bv.x & 0xFFFF0000u);
                        cb[g][2] = __uint_as_float(bv.y << 16), cb[g][3] = __uint_as_float(bv.y & 0xFFFF0000u);
                    } else {
                        cb[g][0] = cb[g][1] = cb[g][2] = cb[g][3] = 0.0f;
                    }
                }
            };
            // (not for int8 with fp32 output: its four passes of one token tile leave no registers for a second set)
            constexpr bool VEC = KIND != 2 && MODE >= 1 && MODE <= 3;
            constexpr bool AHEAD = VEC && !(KIND == 0 && !FP8);
            float ncs[4][4], ncb[4][4];
            if constexpr (AHEAD) fetch(0, ncs, ncb);
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                float cs[4][4], cb[4][4];
                if constexpr (AHEAD) {
#pragma unroll
                    for (int g = 0; g < 4; g++)
#pragma unroll
                        for (int r = 0; r < 4; r++) cs[g][r] = ncs[g][r], cb[g][r] = ncb[g][r];
                    if (j + 1 < TJ) fetch(j + 1, ncs, ncb);
                } else if constexpr (VEC) {
                    fetch(j, cs, cb);
                }
                if constexpr (KIND != 2 && MODE == 4) {
#pragma unroll
                    for (int g = 0; g < 4; g++) chan(j, g, cs[g], cb[g], !FP8, zero);
                }
                if constexpr (KIND == 2) {
#pragma unroll
                    for (int ii = 0; ii < IP; ii++) {
                        const int i = ip + ii;
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            uint8_t* dst = stage + (32 * ii + lm) * ROWB + (32 * j + 8 * g + 4 * lh) * ES;
                            *reinterpret_cast<i32x4*>(dst) = (i32x4){(int)acc[i][j][4 * g], (int)acc[i][j][4 * g + 1],
                                                                      (int)acc[i][j][4 * g + 2], (int)acc[i][j][4 * g + 3]};
                        }
                    }
                } else {
                    float z[IP][4][4];
#pragma unroll
                    for (int ii = 0; ii < IP; ii++)
#pragma unroll
                        for (int g = 0; g < 4; g++)
#pragma unroll
                            for (int r = 0; r < 4; r++) {
                                if constexpr (PLAIN)
                                    z[ii][g][r] = acc[ip + ii][j][4 * g + r] * fp8_scale + 0.0f;  // (+ 0.0f: the bits of the general path, -0.0 included)
                                else if constexpr (FP8)
                                    z[ii][g][r] = acc[ip + ii][j][4 * g + r] * fp8_scale + cb[g][r];
                                else
                                    z[ii][g][r] = (float)acc[ip + ii][j][4 * g + r] * (rscale[ii] * cs[g][r]) + cb[g][r];
                            }
                    if (p.epilogue == NQ_EPI_RELU) {
                        // a real (uniform) branch: one v_max per value when asked for, nothing otherwise
                        asm volatile("" ::: "memory");
#pragma unroll
                        for (int ii = 0; ii < IP; ii++)
#pragma unroll
                            for (int g = 0; g < 4; g++)
#pragma unroll
                                for (int r = 0; r < 4; r++) z[ii][g][r] = z[ii][g][r] > 0.0f ? z[ii][g][r] : 0.0f;
                    }
#pragma unroll
                    for (int ii = 0; ii < IP; ii++)
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            uint8_t* dst = stage + (32 * ii + lm) * ROWB + (32 * j + 8 * g + 4 * lh) * ES;
                            if constexpr (KIND == 0) {
                                *reinterpret_cast<float4*>(dst) =
                                    make_float4(z[ii][g][0], z[ii][g][1], z[ii][g][2], z[ii][g][3]);
                            } else {
                                // v_cvt_pk_bf16_f32: round to nearest even in hardware
                                const bf16x4 pk = __builtin_convertvector(
                                    (f32x4){z[ii][g][0], z[ii][g][1], z[ii][g][2], z[ii][g][3]}, bf16x4);
                                *reinterpret_cast<bf16x4*>(dst) = pk;
                            }
                        }
                }
                asm volatile("" ::: "memory");
            }
            // the region is this wavefront's own and DS operations of a wavefront execute in order:
            // no block barrier, only a fence against compiler reordering
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // ---- LDS -> global: 16 bytes per lane, rows of y contiguous
            constexpr int LPRW = WN * ES / 16;           // lanes per staged row (8, 16 or 32)
            constexpr int RPI = 64 / LPRW;               // rows per wavefront instruction
#pragma unroll
            for (int t = 0; t < 32 * IP / RPI; t++) {
                const int row = t * RPI + lane / LPRW, c16 = lane % LPRW;
                const i32x4 v = *reinterpret_cast<const i32x4*>(stage + row * ROWB + c16 * 16);
                const int m = wm0 + 32 * ip + row;
                const int n = wn0 + c16 * (16 / ES);
                if (full_cols) {
                    if (m < p.M)
                        *reinterpret_cast<i32x4*>(reinterpret_cast<uint8_t*>(p.y) + ((int64_t)m * p.N + n) * ES) = v;
                } else if (m < p.M) {
                    // ragged edge: element by element
#pragma unroll
                    for (int e = 0; e < 16 / ES; e++) {
                        if (n + e >= p.N) break;
                        if constexpr (ES == 2) {
                            const uint32_t wv = (uint32_t)v[e >> 1];
                            reinterpret_cast<uint16_t*>(p.y)[(int64_t)m * p.N + n + e] = (uint16_t)(wv >> (16 * (e & 1)));
                        } else {
                            reinterpret_cast<int32_t*>(p.y)[(int64_t)m * p.N + n + e] = v[e];
                        }
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    };
    using kind_t = std::integral_constant<int, KIND_>;
    if constexpr (KIND_ == 2) {
        emit(kind_t{}, std::integral_constant<int, 4>{});
    } else {
        if (FP8 && !p.bias) emit(kind_t{}, std::integral_constant<int, 0>{});
        else if (!p.chan_vec) emit(kind_t{}, std::integral_constant<int, 4>{});
        else if (!p.bias) emit(kind_t{}, std::integral_constant<int, 1>{});
        else if (p.bias_dtype == NQ_DT_F32) emit(kind_t{}, std::integral_constant<int, 2>{});
        else emit(kind_t{}, std::integral_constant<int, 3>{});
    }
    if (p.stamps) {  // (uniform) entry, first stage landed, loop done, stores acknowledged
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (tid == 0) {
            unsigned long long* o = p.stamps + 4 * (size_t)blockIdx.x;
            o[0] = t_entry, o[1] = t_first, o[2] = t_loop, o[3] = wall_clock64();
        }
    }
}

template <bool FP8, int KIND>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm8_kernel(const Gemm8Params p) {
    gemm8_body<FP8, KIND, 256, 128>(p);
}

template <typename K>
int32_t launch_cfg(K kernel, LdsAttrOnce* attr, const Gemm8Params& p, int bn, int bk, hipStream_t s) {
    const size_t lds = (size_t)2 * (BM + bn) * bk;
    NQ_HIP(set_max_lds_once(*attr, reinterpret_cast<const void*>(kernel), lds));
    hipLaunchKernelGGL(kernel, dim3(p.tiles_m * p.tiles_n), dim3(256), lds, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace

namespace {
unsigned long long* g_stamps = nullptr;  // set by the timeline diagnostic around one call, null otherwise
}

void gemm8_set_stamps(unsigned long long* buf) { g_stamps = buf; }

bool gemm8_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    const bool fp8 = (a.x_dtype == NQ_DT_FP8_E4M3 && L->format == NQ_FMT_FP8_E4M3);
    const bool i8 = (a.x_dtype == NQ_DT_I8 && L->format == NQ_FMT_W8_CHANNEL);
    // the kernel addresses a tile's rows with 32-bit offsets from the tile's base
    return (fp8 || i8) && (L->in % 128 == 0) && a.M >= 64 && (int64_t)L->in * 256 < ((int64_t)1 << 32);
}

int32_t launch_gemm8(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    Gemm8Params p{};
    p.a = reinterpret_cast<const uint8_t*>(a.x);
    p.b = L->d_codes;
    p.y = a.y, p.bias = a.bias;
    p.row_scale = a.x_scale;
    p.col_scale = reinterpret_cast<const float*>(L->d_scales);
    p.tscale = L->scale;
    p.M = a.M, p.N = L->out, p.K = L->in;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    p.tiles_m = (a.M + BM - 1) / BM, p.tiles_n = (L->out + 255) / 256;
    p.stamps = g_stamps;
    const bool i8 = a.x_dtype == NQ_DT_I8;
    p.chan_vec = L->out % 4 == 0 && L->out >= 4 && (!i8 || a.y_dtype == NQ_DT_I32 || (uintptr_t)p.col_scale % 16 == 0) &&
                 (!a.bias || (uintptr_t)a.bias % (a.bias_dtype == NQ_DT_F32 ? 16 : 8) == 0);
    static LdsAttrOnce attr_set[5];
    const bool f32 = a.y_dtype == NQ_DT_F32;
    if (a.x_dtype == NQ_DT_FP8_E4M3)
        return f32 ? launch_cfg(gemm8_kernel<true, 0>, &attr_set[0], p, 256, 128, a.stream)
                   : launch_cfg(gemm8_kernel<true, 1>, &attr_set[1], p, 256, 128, a.stream);
    if (a.y_dtype == NQ_DT_I32) return launch_cfg(gemm8_kernel<false, 2>, &attr_set[4], p, 256, 128, a.stream);
    return f32 ? launch_cfg(gemm8_kernel<false, 0>, &attr_set[2], p, 256, 128, a.stream)
               : launch_cfg(gemm8_kernel<false, 1>, &attr_set[3], p, 256, 128, a.stream);
}

}  // namespace nq
