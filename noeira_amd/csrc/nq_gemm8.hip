// Large-M GEMM over 8-bit operands on the CDNA4 matrix cores:
//     fp8 e4m3 x fp8 e4m3 -> fp32   (v_mfma_f32_16x16x128_f8f6f4)
//     int8     x int8     -> int32  (v_mfma_i32_16x16x64_i8)
//   y[M, N] = epi( (x[M, K] . w[N, K]^T) * scale + bias[N] )
// Both operands are K-contiguous, which is the layout the MFMA wants: a lane
// supplies 32 (int8: 16) consecutive bytes of one row.
//
// Which MFMA.  The call runs at the board's power limit, and on operands that toggle the
// multipliers the 16 x 16 shapes draw less than the 32 x 32 ones for the same arithmetic:
// back to back on register operands, all 256 CUs, e4m3 codes of N(0,1) values, the fp8
// 32x32x64 sustains 4.06 PFLOP/s at 2.00 GHz and the 16x16x128 4.43 at 2.19; uniform int8
// codes: 32x32x32 3.42 POP/s at 1.69 GHz, 16x16x64 4.07 at 2.05 (nq_diag_mfma_rate).  The
// same loop built on the 32 x 32 shapes took 107 us (fp8) and 127 us (int8) for
// 8192 x 4096 x 4096 where this one takes 102 and 114.
//
// Tiling.  (The fp8 form; int8 runs the same tile on 8 wavefronts, described below.)  One workgroup of 4 wavefronts
// (2 x 2) owns a 256 x 256 tile of y;
// each wavefront owns 128 x 128 of it as 8 x 8 MFMA tiles of 16 x 16, i.e. 256
// fp32/int32 accumulators per lane (the AGPR half of the unified register
// file), one workgroup per CU.  A tile this large is what keeps operand traffic
// down: a stage moves 64 KiB from L2 into a CU for 2048 cycles of MFMA work.
//
// K loop.  Stages of BK = 128 bytes: x tile 256 x 128 B and w tile 256 x 128 B
// (64 KiB), double-buffered in LDS (128 of the CU's 160 KiB), filled straight from
// global memory (global_load_lds_dwordx4, 16 per lane per stage): no registers, no
// ds_write.  The registers are a third buffer: a phase (the 64 MFMAs of one k-extent, one
// per stage for fp8, two for int8) multiplies fragments that are all in registers when it
// starts, and requests the next phase's into the registers it frees as it goes - the token
// fragment of row i one MFMA after the row's last, the channel fragments into a second set
// - so that no MFMA waits for an LDS read that was issued less than eleven MFMAs earlier.
// A stage has one barrier, at the start of its row 2: by then its own buffer has been read
// out completely (the requests were made during the stage before), so the barrier both
// proves the next stage landed and frees this stage's buffer for the stage after next.
// The waits before the MFMAs come from a compile-time model of the issue order
// (lds_wait): about ten s_waitcnt per phase.
//
// What the loop's parts cost, measured on this GPU (fp8 8192 x 4096 x 4096, the kernel's
// own clock stamps, parts switched off one at a time; microseconds per stage): whole
// 1.21; without the fragment reads 1.16; without the barrier 1.15; without the transfers
// 0.95 - 0.99; with none of the three 0.90 (MFMAs alone: 0.97 at the rate above).  The
// transfers are the expensive part and it is their bytes, not their timing: two per slot
// instead of one 3 - 4 % slower, all sixteen at once 10 %, spread over two barriers per
// stage no faster; nothing gained by dropping the wait for them (so they do land in
// time), by cache-policy bits (sc0, sc1: the same; nt: 25 % slower), or by another row
// stride (K = 3968 .. 4352: the same time per stage, so no L2 channel is camped on);
// transfers of 1 KiB contiguous from a few KiB per wavefront (L2 hits, one line run
// instead of eight lines) cost half as much.  Moving 64 KiB per stage and CU from L2 is
// 14 TB/s over the chip, and at the power limit that traffic is paid in clock.
//
// Eight wavefronts.  The same tile, stages, layout and epilogue with 8 wavefronts (4 x 2, each 64 x 128: 128
// accumulators per lane, two wavefronts per SIMD, 256 registers each, so one set of registers per fragment and each
// requested again one MFMA after its last reader; ev8_slot below).  Every accumulator still adds its stages in the same
// order: the two forms return the same bits.  int8: 8192 x 4096 x 4096 105 - 108 us against 110 - 112 on the same
// boxes, 8192^3 386 against 407 - 413, and a single round of tiles (M = 2048 over 4096 x 4096) 42 - 43 against 49.5: the
// two short phases per stage of the int8 MFMA leave a lone wavefront waiting more often than the fp8 form's one long
// phase, and a second wavefront on the SIMD fills those waits.  fp8: the same time either way (95.5 - 99 us; N = 11008
// and 8192^3 1 - 2 % slower), so fp8 stays on four.  Both forms take ~1.08 us per stage with half the CUs busy and no
// power limit in play: what is left over the MFMAs' 0.85 is not a lone wavefront's issue order.
//
// In cycles.  The K loop's own reading of the shader clock beside the constant one (fp8, 8192 x 4096 x 4096, all 256
// CUs busy): 2283 cycles per stage at 1.86 - 1.88 GHz, against the 2048 cycles the stage's MFMAs occupy the pipe and
// against 2.18 GHz under the same MFMAs with operands in registers; with half the CUs busy (M = 2048) 2320 cycles at
// 2.19 - 2.24 GHz; int8 on eight wavefronts 2317 cycles at 1.72 - 1.76 GHz (2.05 GHz under its MFMAs alone).  So nine
// tenths of the loop's cycles are MFMA cycles wherever it runs, and what a full chip loses beyond that is clock: the
// transfers and fragment reads are paid in power, not in stalls.
//
// Half tiles.  A launch that fills at most half a round of workgroups (128 tiles of 256 x 256) leaves CUs idle for the
// whole call, and so do the tiles left over after the last full round.  Both go on a 128 x 256 tile instead (4
// wavefronts, 2 x 2, each 64 x 128 with the eight-wavefront form's phase), twice as many workgroups: the call as a
// whole, or the leftover tiles in a second launch when they are whole columns of the last band of row tiles (N = 11008
// at M = 8192: 96 of 1376, 12 columns of 8).  A stage of that tile has half the MFMAs for three quarters of the
// transfers and is shorter than the transfers' way from L2, so it has three stage buffers (48 KiB each) and a stage's
// transfers two stages to land in; even so it is delivery that bounds it once most CUs draw on L2 (fp8, K = 4096: 24.7
// us with 128 workgroups, 26.9 with 192, 31.3 with 256 - against 41 - 43 us for the same calls on 64 .. 128 tiles of
// 256 x 256).  Same sums in the same order: same bits.
//
// Quarter tiles.  Calls whose 128 x 128 tiles fit about a round of workgroups (M = 512 .. 1152 over 4096 x 4096) run the
// body on that tile: 4 wavefronts of 64 x 64, a phase of 16 MFMAs (ev16_slot), four stage buffers of 32 KiB.  fp8 /
// int8 over 4096 x 4096: M = 512 15.8 / 18.0 us, M = 1024 18.1 - 20.2 / 20.2 - 22.3 (a plainer kernel on the same tile, with a
// stage's fragment reads at the head of the stage: 19.5 / 23.4 and 21.3 / 24.5; 256 x 256 tiles: 39 - 48).  Twice the
// bytes from L2 per operation: with all CUs on such tiles a stage is 0.39 - 0.45 us for 0.22 - 0.25 of MFMA, 18 - 21 TB/s
// into LDS over the chip.  launch_gemm8 takes the form of lowest estimated time (estimate_form).
// (int8 is 2 - 2.5 us behind fp8 on this tile.  Its two phases of 16 short MFMAs per stage request the next phase's
// fragments only six to nine MFMAs - about a hundred cycles - ahead; a form with two register sets, one per half of a
// stage, each fragment requested a whole stage ahead, measured the same: 18.3 / 21.3 us at M = 512 / 1024.  Not kept.)
//
// LDS layout.  Row-major [256][128 B] with the eight 16-byte slots of a row
// permuted by slot ^= ((row >> 1) + 6) & 7.  A 128-bit read is served in passes of
// sixteen lanes that are not consecutive lanes (per half of the wavefront the quads of lanes
// 0-3, 12-15, 20-23, 24-27, then 4-7, 8-11, 16-19, 28-31), a pass being conflict-free
// when its lanes touch sixteen different 16-byte slots modulo 256 bytes.  A fragment read
// has lane l on row l % 16 and slot 2 (l / 16) + e (int8: 4 u + l / 16): in each pass every
// row appears once, rows 0-3 and 12-15 with one slot and rows 4-11 with the slot two
// (int8: one) higher, so the permutation must send the row pairs {2,3,4,5} and {0,1,6,7}
// to two sets of slots that are each closed under xor 1 and xor 2: {0,1,2,3} and {4,5,6,7}.
// The bank-conflict counter reads the same for this kernel as for the one before it,
// whose K loop had none (what it counts is the epilogue's staging).
//
// Epilogue.  The MFMA takes the weight fragment as its first operand, so a lane
// ends up with one token and runs of four consecutive channels; results are
// staged per wavefront through LDS and leave as 128-bit stores covering whole
// 256/512-byte row segments of y.  A CU takes such stores (4 rows x 256 B per
// instruction) at 40 - 49 B per cycle when few CUs write, and the chip takes the 32 MiB of
// a round of tiles in 3.1 - 3.5 us at best; 32 rows x 32 B per instruction - what leaves
// the registers without the trip through LDS - is 2.7 times slower per CU.  Built,
// measured against this kernel in the same sessions and not kept: persistent workgroups
// with the K stages streaming across tile boundaries and stores straight from the
// registers (no first-stage wait, but the slower store shape: equal); a finished tile held
// in registers as packed bf16 and stored one piece per stage under the next tile's K loop
// (the moves that rotate the pieces cost the loop what the epilogue saved); workgroups
// started 0 .. 5 us apart so that epilogues do not coincide (equal); one workgroup per CU walking its tiles with the
// LDS-staged stores kept - the next tile's first stage requested into the first buffer under the epilogue, which stages
// in the second (in twice the passes), the second stage requested after it: 2 % slower for fp8, 8 % for int8 (whose
// epilogue's own loads of scales and bias then queue behind the requested stage), on one box in turn.  At the power
// limit, time that one part stops taking is handed back as clock to the others only
// when energy is saved with it.
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
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;


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
    int32_t grid;            // workgroups to launch: the first `grid` tiles of the order (0: all tiles_m x tiles_n)
    int32_t m_base, n_base;  // the first row and channel of the part of y this launch covers (its tiles count from there)
    int32_t y_dtype, bias_dtype, epilogue;
    unsigned long long* stamps;  // a diagnostic: per workgroup, four readings of the constant 100 MHz clock and two of the shader clock, or null
    int32_t chan_vec;  // N % 4 == 0 and col_scale / bias aligned for one 16-byte (bf16 bias: 8-byte) load per 4 channels
};

__device__ __forceinline__ uint16_t f32_to_bf16(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(static_cast<F&&>(f));
    }
}

// ---- the issue order of one phase (64 MFMAs of one k-extent: row i = 0..7 of token fragments, column j = 0..7 of
// channel fragments, MFMA m = 8 i + j), as the waits' model.  Slot m = right after MFMA m.  A phase requests what
// the NEXT phase multiplies: the token fragment x_i into the registers row i has just finished with (one MFMA
// later, so that no request follows the last reader directly), the channel fragments into the second set; x_7
// is read at the start of the phase that uses it.  Nothing is requested in rows 0 and 1: where the next phase lies
// in the other stage buffer, the stage's barrier stands at the start of row 2, and the requests a barrier-free
// phase could have made earlier are kept where they are, so that every phase has one order.
//   event e:   0     1    2    3    4    5    6    7    8    9    10   11   12   13   14   15
//   brings:    x7'   x0   x1   w0   w1   w2   x2   w3   x3   w4   x4   w5   x5   w6   x6   w7   (x7': this phase's own)
__host__ __device__ constexpr int ev_slot(int e) {
    constexpr int s[16] = {0, 16, 17, 18, 19, 20, 24, 27, 32, 35, 40, 43, 48, 51, 56, 59};
    return s[e];
}
__host__ __device__ constexpr int ev_of_x(int i) {  // i <= 6: the event of the previous phase that brought x_i
    constexpr int e[7] = {1, 2, 6, 8, 10, 12, 14};
    return e[i];
}
__host__ __device__ constexpr int ev_of_w(int j) {
    constexpr int e[8] = {3, 4, 5, 7, 9, 11, 13, 15};
    return e[j];
}
// the event (or -1) in slot m
__host__ __device__ constexpr int ev_at(int m) {
    for (int e = 0; e < 16; e++)
        if (ev_slot(e) == m) return e;
    return -1;
}
// The wait in front of MFMA m = 8 i + j, as the number of reads (fragments x reads per fragment) that may still be
// under way, or -1 where what the MFMA needs has landed by an earlier wait of the phase.  Events are numbered
// 0 .. 15 (the phase before) and 16 .. 31 (this phase); LDS returns in the order of issue, so a wait that leaves
// `a` events in flight proves every older one landed.  A phase starts knowing nothing (conservative: a stage's
// barrier waits for everything, but not every phase follows one).  lgkmcnt counts to 15.
__host__ __device__ constexpr int lds_wait(int m_want, int reads_per_fragment, bool barrier_at_16) {
    int landed = 0;  // events 0 .. landed - 1 are known to have landed
    for (int m = 0; m < 64; m++) {
        const int i = m / 8, j = m % 8;
        int issued = 16;
        for (int e = 0; e < 16; e++)
            if (ev_slot(e) < m) issued++;
        const int nx = (i == 7) ? 16 : ev_of_x(i), nw = ev_of_w(j);
        const int need = nx > nw ? nx : nw;
        int w = -1;
        if (barrier_at_16 && m == 16) {
            landed = issued;  // (the barrier's own wait is lgkmcnt(0))
        } else if (need >= landed) {
            int a = issued - 1 - need;                       // events younger than the needed one
            const int cap = 15 / reads_per_fragment;
            if (a > cap) a = cap;
            w = a * reads_per_fragment;
            landed = issued - a;
        }
        if (m == m_want) return w;
    }
    return -1;
}
// A stage's 16 transfers per wavefront leave one at a time in these slots of the stage's last phase (after the barrier,
// in slots that hold no request): slot m -> transfer, or -1.  The CU's address unit takes about 22 cycles per transfer and
// a wavefront that finds it busy stands still with its MFMAs behind it: pairs of transfers per slot measured 3 - 4 %
// slower, all sixteen at once 10 %; spreading them further (over two barriers per stage) brought nothing more.
__host__ __device__ constexpr int dma_at(int m) {
    constexpr int s[16] = {21, 22, 23, 25, 26, 28, 29, 30, 33, 34, 36, 37, 38, 41, 42, 44};
    for (int t = 0; t < 16; t++)
        if (s[t] == m) return t;
    return -1;
}

// ---- the same for the form with eight wavefronts (4 x 2, each 64 x 128 of the tile: 4 token fragments, 8 channel
// fragments, 32 MFMAs per phase, two wavefronts per SIMD so that one's waits stand under the other's MFMAs).  With 128
// accumulators a wavefront has 256 registers in all, so every fragment has ONE set of registers and is requested again
// one MFMA after its last reader.  Order: m -> token fragment i = (m % 16) / 4, channel fragment j = 4 (m / 16) + m % 4:
// channel fragments 0 .. 3 are done with after MFMAs 12 .. 15, token fragment i after 19 + 4 i, channel fragments
// 4 .. 7 after 28 .. 31.  The last two requests of a phase's fragments (w7, x3) fall into the phase itself, slots 0, 1.
//   event e:   0     1     2    3    4    5    6    7    8    9    10   11
//   brings:    w7'   x3'   w0   w1   w2   w3   x0   x1   x2   w4   w5   w6     (': this phase's own)
__host__ __device__ constexpr int ev8_slot(int e) {
    constexpr int s[12] = {0, 1, 13, 14, 15, 16, 20, 24, 28, 29, 30, 31};
    return s[e];
}
__host__ __device__ constexpr int ev8_at(int m) {
    for (int e = 0; e < 12; e++)
        if (ev8_slot(e) == m) return e;
    return -1;
}
// events 0 .. 11: the phase before, 12 .. 23: this phase; barrier_at: the MFMA in front of which the stage's barrier
// (with its lgkmcnt(0)) stands, or -1
__host__ __device__ constexpr int lds_wait8(int m_want, int reads_per_fragment, int barrier_at) {
    int landed = 0;
    for (int m = 0; m < 32; m++) {
        const int i = (m % 16) / 4, j = 4 * (m / 16) + m % 4;
        int issued = 12;
        for (int e = 0; e < 12; e++)
            if (ev8_slot(e) < m) issued++;
        const int nx = i < 3 ? 6 + i : 12 + 1;
        const int nw = j < 4 ? 2 + j : (j < 7 ? 9 + (j - 4) : 12 + 0);
        const int need = nx > nw ? nx : nw;
        int w = -1;
        if (m == barrier_at) {
            landed = issued;
        } else if (need >= landed) {
            int a = issued - 1 - need;
            const int cap = 15 / reads_per_fragment;
            if (a > cap) a = cap;
            w = a * reads_per_fragment;
            landed = issued - a;
        }
        if (m == m_want) return w;
    }
    return -1;
}
// (the barrier in front of MFMA 2, 4, 8 or 12, the transfers in consecutive slots or every other one: the same time)
constexpr int BARRIER8_AT = 8;
// the eight transfers per wavefront and stage: after the barrier, in slots without a request, every other one
// (twelve for the 128 x 256 tile on four wavefronts)
__host__ __device__ constexpr int dma8_at(int m, int n) {
    constexpr int s8[8] = {8, 10, 12, 17, 19, 21, 23, 25};
    constexpr int s12[12] = {8, 9, 10, 11, 12, 17, 18, 19, 21, 22, 23, 25};
    for (int t = 0; t < n; t++)
        if ((n == 8 ? s8[t] : s12[t]) == m) return t;
    return -1;
}

// ---- and for a 128 x 128 tile on four wavefronts (2 x 2, each 64 x 64: 4 token and 4 channel fragments, 16 MFMAs per
// phase), again one register set per fragment.  Order: m -> token fragment i = (m % 8) / 2, channel fragment
// j = 2 (m / 8) + m % 2: channel fragments 0, 1 are done with after MFMAs 6, 7, token fragment i after 9 + 2 i, channel
// fragments 2, 3 after 14, 15.  Each is requested again one MFMA after its last reader; x3 and w3 fall into the phase
// that uses them (slots 0, 1).
//   event e:   0     1     2    3    4    5    6    7
//   brings:    x3'   w3'   w0   w1   x0   x1   x2   w2     (': this phase's own)
__host__ __device__ constexpr int ev16_slot(int e) {
    constexpr int s[8] = {0, 1, 7, 8, 10, 12, 14, 15};
    return s[e];
}
__host__ __device__ constexpr int ev16_at(int m) {
    for (int e = 0; e < 8; e++)
        if (ev16_slot(e) == m) return e;
    return -1;
}
__host__ __device__ constexpr int lds_wait16(int m_want, int reads_per_fragment, int barrier_at) {
    int landed = 0;
    for (int m = 0; m < 16; m++) {
        const int i = (m % 8) / 2, j = 2 * (m / 8) + m % 2;
        int issued = 8;
        for (int e = 0; e < 8; e++)
            if (ev16_slot(e) < m) issued++;
        const int nx = i < 3 ? 4 + i : 8 + 0;
        const int nw = j < 2 ? 2 + j : (j == 2 ? 7 : 8 + 1);
        const int need = nx > nw ? nx : nw;
        int w = -1;
        if (m == barrier_at) {
            landed = issued;
        } else if (need >= landed) {
            int a = issued - 1 - need;
            const int cap = 15 / reads_per_fragment;
            if (a > cap) a = cap;
            w = a * reads_per_fragment;
            landed = issued - a;
        }
        if (m == m_want) return w;
    }
    return -1;
}
constexpr int BARRIER16_AT = 4;
// eight transfers per wavefront and stage behind the barrier: two each after MFMAs 4 and 5, then one per slot that holds
// no request (barrier in front of MFMA 2 or 6, or all eight transfers right behind it: the same time or slower)
__host__ __device__ constexpr int dma16_first(int m) { return m == 4 ? 0 : m == 5 ? 2 : m == 6 ? 4 : m == 9 ? 5 : m == 11 ? 6 : m == 13 ? 7 : -1; }
__host__ __device__ constexpr int dma16_count(int m) { return (m == 4 || m == 5) ? 2 : (m == 6 || m == 9 || m == 11 || m == 13) ? 1 : 0; }

// BN and BK are parameters of the body for the arithmetic's sake; the tile built is 256 x 256 with BK = 128.
// KIND: the output type the epilogue is built for (0 fp32, 1 bf16, 2 raw int32 accumulators); one
// kernel per kind, because with all three in one function the register allocator spills.
template <bool FP8, int KIND_, int BM, int BN, int BK, int WAVES>
__device__ __forceinline__ void gemm8_body(const Gemm8Params& p) {
    constexpr int STAGE_BYTES = (BM + BN) * BK;
    constexpr int SLOTS = BK / 16;     // 16-byte slots per LDS row
    constexpr int WN = BN / 2;         // channels per wavefront
    constexpr int TI = BM / (8 * WAVES), TJ = WN / 16;  // fragments of 16 rows: token rows i, channel columns j
    static_assert(BK == 128 && ((BN == 256 && TJ == 8 && ((BM == 256 && (WAVES == 4 || WAVES == 8)) || (BM == 128 && WAVES == 4))) ||
                                (BN == 128 && BM == 128 && WAVES == 4 && TI == 4 && TJ == 4)),
                  "the phase models are written for these tiles");
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
    const int m0 = p.m_base + tm * BM, n0 = p.n_base + tn * BN;

    // the slot permutation of an LDS row (see the header): rows 16 f + r of any fragment f share it
    auto swz = [](int row) { return (((row >> 1) & 7) + 6) & 7; };

    // ---- global -> LDS, direct (global_load_lds_dwordx4): no register round trip.  One
    // instruction fills 1 KiB of LDS, lane l at byte 16 l, i.e. 1024 / BK rows; wavefront w owns
    // a quarter of the rows of both tiles.  The slot permutation is applied on the global side: the
    // lane that lands in physical slot s of its row fetches logical slot s ^ swz(row).
    typedef __attribute__((address_space(3))) void lptr_t;
    constexpr int DROWS = 1024 / BK;           // rows per instruction
    constexpr int DA = BM / WAVES / DROWS;         // instructions per wavefront and stage, x tile
    constexpr int DB = BN / WAVES / DROWS;         // ... w tile
    static_assert(DA + DB == 16 || DA + DB == 8 || DA + DB == 12, "dma_at() / dma8_at() place every transfer of a wavefront and stage");
    // addresses as a uniform 64-bit tile base (advanced by k0) plus a 32-bit per-lane offset, and
    // the LDS destination as a scalar: two instructions per transfer (set M0, issue)
    const uint8_t* const abase = p.a + (int64_t)m0 * p.K;
    const uint8_t* const bbase = p.b + (int64_t)n0 * p.K;
    uint32_t doff[DA + DB];
#pragma unroll
    for (int t = 0; t < DA; t++) {
        const int row = wave * (BM / WAVES) + t * DROWS + lane / SLOTS;
        const int slot = (lane % SLOTS) ^ swz(row);
        doff[t] = (uint32_t)(min(m0 + row, p.M - 1) - m0) * (uint32_t)p.K + slot * 16;
    }
#pragma unroll
    for (int t = 0; t < DB; t++) {
        const int row = wave * (BN / WAVES) + t * DROWS + lane / SLOTS;
        const int slot = (lane % SLOTS) ^ swz(row);
        doff[DA + t] = (uint32_t)(min(n0 + row, p.N - 1) - n0) * (uint32_t)p.K + slot * 16;
    }
    // transfer t (0 .. DA+DB-1) of a stage: M0 = the LDS address of the 1 KiB the instruction
    // fills (a scalar base of the buffer half plus t KiB), global address = scalar base + lane
    // offset.  Three instructions per transfer.  (M0 is a reserved register the compiler sets itself
    // right before each of its own uses, so writing it here needs no clobber; SCC does.)
    const uint32_t lds_addr0 = (uint32_t)(uintptr_t)(lptr_t*)lds;
    // stage buffers: two of 64 KiB; the 128-row tiles have three of 48 KiB (128 x 256) or four of 32 KiB (128 x 128), so
    // that a stage's transfers have two or three stages of MFMAs to land in (one stage of 32 or 16 MFMAs per wavefront
    // is shorter than their way from L2)
    constexpr int NB = BM == 128 ? (BN == 128 ? 4 : 3) : 2;
    uint32_t dbase[NB][2];  // [buffer][x tile, w tile]: this wavefront's first destination
#pragma unroll
    for (int buf = 0; buf < NB; buf++) {
        dbase[buf][0] = lds_addr0 + buf * STAGE_BYTES + wave * (BM / WAVES) * BK;
        dbase[buf][1] = lds_addr0 + buf * STAGE_BYTES + BM * BK + wave * (BN / WAVES) * BK;
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

    typedef typename std::conditional<FP8, f32x4, i32x4>::type acc_t;
    acc_t acc[TI][TJ];

    // ---- fragments.  fp8 (v_mfma_f32_16x16x128_f8f6f4): the whole 128-byte k-extent of a stage is ONE phase; lane
    // l supplies bytes [32 c, 32 c + 32) of row l % 16, c = l / 16: slots 2 c and 2 c + 1, two 128-bit reads.  int8
    // (v_mfma_i32_16x16x64_i8): two phases of 64 bytes per stage, bytes [16 c, 16 c + 16) of the phase's half: slot
    // 4 u + c, one read.  A fragment is 16 rows x 128 B = 2 KiB of a tile: the immediate offset of the read.
    constexpr int PH = FP8 ? 1 : 2;          // phases per stage
    constexpr int R = FP8 ? 2 : 1;           // 128-bit reads per fragment
    const int frow = lane & 15, fc = lane >> 4;
    const int fsw = swz(frow);
    // LDS byte addresses of this lane's reads: [buffer][u], u = half of the fragment (fp8) or phase of the stage (int8)
    uint32_t aaddr[NB][2], baddr[NB][2];
#pragma unroll
    for (int buf = 0; buf < NB; buf++)
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const uint32_t so = (uint32_t)(((FP8 ? 2 * fc + u : 4 * u + fc) ^ fsw) << 4);
            aaddr[buf][u] = lds_addr0 + buf * STAGE_BYTES + (wm * (16 * TI) + frow) * BK + so;
            baddr[buf][u] = lds_addr0 + buf * STAGE_BYTES + BM * BK + (wn * WN + frow) * BK + so;
        }
    i32x4 xf[TI][R], wf[WAVES == 4 ? 2 : 1][TJ][R];
#define NQ_LDS_READ(dst, addr, imm) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm))
#define NQ_LDS_WAIT(n) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n))
    // zc: the accumulator's first MFMA of the tile (C = 0)
    auto mma = [&](auto zc, int i, int j, const i32x4(&a)[R], const i32x4(&b)[R]) {
        constexpr bool ZERO = decltype(zc)::value;
        if constexpr (FP8) {
            const i32x8 av = {a[0][0], a[0][1], a[0][2], a[0][3], a[1][0], a[1][1], a[1][2], a[1][3]};
            const i32x8 bv = {b[0][0], b[0][1], b[0][2], b[0][3], b[1][0], b[1][1], b[1][2], b[1][3]};
            if constexpr (ZERO)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, acc_t{}, 0, 0, 0, 0, 0, 0);
            else
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, acc[i][j], 0, 0, 0, 0, 0, 0);
        } else {
            // (inline assembly with the accumulator tied to itself: for this four-pass MFMA the compiler keeps result
            // and addend apart, and with all 256 accumulator registers live that turns into a rotation through the
            // vector registers, two copies per MFMA.  Consecutive MFMAs never share an accumulator, and the
            // operands come from LDS reads whose wait stands in front, so no hazard is hidden from the compiler.)
            auto& c = acc;
            if constexpr (ZERO)
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, 0" : "=a"(c[i][j]) : "v"(b[0]), "v"(a[0]));
            else
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c[i][j]) : "v"(b[0]), "v"(a[0]));
        }
    };
    // token fragment i / channel fragment j of (buffer, phase) into the given registers
    auto read_x = [&](auto ic, auto bufc, auto phc) {
        constexpr int i = decltype(ic)::value, BUF = decltype(bufc)::value, PHI = decltype(phc)::value;
        auto& x = xf;  // (named outside the asm statements so that the lambda captures them)
#pragma unroll
        for (int e = 0; e < R; e++) {
            const uint32_t addr = aaddr[BUF][FP8 ? e : PHI];
            NQ_LDS_READ(x[i][e], addr, i * 16 * BK);
        }
    };
    auto read_w = [&](auto setc, auto jc, auto bufc, auto phc) {
        constexpr int SET = decltype(setc)::value, j = decltype(jc)::value, BUF = decltype(bufc)::value, PHI = decltype(phc)::value;
        auto& w = wf;
#pragma unroll
        for (int e = 0; e < R; e++) {
            const uint32_t addr = baddr[BUF][FP8 ? e : PHI];
            NQ_LDS_READ(w[SET][j][e], addr, j * 16 * BK);
        }
    };
    using std::integral_constant;
    // One phase: the 64 MFMAs of (buffer BUF, phase PHI of its stage) with the requests for the next phase, and in a
    // stage's last phase its barrier (start of row 2: this wavefront's share of the next stage has landed, its reads
    // of this stage are done) followed by the transfers of the stage after next into the buffer just freed.
    // ZERO: the tile's first phase (accumulators start from a literal zero).
    auto phase = [&](auto bufc, auto phc, auto zeroc, bool have2, const uint8_t* srca, const uint8_t* srcb) {
        constexpr int BUF = decltype(bufc)::value, PHI = decltype(phc)::value;
        constexpr bool LAST = PHI == PH - 1;
        constexpr int NBUF = LAST ? BUF ^ 1 : BUF, NPH = LAST ? 0 : PHI + 1;
        constexpr int WS = FP8 ? BUF : PHI;  // the set of channel fragments this phase multiplies
        static_for<64>([&](auto mc) {
            constexpr int m = decltype(mc)::value, i = m / 8, j = m % 8;
            if constexpr (LAST && m == 16) {
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
            } else {
                constexpr int al = lds_wait(m, R, LAST);
                if constexpr (al >= 0) NQ_LDS_WAIT(al);
            }
            __builtin_amdgcn_sched_barrier(0);
            mma(zeroc, i, j, xf[i], wf[WS][j]);
            __builtin_amdgcn_sched_barrier(0);
            constexpr int e = ev_at(m);
            if constexpr (e == 0) {
                read_x(integral_constant<int, 7>{}, bufc, phc);
            } else if constexpr (e > 0) {
                constexpr bool isx = e == 1 || e == 2 || e == 6 || e == 8 || e == 10 || e == 12 || e == 14;
                if constexpr (isx) {
                    constexpr int xi = e == 1 ? 0 : e == 2 ? 1 : e == 6 ? 2 : e == 8 ? 3 : e == 10 ? 4 : e == 12 ? 5 : 6;
                    read_x(integral_constant<int, xi>{}, integral_constant<int, NBUF>{}, integral_constant<int, NPH>{});
                } else {
                    constexpr int wj = e == 3 ? 0 : e == 4 ? 1 : e == 5 ? 2 : e == 7 ? 3 : e == 9 ? 4 : e == 11 ? 5 : e == 13 ? 6 : 7;
                    read_w(integral_constant<int, WS ^ 1>{}, integral_constant<int, wj>{}, integral_constant<int, NBUF>{},
                           integral_constant<int, NPH>{});
                }
            }
            if constexpr (LAST && dma_at(m) >= 0) {
                // (one branch per transfer; the requests above stand in straight code, so that no register with a read
                // under way meets a copy where branches join)
                if (have2) {
                    constexpr int t = dma_at(m);
                    NQ_DMA(t, BUF, srca, srcb);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // A stage's barrier with more than two buffers: the transfers of the `keep` stages after the next one may stay in
    // flight across it (loads return in the order of issue)
    auto barrier_keep = [&](int keep) {
        if (keep >= 2)
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * (DA + DB)) : "memory");
        else if (keep == 1)
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(DA + DB) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    };
    // The same for eight wavefronts: 32 MFMAs, one set of registers per fragment (see ev8_slot).
    auto phase8 = [&](auto bufc, auto phc, auto zeroc, bool have2, int keep, const uint8_t* srca, const uint8_t* srcb) {
        constexpr int BUF = decltype(bufc)::value, PHI = decltype(phc)::value;
        constexpr bool LAST = PHI == PH - 1;
        constexpr int NBUF = LAST ? (BUF + 1) % NB : BUF, NPH = LAST ? 0 : PHI + 1;
        static_for<32>([&](auto mc) {
            constexpr int m = decltype(mc)::value, i = (m % 16) / 4, j = 4 * (m / 16) + m % 4;
            if constexpr (LAST && m == BARRIER8_AT) {
                barrier_keep(keep);
            } else {
                constexpr int al = lds_wait8(m, R, LAST ? BARRIER8_AT : -1);
                if constexpr (al >= 0) NQ_LDS_WAIT(al);
            }
            __builtin_amdgcn_sched_barrier(0);
            mma(zeroc, i, j, xf[i], wf[0][j]);
            __builtin_amdgcn_sched_barrier(0);
            constexpr int e = ev8_at(m);
            using z0 = integral_constant<int, 0>;
            if constexpr (e == 0) {
                read_w(z0{}, integral_constant<int, 7>{}, bufc, phc);
            } else if constexpr (e == 1) {
                read_x(integral_constant<int, 3>{}, bufc, phc);
            } else if constexpr (e >= 2 && e <= 5) {
                read_w(z0{}, integral_constant<int, e - 2>{}, integral_constant<int, NBUF>{}, integral_constant<int, NPH>{});
            } else if constexpr (e >= 6 && e <= 8) {
                read_x(integral_constant<int, e - 6>{}, integral_constant<int, NBUF>{}, integral_constant<int, NPH>{});
            } else if constexpr (e >= 9) {
                read_w(z0{}, integral_constant<int, e - 5>{}, integral_constant<int, NBUF>{}, integral_constant<int, NPH>{});
            }
            if constexpr (LAST && dma8_at(m, DA + DB) >= 0) {
                if (have2) {
                    constexpr int t = dma8_at(m, DA + DB);
                    NQ_DMA(t, BUF, srca, srcb);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // And for the 128 x 128 tile: 16 MFMAs (see ev16_slot).
    auto phase16 = [&](auto bufc, auto phc, auto zeroc, bool have2, int keep, const uint8_t* srca, const uint8_t* srcb) {
        constexpr int BUF = decltype(bufc)::value, PHI = decltype(phc)::value;
        constexpr bool LAST = PHI == PH - 1;
        constexpr int NBUF = LAST ? (BUF + 1) % NB : BUF, NPH = LAST ? 0 : PHI + 1;
        static_for<16>([&](auto mc) {
            constexpr int m = decltype(mc)::value, i = (m % 8) / 2, j = 2 * (m / 8) + m % 2;
            if constexpr (LAST && m == BARRIER16_AT) {
                barrier_keep(keep);
            } else {
                constexpr int al = lds_wait16(m, R, LAST ? BARRIER16_AT : -1);
                if constexpr (al >= 0) NQ_LDS_WAIT(al);
            }
            __builtin_amdgcn_sched_barrier(0);
            mma(zeroc, i, j, xf[i], wf[0][j]);
            __builtin_amdgcn_sched_barrier(0);
            constexpr int e = ev16_at(m);
            using z0 = integral_constant<int, 0>;
            using nb = integral_constant<int, NBUF>;
            using np = integral_constant<int, NPH>;
            if constexpr (e == 0) {
                read_x(integral_constant<int, 3>{}, bufc, phc);
            } else if constexpr (e == 1) {
                read_w(z0{}, integral_constant<int, 3>{}, bufc, phc);
            } else if constexpr (e == 2 || e == 3) {
                read_w(z0{}, integral_constant<int, e - 2>{}, nb{}, np{});
            } else if constexpr (e >= 4 && e <= 6) {
                read_x(integral_constant<int, e - 4>{}, nb{}, np{});
            } else if constexpr (e == 7) {
                read_w(z0{}, integral_constant<int, 2>{}, nb{}, np{});
            }
            if constexpr (LAST && dma16_count(m) > 0) {
                if (have2) {
                    constexpr int t = dma16_first(m);
                    NQ_DMA(t, BUF, srca, srcb);
                    if constexpr (dma16_count(m) == 2) NQ_DMA(t + 1, BUF, srca, srcb);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // one stage, read from buffer BUF; its last phase refills BUF with stage st + NB
    auto stage = [&](auto bufc, auto zeroc, int st, int KT) {
        const bool have2 = st + NB < KT;
        const int keep = max(0, min(NB - 2, KT - st - 2));
        const uint8_t* const srca = abase + (int64_t)(st + NB) * BK;
        const uint8_t* const srcb = bbase + (int64_t)(st + NB) * BK;
        if constexpr (TJ == 4) {
            phase16(bufc, integral_constant<int, 0>{}, zeroc, have2, keep, srca, srcb);
            if constexpr (PH == 2) phase16(bufc, integral_constant<int, 1>{}, std::false_type{}, have2, keep, srca, srcb);
        } else if constexpr (TI == 4) {
            phase8(bufc, integral_constant<int, 0>{}, zeroc, have2, keep, srca, srcb);
            if constexpr (PH == 2) phase8(bufc, integral_constant<int, 1>{}, std::false_type{}, have2, keep, srca, srcb);
        } else {
            phase(bufc, integral_constant<int, 0>{}, zeroc, have2, srca, srcb);
            if constexpr (PH == 2) phase(bufc, integral_constant<int, 1>{}, std::false_type{}, have2, srca, srcb);
        }
    };

    const int KT = p.K / BK;
    {
        // stage 0 now, stage 1 on its way during all of stage 0
        const uint8_t* srca = abase;
        const uint8_t* srcb = bbase;
#define NQ_DMA_ALL(buf)                                                                            \
    NQ_DMA(0, buf, srca, srcb); NQ_DMA(1, buf, srca, srcb); NQ_DMA(2, buf, srca, srcb);            \
    NQ_DMA(3, buf, srca, srcb); NQ_DMA(4, buf, srca, srcb); NQ_DMA(5, buf, srca, srcb);            \
    NQ_DMA(6, buf, srca, srcb); NQ_DMA(7, buf, srca, srcb);                                        \
    if constexpr (DA + DB >= 12) {                                                                 \
        NQ_DMA(8, buf, srca, srcb); NQ_DMA(9, buf, srca, srcb); NQ_DMA(10, buf, srca, srcb);       \
        NQ_DMA(11, buf, srca, srcb);                                                               \
    }                                                                                              \
    if constexpr (DA + DB == 16) {                                                                 \
        NQ_DMA(12, buf, srca, srcb); NQ_DMA(13, buf, srca, srcb);                                  \
        NQ_DMA(14, buf, srca, srcb); NQ_DMA(15, buf, srca, srcb);                                  \
    }
        NQ_DMA_ALL(0)
        if constexpr (NB >= 3) {
            // all buffers at once; stage 0 has landed when at most the other stages' transfers are out
            if (KT > 1) {
                srca = abase + BK, srcb = bbase + BK;
                NQ_DMA_ALL(1)
            }
            if (KT > 2) {
                srca = abase + 2 * BK, srcb = bbase + 2 * BK;
                NQ_DMA_ALL(2)
            }
            if constexpr (NB == 4) {
                if (KT > 3) {
                    srca = abase + 3 * BK, srcb = bbase + 3 * BK;
                    NQ_DMA_ALL(3)
                }
            }
            const int out = min(KT, NB) - 1;  // stages that may still be on their way
            if (out >= 3)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * (DA + DB)) : "memory");
            else if (out == 2)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (DA + DB)) : "memory");
            else if (out == 1)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DA + DB) : "memory");
            else
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (KT > 1) {
                srca = abase + BK, srcb = bbase + BK;
                NQ_DMA_ALL(1)
            }
        }
#undef NQ_DMA_ALL
    }
    const unsigned long long t_first = wall_clock64();  // stage 0 has landed
    const unsigned long long c_first = p.stamps ? clock64() : 0;  // (the shader clock's own count, for the loop in cycles)
    // what a phase before the first would have requested: all fragments of (buffer 0, phase 0)
    static_for<TI>([&](auto ic) { read_x(ic, integral_constant<int, 0>{}, integral_constant<int, 0>{}); });
    static_for<TJ>([&](auto jc) { read_w(integral_constant<int, 0>{}, jc, integral_constant<int, 0>{}, integral_constant<int, 0>{}); });
    NQ_LDS_WAIT(0);
    stage(integral_constant<int, 0>{}, std::true_type{}, 0, KT);
    if constexpr (NB == 4) {
        for (int st = 1; st < KT;) {
            stage(integral_constant<int, 1>{}, std::false_type{}, st, KT);
            if (++st >= KT) break;
            stage(integral_constant<int, 2>{}, std::false_type{}, st, KT);
            if (++st >= KT) break;
            stage(integral_constant<int, 3>{}, std::false_type{}, st, KT);
            if (++st >= KT) break;
            stage(integral_constant<int, 0>{}, std::false_type{}, st, KT);
            ++st;
        }
    } else if constexpr (NB == 3) {
        for (int st = 1; st < KT;) {
            stage(integral_constant<int, 1>{}, std::false_type{}, st, KT);
            if (++st >= KT) break;
            stage(integral_constant<int, 2>{}, std::false_type{}, st, KT);
            if (++st >= KT) break;
            stage(integral_constant<int, 0>{}, std::false_type{}, st, KT);
            ++st;
        }
    } else {
        int st = 1;
        for (; st + 1 < KT; st += 2) {
            stage(integral_constant<int, 1>{}, std::false_type{}, st, KT);
            stage(integral_constant<int, 0>{}, std::false_type{}, st + 1, KT);
        }
        if (st < KT) stage(integral_constant<int, 1>{}, std::false_type{}, st, KT);  // an even number of stages
    }
    NQ_LDS_WAIT(0);  // requests past the last stage still target registers: let them land
    __syncthreads();  // every wavefront is done with the stage buffers: the epilogue stages through them
    const unsigned long long t_loop = wall_clock64();
    const unsigned long long c_loop = p.stamps ? clock64() : 0;
#undef NQ_DMA
#undef NQ_LDS_READ
#undef NQ_LDS_WAIT

    // ---- epilogue.  The MFMA was issued with the weight fragment as its first operand, so in acc[i][j] a lane
    // holds ONE token m = 16 i + lane % 16 (MFMA column) and the four consecutive channels n = 16 j + 4 (lane / 16)
    // + 0..3 (MFMA rows, registers 0..3).  Per-token work is lane-local and four outputs of a row of y are adjacent.
    // Each wavefront stages its results through its own LDS region as [token][channel] rows, and writes them out as
    // 128-bit stores, 256 B (bf16) or 512 B (fp32 / int32) contiguous per row of y.
    const int wm0 = m0 + wm * (16 * TI), wn0 = n0 + wn * WN;
    const int lm = lane & 15, lq = lane >> 4;
    // whole 16-byte stores wherever the tile's columns all exist and rows of y stay 16-byte aligned
    // (a tile that only M cuts short just skips the rows past M)
    const bool full_cols = (n0 + BN <= p.N) && (p.N % 8 == 0) && (((uintptr_t)p.y & 15) == 0);

    // channel scale and bias for the lane's channels of fragment j (needs n < N: clamped)
    auto chan = [&](int j, float (&cs)[4], float (&cb)[4], bool need_scale, int zero) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int n = min(wn0 + 16 * j + 4 * lq + r, p.N - 1) + zero;
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
        // MODE (uniform over the launch, so chosen once and not per channel fragment: a branch around a load makes
        // the wavefront wait for that load where the branches meet).  0: one scale for the whole tensor and no bias
        // (fp8 x fp8): no channel operands at all; 1 .. 3: the lane's four channels adjacent and aligned, one load
        // per operand - no bias, fp32 bias, bf16 bias; 4: channel by channel
        constexpr int MODE = decltype(plain)::value;
        constexpr bool PLAIN = MODE == 0;
        constexpr int ES = (KIND == 1) ? 2 : 4;      // bytes per output element
        constexpr int IP = (KIND == 1) ? 4 : 2;      // token fragments (of 16) staged per pass
        constexpr int ROWB = WN * ES + 16;           // staged row: the wavefront's channels + pad (bank spread)
        uint8_t* stg = lds + wave * (16 * IP * ROWB);
#pragma unroll
        for (int ip = 0; ip < TI; ip += IP) {
            // ---- registers -> LDS (this wavefront's region only).
            // (a zero the compiler cannot see through, new in every pass: the channel operands do not depend on
            // the pass, and kept across the passes they spill; they are re-read from L1 per pass instead)
            int zero = 0;
            asm volatile("" : "+v"(zero));
            float rscale[IP];
#pragma unroll
            for (int ii = 0; ii < IP; ii++) {
                rscale[ii] = 1.0f;
                if constexpr (!FP8 && KIND != 2) rscale[ii] = p.row_scale[min(wm0 + 16 * (ip + ii) + lm, p.M - 1)];
            }
            auto fetch = [&](int j, float (&cs)[4], float (&cb)[4]) {
                const int nb = min(wn0 + 16 * j + 4 * lq, p.N - 4) + zero;
                if constexpr (!FP8) {
                    const float4 sv = *reinterpret_cast<const float4*>(p.col_scale + nb);
                    cs[0] = sv.x, cs[1] = sv.y, cs[2] = sv.z, cs[3] = sv.w;
                } else {
                    cs[0] = cs[1] = cs[2] = cs[3] = 1.0f;
                }
                if constexpr (MODE == 2) {
                    const float4 bv = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.bias) + nb);
                    cb[0] = bv.x, cb[1] = bv.y, cb[2] = bv.z, cb[3] = bv.w;
                } else if constexpr (MODE == 3) {
                    const uint2 bv = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p.bias) + nb);
                    cb[0] = __uint_as_float(bv.x << 16), cb[1] = __uint_as_float(bv.x & 0xFFFF0000u);
                    cb[2] = __uint_as_float(bv.y << 16), cb[3] = __uint_as_float(bv.y & 0xFFFF0000u);
                } else {
                    cb[0] = cb[1] = cb[2] = cb[3] = 0.0f;
                }
            };
            constexpr bool VEC = KIND != 2 && MODE >= 1 && MODE <= 3;
            // modes 1 .. 3: the operands of two channel fragments are requested together, a pair ahead
            float ncs[2][4], ncb[2][4];
            if constexpr (VEC) fetch(0, ncs[0], ncb[0]), fetch(1, ncs[1], ncb[1]);
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                float cs[4], cb[4];
                if constexpr (VEC) {
#pragma unroll
                    for (int r = 0; r < 4; r++) cs[r] = ncs[j & 1][r], cb[r] = ncb[j & 1][r];
                    if (j + 2 < TJ) fetch(j + 2, ncs[j & 1], ncb[j & 1]);
                }
                if constexpr (KIND != 2 && MODE == 4) chan(j, cs, cb, !FP8, zero);
#pragma unroll
                for (int ii = 0; ii < IP; ii++) {
                    const int i = ip + ii;
                    uint8_t* dst = stg + (16 * ii + lm) * ROWB + (16 * j + 4 * lq) * ES;
                    if constexpr (KIND == 2) {
                        *reinterpret_cast<i32x4*>(dst) = (i32x4){(int)acc[i][j][0], (int)acc[i][j][1], (int)acc[i][j][2], (int)acc[i][j][3]};
                    } else {
                        float z[4];
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            if constexpr (PLAIN)
                                z[r] = acc[i][j][r] * fp8_scale + 0.0f;  // (+ 0.0f: the bits of the general path, -0.0 included)
                            else if constexpr (FP8)
                                z[r] = acc[i][j][r] * fp8_scale + cb[r];
                            else
                                z[r] = (float)acc[i][j][r] * (rscale[ii] * cs[r]) + cb[r];
                        }
                        if (p.epilogue == NQ_EPI_RELU) {
                            // a real (uniform) branch: one v_max per value when asked for, nothing otherwise
                            asm volatile("" ::: "memory");
#pragma unroll
                            for (int r = 0; r < 4; r++) z[r] = z[r] > 0.0f ? z[r] : 0.0f;
                        }
                        if constexpr (KIND == 0) {
                            *reinterpret_cast<float4*>(dst) = make_float4(z[0], z[1], z[2], z[3]);
                        } else {
                            // v_cvt_pk_bf16_f32: round to nearest even in hardware
                            const bf16x4 pk = __builtin_convertvector((f32x4){z[0], z[1], z[2], z[3]}, bf16x4);
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
            constexpr int LPRW = WN * ES / 16;           // lanes per staged row (16 or 32)
            constexpr int RPI = 64 / LPRW;               // rows per wavefront instruction
#pragma unroll
            for (int t = 0; t < 16 * IP / RPI; t++) {
                const int row = t * RPI + lane / LPRW, c16 = lane % LPRW;
                const i32x4 v = *reinterpret_cast<const i32x4*>(stg + row * ROWB + c16 * 16);
                const int m = wm0 + 16 * ip + row;
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
    if (p.stamps) {  // (uniform) entry, first stage landed, loop done, stores acknowledged; the shader clock at the middle two
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (tid == 0) {
            unsigned long long* o = p.stamps + 6 * (size_t)blockIdx.x;
            o[0] = t_entry, o[1] = t_first, o[2] = t_loop, o[3] = wall_clock64();
            o[4] = c_first, o[5] = c_loop;
        }
    }
}

template <bool FP8, int KIND>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm8_kernel(const Gemm8Params p) {
    gemm8_body<FP8, KIND, 256, 256, 128, 4>(p);
}

template <bool FP8, int KIND>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm8w_kernel(const Gemm8Params p) {
    gemm8_body<FP8, KIND, 256, 256, 128, 8>(p);
}

// a 128 x 256 tile on four wavefronts (2 x 2, each 64 x 128 as in the eight-wavefront form): for what fills at most
// half a round of 256 x 256 tiles
template <bool FP8, int KIND>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm8h_kernel(const Gemm8Params p) {
    gemm8_body<FP8, KIND, 128, 256, 128, 4>(p);
}

// a 128 x 128 tile on four wavefronts of 64 x 64: for what fills at most a round of such tiles
template <bool FP8, int KIND>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm8q_kernel(const Gemm8Params p) {
    gemm8_body<FP8, KIND, 128, 128, 128, 4>(p);
}

template <typename K>
int32_t launch_cfg(K kernel, LdsAttrOnce* attr, const Gemm8Params& p, int form, hipStream_t s) {
    // two stage buffers of 64 KiB each (three of 48 for the 128-row tile); the eight-wavefront form's epilogue stages 17 KiB
    // per wavefront
    const size_t lds = form == 8 ? (size_t)8 * 17408 : form == 12 ? (size_t)3 * (128 + 256) * 128 : form == 16 ? (size_t)4 * (128 + 128) * 128 : (size_t)2 * (256 + 256) * 128;
    NQ_HIP(set_max_lds_once(*attr, reinterpret_cast<const void*>(kernel), lds));
    hipLaunchKernelGGL(kernel, dim3(p.grid ? p.grid : p.tiles_m * p.tiles_n), dim3(form == 8 ? 512 : 256), lds, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// form: 4 / 8 = the 256 x 256 tile on that many wavefronts, 12 = the 128 x 256 tile.  kind: 0 fp32, 1 bf16, 2 raw int32
int32_t launch_form(int form, bool fp8, int kind, const Gemm8Params& p, hipStream_t s) {
    static LdsAttrOnce attr[4][5];
    const int f = form == 4 ? 0 : form == 8 ? 1 : form == 12 ? 2 : 3;
    const int k = fp8 ? kind : 2 + kind;
#define NQ_G8_PICK(KERNEL)                                                                     \
    switch (k) {                                                                               \
        case 0: return launch_cfg(KERNEL<true, 0>, &attr[f][0], p, form, s);                   \
        case 1: return launch_cfg(KERNEL<true, 1>, &attr[f][1], p, form, s);                   \
        case 2: return launch_cfg(KERNEL<false, 0>, &attr[f][2], p, form, s);                  \
        case 3: return launch_cfg(KERNEL<false, 1>, &attr[f][3], p, form, s);                  \
        default: return launch_cfg(KERNEL<false, 2>, &attr[f][4], p, form, s);                 \
    }
    if (form == 4) { NQ_G8_PICK(gemm8_kernel) }
    if (form == 8) { NQ_G8_PICK(gemm8w_kernel) }
    if (form == 16) { NQ_G8_PICK(gemm8q_kernel) }
    NQ_G8_PICK(gemm8h_kernel)
#undef NQ_G8_PICK
}

}  // namespace

// What a call takes on each tile form, from measurements over K = 1024 .. 8192, M = 256 .. 8192, N = 4096 .. 11008: rounds
// of 256 workgroups x (a fixed part + a part per stage of 128 bytes of K); the smaller tiles' stages lengthen as more
// than half the CUs draw on L2 at once (`crowd`: the share of the round's workgroups beyond 128).
//   128 x 128 (one round, fp8, K = 4096): 15.7 - 15.9 us on 128 workgroups, 18.1 - 20.2 on 256; int8 18.0 / 20.2 - 22.3
//   128 x 256 (at most 128 tiles of 256 x 256): fp8 24.7 us on 128 workgroups, 26.9 on 192, 29.6 - 31.3 on 256; int8 28.8 / 30.8 / 33.4 - 35.2
//   256 x 256: 41 - 43 us a round fp8 (four wavefronts), 40 - 42 int8 (eight)
namespace {
double estimate_form(int form, int M, int N, int K, bool i8) {
    const double steps = (double)K / 128.0;
    if (form == 16) {
        const int64_t wgs = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
        const int64_t rounds = (wgs + 255) / 256;
        const int64_t in_round = (wgs + rounds - 1) / rounds;
        const double crowd = in_round > 128 ? (double)(in_round - 128) / 128.0 : 0.0;
        return (double)rounds * (5.6 + steps * ((i8 ? 0.385 : 0.32) + 0.08 * crowd));
    }
    const int64_t tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    if (form == 12) {
        const int64_t wgs = (int64_t)((M + 127) / 128) * ((N + 255) / 256);
        const double crowd = wgs > 128 ? (double)(wgs - 128) / 128.0 : 0.0;
        return i8 ? 7.0 + steps * (0.68 + 0.2 * crowd) : 6.5 + steps * (0.58 + 0.21 * crowd);
    }
    return (double)((tiles + 255) / 256) * (i8 ? 9.5 + 1.03 * steps : 10.0 + 1.1 * steps);
}
// the form a call runs on: 16 = 128 x 128 tiles, 12 = 128 x 256 tiles (calls of at most 128 tiles of 256 x 256), else the
// 256 x 256 tile on 4 (fp8) or 8 (int8) wavefronts
int pick_form(int M, int N, int K, bool i8, double* us) {
    const int64_t tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    int form = i8 ? 8 : 4;
    double best = estimate_form(form, M, N, K, i8);
    if (tiles <= 128) {
        const double h = estimate_form(12, M, N, K, i8);
        if (h < best) best = h, form = 12;
    }
    const double q = estimate_form(16, M, N, K, i8);
    if (q < best) best = q, form = 16;
    if (us) *us = best;
    return form;
}
}  // namespace

double gemm8_estimate_us(int M, int N, int K, bool i8) {
    double us = 0.0;
    pick_form(M, N, K, i8, &us);
    return us;
}

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
    p.stamps = a.diag_stamps;
    const bool i8 = a.x_dtype == NQ_DT_I8, fp8 = !i8;
    p.chan_vec = L->out % 4 == 0 && L->out >= 4 && (!i8 || a.y_dtype == NQ_DT_I32 || (uintptr_t)p.col_scale % 16 == 0) &&
                 (!a.bias || (uintptr_t)a.bias % (a.bias_dtype == NQ_DT_F32 ? 16 : 8) == 0);
    const int kind = a.y_dtype == NQ_DT_F32 ? 0 : a.y_dtype == NQ_DT_BF16 ? 1 : 2;
    const int tm = (a.M + 255) / 256, tn = (L->out + 255) / 256;
    const int tiles = tm * tn;
    p.tiles_m = tm, p.tiles_n = tn;
    if (a.diag_gemm8_waves == 12) {  // everything on 128-row tiles
        p.tiles_m = (a.M + 127) / 128;
        return launch_form(12, fp8, kind, p, a.stream);
    }
    if (a.diag_gemm8_waves == 16) {  // everything on 128 x 128 tiles
        p.tiles_m = (a.M + 127) / 128, p.tiles_n = (L->out + 127) / 128;
        return launch_form(16, fp8, kind, p, a.stream);
    }
    // int8 runs on the eight-wavefront form (8192 x 4096 x 4096: 105 - 108 us against 110 - 112; one round of tiles,
    // M = 2048: 42 - 43 against 49.5), fp8 on the four-wavefront form (the two measure the same, 95.5 - 99 us on the
    // same box; N = 11008 and 8192^3 1 - 2 % slower with eight)
    if (a.diag_gemm8_waves || a.diag_stamps) return launch_form(a.diag_gemm8_waves ? a.diag_gemm8_waves : (i8 ? 8 : 4), fp8, kind, p, a.stream);
    const int form = pick_form(a.M, L->out, L->in, i8, nullptr);
    if (form == 16) {
        p.tiles_m = (a.M + 127) / 128, p.tiles_n = (L->out + 127) / 128;
        return launch_form(16, fp8, kind, p, a.stream);
    }
    // What fills at most half a round of workgroups goes on 128 x 256 tiles, twice as many: a call that small as a
    // whole, or the tiles left over after the last full round when they form a rectangle (the kernel deals tiles in
    // bands of 8 row tiles, rows first, so the last `rest` tiles are whole columns of the last band when its row
    // count divides `rest`).  Every accumulator adds the same terms in the same order on either tile: same bits.
    constexpr int CUS = 256;
    if (form == 12) {
        p.tiles_m = (a.M + 127) / 128;
        return launch_form(12, fp8, kind, p, a.stream);
    }
    const int rest = tiles % CUS;
    const int last_band_rows = tm - (tm - 1) / 8 * 8;
    if (tiles > CUS && rest > 0 && rest <= CUS / 2 && rest % last_band_rows == 0 && rest / last_band_rows <= tn) {
        Gemm8Params q = p;
        // (the kernel regroups workgroup ids over its own grid size: a grid of tiles - rest covers exactly the first
        // tiles - rest tiles of the order)
        q.grid = tiles - rest;
        const int32_t rc = launch_form(form, fp8, kind, q, a.stream);
        if (rc != NQ_OK) return rc;
        Gemm8Params t = p;
        t.m_base = (tm - last_band_rows) * 256;
        t.n_base = (tn - rest / last_band_rows) * 256;
        t.tiles_m = (a.M - t.m_base + 127) / 128;
        t.tiles_n = rest / last_band_rows;
        return launch_form(12, fp8, kind, t, a.stream);
    }
    return launch_form(form, fp8, kind, p, a.stream);
}

}  // namespace nq
