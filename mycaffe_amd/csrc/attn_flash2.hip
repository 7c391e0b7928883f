// Fused attention forward for 16-bit storage, head sizes 64 and 128, no mask or the causal one (gfx950).
//
// What bounds this computation on the part is not the matrix cores alone.  Every MFMA of an attention step takes one
// 1 KB operand fragment from LDS (K for the scores, V^T for the output; Q and P stay in registers), the softmax between
// the two products is vector work, and a wavefront issues one instruction every four to five cycles whatever its kind
// (an exponential every twelve): per 64 keys a wavefront with 64 query rows issues about as many cycles of other
// instructions as its MFMAs take.  Vector work of one wavefront does not hide behind the MFMAs of another on the same
// SIMD, only behind its own; and with every unit busy the part runs into its power limit, where time follows the
// number of instructions and bytes moved rather than the longest of the parallel streams (the same kernel is a
// quarter faster on all-zero operands).  The kernel is built around these facts:
//
//  * Two 32-row query tiles per wavefront.  Every K / V fragment read from LDS feeds two MFMAs, one per tile, which
//    halves the LDS traffic per flop.  The fragments are held in registers across the two tiles' phases.
//  * The jobs (tile, 32-key step) of a wavefront run as a three-stage software pipeline inside the wavefront: while the
//    vector ALU does the softmax of job j, the matrix cores do S^T of job j + 1 and O^T += V^T P^T of job j - 1, in a
//    pinned issue order (one scheduling region per MFMA, each followed by a slice of the softmax, the fragment reads of
//    the next phase and a slice of the K / V staging).  Jobs alternate between the two tiles, so a block of 64 keys is
//    four such phases in straight-line code with fixed registers.
//  * The output tiles and the Q fragments live in accumulation registers (MFMA operands may come from either file), the
//    score tiles, weights and K / V fragments in vector registers.  The MFMAs of the pinned phases are inline assembly
//    with the register file of every operand spelled out, because the compiler's own choice for an MFMA result is an
//    accumulation register, which the vector ALU cannot read (sixteen copies per score tile).  Head size 64 fits 256
//    registers, two workgroups per CU; head size 128 takes the whole file, one wavefront per SIMD.
//  * A lean softmax.  Q is multiplied by scale * log2(e) once, when its fragments are loaded, and the weights are
//    exp2(score) with a fixed reference, 0, instead of a running maximum: bf16 and fp32 share their exponent range, so
//    weights far from 1 lose no precision, and a score then costs one v_exp_f32 and half a v_perm_b32 (the bf16 pair
//    is the upper halves of the two floats).  The row sum is formed from the packed pairs with v_dot2c_f32_bf16 (a
//    two-element dot product against ones), i.e. from exactly the weights that multiply V, so rounding the weights
//    down cancels between numerator and denominator.  No step needs the result of another: the jobs of a row may run in
//    any order, and partial sums simply add.
//  * A workgroup one of whose row sums ends outside [2^-18, 2^18] (scaled scores beyond about +-18: weights that exp2
//    cannot hold, or scores large enough for the second rounding of Q to show) computes its rows again the plain way:
//    running maxima, the scale applied to the scores in fp32 (flash2_plain_pass).  Correct for any input, at several
//    times the cost for such a workgroup.
//  * K and V blocks of 64 keys are staged through registers into four LDS stages, rows unpadded, the 16-byte pieces of
//    a row permuted by an XOR of row bits so that both the 128-bit K fragment reads (sixteen rows per access) and the
//    transposing V reads (four rows x 64 bytes per access) fall on distinct banks.  A block is requested from memory a
//    whole block (four phases) before it is written to LDS, a few pieces per phase; one workgroup barrier per block.
//  * Blocks in which some step of the wavefront needs a mask (the diagonal of the causal mask, the ragged end of the
//    keys) run one job after the other.  With the causal mask that block is a different one for every wavefront of the
//    workgroup, so these blocks are kept in their stages and done behind the loop over the blocks, by all wavefronts at
//    once, instead of one wavefront at a time with the others waiting at the block's barrier.
//  * The output leaves through LDS as whole rows, 16 bytes a lane: a lane owns a query, and its own values would be
//    sixteen scattered 8-byte stores.
//
// Scores are computed transposed (S^T = K Q^T), so that a lane owns one query row: register v of a 32 x 32 tile holds
// key 8 (v / 4) + 4 (lane / 32) + v % 4 of query lane % 32.
#include <type_traits>

#include "flash_traits.h"
#include "kernels.h"

namespace mch {

__device__ __forceinline__ float f2_pair_sum(float v)   // v + the value of the lane 32 away; both lanes get the same bits
{
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float f2_pair_max(float v)
{
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float f2_dot2_ones(uint32_t pair, float acc)   // acc + lo(pair) + hi(pair), bf16 pair
{
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(*reinterpret_cast<bf16x2*>(&pair), ones, acc, false);
}
__device__ __forceinline__ uint32_t f2_pack_trunc(float lo, float hi)   // the upper halves of two floats: a bf16 pair
{
    // Rounding towards zero: the row sums are formed from these same pairs, so the one-sided error cancels between the
    // weights and their sum, and v_perm_b32 runs at the full rate where the rounding conversion runs at half of it.
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}
__device__ __forceinline__ u32x4 f2_scale_frag(u32x4 q, float c)   // eight bf16 values times c, rounded back to bf16
{
    uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 4; i++)
        w[i] = pack_bf16x2(__uint_as_float(w[i] << 16) * c, __uint_as_float(w[i] & 0xffff0000u) * c);
    return u32x4{w[0], w[1], w[2], w[3]};
}

// MFMAs of the pinned phases.  "v": vector register, "a": accumulation register.  The compiler cannot see into the
// assembly, so the distances the hardware wants around an MFMA are kept by the order the phases are written in: two
// MFMAs that accumulate onto the same tile are at least one other MFMA apart, and a tile's first other reader is at
// least four MFMAs after its last writer.
__device__ __forceinline__ void f2_mma_s_first(floatx16& d, const u32x4& k, const u32x4& q)   // d (v) = K (v) Q^T (a)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(k), "a"(q));
}
__device__ __forceinline__ void f2_mma_s_acc(floatx16& d, const u32x4& k, const u32x4& q)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q));
}
__device__ __forceinline__ void f2_mma_o_acc(floatx16& o, const u32x4& vt, const u32x4& p)    // o (a) += V^T (v) P^T (v)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(o) : "v"(vt), "v"(p));
}

// Row sums the fast pass accepts.  Multiplying Q by the scale before the product rounds it to bf16 once more, an error
// of |score| 2^-9 at most on a score (in units of log2), and the fixed reference wants weights that are ordinary
// numbers; both ask for moderate scores.  A row sum inside [2^-18, 2^18] means the scores that carry the row are.
static constexpr float F2_HI = 262144.0f;             // 2^18
static constexpr float F2_LO = 3.814697265625e-06f;   // 2^-18

// The plain pass: the rows of one workgroup with a running maximum per row, the scale applied to the scores in fp32,
// one job after the other, K and V blocks of 64 keys copied to LDS one at a time.  Correct for any input; the fast pass
// below hands a workgroup over to it when one of its row sums leaves the accepted range.  Same tiles, same register
// layout of a tile as the fast pass; the compiler's own MFMAs throughout.
template <int HS, int KIND, int NW>
__device__ __forceinline__ void flash2_plain_pass(const FlashArgs& a, int b, int h, int qblock)
{
    typedef FlashTraits<bf16_t> TR;
    constexpr int KF = HS / 16, DT = HS / 32, LD = HS + 8, NT = NW * 64, BM = NW * 64, CPRW = HS / 8;
    extern __shared__ __attribute__((aligned(1024))) unsigned char f2_smem[];
    bf16_t* Ks = reinterpret_cast<bf16_t*>(f2_smem);
    bf16_t* Vs = Ks + 64 * LD;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const size_t bh = (size_t)b * a.H + h;
    const bf16_t* qp = (const bf16_t*)a.q + bh * a.Tq * HS;
    const bf16_t* kp = (const bf16_t*)a.k + bh * a.Tk * HS;
    const bf16_t* vp = (const bf16_t*)a.v + bh * a.Tk * HS;
    const int row0 = qblock * BM + 64 * wave;
    const int nsteps = (a.Tk + 31) >> 5;
    const int kend = KIND == 1 ? min(a.Tk, qblock * BM + BM) : a.Tk;
    const int nkb = (kend + 63) >> 6;
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // one tile after the other (the keys are walked twice): this path is rare, and its registers must not weigh on
    // the kernel that holds it
#pragma unroll 1
    for (int x = 0; x < 2; x++) {
        const int qbase = row0 + 32 * x;
        const int njobs = KIND == 1 ? min((qbase >> 5) + 1, nsteps) : nsteps;
        u32x4 qf[KF];
        floatx16 o[DT];
        float m = -INFINITY, l = 0.f;
        {
            const int row = min(qbase + l32, a.Tq - 1);
#pragma unroll
            for (int f = 0; f < KF; f++) qf[f] = *(const u32x4*)(qp + (size_t)row * HS + f * 16 + half * 8);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) o[dt] = zero16;
        }
        for (int kb = 0; kb < nkb; kb++) {
            __syncthreads();   // everybody has left the previous block (and, the first time, the stages of the fast pass)
            for (int e = tid; e < 64 * CPRW; e += NT) {
                const int row = e / CPRW, cp = e % CPRW, grow = min(kb * 64 + row, a.Tk - 1);
                *(u32x4*)(Ks + row * LD + cp * 8) = *(const u32x4*)(kp + (size_t)grow * HS + cp * 8);
                *(u32x4*)(Vs + row * LD + cp * 8) = *(const u32x4*)(vp + (size_t)grow * HS + cp * 8);
            }
            __syncthreads();
#pragma unroll 1
            for (int j = 0; j < 2; j++) {
                const int step = 2 * kb + j;
                if (step >= njobs) continue;
                const bf16_t* kst = Ks + (32 * j + l32) * LD + half * 8;
                floatx16 sc = zero16;
#pragma unroll
                for (int f = 0; f < KF; f++) sc = TR::mma(*(const u32x4*)(kst + f * 16), qf[f], sc);
                float mx = -INFINITY;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int key = step * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
                    sc[v] *= a.c;
                    if ((KIND == 1 && key > qbase + l32) || key >= a.Tk) sc[v] = -INFINITY;
                    mx = fmaxf(mx, sc[v]);
                }
                mx = fmaxf(f2_pair_max(mx), m);
                const float mnew = mx > -INFINITY ? mx : 0.f;   // no visible key yet: weights exp2(-inf - 0) = 0
                const float alpha = __builtin_amdgcn_exp2f(m - mnew);
                m = mx;
                float rs = 0.f;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    sc[v] = __builtin_amdgcn_exp2f(sc[v] - mnew);
                    rs += sc[v];
                }
                l = l * alpha + rs;
                const u32x4 p0 = TR::pack_p(sc, 0), p1 = TR::pack_p(sc, 1);
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                    for (int v = 0; v < 16; v++) o[dt][v] *= alpha;
                    const bf16_t* tile = Vs + 32 * j * LD + 32 * dt;
                    o[dt] = TR::mma(TR::load_vt_rowmajor(tile, LD, 0, lane), p0, o[dt]);
                    o[dt] = TR::mma(TR::load_vt_rowmajor(tile, LD, 1, lane), p1, o[dt]);
                }
            }
        }
        const int qrow = qbase + l32;
        const float lt = f2_pair_sum(l);
        const float inv = 1.0f / lt;
        const float mr = m > -INFINITY ? m : 0.f;
        if (a.lse2 && qrow < a.Tq && half == 0) a.lse2[bh * a.Tq + qrow] = mr + __log2f(lt);
        if (qrow < a.Tq) {
            bf16_t* yr = (bf16_t*)a.y + attn_y_row(a.yMerged, b, h, a.H, a.Tq, qrow, HS);
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    TR::store4(yr + 32 * dt + 8 * g + 4 * half, o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv,
                               o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv);
        }
    }
}

// KIND 0: no mask, 1: causal (query i sees keys 0 .. i).  NW wavefronts, two adjacent 32-row tiles each: a workgroup
// owns 64 NW query rows of one (batch, head).
template <int HS, int KIND, int NW>
__global__ __launch_bounds__(NW * 64, HS == 64 ? 2 : 1) void flash2_bf16_kernel(FlashArgs a)
{
    typedef FlashTraits<bf16_t> TR;
    constexpr int NST = 4;                        // LDS stages of 64 keys
    constexpr int ROWB = HS * 2;                  // bytes of a K / V row
    constexpr int BLKB = 64 * ROWB, VBASE = NST * BLKB, STEPB = 32 * ROWB;
    constexpr int KF = HS / 16, DT = HS / 32, NPV = 2 * DT, NSLOT = KF + NPV, EPS = 16 / NSLOT;
    constexpr int NT = NW * 64, BM = NW * 64;
    constexpr int CPRW = ROWB / 16;               // 16-byte pieces per row
    constexpr int CPW = 64 * CPRW / NT;           // pieces of a block and operand per lane
    static_assert((64 * CPRW) % NT == 0 && (HS == 64 || HS == 128) && KF == NPV && 2 * CPW <= NSLOT && (NST & (NST - 1)) == 0, "tile / wavefront mismatch");
    extern __shared__ __attribute__((aligned(1024))) unsigned char f2_smem[];   // K stages, V stages, second-pass flag

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5, i16 = lane & 15, g16 = (lane >> 4) & 1;
    const int nqb = (a.Tq + BM - 1) / BM;
    int qblock, h, b;
    if (KIND == 1) {
        // heaviest query block first across all (batch, head) pairs
        const int nbh = a.B * a.H;
        const int rank = flash_causal_rank(HS == 64 ? 2 : 1);   // workgroups a CU holds at once
        int ibh;
        flash_causal_map(rank, nbh, nqb, a.causalGroup, &qblock, &ibh);
        b = ibh / a.H;
        h = ibh % a.H;
    } else {
        qblock = blockIdx.x;
        h = blockIdx.y;
        b = blockIdx.z;
    }
    const size_t bh = (size_t)b * a.H + h;
    const bf16_t* qp = (const bf16_t*)a.q + bh * a.Tq * HS;
    const unsigned char* kp = (const unsigned char*)a.k + bh * a.Tk * ROWB;
    const unsigned char* vp = (const unsigned char*)a.v + bh * a.Tk * ROWB;

    // the wavefront's two tiles (0: rows row0 .. + 31, 1: the 32 rows after them) and their numbers of 32-key steps
    const int row0 = qblock * BM + 64 * wave;
    const int nsteps = (a.Tk + 31) >> 5;
    const int nA = KIND == 1 ? min((row0 >> 5) + 1, nsteps) : nsteps;
    const int nB = KIND == 1 ? min((row0 >> 5) + 2, nsteps) : nsteps;
    // steps 0 .. nplain - 1 need no mask in either tile
    const int nplain = KIND == 1 ? min(row0 >> 5, a.Tk >> 5) : a.Tk >> 5;
    const int kend = KIND == 1 ? min(a.Tk, qblock * BM + BM) : a.Tk;
    const int nkb = (kend + 63) >> 6;

    // ---- staging: piece e = tid + NT i of a block is 16-byte piece e % CPRW of key e / CPRW; in LDS it sits at piece
    // position (e % CPRW) ^ swizzle(row) of its row -------------------------------------------------------------------
    unsigned srcOff[CPW], dstK[CPW], dstV[CPW];
#pragma unroll
    for (int i = 0; i < CPW; i++) {
        const int e = tid + NT * i, row = e / CPRW, cp = e % CPRW;
        const int swK = HS == 64 ? (row >> 1) & 7 : row & 15;
        const int swV = HS == 64 ? 4 * ((row >> 1) & 1) : 4 * (row & 3);
        srcOff[i] = row * ROWB + (cp << 4);
        dstK[i] = row * ROWB + ((cp ^ swK) << 4);
        dstV[i] = VBASE + row * ROWB + ((cp ^ swV) << 4);
    }
    // Staging registers: piece i of the K block (i < CPW) or the V block (i >= CPW) on its way from memory to LDS.
    // gload_any takes any block number (rows past the last key repeat it: the mask hides them); gload_full wants a block
    // that lies inside the keys, given by its byte offset, and costs no vector arithmetic.
    u32x4 st[2 * CPW];
    const int lastRowOff = (a.Tk - 1) * ROWB;
    auto gload_any = [&](u32x4& dst, int kb, int i) {
        const unsigned so = srcOff[i % CPW];
        const unsigned off = (unsigned)min(kb * BLKB + (int)(so & ~(unsigned)(ROWB - 1)), lastRowOff) + (so & (ROWB - 1));
        dst = *(const u32x4*)((i < CPW ? kp : vp) + off);
    };
    auto gload_full = [&](u32x4& dst, unsigned blockOff, int i) {
        dst = *(const u32x4*)((i < CPW ? kp : vp) + (size_t)blockOff + srcOff[i % CPW]);
    };
    auto sstore_piece = [&](const u32x4& src, int stageOff, int i) {
        *(u32x4*)(f2_smem + stageOff + (i < CPW ? dstK[i] : dstV[i - CPW])) = src;
    };
    auto stage_of = [&](int kb) { return (kb & (NST - 1)) * BLKB; };

    // ---- Q fragments, multiplied by scale * log2(e) ----------------------------------------------------------------
    u32x4 qf[2][KF];
#pragma unroll
    for (int x = 0; x < 2; x++) {
        const int row = min(row0 + 32 * x + l32, a.Tq - 1);
#pragma unroll
        for (int f = 0; f < KF; f++) qf[x][f] = *(const u32x4*)(qp + (size_t)row * HS + f * 16 + half * 8);
    }

    // ---- fragment addresses in LDS ----------------------------------------------------------------------------------
    // K fragment f of a step: row 32 (step & 1) + l32 of the step's block, piece 2 f + half
    int klane[KF];
#pragma unroll
    for (int f = 0; f < KF; f++) klane[f] = l32 * ROWB + (((2 * f + half) ^ (HS == 64 ? (l32 >> 1) & 7 : l32 & 15)) << 4);
    // V^T fragment (tt, dt): two transposing reads of four keys each; this lane supplies row 16 tt + 4 half + i16 / 4
    // (+ 8 for the second read), bytes 64 dt + 32 g16 + 8 (i16 % 4) .. + 7 of it
    int vlane[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
        vlane[dt] = VBASE + (4 * half + (i16 >> 2)) * ROWB + ((dt ^ (HS == 64 ? (i16 >> 3) & 1 : (i16 >> 2) & 3)) << 6) + g16 * 32 + (i16 & 3) * 8;
    // off: byte offset of the step inside the stages (stage of its block, plus half a block for an odd step)
    auto ldK = [&](int f, int off) -> u32x4 { return *(const u32x4*)(f2_smem + klane[f] + off); };
    auto ldV = [&](int idx, int off) -> u32x4 {   // idx = tt * DT + dt
        const bf16_t* p = (const bf16_t*)(f2_smem + vlane[idx % DT] + off + (idx / DT) * 16 * ROWB);
        const uint2 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 8 * HS);
        return u32x4{lo.x, lo.y, hi.x, hi.y};
    };

    // ---- state ------------------------------------------------------------------------------------------------------
    // o[X]: output tiles, sb[X]: scores of tile X's next job, pkb[X]: packed weights of tile X's latest job,
    // fr: the K fragments (0 .. KF) and V^T fragments (KF ..) the coming MFMAs multiply with,
    // ls[X]: the row sums so far (two partial sums each, so that consecutive additions do not wait for each other)
    floatx16 o[2][DT], sb[2];
    u32x4 pkb[2][2], fr[NSLOT];
    float ls[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
    float exc0 = 0.f, exc1 = 0.f;   // the last two exponentials of the latest pinned phase, not yet packed
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // The block that travels to stage_of(j) as "block j".  Past the last block it is the block that lives in that stage
    // already (the same bytes once more), so that after the last block the stages still hold the last NST blocks.
    auto staged_block = [&](int j) { return j < nkb ? j : max(j - NST, 0); };
    // Blocks kb0 and kb0 + 1 into their stages, block kb0 + 2 requested: what every loop below expects going in.  The
    // second block travels through the fragment registers, free at this point.  Ends with a barrier.
    auto fill_stages = [&](int kb0) {
#pragma unroll
        for (int i = 0; i < 2 * CPW; i++) gload_any(st[i], kb0, i);
#pragma unroll
        for (int i = 0; i < 2 * CPW; i++) gload_any(fr[i], staged_block(kb0 + 1), i);
#pragma unroll
        for (int i = 0; i < 2 * CPW; i++) sstore_piece(st[i], stage_of(kb0), i);
#pragma unroll
        for (int i = 0; i < 2 * CPW; i++) gload_any(st[i], staged_block(kb0 + 2), i);
#pragma unroll
        for (int i = 0; i < 2 * CPW; i++) sstore_piece(fr[i], stage_of(kb0 + 1), i);
        __syncthreads();
    };
    // one block of the plain loops: block kb + 2 from the staging registers to its stage, block kb + 3 requested
    auto stage_step = [&](int kb) {
#pragma unroll
        for (int i = 0; i < 2 * CPW; i++) sstore_piece(st[i], stage_of(kb + 2), i);
#pragma unroll
        for (int i = 0; i < 2 * CPW; i++) gload_any(st[i], staged_block(kb + 3), i);
    };

    if (tid == 0) *reinterpret_cast<int*>(f2_smem + 2 * VBASE) = 0;   // the second-pass flag
    fill_stages(0);
#pragma unroll
    for (int x = 0; x < 2; x++)
#pragma unroll
        for (int f = 0; f < KF; f++) qf[x][f] = f2_scale_frag(qf[x][f], a.c);
#pragma unroll
    for (int x = 0; x < 2; x++) {
        sb[x] = zero16;
        asm volatile("" : "+v"(sb[x]));
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            o[x][dt] = zero16;
            asm volatile("" : "+a"(o[x][dt]));
        }
        pkb[x][0] = pkb[x][1] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int f = 0; f < KF; f++) asm volatile("" : "+a"(qf[x][f]));
    }
#pragma unroll
    for (int j = 0; j < NSLOT; j++) fr[j] = u32x4{0u, 0u, 0u, 0u};

    // softmax of one job, one instruction after the other: weights into pk, their sum into the row sums
    auto soft_seq = [&](auto x_, int step, bool plain, floatx16& sc, u32x4 (&pk)[2]) {
        constexpr int X = decltype(x_)::value;
        if (!plain) {
            const int qrow = row0 + 32 * X + l32, k0 = step * 32;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int key = k0 + 8 * (v >> 2) + 4 * half + (v & 3);
                if ((KIND == 1 && key > qrow) || key >= a.Tk) sc[v] = -INFINITY;
            }
        }
        uint32_t w[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            w[q] = f2_pack_trunc(__builtin_amdgcn_exp2f(sc[2 * q]), __builtin_amdgcn_exp2f(sc[2 * q + 1]));
            ls[X][q & 1] = f2_dot2_ones(w[q], ls[X][q & 1]);
        }
        pk[0] = u32x4{w[0], w[1], w[2], w[3]};
        pk[1] = u32x4{w[4], w[5], w[6], w[7]};
    };
    auto pv_regs = [&](auto x_) {   // O^T += V^T P^T of tile X's latest job, V^T fragments from fr[KF ..)
        constexpr int X = decltype(x_)::value;
#pragma unroll
        for (int idx = 0; idx < NPV; idx++) f2_mma_o_acc(o[X][idx % DT], fr[KF + idx], pkb[X][idx / DT]);
    };
    // one whole job, nothing overlapped: used where a step needs a mask.  off: the step's byte offset in the stages
    auto cold_job = [&](auto x_, int step, int off) {
        constexpr int X = decltype(x_)::value;
        floatx16 t = zero16;
#pragma unroll
        for (int f = 0; f < KF; f++) t = TR::mma(ldK(f, off), qf[X][f], t);
        asm volatile("" : "+v"(t));   // the score tiles live in vector registers throughout
        sb[X] = t;
        const bool plain = !(KIND == 1 && step * 32 + 31 > row0 + 32 * X) && step * 32 + 32 <= a.Tk;
        soft_seq(x_, step, plain, sb[X], pkb[X]);
#pragma unroll
        for (int idx = 0; idx < NPV; idx++) f2_mma_o_acc(o[X][idx % DT], ldV(idx, off), pkb[X][idx / DT]);
    };

    // One pinned phase of NSLOT slots, an MFMA each: the softmax of tile TS's job (scores sb[TS] -> weights pkb[TS]) next
    // to the other tile's MFMAs - S^T of its next job (into sb[1 - TS]) and O^T += V^T P^T of its latest one (weights
    // pkb[1 - TS]) - all on the fragments in fr.  The softmax is spread evenly: EPS exponentials a slot, a pair packed one
    // slot after its second exponential and added to the row sum a slot after that; what would fall behind the last slot
    // is done in the first slots of the next phase (the last pair of the previous phase's job, whose weights the MFMAs
    // of this phase need no earlier than slot 2 DT + 1).
    // RELOAD: behind every MFMA the fragment it used is replaced by the one at byte offset koff / voff.
    // PH (0 .. 3): the phase's share of the staging - pieces PH * PPP .. of the block two ahead go from their registers
    // to the stage at sOff, and the same pieces of the block three ahead (byte offset gOff) are requested.
    constexpr int PPP = 2 * CPW / 4;
    static_assert(2 * CPW % 4 == 0 && PPP <= NSLOT / 2, "staging pieces per phase");
    auto hot_phase = [&](auto ts_, auto reload_, auto ph_, int koff, int voff, int sOff, unsigned gOff) {
        constexpr int TS = decltype(ts_)::value, TO = 1 - TS, PH = decltype(ph_)::value;
        constexpr bool RELOAD = decltype(reload_)::value;
        floatx16& sc = sb[TS];
        float ex[16];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NSLOT; j++) {
            // even slots: S^T, odd slots: O^T (see f2_mma_s_first)
            if (!(j & 1)) {
                const int f = j >> 1;
                if (f == 0) f2_mma_s_first(sb[TO], fr[f], qf[TO][f]);
                else f2_mma_s_acc(sb[TO], fr[f], qf[TO][f]);
                if (RELOAD) fr[f] = ldK(f, koff);
            } else {
                const int idx = j >> 1;
                f2_mma_o_acc(o[TO][idx % DT], fr[KF + idx], pkb[TO][idx / DT]);
                if (RELOAD) fr[KF + idx] = ldV(idx, voff);
            }
            if ((j & 1) && (j >> 1) < PPP) {
                const int i = PH * PPP + (j >> 1);
                sstore_piece(st[i], sOff, i);
                gload_full(st[i], gOff, i);
            }
#pragma unroll
            for (int e = j * EPS; e < (j + 1) * EPS; e++) {
                ex[e] = __builtin_amdgcn_exp2f(sc[e]);
                asm volatile("" : "+v"(ex[e]));   // keeps the instruction in this slot
            }
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const int cs = (2 * q + 1) / EPS + 1;   // the slot that packs pair q, the next one adds it up
                if (cs == j) {
                    uint32_t w = f2_pack_trunc(ex[2 * q], ex[2 * q + 1]);
                    asm volatile("" : "+v"(w));
                    pkb[TS][q >> 2][q & 3] = w;
                }
                if (cs == j + NSLOT) {                  // q == 7 of the previous phase's job
                    uint32_t w = f2_pack_trunc(exc0, exc1);
                    asm volatile("" : "+v"(w));
                    pkb[TO][q >> 2][q & 3] = w;
                }
                if (cs + 1 == j) {
                    ls[TS][q & 1] = f2_dot2_ones(pkb[TS][q >> 2][q & 3], ls[TS][q & 1]);
                    asm volatile("" : "+v"(ls[TS][q & 1]));
                }
                if (cs + 1 == j + NSLOT) {
                    ls[TO][q & 1] = f2_dot2_ones(pkb[TO][q >> 2][q & 3], ls[TO][q & 1]);
                    asm volatile("" : "+v"(ls[TO][q & 1]));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        exc0 = ex[14];
        exc1 = ex[15];
    };
    // what the last pinned phase (softmax of tile X) left for the first slots of a next one
    auto hot_tail = [&](auto x_) {
        constexpr int X = decltype(x_)::value;
        pkb[X][1][3] = f2_pack_trunc(exc0, exc1);
#pragma unroll
        for (int q = 0; q < 8; q++)
            if ((2 * q + 1) / EPS + 2 >= NSLOT) ls[X][q & 1] = f2_dot2_ones(pkb[X][q >> 2][q & 3], ls[X][q & 1]);
        exc0 = exc1 = 0.f;
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    typedef std::integral_constant<int, 2> I2;
    typedef std::integral_constant<int, 3> I3;
    typedef std::integral_constant<bool, false> BF;
    typedef std::integral_constant<bool, true> BT;

    // the K fragments of step 0, and with them S^T of tile 0's first job
#pragma unroll
    for (int f = 0; f < KF; f++) fr[f] = ldK(f, 0);
    {
        floatx16 t = zero16;
#pragma unroll
        for (int f = 0; f < KF; f++) t = TR::mma(fr[f], qf[0][f], t);
        asm volatile("" : "+v"(t));
        sb[0] = t;
    }

    // Blocks whose two steps need no mask in either tile: four pinned phases each.  Going in, sb[0] holds tile 0's scores
    // of the block's first step; tile 1's latest weights (pkb[1], their V^T fragments in fr) are multiplied in the first
    // phase - zeros before the first block.
    // Staging.  Going into block kb, blocks kb and kb + 1 are in their stages and the staging registers hold block
    // kb + 2.  During the block they are written to the stage that block kb - 2 had - every wavefront left it before the
    // barrier of block kb - 1 - and are read from the second half of block kb + 1 on, behind that block's barrier.
    // The pinned phases request whole blocks only; a block cut short by the end of the keys is requested by the plain
    // loop, so the pinned phases stop four blocks before such a block.
    // The last NST blocks are still in their stages when the loop over the blocks ends.  What a wavefront has to do with
    // them one job after the other - the diagonal of the causal mask, which is a different block for every wavefront of
    // the workgroup - it does behind the loop, all wavefronts at once, instead of inside it with the others waiting at
    // the block's barrier (the jobs of a row may run in any order: the weights have a fixed reference).
    const int nFull = a.Tk >> 6;
    int kb = 0;
    int nhot = min(nkb, nplain >> 1);
    if (nkb > nFull) nhot = min(nhot, nkb - 4);
    for (; kb < nhot; kb++) {
        const int cur = stage_of(kb), nxt = stage_of(kb + 1), wst = stage_of(kb + 2);
        const unsigned gOff = (unsigned)min(staged_block(kb + 3), nFull - 1) * BLKB;
        hot_phase(I0{}, BT{}, I0{}, cur + STEPB, cur, wst, gOff);
        hot_phase(I1{}, BF{}, I1{}, 0, 0, wst, gOff);
        __syncthreads();
        hot_phase(I0{}, BT{}, I2{}, nxt, cur + STEPB, wst, gOff);
        hot_phase(I1{}, BF{}, I3{}, 0, 0, wst, gOff);
    }
    hot_tail(I1{});
    pv_regs(I1{});
    // the remaining blocks (diagonal of the causal mask, ragged end of the keys), one job after the other
    auto cold_block = [&](int kb) {
        const int t0 = 2 * kb, cur = stage_of(kb);
        if (t0 < nA) cold_job(I0{}, t0, cur);
        if (t0 < nB) cold_job(I1{}, t0, cur);
        if (t0 + 1 < nA) cold_job(I0{}, t0 + 1, cur + STEPB);
        if (t0 + 1 < nB) cold_job(I1{}, t0 + 1, cur + STEPB);
    };
    const int kbLate = max(kb, nkb - NST);   // from here on the wavefront's blocks wait for the end of the loop
    for (; kb < nkb; kb++) {
        stage_step(kb);
        if (kb < kbLate) cold_block(kb);
        __syncthreads();
    }
    for (kb = kbLate; kb < nkb; kb++) cold_block(kb);

    // ---- a workgroup one of whose rows does not suit the fast pass computes its rows again the plain way -----------------
    // Only the final sums matter: a sum inside the accepted range means the row's largest weight was an ordinary number,
    // and weights that are tiny next to it are as good as the zeros they may have become.
    float lsum[2];
    bool bad = false;
#pragma unroll
    for (int x = 0; x < 2; x++) {
        lsum[x] = ls[x][0] + ls[x][1];
        const float lt = f2_pair_sum(lsum[x]);
        bad = bad || !(lt >= F2_LO && lt <= F2_HI);
    }
    int* flag = reinterpret_cast<int*>(f2_smem + 2 * VBASE);
    if (__any(bad) && lane == 0) *flag = 1;
    __syncthreads();
    if (*flag != 0) {   // uniform over the workgroup
        flash2_plain_pass<HS, KIND, NW>(a, b, h, qblock);
        return;
    }

    // ---- epilogue: y[query, dim] = O^T[dim, query] / l; register v of tile dt is dim 32 dt + 8 (v / 4) + 4 half + v % 4.
    // A lane owns a query, so its values are scattered over the row; they go through the wavefront's own 64 rows of LDS
    // (the stages are free: every wavefront is past the barrier above) and leave as whole rows, 16 bytes a lane.  The
    // 16-byte pieces of a row are permuted by the row number so that neither side piles up on a few banks.
    static_assert(NW * BLKB <= 2 * VBASE, "one block of LDS per wavefront");
    unsigned char* ybuf = f2_smem + wave * BLKB;
#pragma unroll
    for (int x = 0; x < 2; x++) {
        const int r = 32 * x + l32, qrow = row0 + r;
        const float lt = f2_pair_sum(lsum[x]);
        const float inv = 1.0f / lt;
        if (a.lse2 && qrow < a.Tq && half == 0) a.lse2[bh * a.Tq + qrow] = __log2f(lt);
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint2 w;
                w.x = pack_bf16x2(o[x][dt][4 * g] * inv, o[x][dt][4 * g + 1] * inv);
                w.y = pack_bf16x2(o[x][dt][4 * g + 2] * inv, o[x][dt][4 * g + 3] * inv);
                *(uint2*)(ybuf + r * ROWB + (((4 * dt + g) ^ (r & (CPRW - 1))) << 4) + 8 * half) = w;
            }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int i = 0; i < CPRW; i++) {
        const int e = lane + 64 * i, r = e / CPRW, piece = e % CPRW, qrow = row0 + r;
        const u32x4 w = *(const u32x4*)(ybuf + r * ROWB + ((piece ^ (r & (CPRW - 1))) << 4));
        if (qrow < a.Tq) *(u32x4*)((bf16_t*)a.y + attn_y_row(a.yMerged, b, h, a.H, a.Tq, qrow, HS) + piece * 8) = w;
    }
}

template <int HS, int KIND, int NW> static hipError_t flash2_launch_cfg(hipStream_t s, const FlashArgs& f)
{
    constexpr int BM = NW * 64, LDSB = 2 * 4 * 64 * HS * 2 + 16;   // four K and four V stages, the second-pass flag
    static bool attr = false;
    if (!attr) {
        hipError_t e = hipFuncSetAttribute((const void*)flash2_bf16_kernel<HS, KIND, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, LDSB);
        if (e != hipSuccess) return e;
        attr = true;
    }
    const int nqb = (f.Tq + BM - 1) / BM;
    const dim3 grid = KIND == 1 ? dim3(nqb * f.H * f.B, 1, 1) : dim3(nqb, f.H, f.B);
    hipLaunchKernelGGL((flash2_bf16_kernel<HS, KIND, NW>), grid, NW * 64, LDSB, s, f);
    return hipGetLastError();
}

// bf16, head size 64 or 128, no mask or causal with Tq == Tk.  f as prepared by attn_flash_launch.
hipError_t attn_flash2_launch(hipStream_t s, const FlashArgs& f, int hs, bool causal, bool* handled)
{
    *handled = false;
    if (causal && f.Tq != f.Tk) return hipSuccess;
    if ((long long)f.Tk * hs * 2 >= (1ll << 31)) return hipSuccess;
    *handled = true;
    if (hs == 64) return causal ? flash2_launch_cfg<64, 1, 4>(s, f) : flash2_launch_cfg<64, 0, 4>(s, f);
    return causal ? flash2_launch_cfg<128, 1, 4>(s, f) : flash2_launch_cfg<128, 0, 4>(s, f);
}

}  // namespace mch
