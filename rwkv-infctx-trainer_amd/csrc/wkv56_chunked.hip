// WKV5 / WKV6 in blocked form on the matrix cores (bf16 operands, fp32 state).
//
// A (batch, head) sequence is walked in blocks of 16 tokens.  Inside a block, with
// incl_t / excl_t the inclusive / exclusive running sums of log w from the block's
// start and b their total:
//
//   y_t = (r_t e^{excl_t}) S  +  sum_{s<t} [(r_t e^{excl_t}) . (k_s e^{-incl_s})] v_s  +  (r_t . u k_t) v_t
//   S  <- e^{b} o S + sum_s (k_s e^{b-incl_s})^T v_s
//
// log w >= ln 0.005, so excl_t >= -79.5 for every token of a block and -incl_s <= 79.5
// for every s that has a later token in its block: all scaled factors stay inside
// the bf16/fp32 range without the fp64 the reference needs for its 128-token chunks
// (RWKV-v5/src/module/rwkv_inner.py:91-93).  The contractions are 16x16x32 bf16
// MFMAs; the state lives in MFMA accumulators for the whole sequence and enters the
// next product straight from registers (the accumulator layout of a 16x16 tile is
// the B-operand layout).
//
// Precision: every operand that is not already an exact bf16 input (decay-scaled
// r and k, the masked intra-block matrices, the state and its gradient) is fed
// to the matrix cores as a bf16 head plus a bf16 remainder (x ~= hi + lo, 16
// mantissa bits) and the products hi*hi + lo*hi + hi*lo are accumulated in fp32,
// two 16-deep products per 16x16x32 instruction.  This is what keeps the decay
// gradient, a difference of large running sums, at fp32-like accuracy.
//
// The scaled operands are prepared 64 tokens at a time and laid out in LDS as
// [token][channel] tiles whose rows are padded to 68 elements, which makes every 8-byte
// MFMA operand fragment read conflict-free, both the plain ones (tokens along M or N)
// and the transposing ones (tokens along the contraction).
//
// The main kernels run 16 wavefronts per workgroup, four per SIMD: one wavefront alone
// issues a vector instruction only every six to eight cycles, so the work of a step is
// cut into independent pieces (per 16-token block, per 16 channels) for different
// wavefronts, and only the short serial recurrences stay with one wavefront each.
// Global memory is always touched in full 128-byte rows (16 lanes x 8 bytes = the 64
// channels of one token and head).
//
// Time-parallel split: a sequence is cut into segments that run as separate
// workgroups; a light pass leaves each piece's effect on a state handed in
// (S_out = decay o S_in + delta), a small kernel chains the summaries into the state
// at the start of every segment.  Backward does the same with the state gradient.
#include "common.h"
#include <type_traits>

namespace wkv {
namespace chunked {

// optional per-phase cycle counts of workgroup 0 (development aid, off by default; build with EXTRA=-DWKV_PHASE_TIMING).
// forward16:  p5 top of the step, p0 prepare, p1 wait, p2 chains / builders, p3 wait, p4 finish
// backward16: p5 top of the step (the prefetched inputs arrive), p6 results of the step before written out, p7 running
//             sum inside the wavefronts + the wait for the others', p0 rest of prepare, p1 wait, p2 chains / builders,
//             p3 wait, p4 block phase
// summary_pass (all four wavefronts print): p0 prepare (with the wait for the prefetched inputs), p1 wait, p2 the next
//             step's loads issued + the decay bookkeeping of wavefront 0, p3 the four blocks' MFMAs and the update of X,
//             p4 wait
#ifdef WKV_PHASE_TIMING
#define PT_DECL long long pt_[8] = {0, 0, 0, 0, 0, 0, 0, 0}; long long pt_last_ = clock64();
#define PT_MARK(i) { const long long now_ = clock64(); pt_[i] += now_ - pt_last_; pt_last_ = now_; }
#define PT_PRINT(name) if (blockIdx.x == 0 && (threadIdx.x & 255) == 0) printf("%s[%d]: p0 %lld p1 %lld p2 %lld p3 %lld p4 %lld p5 %lld p6 %lld p7 %lld\n", name, (int)threadIdx.x, pt_[0], pt_[1], pt_[2], pt_[3], pt_[4], pt_[5], pt_[6], pt_[7]);
#define PT_PRINT_WAVES(name) if (blockIdx.x == 0 && (threadIdx.x & 63) == 0) printf("%s[%d]: p0 %lld p1 %lld p2 %lld p3 %lld p4 %lld\n", name, (int)threadIdx.x, pt_[0], pt_[1], pt_[2], pt_[3], pt_[4]);
#else
#define PT_DECL
#define PT_MARK(i)
#define PT_PRINT(name)
#define PT_PRINT_WAVES(name)
#endif

// (lds_barrier(): the workgroup barrier of these kernels, whose wavefronts talk to each other through LDS alone)

typedef short s4 __attribute__((ext_vector_type(4)));
typedef short s8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int SB = 64;        // tokens prepared per staging step
constexpr int LD = 68;        // padded row length of a 64x64 bf16 tile in LDS
constexpr int NT_F = 256;     // summary passes: 4 wavefronts

// One 16-deep product, D[m][n] += sum_k A[m][k] B[k][n].  Issued as a 16x16x32 MFMA
// with a zero upper half: on gfx950 a 16x16x16 MFMA chained on the accumulator of a
// 16x16x32 one returned corrupted rows in this kernel, and both cost one issue slot.
__device__ __forceinline__ f4 mma(s4 a, s4 b, f4 c) {
    const s8 av = {a[0], a[1], a[2], a[3], 0, 0, 0, 0};
    const s8 bv = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, av), __builtin_bit_cast(b8, bv), c, 0, 0, 0);
}
// two 16-deep products in one 16x16x32 instruction: D += A0 B0 + A1 B1
__device__ __forceinline__ f4 mma2(s4 a0, s4 a1, s4 b0, s4 b1, f4 c) {
    const s8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
    const s8 b = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
}
// lane (g = lane/16, n = lane%16) supplies A[n][4g..4g+3] and B[4g..4g+3][n], receives D[4g..4g+3][n]
__device__ __forceinline__ s4 frag(const uint16_t *tile, int row, int col) {
    return *reinterpret_cast<const s4 *>(tile + row * LD + col);
}
__device__ __forceinline__ float bf2f(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ float bf_lo(uint32_t p) { return __uint_as_float(p << 16); }          // element 0 of a pair
__device__ __forceinline__ float bf_hi(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }  // element 1
__device__ __forceinline__ s4 as_s4(uint32_t a, uint32_t b) {
    const uint2 x = make_uint2(a, b);
    return __builtin_bit_cast(s4, x);
}
// x ~= hi + lo with both parts bf16: 16 mantissa bits instead of 8
__device__ __forceinline__ void split2(float a, float b, uint32_t &hi, uint32_t &lo) {
    hi = bf16_pack2(a, b);
    lo = bf16_pack2(a - bf_lo(hi), b - bf_hi(hi));
}
__device__ __forceinline__ void split4(f4 x, s4 &hi, s4 &lo) {
    uint32_t h0, l0, h1, l1;
    split2(x[0], x[1], h0, l0);
    split2(x[2], x[3], h1, l1);
    hi = as_s4(h0, h1);
    lo = as_s4(l0, l1);
}
// The builders' r operand of the masked intra-block matrix: (r e^{excl}) e^{-b} = r e^{excl-b}, from the head/remainder
// fragments of r e^{excl} (four keys of one token) and e^{-b} of those keys, as head + remainder again.  With
// k e^{b-incl} as the other operand the product is r k e^{excl_t - incl_s}, at most |r k| where it is used (s < t).
// A block's first token has no earlier token; its row is zeroed (its exponent -b is the only one beyond 79.5).
__device__ __forceinline__ void scale_split(s4 hi, s4 lo, float4 f, bool zero, s4 &oh, s4 &ol) {
    const uint2 h = __builtin_bit_cast(uint2, hi), l = __builtin_bit_cast(uint2, lo);
    float x0 = (bf_lo(h.x) + bf_lo(l.x)) * f.x, x1 = (bf_hi(h.x) + bf_hi(l.x)) * f.y;
    float x2 = (bf_lo(h.y) + bf_lo(l.y)) * f.z, x3 = (bf_hi(h.y) + bf_hi(l.y)) * f.w;
    if (zero) x0 = x1 = x2 = x3 = 0.f;
    uint32_t h0, l0, h1, l1;
    split2(x0, x1, h0, l0);
    split2(x2, x3, h1, l1);
    oh = as_s4(h0, h1);
    ol = as_s4(l0, l1);
}
// Result rows leave with the non-temporal hint: they are not read again by these kernels, and left to the default
// policy they push the inputs that the backward pass reads a second time out of the last-level cache.
__device__ __forceinline__ void store_row(bf16 *p, uint2 v) {
    typedef unsigned int u2 __attribute__((ext_vector_type(2)));
    __builtin_nontemporal_store(u2{v.x, v.y}, reinterpret_cast<u2 *>(p));
}
__device__ __forceinline__ void store_row(bf16 *p, const float (&x)[4]) { store_row(p, make_uint2(bf16_pack2(x[0], x[1]), bf16_pack2(x[2], x[3]))); }
__device__ __forceinline__ void store_row(float *p, const float (&x)[4]) {
    typedef float f4_ __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(f4_{x[0], x[1], x[2], x[3]}, reinterpret_cast<f4_ *>(p));
}
__device__ __forceinline__ float group_sum4(float x) {      // over the 4 lane groups of 16
    x += __shfl_xor(x, 16);
    x += __shfl_xor(x, 32);
    return x;
}

// The raw decay of one token's four channels as it waits in registers between fetch and use: fp32, or bf16 as a
// mixed-precision TimeMix hands it over (W16; converted where it is used, so the prefetch holds half the registers
// and moves half the bytes).  For the time-invariant decay the same slot carries the constant log decay.
// Element `o` of a sequence whose first element `p` points at, `p` being the same for all lanes: the byte offset is
// formed in 32 bits, so the access takes the scalar base + 32-bit lane offset form and no lane holds a 64-bit address
// (the launchers refuse a sequence of 2^30 elements or more per batch entry).
template <class P> __device__ __forceinline__ P *seq_at(P *p, uint32_t o) {
    using Byte = typename std::conditional<std::is_const<P>::value, const char, char>::type;
    return reinterpret_cast<P *>(reinterpret_cast<Byte *>(p) + o * (uint32_t)sizeof(P));
}
template <bool W16> struct WReg;
template <> struct WReg<false> {
    float4 v;
    static __device__ __forceinline__ WReg load(const void *w, uint32_t o) {
        return WReg{*reinterpret_cast<const float4 *>(seq_at(static_cast<const float *>(w), o))};
    }
    // The same as two 8-byte loads, for a value that stays in flight across a phase short of registers: a 16-byte load
    // wants four consecutive registers, which the allocator there gives only at the price of copies that wait for the
    // load on the spot.
    static __device__ __forceinline__ WReg load_in_halves(const void *w, uint32_t o) {
        typedef float f2 __attribute__((ext_vector_type(2)));
        uint32_t o2 = o + 2;
        asm volatile("" : "+v"(o2));          // (opaque: the two loads are not seen to be adjacent, so they are not merged)
        const f2 a = *reinterpret_cast<const f2 *>(seq_at(static_cast<const float *>(w), o));
        const f2 b = *reinterpret_cast<const f2 *>(seq_at(static_cast<const float *>(w), o2));
        return WReg{make_float4(a[0], a[1], b[0], b[1])};
    }
    static __device__ __forceinline__ WReg from(float4 x) { return WReg{x}; }
    __device__ __forceinline__ float4 f4() const { return v; }
};
template <> struct WReg<true> {
    uint2 v;
    static __device__ __forceinline__ WReg load(const void *w, uint32_t o) {
        return WReg{*reinterpret_cast<const uint2 *>(seq_at(static_cast<const bf16 *>(w), o))};
    }
    static __device__ __forceinline__ WReg load_in_halves(const void *w, uint32_t o) { return load(w, o); }
    static __device__ __forceinline__ WReg from(float4 x) { return WReg{make_uint2(bf16_pack2(x.x, x.y), bf16_pack2(x.z, x.w))}; }
    __device__ __forceinline__ float4 f4() const { return make_float4(bf_lo(v.x), bf_hi(v.x), bf_lo(v.y), bf_hi(v.y)); }
};
#define WKV_NEG_INF4 make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY)
// "These registers are needed HERE": makes the compiler wait for the loads that fill them at this point.  One counter
// covers a wavefront's loads and stores, and a wait the compiler places after a conditional memory operation is
// counted for the path without it: a wait for the step's inputs placed after the (conditional) result stores would
// also wait for those stores to complete.
__device__ __forceinline__ void needed_here(uint2 &a) { asm volatile("" : "+v"(a.x), "+v"(a.y)); }
__device__ __forceinline__ void needed_here(float4 &a) { asm volatile("" : "+v"(a.x), "+v"(a.y), "+v"(a.z), "+v"(a.w)); }

// One segment's summary for the time-parallel split: what the segment does to a
// state handed in, S_out = decay o S_in + delta (forward), or to a state gradient
// handed back (backward).  [key][value] fp32 plus one decay per key.
constexpr int PART = HEAD * HEAD + HEAD;

// ------------------------------------------------------- forward, 16 wavefronts --
// The main forward pass with the work of a 64-token step spread over 16 wavefronts
// (four per SIMD).  A step runs in three phases separated by workgroup barriers:
//
//   prepare   all wavefronts: lane = (one token, four channels), 16 lanes = that token's
//             128-byte row; a block's running log decay is summed inside the wavefront (four
//             tokens) and joined across the block's four wavefronts through LDS.  Every tile
//             is [token][channel]; the operands that the MFMAs want with the tokens along the
//             contraction (k e^{b-incl}, v) come out of the transposing LDS read of gfx950.
//   chains    wavefronts 0-7 own the state for good: wavefront (w, half) holds keys
//             32*half..32*half+31 x values 16w..16w+15 in registers, walks it over the four
//             blocks and leaves its share of  rh S  per block in LDS;
//             wavefronts 8-15 build the masked intra-block matrix of one block each, one half of the
//             keys a wavefront (the two parts are added by the MFMAs of the finish).
//   finish    wavefront (q, w): y of block q, value columns 16w..16w+15 = the two shares
//             + (intra-block matrix) v, converted and stored.
constexpr int NT_F16 = 1024;

struct Fwd16Tiles {
    uint16_t rh[SB * LD];     // r e^{excl}       [token][key]  bf16 head / remainder
    uint16_t rhl[SB * LD];
    uint16_t kh[SB * LD];    // k e^{b-incl}     [token][key]   (read both ways)
    uint16_t khl[SB * LD];
    uint16_t v[SB * LD];     // v                [token][value] (read transposed)
    float dec[4][HEAD];       // e^{b} per block and key
    float ent[4][HEAD];       // e^{-b}
    float rho[SB];            // r . (u o k) per token
    uint4 amat[2][4][64];     // masked intra-block matrix of each block, one part per half of the keys, as A-operand fragments (head, remainder)
    float4 yi[2][4][4][64];   // rh S per key half, block, value quarter: accumulator layout, one float4 per lane
    float wtot[16][HEAD];     // per wavefront (four tokens) and channel: sum of log w, for the block-wide running sum
};

__device__ __forceinline__ float row_prefix_sum(float x) {      // inclusive, over the 16 lanes of a DPP row
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x111, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x112, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x114, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x118, 0xf, 0xf, true));
    return x;
}
// inclusive sum over the lanes n..15 of a DPP row (the later tokens of a block when a row's lanes are its 16 tokens)
__device__ __forceinline__ float row_suffix_sum(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x101, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x102, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x104, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x108, 0xf, 0xf, true));
    return x;
}
// Index into a [token][64 keys] fp32 table of the backward kernel.  The tables are written one token row per 16 lanes
// (four keys a lane) by the preparing lanes and read one token per lane (four keys) by the block phase; without the
// exchange of 16-byte pieces inside a row by the row number, the second pattern would put the sixteen lanes of a group
// (sixteen consecutive rows, the same columns) on the same banks.
__device__ __forceinline__ int swz(int row, int col) { return row * HEAD + (col ^ ((row & 15) << 2)); }
// Transposing 8-byte LDS read: with every lane (g, a) of a 16-lane group pointing at
// tile[row0 + 4g + a/4][col0 + 4(a%4) ..+3], lane (g, n) receives tile[row0 + 4g + i][col0 + n], i = 0..3:
// an MFMA operand fragment with the rows along the contraction.  `off` = the lane's share of the address.
__device__ __forceinline__ int tr_lane_offset(int lane, int ld) {
    const int a = lane & 15, g = lane >> 4;
    return (4 * g + (a >> 2)) * ld + 4 * (a & 3);
}
__device__ __forceinline__ s4 frag_tr(const uint16_t *tile, int off) {
    typedef s4 __attribute__((address_space(3))) lds_s4;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4 *)(tile + off));
}

// Preparing role of the 16-wavefront kernels: a lane holds one token and four channels;
// the 16 lanes of a DPP row are the 64 channels of that token (one 128-byte row of the
// (B,T,C) bf16 tensors, so every global access is a full row segment); wavefront w has the
// tokens 4w..4w+3 of the step, four wavefronts make a 16-token block.
// Block-wide running sum of log w in two halves, so that the exchange across the four wavefronts of a block
// rides on a barrier the step has anyway:
//   scan_local  (at the end of the previous step, on the prefetched w): log w of the lane's token -> running sum
//               inside the wavefront (two shuffles); the wavefront's total goes to `wtot` in LDS;
//   scan_join   (at the start of the step, after that barrier): adds the totals of the earlier wavefronts of the
//               block (inc = inclusive running sum inside the block) and forms the block total (tot).
// All of these are in base-2 units (log2 w), so that every exponential is one v_exp_f32.
__device__ __forceinline__ void scan_local(const float (&l)[4], float (&inc)[4], float (*wtot)[HEAD], int w16, int g, int n) {
#pragma unroll
    for (int c = 0; c < 4; c++) {
        float x = l[c];
        const float u1 = __shfl_up(x, 16);
        x += g >= 1 ? u1 : 0.f;
        const float u2 = __shfl_up(x, 32);
        x += g >= 2 ? u2 : 0.f;
        inc[c] = x;
    }
    if (g == 3) *reinterpret_cast<float4 *>(&wtot[w16][4 * n]) = make_float4(inc[0], inc[1], inc[2], inc[3]);
}
__device__ __forceinline__ void scan_join(float (&inc)[4], float (&tot)[4], const float (*wtot)[HEAD], int w16, int n) {
    const int w0 = w16 & ~3, pos = w16 & 3;       // wavefront-uniform: the branches below are scalar
    const float4 t0 = *reinterpret_cast<const float4 *>(&wtot[w0][4 * n]), t1 = *reinterpret_cast<const float4 *>(&wtot[w0 + 1][4 * n]);
    const float4 t2 = *reinterpret_cast<const float4 *>(&wtot[w0 + 2][4 * n]), t3 = *reinterpret_cast<const float4 *>(&wtot[w0 + 3][4 * n]);
    const float a[4] = {t0.x + t1.x, t0.y + t1.y, t0.z + t1.z, t0.w + t1.w};
    tot[0] = a[0] + (t2.x + t3.x); tot[1] = a[1] + (t2.y + t3.y); tot[2] = a[2] + (t2.z + t3.z); tot[3] = a[3] + (t2.w + t3.w);
    if (pos == 1) {
        inc[0] += t0.x; inc[1] += t0.y; inc[2] += t0.z; inc[3] += t0.w;
        asm volatile("" ::: "memory");      // keeps the branch a branch (no select form with all the additions)
    } else if (pos == 2) {
        inc[0] += a[0]; inc[1] += a[1]; inc[2] += a[2]; inc[3] += a[3];
        asm volatile("" ::: "memory");
    } else if (pos == 3) {
        inc[0] += a[0] + t2.x; inc[1] += a[1] + t2.y; inc[2] += a[2] + t2.z; inc[3] += a[3] + t2.w;
        asm volatile("" ::: "memory");
    }
}

// -------------------------------------------------------------- summary passes --
// Time-parallel split.  One piece (`pps` steps) of a segment, from a zero state
// (gradient): what the piece does to a state handed in, X_out = decay o X_in + delta.
//   BACKWARD = false: state summary over pieces of the segments 0..nseg-2 (reads k, v, w):
//                     delta = sum over the piece's tokens s of (k_s e^{(decay from s to the piece's end)})^T v_s;
//   BACKWARD = true:  state-gradient summary over pieces of the segments 1..nseg-1 (reads r, gy, w):
//                     delta = sum over t of (r_t e^{(decay from the piece's start to t)})^T gy_t.
// The main kernels chain the pieces in their prologues (chain_state / chain_gradient).  Four wavefronts; wavefront w prepares block w of
// a step (lane = four consecutive tokens x four channels, 16 lanes = one 128-byte row, the
// running log decay inside the lane and two shuffles across) and owns value columns
// 16w..16w+15 of X.  Tiles are [token][channel]; the MFMA operands come out of the
// transposing LDS read.
//
// The steps of a piece are walked AWAY from the boundary the summary is for (the state pass from the piece's
// last step to its first, the gradient pass from its first to its last): a step's contribution T (its four
// blocks chained from zero) enters as  X += e^{R} o T  with R the log decay between the step and the boundary,
// which only grows in size.  Once e^{R} is below 2^-56 for every key, what is left of the piece cannot change
// X any more (fp32 keeps 24 bits) and the walk stops; the piece's decay is then reported as exactly 0, which
// tells whoever chains the summaries that nothing beyond this piece matters.  With a decay that forgets within
// a few hundred tokens every piece reads a few steps instead of all of its steps; with a decay close to 1
// nothing stops early and the pass costs what a full pass costs.
struct PassTiles {
    uint16_t a[SB * LD];      // forward: k e^{b-incl};  backward: r e^{excl}     [token][key]   bf16 head of the value
    uint16_t al[SB * LD];     //                                                                 bf16 remainder
    uint16_t b[SB * LD];      // forward: v;             backward: gy             [token][value]
    float dec[4][HEAD];       // e^{b} per block and key
    float tot[4][HEAD];       // b
    float fac[2][HEAD];       // e^{R} per key for this step / the next one
    int stop;
};
constexpr float PASS_CUT_LOG2 = -56.f;

template <bool PER_TOKEN_W, bool BACKWARD, bool W16>
__global__ __launch_bounds__(NT_F) void summary_pass(int bh0, int Tlen, int C, int H, int nseg, int sps, int m, int pps,
        const bf16 *__restrict__ a_in, const bf16 *__restrict__ b_in, const void *__restrict__ wraw,
        float *__restrict__ part, int floor_decay)
{
    __shared__ __align__(16) PassTiles sm;
    const int units = (nseg - 1) * m;       // workgroups per (batch, head)
    const int bh = bh0 + blockIdx.x / units, piece = (BACKWARD ? m : 0) + blockIdx.x % units, seg = piece / m, j = piece % m;
    const int b = bh / H, h = bh % H;
    const int tid = threadIdx.x, wv = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 4, n = lane & 15;
    {       // the streams of this (batch, head): from here on every address is a 32-bit offset into its sequence
        const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
        a_in += base; b_in += base;
        if (PER_TOKEN_W) wraw = W16 ? (const void *)(static_cast<const bf16 *>(wraw) + base) : (const void *)(static_cast<const float *>(wraw) + base);
    }
    const int nsb = (Tlen + SB - 1) / SB;
    const int sb0 = seg * sps + j * pps, sb1 = min(min(nsb, (seg + 1) * sps), sb0 + pps);
    const int nsteps = sb1 - sb0;

    // X[kk][e] = X[key 16kk+4g+e][value 16wv+n]
    f4 X[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) X[kk] = f4{0.f, 0.f, 0.f, 0.f};
    float R = 0.f;                          // wavefront 0, lane = key: log2 of the decay between the boundary and the next step
    // preparing role: tokens tok0..tok0+3 of the step (block wv), channels c4..c4+3
    const int c4 = 4 * n, tok0 = 16 * wv + 4 * g;
    float4 l_const = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!PER_TOKEN_W) {
        const float4 w4 = *reinterpret_cast<const float4 *>(static_cast<const float *>(wraw) + h * HEAD + c4);
        l_const = make_float4(log2_decay(w4.x, floor_decay), log2_decay(w4.y, floor_decay), log2_decay(w4.z, floor_decay),
                              log2_decay(w4.w, floor_decay));
    }
    uint2 pa[4], pb[4];
    WReg<W16> pw[4];
    auto fetch = [&](int sb) {
#pragma unroll
        for (int x = 0; x < 4; x++) {
            const int t = sb * SB + tok0 + x;
            if (t < Tlen) {
                const uint32_t o = (uint32_t)t * C + c4;
                pa[x] = *reinterpret_cast<const uint2 *>(seq_at(a_in, o));
                pb[x] = *reinterpret_cast<const uint2 *>(seq_at(b_in, o));
                pw[x] = PER_TOKEN_W ? WReg<W16>::load(wraw, o) : WReg<W16>::from(l_const);
            } else {
                pa[x] = pb[x] = make_uint2(0u, 0u);
                pw[x] = WReg<W16>::from(PER_TOKEN_W ? WKV_NEG_INF4 : make_float4(0.f, 0.f, 0.f, 0.f));
            }
        }
    };
    const int tro = tr_lane_offset(lane, LD);
    // the state pass walks back in time, the gradient pass forward
    auto step_at = [&](int it) { return BACKWARD ? sb0 + it : sb1 - 1 - it; };
    if (nsteps > 0) fetch(step_at(0));
    if (tid < HEAD) sm.fac[0][tid] = 1.f;
    if (tid == 0) sm.stop = 0;
    bool stopped = false;
    PT_DECL
    for (int it = 0; it < nsteps; it++) {
        const int par = it & 1;
        {
            float l[4][4], inc[4][4], run[4] = {0.f, 0.f, 0.f, 0.f}, tot[4];
#pragma unroll
            for (int x = 0; x < 4; x++) {
                const float4 pf = pw[x].f4();
                const float lw4[4] = {pf.x, pf.y, pf.z, pf.w};
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    l[x][c] = PER_TOKEN_W ? log2_decay(lw4[c], floor_decay) : lw4[c];
                    run[c] += l[x][c];
                    inc[x][c] = run[c];
                }
            }
#pragma unroll
            for (int c = 0; c < 4; c++) {          // the lanes g-1, g-2, g-3 hold the earlier tokens of the block
                float x = run[c];
                const float u1 = __shfl_up(x, 16);
                x += g >= 1 ? u1 : 0.f;
                const float u2 = __shfl_up(x, 32);
                x += g >= 2 ? u2 : 0.f;
                tot[c] = __shfl(x, lane | 48);
                run[c] = x - run[c];               // what comes before this lane's tokens
            }
#pragma unroll
            for (int x = 0; x < 4; x++) {
                const float af[4] = {bf_lo(pa[x].x), bf_hi(pa[x].x), bf_lo(pa[x].y), bf_hi(pa[x].y)};
                float sc[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const float ic = inc[x][c] + run[c];
                    sc[c] = af[c] * exp2_fast(BACKWARD ? ic - l[x][c] : tot[c] - ic);       // r e^{excl}  /  k e^{b-incl}
                }
                uint32_t h0, l0, h1, l1;
                const int o = (tok0 + x) * LD + c4;
                split2(sc[0], sc[1], h0, l0); split2(sc[2], sc[3], h1, l1);
                *reinterpret_cast<uint2 *>(&sm.a[o]) = make_uint2(h0, h1);
                *reinterpret_cast<uint2 *>(&sm.al[o]) = make_uint2(l0, l1);
                *reinterpret_cast<uint2 *>(&sm.b[o]) = pb[x];
            }
            if (g == 3) {
                *reinterpret_cast<float4 *>(&sm.tot[wv][c4]) = make_float4(tot[0], tot[1], tot[2], tot[3]);
                *reinterpret_cast<float4 *>(&sm.dec[wv][c4]) = make_float4(exp2_fast(tot[0]), exp2_fast(tot[1]), exp2_fast(tot[2]), exp2_fast(tot[3]));
            }
        }
        PT_MARK(0)
        lds_barrier();
        PT_MARK(1)
        if (it + 1 < nsteps) fetch(step_at(it + 1));          // next step's loads fly during the MFMA phase
        if (wv == 0) {      // lane = key: the decay up to the next step, and whether anything later can still matter
            R += (sm.tot[0][lane] + sm.tot[1][lane]) + (sm.tot[2][lane] + sm.tot[3][lane]);
            sm.fac[par ^ 1][lane] = exp2_fast(R);
            if (__builtin_amdgcn_ballot_w64(R >= PASS_CUT_LOG2) == 0 && lane == 0) sm.stop = 1;
        }
        PT_MARK(2)
        // the step's own contribution, its four blocks chained from zero (first to last going forward, last to first going back)
        f4 Tt[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int blk = BACKWARD ? 3 - i : i;
            const s4 b_op = frag_tr(sm.b, tro + (16 * blk) * LD + 16 * wv);
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                if (i == 0) {
                    Tt[kk] = f4{0.f, 0.f, 0.f, 0.f};
                } else {
                    const float4 d4 = *reinterpret_cast<const float4 *>(&sm.dec[blk][16 * kk + 4 * g]);
                    Tt[kk][0] *= d4.x; Tt[kk][1] *= d4.y; Tt[kk][2] *= d4.z; Tt[kk][3] *= d4.w;
                }
                Tt[kk] = mma2(frag_tr(sm.a, tro + (16 * blk) * LD + 16 * kk), frag_tr(sm.al, tro + (16 * blk) * LD + 16 * kk),
                              b_op, b_op, Tt[kk]);
            }
        }
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const float4 f = *reinterpret_cast<const float4 *>(&sm.fac[par][16 * kk + 4 * g]);
            X[kk][0] = fmaf(f.x, Tt[kk][0], X[kk][0]); X[kk][1] = fmaf(f.y, Tt[kk][1], X[kk][1]);
            X[kk][2] = fmaf(f.z, Tt[kk][2], X[kk][2]); X[kk][3] = fmaf(f.w, Tt[kk][3], X[kk][3]);
        }
        PT_MARK(3)
        lds_barrier();
        PT_MARK(4)
        if (sm.stop) { stopped = true; break; }
    }
    PT_PRINT_WAVES(BACKWARD ? "gradient summary" : "state summary")
    float *pp = part + ((size_t)bh * nseg * m + piece) * PART;
#pragma unroll
    for (int kk = 0; kk < 4; kk++)
#pragma unroll
        for (int e = 0; e < 4; e++) pp[(16 * kk + 4 * g + e) * HEAD + 16 * wv + n] = X[kk][e];
    if (wv == 0) pp[HEAD * HEAD + lane] = stopped ? 0.f : exp2_fast(R);
}

// Chaining the piece summaries, done by the main kernels for the state elements a lane holds.  A lane's
// elements are X[i] = X[key ki[i]][value vi[i]], i < N.
//   chain_state:    the state at the start of segment `seg` = the summaries of the pieces before it applied in
//                   order to the state handed in.  Walked from the nearest piece backwards,
//                       S = D_p + d_p o (D_{p-1} + d_{p-1} o ( ... + d_0 o S_in)),
//                   i.e. S = sum_q (prod_{q < q' <= p} d_q') o D_q, so that the walk ends as soon as the running product
//                   of the decays is 0 for all of the lane's keys (a piece that forgot everything reports exactly 0).
//   chain_gradient: the state gradient at the end of segment `seg`, from the pieces after it and the gradient handed in,
//                   walked forward in the same way.
// The summaries are read two pieces at a time, deltas and decays together, so that the common cases (the nearest piece
// forgot everything; two pieces per segment) take one round trip to memory.  ONE_KEY: all N elements share the key ki[0].
template <int N, bool ONE_KEY>
__device__ __forceinline__ void chain_summaries(float (&X)[N], const int (&ki)[N], const int (&vi)[N], const float *__restrict__ pieces,
                                                int first, int count, int dir, const float *__restrict__ ends) {
    constexpr int NK = ONE_KEY ? 1 : N;
    float run[NK];
#pragma unroll
    for (int i = 0; i < N; i++) X[i] = 0.f;
#pragma unroll
    for (int k = 0; k < NK; k++) run[k] = 1.f;
    bool alive = true;
    for (int x = 0; x < count && alive; x += 2) {
        float d[2][N], dc[2][NK];
#pragma unroll
        for (int bb = 0; bb < 2; bb++) {
            const float *q = pieces + (size_t)(first + dir * min(x + bb, count - 1)) * PART;
#pragma unroll
            for (int i = 0; i < N; i++) d[bb][i] = q[ki[i] * HEAD + vi[i]];
#pragma unroll
            for (int k = 0; k < NK; k++) dc[bb][k] = q[HEAD * HEAD + ki[k]];
        }
#pragma unroll
        for (int bb = 0; bb < 2; bb++) {
            if (x + bb < count && alive) {
                bool any = false;
#pragma unroll
                for (int i = 0; i < N; i++) X[i] = fmaf(run[ONE_KEY ? 0 : i], d[bb][i], X[i]);
#pragma unroll
                for (int k = 0; k < NK; k++) { run[k] *= dc[bb][k]; any |= run[k] != 0.f; }
                alive = any;
            }
        }
    }
    if (alive && ends) {
#pragma unroll
        for (int i = 0; i < N; i++) X[i] = fmaf(run[ONE_KEY ? 0 : i], ends[ki[i] * HEAD + vi[i]], X[i]);
    }
}

// ALL_WHOLE (time-invariant decay only): the sequence is a whole number of 64-token steps, so the general way of
// a step with missing tokens is left out of the kernel, and with it the registers it keeps alive across the loop.
template <bool PER_TOKEN_W, bool W16, bool ALL_WHOLE = false>
__global__ __launch_bounds__(NT_F16) void forward16(int bh0, int Tlen, int C, int H, int nseg, int sps, int m,
        const bf16 *__restrict__ r, const bf16 *__restrict__ k, const bf16 *__restrict__ v,
        const void *__restrict__ wraw, const float *__restrict__ u, const float *__restrict__ s_in,
        bf16 *__restrict__ y, float *__restrict__ s_out, float *__restrict__ ckpt, const float *__restrict__ part,
        int floor_decay)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Fwd16Tiles &sm = *reinterpret_cast<Fwd16Tiles *>(smem_raw);
    const int bh = bh0 + blockIdx.x / nseg, seg = blockIdx.x % nseg, b = bh / H, h = bh % H;
    const int tid = threadIdx.x, w16 = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 4, n = lane & 15;
    const int q = w16 >> 2, wv = w16 & 3;          // block and quarter for preparing and finishing
    const bool chain = w16 < 8;                    // the other eight build the intra-block matrices: block wv, key half (w16 >> 2) & 1
    const int hk = w16 >> 2;                       // chain wavefronts: key half
    {       // the streams of this (batch, head): from here on every address is a 32-bit offset into its sequence
        const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
        r += base; k += base; v += base; y += base;
        if (PER_TOKEN_W) wraw = W16 ? (const void *)(static_cast<const bf16 *>(wraw) + base) : (const void *)(static_cast<const float *>(wraw) + base);
    }
    const int nsb = (Tlen + SB - 1) / SB;
    const int sb0 = seg * sps, sb1 = min(nsb, (seg + 1) * sps);

    // chain wavefronts: S[j][e] = S[key 32hk+16j+4g+e][value 16wv+n]
    f4 S[2] = {f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}};
    if (chain) {
        if (seg == 0) {
            const float *sp = s_in + (size_t)bh * HEAD * HEAD;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) S[j][e] = sp[(32 * hk + 16 * j + 4 * g + e) * HEAD + 16 * wv + n];
        } else {      // the summaries of the pieces before this segment, chained onto the state handed in
            float X[8];
            int ki[8], vi[8];
#pragma unroll
            for (int i = 0; i < 8; i++) { ki[i] = 32 * hk + 16 * (i >> 2) + 4 * g + (i & 3); vi[i] = 16 * wv + n; }
            chain_summaries<8, false>(X, ki, vi, part + (size_t)bh * nseg * m * PART, seg * m - 1, seg * m, -1,
                               s_in + (size_t)bh * HEAD * HEAD);
#pragma unroll
            for (int i = 0; i < 8; i++) S[i >> 2][i & 3] = X[i];
        }
    }
    // preparing role: token tok of the step (block q), channels c4..c4+3
    const int c4 = 4 * n, tok = 4 * w16 + g;

    float4 l_const = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!PER_TOKEN_W) {
        const float4 w4 = *reinterpret_cast<const float4 *>(static_cast<const float *>(wraw) + h * HEAD + c4);
        l_const = make_float4(log2_decay(w4.x, floor_decay), log2_decay(w4.y, floor_decay), log2_decay(w4.z, floor_decay),
                              log2_decay(w4.w, floor_decay));
    }
    // the inputs of this lane's token, fetched two steps ahead into two register sets used in turn
    struct Row { uint2 r, k, v; WReg<W16> w; };
    Row rowA, rowB;
    auto fetch = [&](int sb, Row &x) __attribute__((always_inline)) {
        const int t = sb * SB + tok;
        if (t < Tlen) {
            const uint32_t o = (uint32_t)t * C + c4;
            x.r = *reinterpret_cast<const uint2 *>(seq_at(r, o));
            x.k = *reinterpret_cast<const uint2 *>(seq_at(k, o));
            x.v = *reinterpret_cast<const uint2 *>(seq_at(v, o));
            x.w = PER_TOKEN_W ? WReg<W16>::load(wraw, o) : WReg<W16>::from(l_const);
        } else {
            x.r = x.k = x.v = make_uint2(0u, 0u);
            x.w = WReg<W16>::from(PER_TOKEN_W ? WKV_NEG_INF4 : make_float4(0.f, 0.f, 0.f, 0.f));
        }
    };
    const int tro = tr_lane_offset(lane, LD);
    // the slot of this wavefront's two state tiles in a checkpoint (accumulator layout)
    const size_t ck_off = (size_t)bh * (nsb + 1) * HEAD * HEAD;

    bool have_y = false;
    fetch(sb0, rowA);
    if (sb0 + 1 < sb1) fetch(sb0 + 1, rowB);
    // log w of this lane's token and its running sum inside the wavefront, always one step ahead (see scan_local)
    float lc[4], ic[4];
    auto scan_ahead = [&](const WReg<W16> &pwr) __attribute__((always_inline)) {
        const float4 pw = pwr.f4();
        lc[0] = pw.x; lc[1] = pw.y; lc[2] = pw.z; lc[3] = pw.w;
        if (PER_TOKEN_W) {
#pragma unroll
            for (int c = 0; c < 4; c++) lc[c] = log2_decay(lc[c], floor_decay);
        }
        scan_local(lc, ic, sm.wtot, w16, g, n);
    };
    // Time-invariant decay (WKV5): in a step with all 64 tokens present the scaling factors depend only on the
    // token's place p in its block, e^{excl} = w^p and e^{b-incl} = w^(15-p), and the block's decay is w^16: a lane
    // keeps its eight factors for the whole kernel and needs no running sum and no exponential per step.
    float Fr[4] = {1.f, 1.f, 1.f, 1.f}, Fk[4] = {1.f, 1.f, 1.f, 1.f};
    if (!PER_TOKEN_W) {
        const float lcst[4] = {l_const.x, l_const.y, l_const.z, l_const.w};
        const int pl = tok & 15;
#pragma unroll
        for (int c = 0; c < 4; c++) { Fr[c] = exp2_fast(pl * lcst[c]); Fk[c] = exp2_fast((15 - pl) * lcst[c]); }
        if (pl == 15) {
            *reinterpret_cast<float4 *>(&sm.dec[q][c4]) = make_float4(exp2_fast(16.f * lcst[0]), exp2_fast(16.f * lcst[1]), exp2_fast(16.f * lcst[2]), exp2_fast(16.f * lcst[3]));
            *reinterpret_cast<float4 *>(&sm.ent[q][c4]) = make_float4(exp2_fast(-16.f * lcst[0]), exp2_fast(-16.f * lcst[1]), exp2_fast(-16.f * lcst[2]), exp2_fast(-16.f * lcst[3]));
        }
    }
    auto whole_step = [&](int sb) { return ALL_WHOLE ? true : !PER_TOKEN_W && (sb + 1) * SB <= Tlen; };       // scalar
#pragma unroll
    for (int c = 0; c < 4; c++) lc[c] = ic[c] = 0.f;
    if (!whole_step(sb0)) scan_ahead(rowA.w);
    lds_barrier();
    PT_DECL
    // one step; `cur` holds its inputs (and takes those of the step after the next), `nxt` those of the next step
    auto do_step = [&](const int sb, Row &cur, const Row &nxt) __attribute__((always_inline)) {
        const uint2 pr = cur.r, pk = cur.k, pv = cur.v;
        PT_MARK(5)
        // ---------------- prepare the scaled operands of this lane's token
        {
            float l[4] = {lc[0], lc[1], lc[2], lc[3]}, inc[4] = {ic[0], ic[1], ic[2], ic[3]}, tot[4];
            const float rf[4] = {bf_lo(pr.x), bf_hi(pr.x), bf_lo(pr.y), bf_hi(pr.y)};
            const float kf[4] = {bf_lo(pk.x), bf_hi(pk.x), bf_lo(pk.y), bf_hi(pk.y)};
            const float4 u4 = *reinterpret_cast<const float4 *>(u + h * HEAD + c4);
            const float uf[4] = {u4.x, u4.y, u4.z, u4.w};
            if (have_y) {      // y of the previous step waits in the rh tile: out as full rows, by the lanes that overwrite it next
                const int t = (sb - 1) * SB + tok;
                if (t < Tlen) store_row(seq_at(y, (uint32_t)t * C + c4), *reinterpret_cast<const uint2 *>(&sm.rh[tok * LD + c4]));
            }
            const bool whole = whole_step(sb);
            float rhv[4], khv[4], p = 0.f;
            if (whole) {
#pragma unroll
                for (int c = 0; c < 4; c++) { rhv[c] = rf[c] * Fr[c]; khv[c] = kf[c] * Fk[c]; }
            } else {
                scan_join(inc, tot, sm.wtot, w16, n);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    rhv[c] = rf[c] * exp2_fast(inc[c] - l[c]);
                    khv[c] = kf[c] * exp2_fast(tot[c] - inc[c]);
                }
            }
#pragma unroll
            for (int c = 0; c < 4; c++) p = fmaf(rf[c] * uf[c], kf[c], p);
            uint32_t h0, l0, h1, l1;
            const int o = tok * LD + c4, ot = tok * LD + c4;
            split2(rhv[0], rhv[1], h0, l0); split2(rhv[2], rhv[3], h1, l1);
            *reinterpret_cast<uint2 *>(&sm.rh[o]) = make_uint2(h0, h1);
            *reinterpret_cast<uint2 *>(&sm.rhl[o]) = make_uint2(l0, l1);
            split2(khv[0], khv[1], h0, l0); split2(khv[2], khv[3], h1, l1);
            *reinterpret_cast<uint2 *>(&sm.kh[ot]) = make_uint2(h0, h1);
            *reinterpret_cast<uint2 *>(&sm.khl[ot]) = make_uint2(l0, l1);
            *reinterpret_cast<uint2 *>(&sm.v[ot]) = pv;
            if (!whole && (w16 & 3) == 3) {       // wavefront-uniform: only the wavefront with the block's last token
                if (g == 3) {
                    *reinterpret_cast<float4 *>(&sm.dec[q][c4]) = make_float4(exp2_fast(tot[0]), exp2_fast(tot[1]), exp2_fast(tot[2]), exp2_fast(tot[3]));
                    *reinterpret_cast<float4 *>(&sm.ent[q][c4]) = make_float4(exp2_fast(-tot[0]), exp2_fast(-tot[1]), exp2_fast(-tot[2]), exp2_fast(-tot[3]));
                }
            }
            p = row_prefix_sum(p);           // lane 15 of the row ends with the sum over the 64 channels
            if (n == 15) sm.rho[tok] = p;
        }
        PT_MARK(0)
        lds_barrier();
        PT_MARK(1)
        if (sb + 2 < sb1) fetch(sb + 2, cur);     // these loads have two steps to arrive

        if (chain) {
            if (ckpt) {       // state at the start of this step, 16 bytes per lane and tile
                float4 *cp = reinterpret_cast<float4 *>(ckpt + ck_off + (size_t)sb * HEAD * HEAD) + (wv * 4 + 2 * hk) * 64 + lane;
                cp[0] = make_float4(S[0][0], S[0][1], S[0][2], S[0][3]);
                cp[64] = make_float4(S[1][0], S[1][1], S[1][2], S[1][3]);
            }
            // ---------------- the state over the four blocks; per block this half's share of rh S
#pragma unroll
            for (int blk = 0; blk < 4; blk++) {
                const int row = 16 * blk + n, ca = 32 * hk + 4 * g, cb = ca + 16;
                s4 s0h, s0l, s1h, s1l;
                split4(S[0], s0h, s0l);
                split4(S[1], s1h, s1l);
                const s4 r0 = frag(sm.rh, row, ca), r1 = frag(sm.rh, row, cb);
                const s4 r0l = frag(sm.rhl, row, ca), r1l = frag(sm.rhl, row, cb);
                f4 y0 = {0.f, 0.f, 0.f, 0.f}, y1 = y0, y2 = y0;
                y2 = mma2(r0l, r1l, s0h, s1h, y2);
                y0 = mma2(r0, r1, s0h, s1h, y0);
                y1 = mma2(r0, r1, s0l, s1l, y1);
                // S <- e^{b} o S + (k e^{b-incl})^T v
                const s4 v_op = frag_tr(sm.v, tro + (16 * blk) * LD + 16 * wv);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const float4 d4 = *reinterpret_cast<const float4 *>(&sm.dec[blk][32 * hk + 16 * j + 4 * g]);
                    S[j][0] *= d4.x; S[j][1] *= d4.y; S[j][2] *= d4.z; S[j][3] *= d4.w;
                    S[j] = mma2(frag_tr(sm.kh, tro + (16 * blk) * LD + 32 * hk + 16 * j),
                                frag_tr(sm.khl, tro + (16 * blk) * LD + 32 * hk + 16 * j), v_op, v_op, S[j]);
                }
                y0 += y1 + y2;
                sm.yi[hk][blk][wv][lane] = make_float4(y0[0], y0[1], y0[2], y0[3]);
            }
        } else {
            // ---------------- the masked intra-block matrix of block wv, once for everybody, as the sum of two
            // matrices (one per half of the keys, each by its own wavefront):
            // A^T[s][t] = sum_i (k e^{b-incl})[s][i] (r e^{excl-b})[t][i]; lane gets s = 4g+e, t = n
            const int row = 16 * wv + n, kh2 = (w16 >> 2) & 1;
            f4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0, a2 = a0;
            const int ca = 32 * kh2 + 4 * g, cb = ca + 16;
            // every LDS operand first, in one batch: a fetch issued where it is used costs the phase its latency
            const s4 k0 = frag(sm.kh, row, ca), k1 = frag(sm.kh, row, cb), k0l = frag(sm.khl, row, ca), k1l = frag(sm.khl, row, cb);
            const s4 ra = frag(sm.rh, row, ca), ral = frag(sm.rhl, row, ca), rb = frag(sm.rh, row, cb), rbl = frag(sm.rhl, row, cb);
            const float4 ea = *reinterpret_cast<const float4 *>(&sm.ent[wv][ca]), eb = *reinterpret_cast<const float4 *>(&sm.ent[wv][cb]);
            const float rho_t = kh2 ? 0.f : sm.rho[row];       // the diagonal goes with the first half
            __builtin_amdgcn_sched_barrier(0);
            {
                s4 r0, r1, r0l, r1l;
                scale_split(ra, ral, ea, n == 0, r0, r0l);
                scale_split(rb, rbl, eb, n == 0, r1, r1l);
                a0 = mma2(k0, k1, r0, r1, a0);
                a1 = mma2(k0l, k1l, r0, r1, a1);
                a2 = mma2(k0, k1, r0l, r1l, a2);
            }
            f4 at = a0 + (a1 + a2);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int s_ = 4 * g + e;
                at[e] = s_ < n ? at[e] : (s_ == n ? rho_t : 0.f);
            }
            uint32_t h0, l0, h1, l1;                        // A[t = n][s = 4g..4g+3] as head + remainder
            split2(at[0], at[1], h0, l0);
            split2(at[2], at[3], h1, l1);
            sm.amat[kh2][wv][lane] = make_uint4(h0, h1, l0, l1);
        }
        PT_MARK(2)
        lds_barrier();
        PT_MARK(3)

        // ---------------- y of block q, value columns 16wv..16wv+15
        if (y) {
            const float4 ya = sm.yi[0][q][wv][lane], yb = sm.yi[1][q][wv][lane];
            const uint4 am = sm.amat[0][q][lane], am2 = sm.amat[1][q][lane];
            const s4 v_op = frag_tr(sm.v, tro + (16 * q) * LD + 16 * wv);
            f4 yt = {ya.x + yb.x, ya.y + yb.y, ya.z + yb.z, ya.w + yb.w};
            yt = mma2(as_s4(am.x, am.y), as_s4(am.z, am.w), v_op, v_op, yt);
            yt = mma2(as_s4(am2.x, am2.y), as_s4(am2.z, am2.w), v_op, v_op, yt);
            // into the rh tile (nobody reads it any more in this step), [token][value]; it leaves as full rows
#pragma unroll
            for (int e = 0; e < 4; e++) sm.rh[(16 * q + 4 * g + e) * LD + 16 * wv + n] = bf16_bits(yt[e]);
        }
        if (sb + 1 < sb1 && !whole_step(sb + 1)) scan_ahead(nxt.w);
        PT_MARK(4)
        lds_barrier();
        have_y = y != nullptr;
    };
    for (int sb = sb0; sb < sb1; sb += 2) {
        do_step(sb, rowA, rowB);
        if (sb + 1 < sb1) do_step(sb + 1, rowB, rowA);
    }
    if (have_y) {
        const int t = (sb1 - 1) * SB + tok;
        if (t < Tlen) store_row(seq_at(y, (uint32_t)t * C + c4), *reinterpret_cast<const uint2 *>(&sm.rh[tok * LD + c4]));
    }
    PT_PRINT("fwd16")
    if (chain && seg == nseg - 1) {
        if (ckpt) {       // the final state takes the slot after the last step
            float4 *cp = reinterpret_cast<float4 *>(ckpt + ck_off + (size_t)nsb * HEAD * HEAD) + (wv * 4 + 2 * hk) * 64 + lane;
            cp[0] = make_float4(S[0][0], S[0][1], S[0][2], S[0][3]);
            cp[64] = make_float4(S[1][0], S[1][1], S[1][2], S[1][3]);
        }
        if (s_out) {
            float *op = s_out + (size_t)bh * HEAD * HEAD;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) op[(32 * hk + 16 * j + 4 * g + e) * HEAD + 16 * wv + n] = S[j][e];
        }
    }
}

// ------------------------------------------------------ backward, 16 wavefronts --
// Walks the 64-token steps of a segment from the last to the first.  With S the state
// at a block's start, G the gradient of the state at a block's end, P[t][s] = gy_t . v_s,
// rh = r e^{excl}, kh = k e^{b-incl}:
//
//   gr_t = e^{excl_t} (gy_t S^T) + e^{excl_t-b} sum_{s<t} P[t][s] kh_s + u k_t P[t][t]
//   gk_s = e^{-incl_s} sum_{t>s} P[t][s] rh_t + e^{b-incl_s} (v_s G^T) + u r_s P[s][s]
//   gv_s = sum_{t>=s} A~[t][s] gy_t + kh_s G          (A~ = the forward's masked matrix)
//   G   <- e^{b} o G + rh^T gy
//
// and the decay gradient from the running sum  A_{t-1} = A_t + r_t gr_t - k_t gk_t,
// dL/dlog w_t = A_t - k_t (gk_t - u r_t P[t][t]).
//
// The work of a step is spread over 16 wavefronts (four per SIMD) so that no single
// wavefront's instruction stream is the critical path.  A step runs in three phases
// separated by workgroup barriers:
//
//   prepare   all wavefronts: lane = (one token, four channels), 16 lanes = one 128-byte
//             row of the inputs; every tile is [token][channel]; fragments with the tokens
//             along the contraction come from the transposing LDS read.
//   chains    wavefronts  0-3  walk the state forward from the step's checkpoint and
//                              leave  Q1 = gy S^T  of each block in LDS;
//             wavefronts  4-7  walk the state gradient backward (value-major copy) and
//                              leave  Q4 = v G^T;
//             wavefronts  8-11 walk the key-major copy and keep  kh G  in registers;
//             wavefronts 12-15 build, per block, the masked matrices P, P^T and A~ once
//                              for everybody.
//   blocks    wavefront (q, w): gr, gk and the decay gradient of block q, keys
//             16w..16w+15; wavefronts 8-11 also finish gv.
//
// Results go back into LDS tiles that are no longer read ([token][channel]) and leave
// as full rows at the start of the next step, written by the lanes that overwrite them.
//
// The running sum of the decay gradient is anchored once per segment (at the segment's
// end, from the state checkpoint there and the gradient handed in: sum_j G o S) and
// carried from step to step in LDS; inside a step every block sums its own tokens and
// the blocks are joined through LDS.
struct Bwd16Tiles {
    uint16_t gy[SB * LD];    // gy              [token][value]
    uint16_t v[SB * LD];     // v               [token][value]
    uint16_t rh[SB * LD];    // r e^{excl}      [token][key]   head / remainder
    uint16_t rhl[SB * LD];
    uint16_t kh[SB * LD];    // k e^{b-incl}    [token][key]
    uint16_t khl[SB * LD];
    float incl[SB * HEAD];   // inclusive running log decay inside the block [token][key]; after the block phase the inside-block part of the decay gradient
    float lw[SB * HEAD];     // log w                                         [token][key]
    uint32_t rk[SB * HEAD];  // r and k as they came (bf16 pair: r low, k high)                 [token][key]
    float tot[4][HEAD];      // b per block and key
    float dec[4][HEAD];      // e^{b}
    float ent[4][HEAD];      // e^{-b}
    float rho[SB];           // r . (u o k) per token
    float ub[HEAD];
    float wtot[16][HEAD];    // per wavefront (four tokens) and channel: sum of log w, for the block-wide running sum
    float q1[SB * HEAD];     // gy S^T          [token][key]
    float q4[SB * HEAD];     // v G^T           [token][key]
    uint4 pfr[4][2][64];     // per block: P^T masked to s < t, P masked to t > s, as A-operand fragments (head, remainder)
    float pdiag[4][16];      // P[t][t]
    uint4 amat[4][64];       // A~ masked to t >= s (diagonal r.(u o k)), A-operand fragments (head, remainder)
    float tots[4][HEAD];     // per block and key: sum over the block's tokens of r gr - k gk
    float arun[2][HEAD];     // the running sum of the decay gradient at the end of a step (two copies, used in turn)
    float red[4][HEAD];      // gu partial sums of the four block groups
    float4 kg3[4][64];       // kh G of the step's last block, parked here by wavefronts 8-11 (they are short of registers)
};
constexpr int NT_B16 = 1024;
// Re-derives the lane-dependent indices from an opaque copy of the lane id, so that the
// address arithmetic of a phase stays inside the phase instead of being hoisted out of the
// step loop into registers that live (and spill) across the whole kernel.
#define WKV_LOCAL_LANE                                                                                        \
    int lane_v_ = lane0;                                                                                      \
    asm volatile("" : "+v"(lane_v_));                                                                         \
    const int lane = lane_v_, g = lane >> 4, n = lane & 15, own = 16 * wv + n, c4 = 4 * n,                     \
              tok = 4 * w16 + g, tro = tr_lane_offset(lane, LD);                                              \
    (void)tro; (void)c4; (void)tok; (void)own;

template <bool PER_TOKEN_W, bool W16, bool ALL_WHOLE = false>
__global__ __launch_bounds__(NT_B16) void backward16(int bh0, int Tlen, int C, int H, int nseg, int sps, int m,
        const bf16 *__restrict__ r, const bf16 *__restrict__ k, const bf16 *__restrict__ v,
        const void *__restrict__ wraw, const float *__restrict__ u, const bf16 *__restrict__ gy,
        const float *__restrict__ gs_out, const float *__restrict__ ckpt, const float *__restrict__ gpart,
        bf16 *__restrict__ gr, bf16 *__restrict__ gk, bf16 *__restrict__ gv, void *__restrict__ gw_tok,
        float *__restrict__ gw_part, float *__restrict__ gu_part, float *__restrict__ gs_in, int floor_decay)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Bwd16Tiles &sm = *reinterpret_cast<Bwd16Tiles *>(smem_raw);
    const int bh = bh0 + blockIdx.x / nseg, seg = blockIdx.x % nseg, b = bh / H, h = bh % H;
    const int tid = threadIdx.x, w16 = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 4, n = lane & 15;
    const int role = w16 >> 2, q = role, wv = w16 & 3;      // chain role; block (for preparing and for the block phase); quarter
    {       // the streams of this (batch, head): from here on every address is a 32-bit offset into its sequence
        const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
        r += base; k += base; v += base; gy += base; gr += base; gk += base; gv += base;
        if (PER_TOKEN_W) {
            wraw = W16 ? (const void *)(static_cast<const bf16 *>(wraw) + base) : (const void *)(static_cast<const float *>(wraw) + base);
            gw_tok = W16 ? (void *)(static_cast<bf16 *>(gw_tok) + base) : (void *)(static_cast<float *>(gw_tok) + base);
        }
    }
    const int nsb = (Tlen + SB - 1) / SB;
    const int sb0 = seg * sps, sb1 = min(nsb, (seg + 1) * sps);
    const int own = 16 * wv + n;               // key (or, for the key-major gradient, value) channel of this lane
    const float *ck_lane = ckpt + (size_t)bh * (nsb + 1) * HEAD * HEAD + (wv * 64 + 16 * (n >> 2) + 4 * g) * 4 + (n & 3);

    // One register tile set per wavefront, by role:
    //   wavefronts 0-3:   the state,   G[kk][e] = S[key own][value 16kk+4g+e]  (reloaded from the checkpoint every step)
    //   wavefronts 4-7:   its gradient, G[kk][e] = G[key own][value 16kk+4g+e]
    //   wavefronts 8-11:  its gradient, G[kk][e] = G[key 16kk+4g+e][value own]
    f4 G[4] = {f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}};
    {
        // the last segment starts from gs_out, an earlier one from the summaries of the pieces after it chained onto gs_out
        float X[16];
        bool have = false;
        if (role < 3) {
            if (seg == nseg - 1) {
                have = gs_out != nullptr;
                if (have) {
                    const float *gp = gs_out + (size_t)bh * HEAD * HEAD;
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int x = 16 * (i >> 2) + 4 * g + (i & 3);
                        X[i] = role == 2 ? gp[x * HEAD + own] : gp[own * HEAD + x];
                    }
                }
            } else if (role == 1) {      // the summaries are read and chained once, by the value-major wavefronts
                int ki[16], vi[16];
#pragma unroll
                for (int i = 0; i < 16; i++) { ki[i] = own; vi[i] = 16 * (i >> 2) + 4 * g + (i & 3); }
                const float *pcs = gpart + (size_t)bh * nseg * m * PART, *ends = gs_out ? gs_out + (size_t)bh * HEAD * HEAD : nullptr;
                chain_summaries<16, true>(X, ki, vi, pcs, (seg + 1) * m, (nseg - 1 - seg) * m, 1, ends);
#pragma unroll
                for (int i = 0; i < 16; i++) sm.q1[swz(own, vi[i])] = X[i];      // (the table is not in use yet)
            }
        }
        if (seg != nseg - 1) {           // ... and handed to the other two roles through LDS, each in its own layout
            lds_barrier();
            if (role == 0 || role == 2) {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int x = 16 * (i >> 2) + 4 * g + (i & 3);
                    X[i] = role == 2 ? sm.q1[swz(x, own)] : sm.q1[swz(own, x)];
                }
            }
            have = role < 3;
        }
        if (have && (role == 1 || role == 2)) {
#pragma unroll
            for (int i = 0; i < 16; i++) G[i >> 2][i & 3] = X[i];
        }
        if (role == 0) {       // anchor of the decay-gradient sum at the segment's end: sum_j G o S
            float a = 0.f;
            if (have) {
                const float *cp = ck_lane + (size_t)sb1 * HEAD * HEAD;
#pragma unroll
                for (int i = 0; i < 16; i++) a = fmaf(X[i], cp[(i >> 2) * 1024 + (i & 3) * 4], a);
            }
            a = group_sum4(a);
            if (g == 0) sm.arun[0][own] = a;
        }
    }
    float gu_acc[4] = {0.f, 0.f, 0.f, 0.f};      // block phase: this lane's token, keys 16wv+4g..+3
    const float4 u4 = *reinterpret_cast<const float4 *>(u + h * HEAD + 16 * wv + 4 * g);      // the bonus of those keys
    // Time-invariant w: its gradient is the SUM over tokens of dL/dlog w_t = A_t - z_t, A_t = A(segment end) + sum_{s>t} c_s,
    // and  sum_t A_t = (tokens) A(segment end) + sum_s (tokens before s) c_s:  no running sum, no per-token values, just
    // one weighted sum per lane (block phase: this lane's token, keys 16wv+4g..+3).
    float gw_acc[4] = {0.f, 0.f, 0.f, 0.f};

    // preparing role: token tok of the step (block q), channels c4..c4+3 (one 128-byte row per 16 lanes)
    const int c4 = 4 * n, tok = 4 * w16 + g;

    bool have_out = false;
    uint2 pr, pk, pv, pg;
    WReg<W16> pw = WReg<W16>::from(make_float4(0.f, 0.f, 0.f, 0.f));      // per-token decay only (the time-invariant one is read where it is used)
    auto fetch = [&](int sb, int tok, int c4) {       // (tok, c4 handed in: see WKV_LOCAL_LANE)
        const int t = sb * SB + tok;
        if (t < Tlen) {
            const uint32_t o = (uint32_t)t * C + c4;
            pr = *reinterpret_cast<const uint2 *>(seq_at(r, o));
            pk = *reinterpret_cast<const uint2 *>(seq_at(k, o));
            pv = *reinterpret_cast<const uint2 *>(seq_at(v, o));
            pg = *reinterpret_cast<const uint2 *>(seq_at(gy, o));
            if (PER_TOKEN_W) pw = WReg<W16>::load(wraw, o);
        } else {
            pr = pk = pv = pg = make_uint2(0u, 0u);
            if (PER_TOKEN_W) pw = WReg<W16>::from(WKV_NEG_INF4);
        }
    };
    // the same without a branch (the token clamped into the sequence): for the fetches inside the step loop, whose steps
    // are whole; a wait the compiler places after a conditional load is counted for the path without it
    auto fetch_whole = [&](int sb, int tok, int c4) {
        const int t = min(sb * SB + tok, Tlen - 1);
        const uint32_t o = (uint32_t)t * C + c4;
        pr = *reinterpret_cast<const uint2 *>(seq_at(r, o));
        pk = *reinterpret_cast<const uint2 *>(seq_at(k, o));
        pv = *reinterpret_cast<const uint2 *>(seq_at(v, o));
        pg = *reinterpret_cast<const uint2 *>(seq_at(gy, o));
        if (PER_TOKEN_W) pw = WReg<W16>::load_in_halves(wraw, o);
    };
    const int lane0 = lane;
    // gr, gk, gv of a finished step wait in the rh, kh, v tiles, [token][channel]; they leave as full rows, written
    // by the lanes that overwrite those entries next.  The decay gradient is finished on the way out:
    //   dL/dlog w_t = (running sum at the end of the token's block) + (inside-block part, waiting in the incl table),
    // the first being the sum at the step's end (arun[par]) plus the totals of the step's later blocks.
    auto write_out = [&](int sb, int tok, int c4, int par) {
        const int t = sb * SB + tok;
        if (!PER_TOKEN_W) {         // nothing per token to finish: gr, gk, gv only
            if (t < Tlen) {
                const uint32_t o = (uint32_t)t * C + c4;
                store_row(seq_at(gr, o), *reinterpret_cast<const uint2 *>(&sm.rh[tok * LD + c4]));
                store_row(seq_at(gk, o), *reinterpret_cast<const uint2 *>(&sm.kh[tok * LD + c4]));
                store_row(seq_at(gv, o), *reinterpret_cast<const uint2 *>(&sm.v[tok * LD + c4]));
            }
            return;
        }
        float4 A = *reinterpret_cast<const float4 *>(&sm.arun[par][c4]);
        const float4 t1 = *reinterpret_cast<const float4 *>(&sm.tots[1][c4]), t2 = *reinterpret_cast<const float4 *>(&sm.tots[2][c4]);
        const float4 t3 = *reinterpret_cast<const float4 *>(&sm.tots[3][c4]);
        if (w16 == 0) {             // wavefront-uniform
            if (tok == 0) {         // the sum at the end of the step before (in time): into the other copy
                const float4 t0 = *reinterpret_cast<const float4 *>(&sm.tots[0][c4]);
                *reinterpret_cast<float4 *>(&sm.arun[par ^ 1][c4]) =
                    make_float4(A.x + ((t0.x + t1.x) + (t2.x + t3.x)), A.y + ((t0.y + t1.y) + (t2.y + t3.y)),
                                A.z + ((t0.z + t1.z) + (t2.z + t3.z)), A.w + ((t0.w + t1.w) + (t2.w + t3.w)));
            }
        }
        if (q < 3) { A.x += t3.x; A.y += t3.y; A.z += t3.z; A.w += t3.w; }
        if (q < 2) { A.x += t2.x; A.y += t2.y; A.z += t2.z; A.w += t2.w; }
        if (q < 1) { A.x += t1.x; A.y += t1.y; A.z += t1.z; A.w += t1.w; }
        const float4 D = *reinterpret_cast<const float4 *>(&sm.incl[swz(tok, c4)]);
        A.x += D.x; A.y += D.y; A.z += D.z; A.w += D.w;
        if (t < Tlen) {
            const uint32_t o = (uint32_t)t * C + c4;
            store_row(seq_at(gr, o), *reinterpret_cast<const uint2 *>(&sm.rh[tok * LD + c4]));
            store_row(seq_at(gk, o), *reinterpret_cast<const uint2 *>(&sm.kh[tok * LD + c4]));
            store_row(seq_at(gv, o), *reinterpret_cast<const uint2 *>(&sm.v[tok * LD + c4]));
            {                       // dL/dw_raw = dL/dlog w x log w (natural logarithm); nothing where the floor holds
                const float4 l4 = *reinterpret_cast<const float4 *>(&sm.lw[swz(tok, c4)]);
                const float lf[4] = {l4.x, l4.y, l4.z, l4.w};
                float f[4];
#pragma unroll
                for (int c = 0; c < 4; c++) f[c] = (floor_decay && lf[c] <= LOG2_W_FLOOR) ? 0.f : lf[c] * LN2;
                const float gw4[4] = {A.x * f[0], A.y * f[1], A.z * f[2], A.w * f[3]};
                if (W16) store_row(seq_at(static_cast<bf16 *>(gw_tok), o), gw4);
                else store_row(seq_at(static_cast<float *>(gw_tok), o), gw4);
            }
        }
    };
    int par = 0;

    // Time-invariant decay (WKV5): in a step with all 64 tokens present the scaling factors depend only on the
    // token's place p in its block, e^{excl} = w^p and e^{b-incl} = w^(15-p), and every block decays by w^16.  They
    // are kept as two [16][64] tables in the (then unused) log w table; such a step needs no running sum, no
    // exponential and one barrier less.  A step with missing tokens (the last of the sequence) takes the general way
    // and overwrites the tables.
    float *const tab_r = sm.lw, *const tab_k = sm.lw + 16 * HEAD;
    bool tables_valid = false;
    auto whole_step = [&](int sb) { return ALL_WHOLE ? true : !PER_TOKEN_W && (sb + 1) * SB <= Tlen; };       // scalar

    fetch(sb1 - 1, tok, c4);
    if (tid < HEAD) sm.ub[tid] = u[h * HEAD + tid];
    lds_barrier();
    PT_DECL
    for (int sb = sb1 - 1; sb >= sb0; sb--) {
      PT_MARK(5)
      const bool whole = whole_step(sb);
      if (whole && !tables_valid) {
          const int key = tid & 63, pl = tid >> 6;
          const float lk = log2_decay(static_cast<const float *>(wraw)[h * HEAD + key], floor_decay);
          tab_r[swz(pl, key)] = exp2_fast(pl * lk);
          tab_k[swz(pl, key)] = exp2_fast((15 - pl) * lk);
          if (pl < 4) {
              sm.tot[pl][key] = 16.f * lk;
              sm.dec[pl][key] = exp2_fast(16.f * lk);
              sm.ent[pl][key] = exp2_fast(-16.f * lk);
          }
          tables_valid = true;
          lds_barrier();
      }
      if (!whole) tables_valid = false;
      {
        WKV_LOCAL_LANE
        needed_here(pr); needed_here(pk); needed_here(pv); needed_here(pg);
        if (PER_TOKEN_W) needed_here(pw.v);
        // the step's checkpoint: loads issued now are back when the chains start
        if (role == 0) {
            const float *ck_lane = ckpt + (size_t)bh * (nsb + 1) * HEAD * HEAD + (wv * 64 + 16 * (n >> 2) + 4 * g) * 4 + (n & 3);
            const float *cp = ck_lane + (size_t)sb * HEAD * HEAD;
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
#pragma unroll
                for (int e = 0; e < 4; e++) G[kk][e] = cp[kk * 1024 + e * 4];
        }
        // ---------------- prepare the operands of this lane's token
        {
            const float4 pf = pw.f4();
            float l[4] = {pf.x, pf.y, pf.z, pf.w}, inc[4], tot[4];
            const float rf[4] = {bf_lo(pr.x), bf_hi(pr.x), bf_lo(pr.y), bf_hi(pr.y)};
            const float kf[4] = {bf_lo(pk.x), bf_hi(pk.x), bf_lo(pk.y), bf_hi(pk.y)};
            const float4 u4 = *reinterpret_cast<const float4 *>(&sm.ub[c4]);
            const float uf[4] = {u4.x, u4.y, u4.z, u4.w};
            if (PER_TOKEN_W) {
#pragma unroll
                for (int c = 0; c < 4; c++) l[c] = log2_decay(l[c], floor_decay);
            } else if (!whole) {       // a step with missing tokens: they count as w = 1
                const float4 w4 = *reinterpret_cast<const float4 *>(static_cast<const float *>(wraw) + h * HEAD + c4);
                const bool in = sb * SB + tok < Tlen;
                l[0] = in ? log2_decay(w4.x, floor_decay) : 0.f; l[1] = in ? log2_decay(w4.y, floor_decay) : 0.f;
                l[2] = in ? log2_decay(w4.z, floor_decay) : 0.f; l[3] = in ? log2_decay(w4.w, floor_decay) : 0.f;
            }
            PT_MARK(5)
            if (have_out) { write_out(sb + 1, tok, c4, par); par ^= 1; }
            PT_MARK(6)
            float rhv[4], khv[4], p = 0.f;
            if (whole) {
                const float4 fr = *reinterpret_cast<const float4 *>(&tab_r[swz(tok & 15, c4)]);
                const float4 fk = *reinterpret_cast<const float4 *>(&tab_k[swz(tok & 15, c4)]);
                rhv[0] = rf[0] * fr.x; rhv[1] = rf[1] * fr.y; rhv[2] = rf[2] * fr.z; rhv[3] = rf[3] * fr.w;
                khv[0] = kf[0] * fk.x; khv[1] = kf[1] * fk.y; khv[2] = kf[2] * fk.z; khv[3] = kf[3] * fk.w;
            } else {
                scan_local(l, inc, sm.wtot, w16, g, n);      // (the one-step-ahead form of forward16 costs registers this kernel lacks)
                lds_barrier();
                PT_MARK(7)
                scan_join(inc, tot, sm.wtot, w16, n);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    rhv[c] = rf[c] * exp2_fast(inc[c] - l[c]);
                    khv[c] = kf[c] * exp2_fast(tot[c] - inc[c]);
                }
            }
#pragma unroll
            for (int c = 0; c < 4; c++) p = fmaf(rf[c] * uf[c], kf[c], p);
            uint32_t h0, l0, h1, l1;
            const int o = tok * LD + c4;
            *reinterpret_cast<uint2 *>(&sm.gy[o]) = pg;
            *reinterpret_cast<uint2 *>(&sm.v[o]) = pv;
            split2(rhv[0], rhv[1], h0, l0); split2(rhv[2], rhv[3], h1, l1);
            *reinterpret_cast<uint2 *>(&sm.rh[o]) = make_uint2(h0, h1);
            *reinterpret_cast<uint2 *>(&sm.rhl[o]) = make_uint2(l0, l1);
            split2(khv[0], khv[1], h0, l0); split2(khv[2], khv[3], h1, l1);
            *reinterpret_cast<uint2 *>(&sm.kh[o]) = make_uint2(h0, h1);
            *reinterpret_cast<uint2 *>(&sm.khl[o]) = make_uint2(l0, l1);
            *reinterpret_cast<uint4 *>(&sm.rk[swz(tok, c4)]) =
                make_uint4((pr.x & 0xffffu) | (pk.x << 16), (pr.x >> 16) | (pk.x & 0xffff0000u),
                           (pr.y & 0xffffu) | (pk.y << 16), (pr.y >> 16) | (pk.y & 0xffff0000u));
            if (!whole) {
                *reinterpret_cast<float4 *>(&sm.incl[swz(tok, c4)]) = make_float4(inc[0], inc[1], inc[2], inc[3]);
                *reinterpret_cast<float4 *>(&sm.lw[swz(tok, c4)]) = make_float4(l[0], l[1], l[2], l[3]);
            }
            if (!whole && (w16 & 3) == 3) {       // wavefront-uniform: only the wavefront with the block's last token
                if (g == 3) {
                    *reinterpret_cast<float4 *>(&sm.tot[q][c4]) = make_float4(tot[0], tot[1], tot[2], tot[3]);
                    *reinterpret_cast<float4 *>(&sm.dec[q][c4]) = make_float4(exp2_fast(tot[0]), exp2_fast(tot[1]), exp2_fast(tot[2]), exp2_fast(tot[3]));
                    *reinterpret_cast<float4 *>(&sm.ent[q][c4]) = make_float4(exp2_fast(-tot[0]), exp2_fast(-tot[1]), exp2_fast(-tot[2]), exp2_fast(-tot[3]));
                }
            }
            p = row_prefix_sum(p);           // lane 15 of the row ends with the sum over the 64 channels
            if (n == 15) sm.rho[tok] = p;
        }
      }
        PT_MARK(0)
        lds_barrier();
        PT_MARK(1)

        f4 KG[4];                    // wavefronts 8-11: kh G per block, KG[q][e] at [token 4g+e][value own]
      {
        WKV_LOCAL_LANE
        fetch_whole(max(sb - 1, sb0), tok, c4);      // (the segment's first step fetches itself once more: unused)
        if (role == 0) {
            // ---------------- state chain, first block to last; Q1[t][key own] = sum_j gy[t][j] S[key own][j]
#pragma unroll
            for (int qq = 0; qq < 4; qq++) {
                f4 qa = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < 4; kk += 2) {
                    s4 s0h, s0l, s1h, s1l;
                    split4(G[kk], s0h, s0l);
                    split4(G[kk + 1], s1h, s1l);
                    const s4 y0 = frag(sm.gy, 16 * qq + n, 16 * kk + 4 * g), y1 = frag(sm.gy, 16 * qq + n, 16 * kk + 16 + 4 * g);
                    qa = mma2(s0l, s1l, y0, y1, qa);       // (the state as the A operand: the product comes out as [key][token])
                    qa = mma2(s0h, s1h, y0, y1, qa);
                }
                *reinterpret_cast<float4 *>(&sm.q1[swz(16 * qq + n, 16 * wv + 4 * g)]) = make_float4(qa[0], qa[1], qa[2], qa[3]);
                if (qq < 3) {
                    const float dq = sm.dec[qq][own];
                    const s4 khf = frag_tr(sm.kh, tro + (16 * qq) * LD + 16 * wv), khfl = frag_tr(sm.khl, tro + (16 * qq) * LD + 16 * wv);
#pragma unroll
                    for (int kk = 0; kk < 4; kk++) {
                        G[kk] = G[kk] * dq;
                        const s4 vf_ = frag_tr(sm.v, tro + (16 * qq) * LD + 16 * kk);
                        G[kk] = mma2(vf_, vf_, khf, khfl, G[kk]);
                    }
                }
            }
        } else if (role == 1) {
            // ---------------- state-gradient chain (value-major), last block to first; Q4[s][key own] = sum_j v[s][j] G[key own][j]
#pragma unroll
            for (int qq = 3; qq >= 0; qq--) {
                f4 q4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < 4; kk += 2) {
                    s4 g0h, g0l, g1h, g1l;
                    split4(G[kk], g0h, g0l);
                    split4(G[kk + 1], g1h, g1l);
                    const s4 v0 = frag(sm.v, 16 * qq + n, 16 * kk + 4 * g), v1 = frag(sm.v, 16 * qq + n, 16 * kk + 16 + 4 * g);
                    q4 = mma2(g0l, g1l, v0, v1, q4);
                    q4 = mma2(g0h, g1h, v0, v1, q4);
                }
                *reinterpret_cast<float4 *>(&sm.q4[swz(16 * qq + n, 16 * wv + 4 * g)]) = make_float4(q4[0], q4[1], q4[2], q4[3]);
                const float dq = sm.dec[qq][own];
                const s4 rhTf = frag_tr(sm.rh, tro + (16 * qq) * LD + 16 * wv), rhTfl = frag_tr(sm.rhl, tro + (16 * qq) * LD + 16 * wv);
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {      // G <- e^{b} o G + rh^T gy
                    G[kk] = G[kk] * dq;
                    const s4 gT_ = frag_tr(sm.gy, tro + (16 * qq) * LD + 16 * kk);
                    G[kk] = mma2(gT_, gT_, rhTf, rhTfl, G[kk]);
                }
            }
        } else if (role == 2) {
            // ---------------- state-gradient chain (key-major), last block to first; KG[s][value own] = sum_i kh[s][i] G[i][value own]
#pragma unroll
            for (int qq = 3; qq >= 0; qq--) {
                const int row = 16 * qq + n;
                // The LDS operands of the block's products are fetched before the arithmetic on G starts: this wavefront
                // is the longest of the phase and walks a dependent sequence, so a fetch issued where it is used costs
                // the whole step its latency.
                s4 kh_[4], kl_[4];
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {
                    kh_[kk] = frag(sm.kh, row, 16 * kk + 4 * g);
                    kl_[kk] = frag(sm.khl, row, 16 * kk + 4 * g);
                }
                __builtin_amdgcn_sched_barrier(0);
                f4 g0 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < 4; kk += 2) {
                    s4 g0h, g0l, g1h, g1l;
                    split4(G[kk], g0h, g0l);
                    split4(G[kk + 1], g1h, g1l);
                    g0 = mma2(g0l, g1l, kh_[kk], kh_[kk + 1], g0);       // (the gradient as the A operand: [value][token])
                    g0 = mma2(g0h, g1h, kl_[kk], kl_[kk + 1], g0);
                    g0 = mma2(g0h, g1h, kh_[kk], kh_[kk + 1], g0);
                }
                KG[qq] = g0;
                if (qq == 3) sm.kg3[wv][lane] = make_float4(KG[3][0], KG[3][1], KG[3][2], KG[3][3]);
                const s4 gyTf = frag_tr(sm.gy, tro + (16 * qq) * LD + 16 * wv);
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {      // G <- e^{b} o G + rh^T gy
                    const float4 d4 = *reinterpret_cast<const float4 *>(&sm.dec[qq][16 * kk + 4 * g]);
                    G[kk][0] *= d4.x; G[kk][1] *= d4.y; G[kk][2] *= d4.z; G[kk][3] *= d4.w;
                    G[kk] = mma2(frag_tr(sm.rh, tro + (16 * qq) * LD + 16 * kk), frag_tr(sm.rhl, tro + (16 * qq) * LD + 16 * kk),
                                 gyTf, gyTf, G[kk]);
                }
                __builtin_amdgcn_sched_barrier(0);      // one block at a time: keeps the register need of the chain bounded
            }
        } else {
            // ---------------- the masked matrices of block wv, once for everybody
            // (the LDS operands of each matrix are fetched together and ahead of their use: the builders are, with the
            // key-major chain, the longest wavefronts of the phase, and a fetch issued where it is used costs the whole
            // step its latency)
            const int row = 16 * wv + n;
            s4 gyf[4], vf[4], rhf[4], rlf[4], khf[4], klf[4];
            float4 en[4];
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                gyf[kk] = frag(sm.gy, row, 16 * kk + 4 * g);
                vf[kk] = frag(sm.v, row, 16 * kk + 4 * g);
            }
            // pt[e] = P[t = 4g+e][s = n],  ptT[e] = P[t = n][s = 4g+e],  P[t][s] = gy_t . v_s
            f4 pt = {0.f, 0.f, 0.f, 0.f}, ptT = pt;
            pt = mma2(gyf[0], gyf[1], vf[0], vf[1], pt);
            ptT = mma2(vf[0], vf[1], gyf[0], gyf[1], ptT);
            pt = mma2(gyf[2], gyf[3], vf[2], vf[3], pt);
            ptT = mma2(vf[2], vf[3], gyf[2], gyf[3], ptT);
            f4 pm, pTm;
            {
                const int e_diag = n & 3;
                if ((n >> 2) == g) sm.pdiag[wv][n] = e_diag == 0 ? pt[0] : e_diag == 1 ? pt[1] : e_diag == 2 ? pt[2] : pt[3];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int x = 4 * g + e;
                    pm[e] = x > n ? pt[e] : 0.f;        // later tokens t > s
                    pTm[e] = x < n ? ptT[e] : 0.f;      // earlier tokens s < t
                }
                uint32_t h0, l0, h1, l1;
                split2(pTm[0], pTm[1], h0, l0); split2(pTm[2], pTm[3], h1, l1);
                sm.pfr[wv][0][lane] = make_uint4(h0, h1, l0, l1);
                split2(pm[0], pm[1], h0, l0); split2(pm[2], pm[3], h1, l1);
                sm.pfr[wv][1][lane] = make_uint4(h0, h1, l0, l1);
            }
            __builtin_amdgcn_sched_barrier(0);
            // A~[t = 4g+e][s = n] = (r e^{excl-b})_t . (k e^{b-incl})_s; its operands all at once
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                rhf[kk] = frag(sm.rh, row, 16 * kk + 4 * g);
                rlf[kk] = frag(sm.rhl, row, 16 * kk + 4 * g);
                khf[kk] = frag(sm.kh, row, 16 * kk + 4 * g);
                klf[kk] = frag(sm.khl, row, 16 * kk + 4 * g);
                en[kk] = *reinterpret_cast<const float4 *>(&sm.ent[wv][16 * kk + 4 * g]);
            }
            const float rho_s = sm.rho[row];
            __builtin_amdgcn_sched_barrier(0);
            f4 at = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < 4; kk += 2) {
                s4 r0, r1, r0l, r1l;
                scale_split(rhf[kk], rlf[kk], en[kk], n == 0, r0, r0l);
                scale_split(rhf[kk + 1], rlf[kk + 1], en[kk + 1], n == 0, r1, r1l);
                at = mma2(r0l, r1l, khf[kk], khf[kk + 1], at);
                at = mma2(r0, r1, klf[kk], klf[kk + 1], at);
                at = mma2(r0, r1, khf[kk], khf[kk + 1], at);
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int x = 4 * g + e;
                at[e] = x > n ? at[e] : (x == n ? rho_s : 0.f);
            }
            uint32_t h0, l0, h1, l1;
            split2(at[0], at[1], h0, l0); split2(at[2], at[3], h1, l1);
            sm.amat[wv][lane] = make_uint4(h0, h1, l0, l1);
        }
      }
        PT_MARK(2)
        lds_barrier();
        PT_MARK(3)

      {
        WKV_LOCAL_LANE
        // In this phase the products come out transposed, [channel][token]: a lane holds four consecutive channels
        // of one token (token 16 blk + n, channels 16 wv + 4 g ..), so every table access is one 16-byte piece, the
        // results go into their tiles eight bytes at a time, and the sums over a block's tokens run along a DPP row.
        if (role == 2) {
            // ---------------- gv[s][value] = kh G + sum_{t>=s} A~[t][s] gy[t], values 16wv..16wv+15
#pragma unroll
            for (int qq = 0; qq < 4; qq++) {
                const uint4 am = sm.amat[qq][lane];
                const s4 gyTf = frag_tr(sm.gy, tro + (16 * qq) * LD + 16 * wv);
                f4 kgq = KG[qq < 3 ? qq : 0];
                if (qq == 3) { const float4 t4 = sm.kg3[wv][lane]; kgq = f4{t4.x, t4.y, t4.z, t4.w}; }
                const f4 gvt = mma2(gyTf, gyTf, as_s4(am.x, am.y), as_s4(am.z, am.w), kgq);
                *reinterpret_cast<uint2 *>(&sm.v[(16 * qq + n) * LD + 16 * wv + 4 * g]) =
                    make_uint2(bf16_pack2(gvt[0], gvt[1]), bf16_pack2(gvt[2], gvt[3]));      // v is not read any more
            }
        }
        // ---------------- block q, token 16q+n, keys 16wv+4g..+3: gr, gk, decay gradient
        {
            const uint4 pa = sm.pfr[q][0][lane], pb = sm.pfr[q][1][lane];
            const s4 pT_h = as_s4(pa.x, pa.y), pT_l = as_s4(pa.z, pa.w), pm_h = as_s4(pb.x, pb.y), pm_l = as_s4(pb.z, pb.w);
            const s4 khTf = frag_tr(sm.kh, tro + (16 * q) * LD + 16 * wv), khTfl = frag_tr(sm.khl, tro + (16 * q) * LD + 16 * wv);
            const s4 rhTf = frag_tr(sm.rh, tro + (16 * q) * LD + 16 * wv), rhTfl = frag_tr(sm.rhl, tro + (16 * q) * LD + 16 * wv);
            f4 q2 = {0.f, 0.f, 0.f, 0.f}, q3 = q2;
            q2 = mma(khTfl, pT_h, q2);
            q3 = mma(rhTfl, pm_h, q3);
            q2 = mma2(khTf, khTf, pT_h, pT_l, q2);      // sum_{s<t} P[t][s] kh_s   at [key][t]
            q3 = mma2(rhTf, rhTf, pm_h, pm_l, q3);      // sum_{t>s} P[t][s] rh_t   at [key][s]
            const int tk = 16 * q + n, k4 = 16 * wv + 4 * g, ti = swz(tk, k4);
            const float4 tot4 = *reinterpret_cast<const float4 *>(&sm.tot[q][k4]), ent4 = *reinterpret_cast<const float4 *>(&sm.ent[q][k4]);
            const float4 q1v = *reinterpret_cast<const float4 *>(&sm.q1[ti]), q4v = *reinterpret_cast<const float4 *>(&sm.q4[ti]);
            const uint4 rk4 = *reinterpret_cast<const uint4 *>(&sm.rk[ti]);
            const float pd = sm.pdiag[q][n];
            float E1[4], E2[4];
            if (whole) {
                const float4 fr = *reinterpret_cast<const float4 *>(&tab_r[swz(n, k4)]), fk = *reinterpret_cast<const float4 *>(&tab_k[swz(n, k4)]);
                E1[0] = fr.x; E1[1] = fr.y; E1[2] = fr.z; E1[3] = fr.w;
                E2[0] = fk.x; E2[1] = fk.y; E2[2] = fk.z; E2[3] = fk.w;
            } else {
                const float4 in4 = *reinterpret_cast<const float4 *>(&sm.incl[ti]), lw4 = *reinterpret_cast<const float4 *>(&sm.lw[ti]);
                E1[0] = exp2_fast(in4.x - lw4.x); E1[1] = exp2_fast(in4.y - lw4.y); E1[2] = exp2_fast(in4.z - lw4.z); E1[3] = exp2_fast(in4.w - lw4.w);
                E2[0] = exp2_fast(tot4.x - in4.x); E2[1] = exp2_fast(tot4.y - in4.y); E2[2] = exp2_fast(tot4.z - in4.z); E2[3] = exp2_fast(tot4.w - in4.w);
            }
            const float entf[4] = {ent4.x, ent4.y, ent4.z, ent4.w}, uf[4] = {u4.x, u4.y, u4.z, u4.w};
            const float q1f[4] = {q1v.x, q1v.y, q1v.z, q1v.w}, q4f[4] = {q4v.x, q4v.y, q4v.z, q4v.w};
            const uint32_t rkf[4] = {rk4.x, rk4.y, rk4.z, rk4.w};
            float c[4], z[4], grv[4], gkv[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float rr = bf_lo(rkf[e]), kr = bf_hi(rkf[e]), upd = uf[e] * pd;
                grv[e] = E1[e] * (q1f[e] + entf[e] * q2[e]) + upd * kr;
                const float gkn = E2[e] * (entf[e] * q3[e] + q4f[e]);
                gkv[e] = gkn + upd * rr;
                c[e] = rr * grv[e] - kr * gkv[e];
                z[e] = kr * gkn;
                gu_acc[e] = fmaf(rr * kr, pd, gu_acc[e]);
            }
            // this wavefront was the only reader left of its (block, quarter) corner of the rh and kh tiles
            *reinterpret_cast<uint2 *>(&sm.rh[tk * LD + k4]) = make_uint2(bf16_pack2(grv[0], grv[1]), bf16_pack2(grv[2], grv[3]));
            *reinterpret_cast<uint2 *>(&sm.kh[tk * LD + k4]) = make_uint2(bf16_pack2(gkv[0], gkv[1]), bf16_pack2(gkv[2], gkv[3]));
            if (PER_TOKEN_W) {
                // dL/dlog w_t = A_t - z_t with A_t = A(end of block) + sum over the block's later tokens of c
                float dpart[4], all[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float incl_suf = row_suffix_sum(c[e]);          // c of this token and the later ones
                    dpart[e] = (incl_suf - c[e]) - z[e];
                    all[e] = incl_suf;                                    // (lane n = 0: the whole block)
                }
                // (the incl entries of this block and quarter had this wavefront as their only reader)
                *reinterpret_cast<float4 *>(&sm.incl[ti]) = make_float4(dpart[0], dpart[1], dpart[2], dpart[3]);
                if (n == 0) *reinterpret_cast<float4 *>(&sm.tots[q][k4]) = make_float4(all[0], all[1], all[2], all[3]);
            } else {
                const float before = (float)((sb - sb0) * SB + tk);      // tokens of the segment before this one
#pragma unroll
                for (int e = 0; e < 4; e++) gw_acc[e] += fmaf(before, c[e], -z[e]);
            }
        }
      }
        PT_MARK(4)
        lds_barrier();
        have_out = true;
    }
    if (have_out) write_out(sb0, tok, c4, par);

    PT_PRINT("bwd16")
    if (role == 1 && gs_in && seg == 0) {
        float *gp = gs_in + (size_t)bh * HEAD * HEAD + own * HEAD;
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
            *reinterpret_cast<float4 *>(gp + 16 * kk + 4 * g) = make_float4(G[kk][0], G[kk][1], G[kk][2], G[kk][3]);
    }
#pragma unroll
    for (int e = 0; e < 4; e++) gu_acc[e] = row_suffix_sum(gu_acc[e]);       // lane n = 0: the sum over the row's 16 tokens
    if (n == 0) *reinterpret_cast<float4 *>(&sm.red[q][16 * wv + 4 * g]) = make_float4(gu_acc[0], gu_acc[1], gu_acc[2], gu_acc[3]);
    float *gw4 = sm.q1;             // [4][HEAD]; the q1 table is dead by now
    if (!PER_TOKEN_W) {
#pragma unroll
        for (int e = 0; e < 4; e++) gw_acc[e] = row_suffix_sum(gw_acc[e]);
        if (n == 0) *reinterpret_cast<float4 *>(&gw4[q * HEAD + 16 * wv + 4 * g]) = make_float4(gw_acc[0], gw_acc[1], gw_acc[2], gw_acc[3]);
    }
    lds_barrier();
    if (q == 0 && g == 0) {      // partial sums per (batch, segment): [(b*nseg + seg)][C]
        const size_t po = ((size_t)(b * nseg + seg) * H + h) * HEAD + own;
        gu_part[po] = (sm.red[0][own] + sm.red[1][own]) + (sm.red[2][own] + sm.red[3][own]);
        if (!PER_TOKEN_W) {
            bool fl;
            const float l = log_decay(static_cast<const float *>(wraw)[h * HEAD + own], floor_decay, &fl);
            const int ntok = min(Tlen, sb1 * SB) - sb0 * SB;         // tokens of this segment
            const float sum = ((gw4[own] + gw4[HEAD + own]) + (gw4[2 * HEAD + own] + gw4[3 * HEAD + own]))
                              + (float)ntok * sm.arun[0][own];            // arun[0]: the anchor A(segment end), untouched for this w
            gw_part[po] = fl ? 0.f : sum * l;
        }
    }
}

// Sums the per-(batch, segment) partial sums of gu (gw) in a fixed order.  The (batch, head) pairs below nA ran as
// one segment and left theirs in `one` [b][C]; the others ran as nseg segments and left theirs in `many`
// [(b*nseg + seg)][C].
__global__ void sum_partials(int B, int H, int nA, int nseg, const float *__restrict__ one, const float *__restrict__ many,
                             float *__restrict__ out) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, C = H * HEAD;
    if (c >= C) return;
    const int h = c / HEAD;
    float sum = 0.f;
    for (int b = 0; b < B; b++) {
        if (b * H + h < nA) sum += one[(size_t)b * C + c];
        else
            for (int x = 0; x < nseg; x++) sum += many[(size_t)(b * nseg + x) * C + c];
    }
    out[c] = sum;
}

// ------------------------------------------------------------------ launchers --
static size_t round256(size_t x) { return (x + 255) & ~(size_t)255; }
size_t checkpoint_bytes(int B, int Tlen, int H) {
    return (size_t)B * H * ((Tlen + SB - 1) / SB + 1) * HEAD * HEAD * sizeof(float);     // one slot per step + the final state
}

// How many time segments run in parallel for one (batch, head).  More segments mean
// more workgroups (B*H*nseg) to spread over the compute units but also one more light pass
// over (part of) the inputs; the estimate below counts CU rounds times steps
// per segment and prefers fewer segments on ties.  wkv_tune(WKV_TUNE_SEGMENTS) /
// RWKV_WKV_NSEG override it.
constexpr int MAX_SEG = 64;
struct SegPlan { int nseg, sps, m, pps; };     // segments, steps per segment, pieces per segment, steps per piece
inline int &forced_segments() {          // 0 = choose automatically
    static int v = [] { const char *e = getenv("RWKV_WKV_NSEG"); return e ? std::min(std::max(atoi(e), 0), MAX_SEG) : 0; }();
    return v;
}
inline int &forced_piece_steps() {       // 0 = choose automatically
    static int v = [] { const char *e = getenv("RWKV_WKV_PPS"); return e ? std::max(atoi(e), 0) : 0; }();
    return v;
}
// what the summary pass adds to a run in n segments, as a factor on the main kernels' time
// (at worst the pass reads (n-1)/n of the tokens at about 40 % of the main kernels' cost per token)
static double segment_overhead(int n) { return 1.0 + 0.4 * (n - 1) / n; }
static SegPlan plan_segments(int BH, int Tlen, int ncu) {
    const int nsb = (Tlen + SB - 1) / SB;
    const int forced = forced_segments();
    int want = 1;
    if (forced > 0) {
        want = std::min(forced, nsb);
    } else {
        double best = 1e30;
        for (int cand = 1; cand <= 16 && cand * 4 <= std::max(4, nsb); cand++) {
            const int sps = (nsb + cand - 1) / cand;
            const double rounds = (double)((BH * cand + ncu - 1) / ncu);
            const double cost = rounds * (sps + 1) * segment_overhead(cand);
            if (cost < best * 0.97) { best = cost; want = cand; }
        }
    }
    const int sps = (nsb + want - 1) / want;
    const int nseg = (nsb + sps - 1) / sps;
    // the summary pass: cut each segment into pieces until the pass has about 1.5 workgroups per CU
    // (every piece costs one 16 KB summary, so no finer than needed and never below 2 steps)
    int pps = sps;
    if (nseg == 1) return SegPlan{1, sps, 1, sps};
    if (forced_piece_steps() > 0) pps = std::min(sps, forced_piece_steps());
    else
        while (pps >= 4 && (long)BH * (nseg - 1) * ((sps + pps - 1) / pps) < ncu + ncu / 2) pps = (pps + 1) / 2;
    int m = (sps + pps - 1) / pps;
    if (nseg * m > MAX_SEG) { m = std::max(1, MAX_SEG / nseg); pps = (sps + m - 1) / m; m = (sps + pps - 1) / pps; }
    if (nseg * m > MAX_SEG) { m = 1; pps = sps; }
    return SegPlan{nseg, sps, m, pps};
}
// Two groups of (batch, head) pairs.  When B*H is more than a whole number of CU rounds, the whole rounds run their
// sequences in one piece (group A: the first nA pairs, no summary pass at all) and only the remainder is cut in time
// (group B), so that it fills one more, shorter round: 320 pairs = 256 whole + 64 x 4 segments instead of 320 x 4.
struct GroupPlan { int nA; SegPlan a, b; };
static GroupPlan plan_groups(int BH, int Tlen) {
    const int nsb = (Tlen + SB - 1) / SB, ncu = cu_count();
    GroupPlan p{0, SegPlan{1, nsb, 1, nsb}, plan_segments(BH, Tlen, ncu)};
    const int whole = BH / ncu * ncu, rest = BH - whole;
    if (forced_segments() > 0 || whole == 0 || rest == 0) return p;
    const SegPlan r = plan_segments(rest, Tlen, ncu);
    auto cost = [ncu](int bh, const SegPlan &x) {
        return (double)((bh * x.nseg + ncu - 1) / ncu) * (x.sps + 1) * segment_overhead(x.nseg);
    };
    if (cost(whole, p.a) + cost(rest, r) < 0.97 * cost(BH, p.b)) { p.nA = whole; p.b = r; }
    return p;
}
// the piece summaries of a plan: one slot per (batch, head) and piece (slots are indexed by the pair's number in the
// whole batch, so the pairs of group A have unused ones)
static size_t part_bytes(int BH, const GroupPlan &gp) {
    return gp.b.nseg > 1 ? round256((size_t)BH * gp.b.nseg * gp.b.m * PART * sizeof(float)) : 0;
}

// Where things are in a workspace, for the plan in force:  checkpoints | forward piece summaries | backward piece
// summaries | gu, gw partial sums, each (B, C) for the unsplit group and (B*nseg, C) for the split one.  A forward
// call uses the first two regions.  Only the checkpoints pass from a forward call to the backward call that follows,
// and their place and layout depend on the shape alone, not on the plan.
struct Layout { size_t ckpt, part, gpart, sums, forward_total, total; };
static Layout layout(int B, int Tlen, int C, int H, const GroupPlan &gp) {
    Layout L;
    L.ckpt = 0;
    L.part = round256(checkpoint_bytes(B, Tlen, H));
    L.gpart = L.part + part_bytes(B * H, gp);
    L.forward_total = L.gpart;
    L.sums = L.gpart + part_bytes(B * H, gp);
    L.total = L.sums + round256(2 * (size_t)B * (gp.b.nseg + 1) * C * sizeof(float));
    return L;
}
// true when the plan in force cuts some sequence of this shape into time segments
bool splits_time(int BH, int Tlen) { return plan_groups(BH, Tlen).b.nseg > 1; }
size_t forward_workspace(int B, int Tlen, int H) { return layout(B, Tlen, H * HEAD, H, plan_groups(B * H, Tlen)).forward_total; }
size_t backward_workspace(int B, int Tlen, int C, int H) { return layout(B, Tlen, C, H, plan_groups(B * H, Tlen)).total; }

// The 16-wavefront kernels use more LDS than a kernel gets by default.  Raising the limit is a property of the loaded
// code object and is done once per device, from wkv_init() or from the first launch there, whichever comes first.
hipError_t init_kernels() {
    static PerDevice done;
    return done.once([] {
        auto allow = [](const void *kernel, size_t bytes) {
            return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        };
        hipError_t e = allow((const void *)forward16<true, false>, sizeof(Fwd16Tiles));
        if (e == hipSuccess) e = allow((const void *)forward16<true, true>, sizeof(Fwd16Tiles));
        if (e == hipSuccess) e = allow((const void *)forward16<false, false>, sizeof(Fwd16Tiles));
        if (e == hipSuccess) e = allow((const void *)forward16<false, false, true>, sizeof(Fwd16Tiles));
        if (e == hipSuccess) e = allow((const void *)backward16<true, false>, sizeof(Bwd16Tiles));
        if (e == hipSuccess) e = allow((const void *)backward16<true, true>, sizeof(Bwd16Tiles));
        if (e == hipSuccess) e = allow((const void *)backward16<false, false>, sizeof(Bwd16Tiles));
        if (e == hipSuccess) e = allow((const void *)backward16<false, false, true>, sizeof(Bwd16Tiles));
        return e;
    });
}

// ckpt == nullptr: no checkpoints kept;  part == nullptr: the sequences run in one piece each
// w16: the per-token decay is bf16 (per_token only)
hipError_t forward_launch(hipStream_t s, bool per_token, bool w16, int B, int Tlen, int C, int H, const void *r, const void *k,
                          const void *v, const void *w, const float *u, const float *s_in, void *y, float *s_out,
                          float *ckpt, float *part, const GroupPlan &plan, int floor_decay) {
    hipError_t e0 = init_kernels();
    if (e0 != hipSuccess) return e0;
    const int mode = per_token ? (w16 ? 2 : 1) : 0;
    const int nsb = (Tlen + SB - 1) / SB, BH = B * H;
    const GroupPlan gp = part ? plan : GroupPlan{0, SegPlan{1, nsb, 1, nsb}, SegPlan{1, nsb, 1, nsb}};
    const bf16 *rr = (const bf16 *)r, *kk = (const bf16 *)k, *vv = (const bf16 *)v;
    const SegPlan &pl = gp.b;
    const int nB = BH - gp.nA;
    if (pl.nseg > 1) {
        dim3 grid(nB * (pl.nseg - 1) * pl.m), block(NT_F);
        if (mode == 2)
            hipLaunchKernelGGL((summary_pass<true, false, true>), grid, block, 0, s, gp.nA, Tlen, C, H, pl.nseg, pl.sps, pl.m,
                               pl.pps, kk, vv, w, part, floor_decay);
        else if (mode == 1)
            hipLaunchKernelGGL((summary_pass<true, false, false>), grid, block, 0, s, gp.nA, Tlen, C, H, pl.nseg, pl.sps, pl.m,
                               pl.pps, kk, vv, w, part, floor_decay);
        else
            hipLaunchKernelGGL((summary_pass<false, false, false>), grid, block, 0, s, gp.nA, Tlen, C, H, pl.nseg, pl.sps, pl.m,
                               pl.pps, kk, vv, w, part, floor_decay);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    dim3 block16(NT_F16);
    auto launch = [&](int bh0, int n, const SegPlan &x) {
        if (n <= 0) return;
        dim3 grid(n * x.nseg);
        if (mode == 2)
            hipLaunchKernelGGL((forward16<true, true>), grid, block16, sizeof(Fwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps, x.m,
                               rr, kk, vv, w, u, s_in, (bf16 *)y, s_out, ckpt, part, floor_decay);
        else if (mode == 1)
            hipLaunchKernelGGL((forward16<true, false>), grid, block16, sizeof(Fwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps, x.m,
                               rr, kk, vv, w, u, s_in, (bf16 *)y, s_out, ckpt, part, floor_decay);
        else if (Tlen % SB == 0)
            hipLaunchKernelGGL((forward16<false, false, true>), grid, block16, sizeof(Fwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps, x.m,
                               rr, kk, vv, w, u, s_in, (bf16 *)y, s_out, ckpt, part, floor_decay);
        else
            hipLaunchKernelGGL((forward16<false, false>), grid, block16, sizeof(Fwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps, x.m,
                               rr, kk, vv, w, u, s_in, (bf16 *)y, s_out, ckpt, part, floor_decay);
    };
    prof_begin(KID_CHUNK_FORWARD, s);          // (both groups count as the one forward kernel of the call)
    launch(0, gp.nA, gp.a);
    launch(gp.nA, nB, pl);
    prof_end(KID_CHUNK_FORWARD, s);
    return hipGetLastError();
}

// forward with a caller's workspace (or none: one piece per sequence, no checkpoints)
hipError_t forward_launch(hipStream_t s, bool per_token, bool w16, int B, int Tlen, int C, int H, const void *r, const void *k,
                          const void *v, const void *w, const float *u, const float *s_in, void *y, float *s_out,
                          void *workspace, int floor_decay) {
    const GroupPlan gp = plan_groups(B * H, Tlen);
    const Layout L = layout(B, Tlen, C, H, gp);
    char *ws = (char *)workspace;
    return forward_launch(s, per_token, w16, B, Tlen, C, H, r, k, v, w, u, s_in, y, s_out, ws ? (float *)(ws + L.ckpt) : nullptr,
                          (ws && gp.b.nseg > 1) ? (float *)(ws + L.part) : nullptr, gp, floor_decay);
}

hipError_t backward_launch(hipStream_t s, bool per_token, bool w16, int B, int Tlen, int C, int H, const void *r, const void *k,
                           const void *v, const void *w, const float *u, const float *s_in, const void *gy,
                           const float *gs_out, void *gr, void *gk, void *gv, void *gw, float *gu, float *gs_in,
                           void *workspace, bool have_ckpt, int floor_decay) {
    hipError_t e0 = init_kernels();
    if (e0 != hipSuccess) return e0;
    const int BH = B * H, mode = per_token ? (w16 ? 2 : 1) : 0;
    const GroupPlan gp = plan_groups(BH, Tlen);
    const Layout L = layout(B, Tlen, C, H, gp);
    const SegPlan &pl = gp.b;
    char *ws = (char *)workspace;
    float *ckpt = (float *)(ws + L.ckpt), *gpart = (float *)(ws + L.gpart);
    float *gu_one = (float *)(ws + L.sums), *gu_many = gu_one + (size_t)B * C;
    float *gw_one = gu_many + (size_t)B * pl.nseg * C, *gw_many = gw_one + (size_t)B * C;
    if (!have_ckpt) {      // the forward call did not leave its checkpoints here: rebuild them
        hipError_t e = forward_launch(s, per_token, w16, B, Tlen, C, H, r, k, v, w, u, s_in, nullptr, nullptr, ckpt,
                                      pl.nseg > 1 ? (float *)(ws + L.part) : nullptr, gp, floor_decay);
        if (e != hipSuccess) return e;
    }
    const int nB = BH - gp.nA;
    const bf16 *rr = (const bf16 *)r, *kk = (const bf16 *)k, *vv = (const bf16 *)v, *gg = (const bf16 *)gy;
    if (pl.nseg > 1) {
        dim3 grid(nB * (pl.nseg - 1) * pl.m), block(NT_F);
        if (mode == 2)
            hipLaunchKernelGGL((summary_pass<true, true, true>), grid, block, 0, s, gp.nA, Tlen, C, H, pl.nseg, pl.sps, pl.m,
                               pl.pps, rr, gg, w, gpart, floor_decay);
        else if (mode == 1)
            hipLaunchKernelGGL((summary_pass<true, true, false>), grid, block, 0, s, gp.nA, Tlen, C, H, pl.nseg, pl.sps, pl.m,
                               pl.pps, rr, gg, w, gpart, floor_decay);
        else
            hipLaunchKernelGGL((summary_pass<false, true, false>), grid, block, 0, s, gp.nA, Tlen, C, H, pl.nseg, pl.sps, pl.m,
                               pl.pps, rr, gg, w, gpart, floor_decay);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    dim3 block16(NT_B16);
    auto launch = [&](int bh0, int n, const SegPlan &x, float *gw_part, float *gu_part) {
        if (n <= 0) return;
        dim3 grid(n * x.nseg);
        if (mode == 2)
            hipLaunchKernelGGL((backward16<true, true>), grid, block16, sizeof(Bwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps,
                               x.m, rr, kk, vv, w, u, gg, gs_out, ckpt, gpart, (bf16 *)gr, (bf16 *)gk, (bf16 *)gv, gw, gw_part,
                               gu_part, gs_in, floor_decay);
        else if (mode == 1)
            hipLaunchKernelGGL((backward16<true, false>), grid, block16, sizeof(Bwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps,
                               x.m, rr, kk, vv, w, u, gg, gs_out, ckpt, gpart, (bf16 *)gr, (bf16 *)gk, (bf16 *)gv, gw, gw_part,
                               gu_part, gs_in, floor_decay);
        else if (Tlen % SB == 0)
            hipLaunchKernelGGL((backward16<false, false, true>), grid, block16, sizeof(Bwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps,
                               x.m, rr, kk, vv, w, u, gg, gs_out, ckpt, gpart, (bf16 *)gr, (bf16 *)gk, (bf16 *)gv, (void *)nullptr,
                               gw_part, gu_part, gs_in, floor_decay);
        else
            hipLaunchKernelGGL((backward16<false, false>), grid, block16, sizeof(Bwd16Tiles), s, bh0, Tlen, C, H, x.nseg, x.sps,
                               x.m, rr, kk, vv, w, u, gg, gs_out, ckpt, gpart, (bf16 *)gr, (bf16 *)gk, (bf16 *)gv, (void *)nullptr,
                               gw_part, gu_part, gs_in, floor_decay);
    };
    prof_begin(KID_CHUNK_BACKWARD, s);         // (both groups count as the one backward kernel of the call)
    launch(0, gp.nA, gp.a, gw_one, gu_one);
    launch(gp.nA, nB, pl, gw_many, gu_many);
    prof_end(KID_CHUNK_BACKWARD, s);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sum_partials, dim3((C + 255) / 256), dim3(256), 0, s, B, H, gp.nA, pl.nseg, gu_one, gu_many, gu);
    if (!per_token)
        hipLaunchKernelGGL(sum_partials, dim3((C + 255) / 256), dim3(256), 0, s, B, H, gp.nA, pl.nseg, gw_one, gw_many,
                           (float *)gw);
    return hipGetLastError();
}

}  // namespace chunked
}  // namespace wkv
