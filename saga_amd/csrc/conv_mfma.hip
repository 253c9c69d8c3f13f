// Implicit-GEMM convolution on the gfx950 matrix cores (fp16 in, fp32 accumulate), for
// channels-last activations and K,R,S,C filters.
//
//   forward        y[m, k]  = sum_{tap, c} x[pix(m, tap), c] * w[k, tap, c]      m = (n, p, q)
//   backward data  dx[m, c] = sum_{tap, k} dy[pix'(m, tap), k] * wT[c, tap, k]   m = (n, h, w)
//   backward filt  dw[k, tap, c] = sum_m dy[m, k] * x[pix(m, tap), c]
//
// Forward and backward-data share one kernel: a GEMM whose A operand is gathered on the fly
// (im2col is never materialised) and whose B operand is a row-major [Ngemm][taps*Cred] matrix
// with the reduction index contiguous - exactly the K,R,S,C filter for forward, and a
// transposed copy (C,R,S,K) made in the workspace for backward-data.
//
// Tiling: 256 threads = 4 wavefronts; each wavefront owns a (TM*32) x (TN*32) patch built
// from v_mfma_f32_32x32x16_f16 tiles; the block tile is staged through LDS in slices of
// BK = 32 reduction elements, double buffered, with the next slice's global loads issued
// before the current slice's MFMAs.  All global loads are 16-byte vectors along the channel
// axis (the contiguous axis of NHWC), LDS rows are padded to 40 halfs so that the 16-byte
// fragment reads of a wavefront spread over the banks.
// Blocks are renumbered so that consecutive tiles land on the same XCD and share its L2.
#include "conv.hpp"

#include <stdlib.h>
#include <algorithm>
#include <stdio.h>

namespace {

constexpr int BK = 32;        // reduction elements per LDS slice
constexpr int LDK = BK + 8;   // padded LDS row, in halfs (80 bytes, keeps 16-byte alignment)

struct GatherArgs {
    const half_t *a;   // gathered operand (x for forward, dy for backward data)
    const half_t *b;   // [Ngemm][taps * Cred]
    half_t *out;       // [M][ldo]
    int M;             // output rows = N * OH * OW
    int Ngemm;         // output channels
    int Cred;          // channels of the gathered tensor (reduction per tap)
    int IH, IW;        // gathered tensor spatial size
    int OH, OW;        // output spatial size
    int R, S;
    int pad, stride, dil;
    int sshift;        // log2(stride), backward data only
    int lda;           // row pitch of the gathered tensor (elements)
    int ldo;           // row pitch of the output
    float alpha, beta;
    int nblk_n;        // number of block columns
    int nblocks;
    unsigned a_bytes;  // extent of the gathered tensor / of b, for range-checked buffer loads
    unsigned b_bytes;
    int classes;       // backward data: stride*stride residue classes of output pixels (1: none)
    int OHc, OWc, Mc;  // pixel grid and row count of one class (Mc = M when classes == 1)
    int blocks_per_class;
    int nactive;       // classes that get blocks
    unsigned char cls_ids[16]; // residue classes that get blocks (classes with no tap are left out)
    // forward only, optional: y = act(conv * sc[c] + sh[c] (+ z)) with sc = s*rsqrt(v+eps),
    // sh = b - m*sc (batch-norm inference folded into the epilogue)
    const float *bn_s, *bn_b, *bn_m, *bn_v;
    float bn_eps;
    int bn_flags;      // SAGA_BN_RELU | SAGA_BN_ADD
    const half_t *z;   // residual, [M][ldz]
    int ldz;
    // backward data only, optional (kernels instantiated with BQ): the output is the gradient of a batch norm's
    // (+ relu) result and this launch is its only writer.  The epilogue masks it with that relu (recomputed from
    // the norm's input as half(fma(x, s*invstd, b - mean*s*invstd)) > 0, what the forward stored), stores the
    // masked gradient and leaves, per block row and channel, sum(g) and sum(g * (x - mean)) in
    // bq_partial[stats_rows][Ngemm][2]: the first pass of the batch norm's backward.
    const half_t *bq_x; // the norm's input, [M][bq_ldx]
    int bq_ldx;
    const float *bq_mean, *bq_s, *bq_invstd, *bq_b;
    int bq_relu;
    float *bq_partial;  // null: no link
    int no_stage;      // the epilogue stores straight from registers (experiment switch SAGA_HIP_NO_STAGED_STORES)
    int b_krsc;        // conv_rows64_wide<.., FLIP>: b is the filter as the forward pass has it (K,R,S,C), not transposed
    unsigned out_bytes; // extent of out, for the epilogue variant that stores through a range-checked buffer (BUFST)
    float *stats;      // forward only, optional: per block row and output channel, sum and sum of
                       // squares of the stored outputs, [ceil(M / BM)][Ngemm][2]
    int stats_rows;    // out: block rows the launch wrote
};

__device__ __forceinline__ int xcd_remap(int b, int nblocks)
{
    // hardware hands consecutive workgroup ids to the 8 XCDs round-robin; give each XCD a
    // contiguous range of tiles instead
    const int per = nblocks >> 3, rem = nblocks & 7;
    const int xcd = b & 7, slot = b >> 3;
    const int base = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
    return base + slot;
}

template <int BM, int BN, int WGM, int WGN, bool BWD>
__global__ void __launch_bounds__(256) conv_gather_gemm(GatherArgs g)
{
    constexpr int WTM = BM / WGM, WTN = BN / WGN; // wavefront tile
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int AV = BM / 64, BV = BN / 64;     // 16-byte vectors per thread per slice
    static_assert(WGM * WGN == 4, "four wavefronts");
    static_assert(BM % 64 == 0 && BN % 64 == 0, "tile");

    __shared__ __attribute__((aligned(16))) half_t As[2][BM * LDK];
    __shared__ __attribute__((aligned(16))) half_t Bs[2][BN * LDK];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int bid = xcd_remap(blockIdx.x, g.nblocks);
    const int bm = bid / g.nblk_n, bn = bid - bm * g.nblk_n;
    const int m0 = bm * BM, n0 = bn * BN;

    // ---- per-thread load coordinates: vector column kv (8 halfs), rows tid/4 + 64*j
    const int kv = (tid & 3) * 8;
    const int lrow = tid >> 2;
    int a_base[AV], a_y[AV], a_x[AV];
    bool a_ok[AV];
#pragma unroll
    for(int j = 0; j < AV; j++) {
        const int m = m0 + lrow + 64 * j;
        a_ok[j] = m < g.M;
        const int mm = a_ok[j] ? m : 0;
        const int ox = mm % g.OW;
        const int t = mm / g.OW;
        const int oy = t % g.OH;
        const int n = t / g.OH;
        a_base[j] = n * g.IH * g.IW;
        if(BWD) {
            a_y[j] = oy + g.pad;
            a_x[j] = ox + g.pad;
        } else {
            a_y[j] = oy * g.stride - g.pad;
            a_x[j] = ox * g.stride - g.pad;
        }
    }
    const int ktot = g.R * g.S * g.Cred;
    int b_off[BV];
    bool b_ok[BV];
#pragma unroll
    for(int j = 0; j < BV; j++) {
        const int n = n0 + lrow + 64 * j;
        b_ok[j] = n < g.Ngemm;
        b_off[j] = (b_ok[j] ? n : 0) * ktot;
    }

    half8_t ra[AV], rb[BV];
    const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    // slice iterator: tap (r, s) and channel offset c0
    int r = 0, s = 0, c0 = 0;
    const int csteps = (g.Cred + BK - 1) / BK;
    const int KT = g.R * g.S * csteps;

    auto load_slice = [&]() {
        const int c = c0 + kv;
        const bool cok = c < g.Cred;
#pragma unroll
        for(int j = 0; j < AV; j++) {
            int iy, ix;
            bool ok = a_ok[j] && cok;
            if(BWD) {
                const int ty = a_y[j] - r * g.dil, tx = a_x[j] - s * g.dil;
                ok = ok && ty >= 0 && tx >= 0 && ((ty | tx) & (g.stride - 1)) == 0;
                iy = ty >> g.sshift;
                ix = tx >> g.sshift;
            } else {
                iy = a_y[j] + r * g.dil;
                ix = a_x[j] + s * g.dil;
                ok = ok && iy >= 0 && ix >= 0;
            }
            ok = ok && iy < g.IH && ix < g.IW;
            ra[j] = zero;
            if(ok)
                ra[j] = *(const half8_t *)(g.a + (int64_t)(a_base[j] + iy * g.IW + ix) * g.lda + c);
        }
        const int kb = (r * g.S + s) * g.Cred + c;
#pragma unroll
        for(int j = 0; j < BV; j++) {
            rb[j] = zero;
            if(b_ok[j] && cok)
                rb[j] = *(const half8_t *)(g.b + b_off[j] + kb);
        }
    };
    auto advance = [&]() {
        c0 += BK;
        if(c0 >= g.Cred) {
            c0 = 0;
            if(++s == g.S) {
                s = 0;
                ++r;
            }
        }
    };
    auto store_slice = [&](int st) {
#pragma unroll
        for(int j = 0; j < AV; j++)
            *(half8_t *)(&As[st][(lrow + 64 * j) * LDK + kv]) = ra[j];
#pragma unroll
        for(int j = 0; j < BV; j++)
            *(half8_t *)(&Bs[st][(lrow + 64 * j) * LDK + kv]) = rb[j];
    };

    float16_t acc[TM][TN];
#pragma unroll
    for(int i = 0; i < TM; i++)
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][j][v] = 0.0f;

    const int wm = (wave / WGN) * WTM, wn = (wave % WGN) * WTN;
    const int frow = lane & 31, fk = (lane >> 5) * 8;

    load_slice();
    store_slice(0);
    __syncthreads();

    for(int kt = 0; kt < KT; kt++) {
        const int cur = kt & 1;
        if(kt + 1 < KT) {
            advance();
            load_slice();
        }
#pragma unroll
        for(int kk = 0; kk < BK; kk += 16) {
            half8_t fa[TM], fb[TN];
#pragma unroll
            for(int i = 0; i < TM; i++)
                fa[i] = *(const half8_t *)(&As[cur][(wm + i * 32 + frow) * LDK + kk + fk]);
#pragma unroll
            for(int j = 0; j < TN; j++)
                fb[j] = *(const half8_t *)(&Bs[cur][(wn + j * 32 + frow) * LDK + kk + fk]);
#pragma unroll
            for(int i = 0; i < TM; i++)
#pragma unroll
                for(int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if(kt + 1 < KT)
            store_slice(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: accumulator element v of a 32x32 tile sits at row 8*(v/4) + 4*(lane/32) + v%4,
    // column lane%32
    const int ecol = lane & 31, erow = (lane >> 5) * 4;
#pragma unroll
    for(int i = 0; i < TM; i++) {
#pragma unroll
        for(int j = 0; j < TN; j++) {
            const int n = n0 + wn + j * 32 + ecol;
            if(n >= g.Ngemm)
                continue;
#pragma unroll
            for(int v = 0; v < 16; v++) {
                const int m = m0 + wm + i * 32 + (v >> 2) * 8 + erow + (v & 3);
                if(m >= g.M)
                    continue;
                half_t *o = g.out + (int64_t)m * g.ldo + n;
                float val = g.alpha * acc[i][j][v];
                if(g.beta != 0.0f)
                    val += g.beta * (float)*o;
                *o = (half_t)val;
            }
        }
    }
}

// ---------------------------------------------------------------- pipelined variant
//
// Same GEMM, different data movement: global -> LDS goes through the buffer-load-to-LDS path
// (16 bytes per lane, no register staging), which lets STAGES-1 slices be in flight per
// workgroup instead of one, enough to cover HBM latency at 2-3 workgroups per CU.
//  * One such instruction fills 1 KB of LDS contiguously (lane i -> base + 16*i), i.e. 16 rows
//    of one 64-byte slice row each.  Rows are therefore unpadded; bank conflicts of the MFMA
//    fragment reads are avoided by an XOR swizzle of the four 16-byte slots of a row with
//    bits 2..3 of the row number - applied on the way in by choosing WHICH 16 bytes a lane
//    fetches, and on the way out by the fragment read address.
//  * Lanes whose element is padding (outside the image, past M / N / C) use an offset beyond
//    the buffer's num_records: the range check of the buffer load returns zeros for them.
//  * Waits are explicit: loads retire in order, so "at most (STAGES-2) slices outstanding"
//    means the oldest slice has landed.

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// Backward data with stride > 1 is split by the residue class (y % stride, x % stride) of the
// output pixel: inside a class the set of filter taps that reach a pixel is the same for all
// pixels (r = r0, r0+stride, ...), so a block of one class walks only those taps instead of
// multiplying the zeros of the others.  g.classes = stride*stride (1: no split); a class's
// pixels are numbered over the grid OHc x OWc = ceil(OH/stride) x ceil(OW/stride).
//
// The MFMA takes the filter tile as its first operand, so a lane ends up with 4 consecutive
// output CHANNELS of one pixel per accumulator group; v_permlane32_swap pairs the two halves
// of the wave and every lane stores (and, for beta != 0, loads) 16 contiguous bytes.

__device__ __forceinline__ unsigned pack2(float a, float b)
{
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v;
    v[0] = (_Float16)a;
    v[1] = (_Float16)b;
    return __builtin_bit_cast(unsigned, v);
}

// Reads the 32 channels nb .. nb+31 of this lane's pixel row the way the epilogue stores them
// (16 contiguous bytes per lane: the lower half-wave channels 16q .. 16q+7, the upper one
// 16q+8 .. 16q+15) and hands every lane the values of ITS accumulator elements: the same
// half-wave swap as on the way out undoes the regrouping.  All lanes must call it.
// f[v] belongs to channel nb + 8*(v/4) + 4*hi + v%4.
__device__ __forceinline__ void load_row32(const half_t *row, bool ok, int nb, int ncols, int hi, float (&f)[16])
{
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for(int q = 0; q < 2; q++) {
        const int n = nb + 16 * q + 8 * hi;
        u4 o = {0, 0, 0, 0};
        if(ok && n < ncols)
            o = *(const u4 *)(row + n);
        const auto s0 = __builtin_amdgcn_permlane32_swap(o[0], o[2], false, false);
        const auto s1 = __builtin_amdgcn_permlane32_swap(o[1], o[3], false, false);
        const unsigned w[4] = {s0[0], s1[0], s0[1], s1[1]}; // elements 8q .. 8q+7, two per word
#pragma unroll
        for(int e = 0; e < 4; e++) {
            const h2 v = __builtin_bit_cast(h2, w[e]);
            f[8 * q + 2 * e] = (float)v[0];
            f[8 * q + 2 * e + 1] = (float)v[1];
        }
    }
}

// One step of a halving exchange over n live values per lane: the lane with bit M set keeps
// the upper half, its partner the lower half, and each adds what the other held of its half.
// n is a template parameter so that every array index is a constant and the arrays stay in
// registers.  The partner only has to differ in bit M and agree in the bits above it (the bits
// below are exchanged by the later steps), which lets every step run in the vector ALU instead of
// going through the LDS crossbar (ds_bpermute):
//   M = 16: v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows
//           of the second, after which a lane's two results are its own and its partner's value of the
//           half it keeps (the results pass through an opaque statement: hipcc 7.2 otherwise folds the
//           sum of the two results of one swap into twice the first);
//   M = 8, 4: the partner is the mirror lane of the row of 16 / of the half row of 8 (DPP row_mirror,
//           row_half_mirror); M = 2, 1: the lane two / one away inside the quad (DPP quad_perm).
template <int CTRL> __device__ __forceinline__ float dpp_read(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int n, int M, int NV>
__device__ __forceinline__ void halve_exchange(float (&a)[NV], float (&b)[NV], int lane)
{
    static_assert(M == 16 || M == 8 || M == 4 || M == 2 || M == 1, "partner distance");
    if constexpr(M == 16) {
#pragma unroll
        for(int k = 0; k < n / 2; k++) {
            const auto ra = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, a[k]),
                                                             __builtin_bit_cast(unsigned, a[k + n / 2]), false, false);
            const auto rb = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, b[k]),
                                                             __builtin_bit_cast(unsigned, b[k + n / 2]), false, false);
            unsigned a0 = ra[0], a1 = ra[1], b0 = rb[0], b1 = rb[1];
            asm volatile("" : "+v"(a0), "+v"(a1), "+v"(b0), "+v"(b1));
            a[k] = __builtin_bit_cast(float, a0) + __builtin_bit_cast(float, a1);
            b[k] = __builtin_bit_cast(float, b0) + __builtin_bit_cast(float, b1);
        }
    } else {
        constexpr int CTRL = M == 8 ? 0x140 : M == 4 ? 0x141 : M == 2 ? 0x4e : 0xb1;
        const bool up = lane & M;
#pragma unroll
        for(int k = 0; k < n / 2; k++) {
            const float ka = up ? a[k + n / 2] : a[k], sa = up ? a[k] : a[k + n / 2];
            const float kb = up ? b[k + n / 2] : b[k], sb = up ? b[k] : b[k + n / 2];
            a[k] = ka + dpp_read<CTRL>(sa);
            b[k] = kb + dpp_read<CTRL>(sb);
        }
    }
}

// Everything the gather kernels do after their main loop: alpha / beta, the optional batch-norm
// inference fold (+ residual + relu), the 16-byte channel-vector stores and the optional per-channel
// statistics of the stored values.  acc[i][j][v] belongs to row wm + 32*i + lane%32 of the block tile
// and channel n0 + wn + 32*j + 8*(v/4) + 4*(lane/32) + v%4; rowpix(r, ok, pix) names the output pixel of
// row r of the block tile (ok false: nothing is stored).
// Where the output takes 16-byte vectors the values go out through LDS: a wavefront lays its 64x64 tile down
// row by row (128 bytes per row, 16-byte chunks XORed with the row number against bank conflicts) and reads
// it back with eight lanes per row, so that one store instruction writes eight whole 128-byte rows instead of
// 32-byte pieces of 32 rows.  Measured on MI355X at batch 256 (forward): 64 -> 256 channels over 56x56 pixels
// 135 -> 109 us with fully coalesced stores, 128 -> 512 over 28x28 86 -> 74 us.  MASK: rows that are not ok may hold
// non-zero accumulators and have to be kept out of the statistics.  smem: the block's LDS, free for
// reuse once every wavefront has left the main loop (the barriers inside see to that).
// whether gather_epilogue stores through LDS (the producer wavefronts of a block count its barriers)
// (not the 64-channel tiles: their rows are 128 bytes to begin with and the detour measured 3 - 7 % slower)
// Per-channel sum and sum of squares of a wavefront's outputs (as stored, i.e. rounded to fp16), for a batch
// normalisation that follows.  Columns past Ngemm hold zeros in the accumulators and add nothing; so do rows that
// are not ok unless MASK says they may hold anything, in which case they are left out here.  Lanes of one
// half-wave hold different pixels of the same channels: a halving exchange (each step swaps half of the values
// with the lane 16, 8, .. 1 away) leaves every lane - every even lane for 32-channel tiles - with the totals of
// one channel, stats_channel() of the wave tile.
template <int TM, int TN, bool MASK>
__device__ __forceinline__ void stats_lane_totals(float alpha, float16_t (&acc)[TM][TN], const bool (&okr)[TM], int lane,
                                                  float &s_out, float &q_out)
{
    constexpr int NV = TN * 16;
    static_assert(NV == 16 || NV == 32, "stats layout");
    float sv[NV], qv[NV];
#pragma unroll
    for(int j = 0; j < TN; j++)
#pragma unroll
        for(int v = 0; v < 16; v++) {
            float a = 0.0f, q = 0.0f;
            if constexpr(TM == 2) {
                // the two rows of a channel rounded to fp16 as they are stored, in one packed register;
                // sum and sum of squares are one two-element dot product each (fp32 result)
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                h2 pr;
                pr[0] = (!MASK || okr[0]) ? (_Float16)(alpha * acc[0][j][v]) : (_Float16)0;
                pr[1] = (!MASK || okr[1]) ? (_Float16)(alpha * acc[1][j][v]) : (_Float16)0;
                const h2 ones = {(_Float16)1, (_Float16)1};
                a = __builtin_amdgcn_fdot2(pr, ones, 0.0f, false);
                q = __builtin_amdgcn_fdot2(pr, pr, 0.0f, false);
            } else {
#pragma unroll
                for(int i = 0; i < TM; i++) {
                    const float r = (!MASK || okr[i]) ? (float)(half_t)(alpha * acc[i][j][v]) : 0.0f;
                    a += r;
                    q += r * r;
                }
            }
            sv[j * 16 + v] = a;
            qv[j * 16 + v] = q;
        }
    if constexpr(NV == 32) {
        halve_exchange<32, 16>(sv, qv, lane);
        halve_exchange<16, 8>(sv, qv, lane);
        halve_exchange<8, 4>(sv, qv, lane);
        halve_exchange<4, 2>(sv, qv, lane);
        halve_exchange<2, 1>(sv, qv, lane);
    } else {
        halve_exchange<16, 16>(sv, qv, lane);
        halve_exchange<8, 8>(sv, qv, lane);
        halve_exchange<4, 4>(sv, qv, lane);
        halve_exchange<2, 2>(sv, qv, lane);
        sv[0] += dpp_read<0xb1>(sv[0]);
        qv[0] += dpp_read<0xb1>(qv[0]);
    }
    s_out = sv[0];
    q_out = qv[0];
}

// The wavefronts stacked along M are added through LDS (red: WGM * BN pairs) in a fixed order and the block's
// [channel][2] row goes to g.stats[stats_row].  The caller has made sure that nobody still reads what red overlays.
template <int TN, int WGM, int WGN, int BN>
__device__ __forceinline__ void stats_block_write(const GatherArgs &g, char *red_mem, int tid, int lane, int wave, int wn,
                                                  int n0, int stats_row, float s0, float q0)
{
    constexpr int NV = TN * 16;
    const int hi = lane >> 5;
    const int idx = NV == 32 ? (lane & 31) : (lane & 31) >> 1;
    const int chl = 32 * (idx >> 4) + 8 * ((idx & 15) >> 2) + 4 * hi + (idx & 3); // channel inside the wave tile
    typedef float float2_t __attribute__((ext_vector_type(2)));
    float2_t *red = (float2_t *)red_mem;
    if(NV == 32 || (lane & 1) == 0) {
        float2_t v2 = {s0, q0};
        red[(wave / WGN) * BN + wn + chl] = v2;
    }
    __syncthreads();
    if(tid < BN && n0 + tid < g.Ngemm) {
        float2_t t = red[tid];
#pragma unroll
        for(int wy = 1; wy < WGM; wy++)
            t += red[wy * BN + tid];
        *(float2_t *)(g.stats + ((int64_t)stats_row * g.Ngemm + n0 + tid) * 2) = t;
    }
}

template <int TM, int TN, int BN, bool BWD> __device__ __forceinline__ bool stores_staged(const GatherArgs &g)
{
    const bool vec_ok = (g.ldo & 7) == 0 && (g.Ngemm & 7) == 0 && ((uintptr_t)g.out & 15) == 0;
    return TM == 2 && TN == 2 && BN >= 128 && vec_ok && !(BWD && g.classes > 1) && !g.no_stage;
}

// Inference with a folded batch norm: scale = s/sqrt(v+eps) and shift = b - m*scale of the block's BN channels
// as a table in LDS (bnp: 2 * BN floats).  The caller puts barriers around it.
template <int BN> __device__ __forceinline__ void bnfold_table(const GatherArgs &g, float *bnp, int tid, int n0)
{
    if(tid < BN) {
        const int n = n0 + tid;
        float sc = 0.0f, sh = 0.0f;
        if(n < g.Ngemm) {
            sc = g.bn_s[n] * rsqrtf(g.bn_v[n] + g.bn_eps);
            sh = g.bn_b[n] - g.bn_m[n] * sc;
        }
        bnp[tid] = sc;
        bnp[BN + tid] = sh;
    }
}

// BUFST: the direct 16-byte stores go through a range-checked buffer with an out-of-range offset for the lanes that
// have nothing to store, so that every wavefront issues the same number of store instructions whatever its rows
// (a caller that counts outstanding memory operations needs that).
template <int TM, int TN, int WGM, int WGN, int BN, bool BWD, bool MASK, bool BUFST = false, typename RowPix>
__device__ __forceinline__ void gather_epilogue(const GatherArgs &g, float16_t (&acc)[TM][TN], char *smem, int tid, int lane,
                                                int wave, int wm, int wn, int n0, int stats_row, RowPix rowpix)
{
    // (the table sits behind the tiles that the wavefronts stage their outputs in; the stage memory is free
    // after the last slice)
    float *bnp = (float *)(smem + WGM * WGN * TM * 32 * TN * 64);
    if constexpr(!BWD) {
        if(g.bn_s) {
            __syncthreads(); // every wavefront is done reading the last slice
            bnfold_table<BN>(g, bnp, tid, n0);
            __syncthreads();
        }
    }
    // acc[i][j][v]: pixel wm + 32*i + lane%32, channel wn + 32*j + 8*(v/4) + 4*(lane/32) + v%4
    const int hi = lane >> 5;
    bool okr[TM];
    const bool vec_ok = (g.ldo & 7) == 0 && (g.Ngemm & 7) == 0 && ((uintptr_t)g.out & 15) == 0;
    // through LDS (see above): this wavefront's 64 rows of 128 bytes
    constexpr bool CAN_STAGE = TM == 2 && TN == 2 && BN >= 128;
    const bool staged = stores_staged<TM, TN, BN, BWD>(g);
    char *stg = smem + wave * (TM * 32 * TN * 64);
    if(staged && !(!BWD && g.bn_s)) // (the fold's barriers have already seen to it)
        __syncthreads();           // every wavefront is done reading the last slice, which the tiles overwrite
#pragma unroll
    for(int i = 0; i < TM; i++) {
        bool ok;
        int64_t pix;
        rowpix(wm + i * 32 + (lane & 31), ok, pix);
        okr[i] = ok;
        half_t *orow = g.out + pix * g.ldo;
#pragma unroll
        for(int j = 0; j < TN; j++) {
            const int nb = n0 + wn + j * 32;
            if(vec_ok) {
                float f[16];
#pragma unroll
                for(int v = 0; v < 16; v++)
                    f[v] = g.alpha * acc[i][j][v];
                typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
                if(g.beta != 0.0f) {
                    float old[16];
                    load_row32(orow, ok, nb, g.Ngemm, hi, old);
#pragma unroll
                    for(int v = 0; v < 16; v++)
                        f[v] += g.beta * old[v];
                }
                if constexpr(!BWD) {
                    if(g.bn_s) {
                        float zz[16];
                        if(g.bn_flags & SAGA_BN_ADD)
                            load_row32(g.z + pix * g.ldz, ok, nb, g.Ngemm, hi, zz);
#pragma unroll
                        for(int q = 0; q < 4; q++) {
                            // scale and shift of the block's channels were put into LDS after the main loop
                            const int cl = wn + j * 32 + 8 * q + 4 * hi;
                            const float4_t sc = *(const float4_t *)(bnp + cl), sh = *(const float4_t *)(bnp + BN + cl);
#pragma unroll
                            for(int e = 0; e < 4; e++) {
                                float t = __builtin_fmaf(f[4 * q + e], sc[e], sh[e]);
                                if(g.bn_flags & SAGA_BN_ADD)
                                    t += zz[4 * q + e];
                                if(g.bn_flags & SAGA_BN_RELU)
                                    t = (t != t) ? t : fmaxf(t, 0.0f);
                                f[4 * q + e] = t;
                            }
                        }
                    }
                }
                // after the swaps: lower half-wave holds channels 0..7 (then 16..23) of the tile,
                // upper half-wave 8..15 (24..31): one store covers 32 contiguous bytes per pixel
#pragma unroll
                for(int q = 0; q < 2; q++) {
                    const unsigned x0 = pack2(f[8 * q + 0], f[8 * q + 1]), x1 = pack2(f[8 * q + 2], f[8 * q + 3]);
                    const unsigned y0 = pack2(f[8 * q + 4], f[8 * q + 5]), y1 = pack2(f[8 * q + 6], f[8 * q + 7]);
                    const auto s0_ = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
                    const auto s1_ = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
                    const int n = nb + 16 * q + 8 * hi;
                    typedef unsigned u4 __attribute__((ext_vector_type(4)));
                    const u4 o = {s0_[0], s1_[0], s0_[1], s1_[1]};
                    if constexpr(BUFST) {
                        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void *)g.out, 0, g.out_bytes, 0x00020000);
                        const unsigned off = (ok && n < g.Ngemm) ? (unsigned)((pix * g.ldo + n) * 2) : 0x7fffff00u;
                        __builtin_amdgcn_raw_buffer_store_b128(o, ro, off, 0, 0);
                    } else if(staged) {
                        const int row = i * 32 + (lane & 31), chunk = 4 * j + 2 * q + hi;
                        *(u4 *)(stg + row * (TN * 64) + ((chunk ^ (row & 7)) << 4)) = o;
                    } else if(ok && n < g.Ngemm) {
                        *(u4 *)(orow + n) = o;
                    }
                }
            } else if(ok) {
#pragma unroll
                for(int v = 0; v < 16; v++) {
                    const int n = nb + (v >> 2) * 8 + hi * 4 + (v & 3);
                    if(n >= g.Ngemm)
                        continue;
                    float val = g.alpha * acc[i][j][v];
                    if(g.beta != 0.0f)
                        val += g.beta * (float)orow[n];
                    if constexpr(!BWD) {
                        if(g.bn_s) {
                            const float sc = g.bn_s[n] * rsqrtf(g.bn_v[n] + g.bn_eps);
                            val = __builtin_fmaf(val, sc, g.bn_b[n] - g.bn_m[n] * sc);
                            if(g.bn_flags & SAGA_BN_ADD)
                                val += (float)g.z[pix * g.ldz + n];
                            if(g.bn_flags & SAGA_BN_RELU)
                                val = (val != val) ? val : fmaxf(val, 0.0f);
                        }
                    }
                    orow[n] = (half_t)val;
                }
            }
        }
    }
    if constexpr(CAN_STAGE) {
        if(staged) {
            // LDS operations of one wavefront complete in order: its reads below see its writes above
            typedef unsigned u4 __attribute__((ext_vector_type(4)));
            constexpr int CH = TN * 4, RPI_ = 64 / CH; // 16-byte chunks per row, rows per store instruction
            const int chunk = lane % CH;
            const int n = n0 + wn + chunk * 8;
            // (no residue classes here: the pixel number is the row number, and rows * pitch fits 31 bits)
            bool ok0;
            int64_t pix0;
            rowpix(wm + lane / CH, ok0, pix0);
            const int p0 = (int)pix0;
            const int sw = (chunk ^ ((lane / CH) & 7)) << 4; // RPI_ is a multiple of 8: the same for every row of the lane
            static_assert(RPI_ % 8 == 0, "swizzle period");
#pragma unroll
            for(int it = 0; it < TM * 32 / RPI_; it++) {
                const int row = it * RPI_ + lane / CH;
                const int p = p0 + it * RPI_;
                const u4 o = *(const u4 *)(stg + row * (TN * 64) + sw);
                if(p < g.M && n < g.Ngemm)
                    *(u4 *)(g.out + (p * g.ldo + n)) = o;
            }
        }
    }
    // Optional: per-channel sum and sum of squares of this block's outputs, for a batch normalisation that follows
    // (stats_lane_totals, stats_block_write).
    if constexpr(!BWD) {
        if(g.stats) {
            float s0, q0;
            stats_lane_totals<TM, TN, MASK>(g.alpha, acc, okr, lane, s0, q0);
            __syncthreads(); // every wavefront is done reading the last slice (and the folded norm's table)
            stats_block_write<TN, WGM, WGN, BN>(g, smem + WGM * WGN * TM * 32 * TN * 64, tid, lane, wave, wn, n0, stats_row,
                                                s0, q0);
        }
    }
}

// The epilogue of a backward-data launch linked to a batch norm's backward (GatherArgs::bq_*): alpha / beta,
// the norm's relu mask, the 16-byte channel-vector stores of the masked gradient and, per channel, the sums
// of that gradient and of gradient * (x - mean) over the block's rows.  Arguments as in gather_epilogue; the
// output must allow the vector stores.
// Registers decide how many blocks a CU holds, so the work is laid out to need few of them: first every
// accumulator is turned into the fp16 value an unlinked launch would store (two per register, half the
// accumulators' footprint); then the wave tile is walked one 32x32 sub-tile at a time, rows inside
// 32-channel columns, eight elements at a time, and the running sums are kept after the first step of the
// halving exchange (8 per lane and sum instead of 16).  okr / pixr: validity and pixel index of this lane's row
// in row block i (rows * pitch of either tensor fits 31 bits, checked on the host); xraw: bnbwd_prefetch's;
// bnp: bnbwd_table's.
typedef unsigned uint4_t __attribute__((ext_vector_type(4)));

// Mean, and the forward's scale and shift for the relu recompute, of the block's BN channels: written to LDS
// (behind the stage memory) by the first BN threads before the main loop, whose barriers publish it.
template <int BN> __device__ __forceinline__ void bnbwd_table(const GatherArgs &g, float *bnp, int tid, int n0)
{
    if(tid < BN) {
        const int n = n0 + tid;
        float mean = 0.0f, sc = 0.0f, sh = 0.0f;
        if(n < g.Ngemm) {
            mean = g.bq_mean[n];
            if(g.bq_relu) {
                sc = g.bq_s[n] * g.bq_invstd[n];
                sh = __builtin_fmaf(-mean, sc, g.bq_b[n]); // the forward's own expression
            }
        }
        bnp[tid] = mean;
        bnp[BN + tid] = sc;
        bnp[2 * BN + tid] = sh;
    }
}

// The norm's input for the linked epilogue below, fetched by the wavefront before its main loop so that the
// data is in registers when the epilogue starts (four dependent trips to memory per block otherwise, which
// nothing hides once every block of a CU reaches its epilogue at the same time): sub-tile t = j*TM + i
// (row block i, 32-channel column j), two 16-byte vectors each, as the stores of the epilogue are laid out.
template <int TM, int TN, int T0, int T1>
__device__ __forceinline__ void bnbwd_prefetch(const GatherArgs &g, int lane, int wn, int n0, const bool (&okr)[TM],
                                               const int (&pixr)[TM], uint4_t (&xraw)[TM * TN][2])
{
    const int hi = lane >> 5;
#pragma unroll
    for(int t = T0; t < T1; t++) {
        const int j = t / TM, i = t % TM;
        const half_t *row = g.bq_x + pixr[i] * g.bq_ldx;
#pragma unroll
        for(int q = 0; q < 2; q++) {
            const int n = n0 + wn + j * 32 + 16 * q + 8 * hi;
            const uint4_t z = {0, 0, 0, 0};
            xraw[t][q] = z;
            if(okr[i] && n < g.Ngemm)
                xraw[t][q] = *(const uint4_t *)(row + n);
        }
    }
}

template <int TM, int TN, int WGM, int WGN, int BN>
__device__ __forceinline__ void gather_epilogue_bnbwd(const GatherArgs &g, float16_t (&acc)[TM][TN], char *smem, int tid,
                                                      int lane, int wave, int wm, int wn, int n0, int stats_row,
                                                      const bool (&okr)[TM], const int (&pixr)[TM],
                                                      uint4_t (&xraw)[TM * TN][2], const float *bnp)
{
    typedef uint4_t u4;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const int hi = lane >> 5;
    // phase 1: pk[i][j][4q .. 4q+3] = channels 8q .. 8q+7 of this lane's accumulator elements, as stored
    unsigned pk[TM][TN][8];
#pragma unroll
    for(int j = 0; j < TN; j++)
#pragma unroll
        for(int i = 0; i < TM; i++) {
            float f[16];
#pragma unroll
            for(int v = 0; v < 16; v++)
                f[v] = g.alpha * acc[i][j][v];
            if(g.beta != 0.0f) {
                float old[16];
                load_row32(g.out + pixr[i] * g.ldo, okr[i], n0 + wn + j * 32, g.Ngemm, hi, old);
#pragma unroll
                for(int v = 0; v < 16; v++)
                    f[v] += g.beta * old[v];
            }
#pragma unroll
            for(int e = 0; e < 8; e++) {
                pk[i][j][e] = pack2(f[2 * e], f[2 * e + 1]);
                asm volatile("" : "+v"(pk[i][j][e])); // converted here and now: the accumulator is dead from here on
            }
        }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads(); // the parameter table is complete (a block may have had no main-loop barrier to publish it)
    // phase 2
    float sres[TN], qres[TN];
    float sv[8], qv[8];
#pragma unroll
    for(int t = 0; t < TM * TN; t++) {
        const int j = t / TM, i = t % TM;
        const int nb = n0 + wn + j * 32;
        const bool ok = okr[i];
        const u4 (&cur)[2] = xraw[t];
        if(i == 0) {
#pragma unroll
            for(int v = 0; v < 8; v++)
                sv[v] = qv[v] = 0.0f;
        }
        // the norm's input in accumulator order (the same half-wave swap as on the way out, undone):
        // wx[c][2*(e/2) .. ] holds elements 8c + 2*ee, 8c + 2*ee + 1 in word ee
        unsigned wx[2][4];
#pragma unroll
        for(int c = 0; c < 2; c++) {
            const auto s0 = __builtin_amdgcn_permlane32_swap(cur[c][0], cur[c][2], false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(cur[c][1], cur[c][3], false, false);
            wx[c][0] = s0[0]; wx[c][1] = s1[0]; wx[c][2] = s0[1]; wx[c][3] = s1[1];
        }
        // Elements are handled eight at a time: the four of channel group q = half and the four of group
        // q + 2, which are the partners of the first step of the halving exchange (element k with k + 8; the
        // lane with bit 16 set keeps the upper one, its partner 16 lanes away the lower one) - that step is
        // folded into the running sums right away, so only eight gradients and products are live at a time.
#pragma unroll
        for(int half = 0; half < 2; half++) {
            float gf[2][4], gq[2][4];
#pragma unroll
            for(int side = 0; side < 2; side++) {
                const int q = half + 2 * side;
                // the table is read again for every sub-tile (the opaque index keeps the compiler from holding
                // a column's 48 parameters in registers across its rows)
                int cl = wn + j * 32 + 8 * q + 4 * hi;
                asm volatile("" : "+v"(cl));
                const float4_t mean = *(const float4_t *)(bnp + cl), sc = *(const float4_t *)(bnp + BN + cl),
                               sh = *(const float4_t *)(bnp + 2 * BN + cl);
#pragma unroll
                for(int e2 = 0; e2 < 2; e2++) {
                    const unsigned word = pk[i][j][2 * q + e2];
                    const h2 hv = __builtin_bit_cast(h2, word), xv = __builtin_bit_cast(h2, wx[side][2 * half + e2]);
                    unsigned keep = 0;
#pragma unroll
                    for(int h = 0; h < 2; h++) {
                        const int e = 2 * e2 + h;
                        const float xe = (float)xv[h];
                        const bool pos = !g.bq_relu || (float)(half_t)__builtin_fmaf(xe, sc[e], sh[e]) > 0.0f;
                        const bool on = ok && pos;
                        keep |= on ? (h ? 0xffff0000u : 0x0000ffffu) : 0u;
                        const float gv = on ? (float)hv[h] : 0.0f;
                        gf[side][e] = gv;
                        gq[side][e] = gv * (xe - mean[e]);
                    }
                    pk[i][j][2 * q + e2] = word & keep;
                }
            }
            // v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of the
            // second: afterwards the two operands of a lane add up to what it keeps plus what its partner sent
#pragma unroll
            for(int e = 0; e < 4; e++) {
                const auto a = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, gf[0][e]),
                                                                __builtin_bit_cast(unsigned, gf[1][e]), false, false);
                const auto b = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, gq[0][e]),
                                                                __builtin_bit_cast(unsigned, gq[1][e]), false, false);
                // (the four results go through an opaque statement: hipcc 7.2 otherwise folds the sum of the
                // two results of one swap into twice the first)
                unsigned a0 = a[0], a1 = a[1], b0 = b[0], b1 = b[1];
                asm volatile("" : "+v"(a0), "+v"(a1), "+v"(b0), "+v"(b1));
                sv[4 * half + e] += __builtin_bit_cast(float, a0) + __builtin_bit_cast(float, a1);
                qv[4 * half + e] += __builtin_bit_cast(float, b0) + __builtin_bit_cast(float, b1);
            }
            // added here and now (left to itself the compiler postpones the additions to the end of the column
            // and keeps every exchanged value in a register until then)
#pragma unroll
            for(int e = 0; e < 4; e++)
                asm volatile("" : "+v"(sv[4 * half + e]), "+v"(qv[4 * half + e]));
            __builtin_amdgcn_sched_barrier(0);
        }
        // after the swaps: lower half-wave holds channels 0..7 (then 16..23) of the tile,
        // upper half-wave 8..15 (24..31): one store covers 32 contiguous bytes per pixel
        half_t *orow = g.out + pixr[i] * g.ldo;
#pragma unroll
        for(int q = 0; q < 2; q++) {
            const auto s0_ = __builtin_amdgcn_permlane32_swap(pk[i][j][4 * q + 0], pk[i][j][4 * q + 2], false, false);
            const auto s1_ = __builtin_amdgcn_permlane32_swap(pk[i][j][4 * q + 1], pk[i][j][4 * q + 3], false, false);
            const int n = nb + 16 * q + 8 * hi;
            if(ok && n < g.Ngemm) {
                const u4 o = {s0_[0], s1_[0], s0_[1], s1_[1]};
                *(u4 *)(orow + n) = o;
            }
        }
        if(i == TM - 1) {
            // lanes of a half-wave hold different pixels of the same 16 channels: after the remaining halving
            // exchanges each pair of lanes holds one channel's total over the wave tile's rows
            halve_exchange<8, 8>(sv, qv, lane);
            halve_exchange<4, 4>(sv, qv, lane);
            halve_exchange<2, 2>(sv, qv, lane);
            sres[j] = sv[0] + dpp_read<0xb1>(sv[0]);
            qres[j] = qv[0] + dpp_read<0xb1>(qv[0]);
        }
        __builtin_amdgcn_sched_barrier(0); // one sub-tile at a time: interleaving them costs registers
    }
    // pair p = (lane%32)/2 holds, per column j, channel 32*j + 8*(p/4) + 4*hi + p%4 of the wave tile;
    // the wavefronts stacked along M are added through LDS in a fixed order
    typedef float float2_t __attribute__((ext_vector_type(2)));
    float2_t *red = (float2_t *)smem;
    const int p = (lane & 31) >> 1;
    __syncthreads(); // every wavefront is done reading the last slice, which the sums below overwrite
    if((lane & 1) == 0) {
#pragma unroll
        for(int j = 0; j < TN; j++) {
            const float2_t v2 = {sres[j], qres[j]};
            red[(wave / WGN) * BN + wn + 32 * j + 8 * (p >> 2) + 4 * hi + (p & 3)] = v2;
        }
    }
    __syncthreads();
    if(tid < BN && n0 + tid < g.Ngemm) {
        float2_t t = red[tid];
#pragma unroll
        for(int wy = 1; wy < WGM; wy++)
            t += red[wy * BN + tid];
        *(float2_t *)(g.bq_partial + ((int64_t)stats_row * g.Ngemm + n0 + tid) * 2) = t;
    }
}

template <int BM, int BN, int WGM, int WGN, int STAGES, int BKT, bool BWD, int PROD = 0, bool BQ = false>
__global__ void __launch_bounds__(64 * (WGM * WGN + PROD), (BQ && WGM * WGN + PROD == 8) ? 4 : PROD ? (WGM * WGN + PROD + 3) / 4 : 1)
    conv_gather_gemm_dma(GatherArgs g)
{
    constexpr int NW = WGM * WGN;                      // wavefronts per block
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int ROWB = BKT * 2;                      // bytes per LDS row (64 or 128)
    constexpr int SLOTS = ROWB / 16;                   // 16-byte slots per row
    constexpr int RPI = 64 / SLOTS;                    // rows one load instruction fills
    constexpr int RPR = RPI * NW;                      // tile rows one round of loads fills
    constexpr int AV = BM / RPR, BV = BN / RPR;
    constexpr int STAGE_BYTES = (BM + BN) * ROWB;
    constexpr unsigned OOB = 0x7fffff00u;
    static_assert((BKT == 32 || BKT == 64) && RPR % 16 == 0 && AV >= 1 && BV >= 1 && TM >= 1 && TN >= 1, "layout");
    // slot swizzle of a row: 64-byte rows alternate between four bank quarters, so rows
    // 4 apart need different slots; 128-byte rows between two halves, rows 2 apart do
    auto swz_of = [](int row) { return SLOTS == 4 ? (row >> 2) & 3 : (row >> 1) & 7; };

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bid = xcd_remap(blockIdx.x, g.nblocks);
    int py = 0, px = 0, r0 = 0, s0 = 0, nr = g.R, ns = g.S, rstep = 1;
    int PH = g.OH, PW = g.OW; // pixel grid this block's rows are numbered over
    int srow0 = 0;            // first row of this block's class in the per-row sums
    if(BWD && g.classes > 1) {
        // the classes of one tile position are neighbours in block order: they read the same
        // rows of dy and write interleaved pixels of the same rows of dx, which L2 then shares
        const int ci = bid % g.nactive;
        bid /= g.nactive;
        const int cls = g.cls_ids[ci];
        srow0 = ci * (g.blocks_per_class / g.nblk_n);
        py = cls >> g.sshift;
        px = cls & (g.stride - 1);
        r0 = (py + g.pad) & (g.stride - 1);
        s0 = (px + g.pad) & (g.stride - 1);
        nr = r0 < g.R ? (g.R - r0 + g.stride - 1) >> g.sshift : 0;
        ns = s0 < g.S ? (g.S - s0 + g.stride - 1) >> g.sshift : 0;
        rstep = g.stride;
        PH = g.OHc;
        PW = g.OWc;
    }
    const int bm = bid / g.nblk_n, bn = bid - bm * g.nblk_n;
    const int m0 = bm * BM, n0 = bn * BN;
    const int Mloc = BWD ? g.Mc : g.M;

    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void *)g.a, 0, g.a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void *)g.b, 0, g.b_bytes, 0x00020000);

    // Address generation is hoisted out of the main loop: the input position of tap (ri, si)
    // is (iy0 + ri*sy, ix0 + si*sy), sy = dil forward and -1 backward (inside a residue class
    // consecutive taps are one input row / column apart), so a row's byte offset is
    // rowoff + a term that is the same for every lane (kept in scalar registers), and which
    // taps fall inside the image is one bit each of a 64-bit mask computed once per row.
    const int sy = BWD ? -1 : g.dil;
    // a 1x1 filter of stride 1 without padding reads input pixel m for output pixel m: no decoding, one tap
    const bool plain = g.R == 1 && g.S == 1 && g.pad == 0 && g.stride == 1 && g.IH == g.OH && g.IW == g.OW;
    auto row_setup = [&](int m, int kvv, int &ro, unsigned long long &mask) {
        bool ok = m < Mloc;
        if(plain) {
            ro = ((ok ? m : 0) * g.lda + kvv) * 2;
            mask = ok ? 1ull : 0ull;
            return;
        }
        const int mm = ok ? m : 0;
        const int ox = mm % PW;
        const int t = mm / PW;
        const int oy = t % PH;
        const int n = t / PH;
        int iy0, ix0;
        if(BWD) {
            const int y = oy * rstep + py, x = ox * rstep + px;
            ok = ok && y < g.OH && x < g.OW;
            iy0 = (y + g.pad - r0) >> g.sshift;
            ix0 = (x + g.pad - s0) >> g.sshift;
        } else {
            iy0 = oy * g.stride - g.pad;
            ix0 = ox * g.stride - g.pad;
        }
        ro = (((n * g.IH + iy0) * g.IW + ix0) * g.lda + kvv) * 2;
        unsigned long long mk = 0;
        if(ok)
            for(int a = 0; a < nr; a++) {
                const int iy = iy0 + a * sy;
                if(iy < 0 || iy >= g.IH)
                    continue;
                for(int b = 0; b < ns; b++) {
                    const int ix = ix0 + b * sy;
                    if(ix >= 0 && ix < g.IW)
                        mk |= 1ull << (a * ns + b);
                }
            }
        mask = mk;
    };
    const int ktot = g.R * g.S * g.Cred;
    const int csteps = (g.Cred + BKT - 1) / BKT;
    const int KT = nr * ns * csteps;
    const bool ragged = g.Cred % BKT != 0;
    int ri = 0, si = 0, c0 = 0; // tap counters and channel offset of the NEXT slice to be issued

    // With PROD > 0 the block has PROD extra wavefronts that do nothing but issue the loads:
    // a load-to-LDS instruction holds its wavefront at issue until the memory pipeline takes
    // it, and in a wavefront that also feeds the matrix unit that wait is lost matrix time.
    // Producers and consumers meet at one barrier per reduction slice: after barrier kt
    // slice kt is in LDS and the stage of slice kt-1 is free for slice kt+STAGES-1.
    if constexpr(PROD > 0) {
        static_assert(BKT == 32 && (BM / 16) % PROD == 0 && (BN / 16) % PROD == 0, "producer split");
        if(wave >= NW) {
            constexpr int PA = BM / 16 / PROD, PB = BN / 16 / PROD; // 16-row pieces per producer
            const int pw = wave - NW;
            const int prow = lane >> 2;
            const int pkv = ((lane & 3) ^ swz_of(prow)) * 8;
            int ro[PA], bo[PB];
            unsigned long long mk[PA];
            bool bok[PB];
#pragma unroll
            for(int i = 0; i < PA; i++)
                row_setup(m0 + (pw * PA + i) * 16 + prow, pkv, ro[i], mk[i]);
#pragma unroll
            for(int i = 0; i < PB; i++) {
                const int n = n0 + (pw * PB + i) * 16 + prow;
                bok[i] = n < g.Ngemm;
                bo[i] = ((bok[i] ? n : 0) * ktot + pkv) * 2;
            }
            // Per tap: the byte offset of every piece this lane loads, or OOB where the tap falls outside
            // the image or the row / column lies beyond the tensor; the slice's channel offset rides in
            // the load's scalar offset.  Only a channel count that is no multiple of the slice depth makes
            // the offsets depend on the slice (its last slice per tap is ragged): then they are rebuilt
            // for every slice.
            unsigned av[PA], bv[PB];
            auto tap_setup = [&]() {
                const bool cok = !ragged || c0 + pkv < g.Cred;
                const int tapoff = ((ri * g.IW + si) * sy * g.lda) * 2; // same for all lanes
                const int tap = ri * ns + si;
#pragma unroll
                for(int i = 0; i < PA; i++)
                    av[i] = (cok && ((mk[i] >> tap) & 1)) ? (unsigned)(ro[i] + tapoff) : OOB;
                const int r = r0 + ri * rstep, s = s0 + si * rstep;
                const int kb = (r * g.S + s) * g.Cred * 2;
#pragma unroll
                for(int i = 0; i < PB; i++)
                    bv[i] = (bok[i] && cok) ? (unsigned)(bo[i] + kb) : OOB;
            };
            auto step_cursor = [&]() {
                bool newtap = false;
                c0 += BKT;
                if(c0 >= g.Cred) {
                    c0 = 0;
                    newtap = true;
                    if(++si == ns) {
                        si = 0;
                        ++ri;
                    }
                }
                if((newtap || ragged) && ri < nr)
                    tap_setup();
            };
            auto produce = [&](int stage) {
                char *sa = smem + stage * STAGE_BYTES + pw * PA * 16 * ROWB;
                char *sb = smem + stage * STAGE_BYTES + BM * ROWB + pw * PB * 16 * ROWB;
                const int koff = c0 * 2;
#pragma unroll
                for(int i = 0; i < PA; i++) {
                    const unsigned off = av[i]; // (a captured array element passed directly makes the host pass drop the kernel)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(sa + i * 16 * ROWB), 16, off, koff, 0, 0);
                }
#pragma unroll
                for(int i = 0; i < PB; i++) {
                    const unsigned off = bv[i];
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(sb + i * 16 * ROWB), 16, off, koff, 0, 0);
                }
                step_cursor();
            };
            if(KT > 0)
                tap_setup();
#pragma unroll
            for(int st = 0; st < STAGES - 1; st++)
                if(st < KT)
                    produce(st);
            // unrolled by the stage count: every stage address is a constant
            for(int kt0 = 0; kt0 < KT; kt0 += STAGES) {
#pragma unroll
                for(int u = 0; u < STAGES; u++) {
                    const int kt = kt0 + u;
                    if(kt >= KT)
                        break;
                    if(kt + STAGES - 2 < KT)
                        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((PA + PB) * (STAGES - 2)) : "memory");
                    else
                        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
                    if(kt + STAGES - 1 < KT)
                        produce((u + STAGES - 1) % STAGES);
                }
            }
            if constexpr(!BQ) {
                if(!BWD && g.bn_s) { // the two barriers around the folded batch norm's parameter table
                    __syncthreads();
                    __syncthreads();
                } else if(stores_staged<TM, TN, BN, BWD>(g)) { // the one in front of the output tiles in LDS
                    __syncthreads();
                }
                if(!BWD && g.stats) { // the two barriers of the statistics epilogue
                    __syncthreads();
                    __syncthreads();
                }
            }
            if constexpr(BQ) { // the parameter table's barrier and the two of the sums
                __syncthreads();
                __syncthreads();
                __syncthreads();
            }
            return;
        }
    }

    // (PROD == 0) this lane fills slot (tid % SLOTS) of row lrow (+RPR per round) and fetches
    // the logical channel vector that the swizzle assigns to that slot
    const int lrow = tid / SLOTS;
    const int kv = ((tid % SLOTS) ^ swz_of(lrow)) * 8;
    int rowoff[AV];
    unsigned long long amask[AV];
    int b_off[BV];
    bool b_ok[BV];
    if constexpr(PROD == 0) {
#pragma unroll
        for(int j = 0; j < AV; j++)
            row_setup(m0 + lrow + RPR * j, kv, rowoff[j], amask[j]);
#pragma unroll
        for(int j = 0; j < BV; j++) {
            const int n = n0 + lrow + RPR * j;
            b_ok[j] = n < g.Ngemm;
            b_off[j] = ((b_ok[j] ? n : 0) * ktot + kv) * 2;
        }
    }

    // one slice = AV + BV load instructions ("pieces"); issue_piece(stage, p) emits piece p of
    // the next slice, step_cursor() moves on once all its pieces are out.  As in the producer
    // branch the per-lane offsets are fixed per tap and the slice's channel offset is scalar.
    unsigned av[AV], bv[BV];
    auto tap_setup = [&]() {
        const bool cok = !ragged || c0 + kv < g.Cred;
        const int tapoff = ((ri * g.IW + si) * sy * g.lda) * 2; // same for all lanes
        const int tap = ri * ns + si;
#pragma unroll
        for(int j = 0; j < AV; j++)
            av[j] = (cok && ((amask[j] >> tap) & 1)) ? (unsigned)(rowoff[j] + tapoff) : OOB;
        const int r = r0 + ri * rstep, s = s0 + si * rstep;
        const int kb = (r * g.S + s) * g.Cred * 2;
#pragma unroll
        for(int j = 0; j < BV; j++)
            bv[j] = (b_ok[j] && cok) ? (unsigned)(b_off[j] + kb) : OOB;
    };
    auto step_cursor = [&]() {
        bool newtap = false;
        c0 += BKT;
        if(c0 >= g.Cred) {
            c0 = 0;
            newtap = true;
            if(++si == ns) {
                si = 0;
                ++ri;
            }
        }
        if((newtap || ragged) && ri < nr)
            tap_setup();
    };
    auto issue_piece = [&](int stage, int p) {
        char *sa = smem + stage * STAGE_BYTES;
        char *sb = sa + BM * ROWB;
        const int koff = c0 * 2;
        // (the offset goes through a local: a captured array element passed directly makes the host pass drop the kernel)
        if(p < AV) {
            const unsigned off = av[p];
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(sa + (p * RPR + wave * RPI) * ROWB), 16, off, koff, 0, 0);
        } else {
            const unsigned off = bv[p - AV];
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(sb + ((p - AV) * RPR + wave * RPI) * ROWB), 16, off, koff, 0, 0);
        }
    };
    auto issue = [&](int stage) {
#pragma unroll
        for(int p = 0; p < AV + BV; p++)
            issue_piece(stage, p);
        step_cursor();
    };

    float16_t acc[TM][TN];
#pragma unroll
    for(int i = 0; i < TM; i++)
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][j][v] = 0.0f;

    const int wm = (wave / WGN) * WTM, wn = (wave % WGN) * WTN;
    auto rowpix = [&](int mrow, bool &ok, int64_t &pix) {
        const int m = m0 + mrow;
        ok = m < Mloc;
        pix = m;
        if(BWD && g.classes > 1) {
            const int mm = ok ? m : 0;
            const int ox = mm % PW;
            const int t = mm / PW;
            const int oy = t % PH;
            const int n = t / PH;
            const int y = oy * rstep + py, x = ox * rstep + px;
            ok = ok && y < g.OH && x < g.OW;
            pix = ((int64_t)n * g.OH + y) * g.OW + x;
        }
    };
    // linked to a batch norm's backward: that norm's input for this wavefront's tile is requested now and
    // arrives while the main loop runs
    bool bq_ok[BQ ? TM : 1];
    int bq_pix[BQ ? TM : 1];
    uint4_t bq_x[BQ ? TM * TN : 1][2];
    float *bq_tab = (float *)(smem + STAGES * (BM + BN) * BKT * 2);
    if constexpr(BQ) {
#pragma unroll
        for(int i = 0; i < TM; i++) {
            int64_t pix;
            rowpix(wm + i * 32 + (lane & 31), bq_ok[i], pix);
            bq_pix[i] = (int)pix;
        }
        bnbwd_table<BN>(g, bq_tab, tid, n0);
        // (wavefronts that also issue the main loop's loads have no registers to spare: they ask after the loop)
        if constexpr(PROD > 0)
            bnbwd_prefetch<TM, TN, 0, TM * TN>(g, lane, wn, n0, bq_ok, bq_pix, bq_x);
    }
    const int frow = lane & 31;
    const int swz = swz_of(frow);
    // byte offset inside a row of this lane's fragment vector for MFMA step kk (k = 16*kk ..)
    constexpr int KS = BKT / 16;
    int fo[KS];
#pragma unroll
    for(int kk = 0; kk < KS; kk++)
        fo[kk] = ((2 * kk + (lane >> 5)) ^ swz) * 16;

    if constexpr(PROD == 0) {
        if(KT > 0)
            tap_setup();
#pragma unroll
        for(int st = 0; st < STAGES - 1; st++)
            if(st < KT)
                issue(st);
    }

    constexpr int NP = PROD ? 0 : AV + BV, NQ = KS * TM * TN; // load pieces and MFMAs per iteration
    // unrolled by the stage count: the stage a slice is read from and the one the next loads go to are
    // constants, so the LDS addresses are one register per operand and k-step plus immediate offsets
    for(int kt0 = 0; kt0 < KT; kt0 += STAGES) {
#pragma unroll
        for(int u = 0; u < STAGES; u++) {
            const int kt = kt0 + u;
            if(kt >= KT)
                break;
            // oldest outstanding slice = kt; newer ones may stay in flight
            // (a plain __syncthreads() would make the compiler drain every outstanding load)
            if constexpr(PROD > 0)
                asm volatile("s_barrier" ::: "memory");
            else if(kt + STAGES - 2 < KT)
                asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(NP * (STAGES - 2)) : "memory");
            else
                asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
            const bool more = !PROD && kt + STAGES - 1 < KT;
            const int nst = (u + STAGES - 1) % STAGES;
            const char *sa = smem + u * STAGE_BYTES;
            const char *sb = sa + BM * ROWB;
            half8_t fa[KS][TM], fb[KS][TN];
#pragma unroll
            for(int kk = 0; kk < KS; kk++) {
#pragma unroll
                for(int i = 0; i < TM; i++)
                    fa[kk][i] = *(const half8_t *)(sa + (wm + i * 32 + frow) * ROWB + fo[kk]);
#pragma unroll
                for(int j = 0; j < TN; j++)
                    fb[kk][j] = *(const half8_t *)(sb + (wn + j * 32 + frow) * ROWB + fo[kk]);
            }
            // the next slice's loads go out between the MFMAs, so that a load waiting for the
            // memory pipeline does not hold back this wavefront's matrix work
#pragma unroll
            for(int q = 0; q < NQ; q++) {
                const int kk = q / (TM * TN), i = (q / TN) % TM, j = q % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk][j], fa[kk][i], acc[i][j], 0, 0, 0);
#pragma unroll
                for(int p = 0; p < NP; p++)
                    if(q == (p * NQ) / (NP ? NP : 1)) {
                        __builtin_amdgcn_sched_barrier(0);
                        if(more)
                            issue_piece(nst, p);
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
            if(more)
                step_cursor();
        }
    }

    if constexpr(BQ && PROD == 0)
        bnbwd_prefetch<TM, TN, 0, TM * TN>(g, lane, wn, n0, bq_ok, bq_pix, bq_x);
    if constexpr(BQ)
        gather_epilogue_bnbwd<TM, TN, WGM, WGN, BN>(g, acc, smem, tid, lane, wave, wm, wn, n0, srow0 + bm, bq_ok, bq_pix,
                                                    bq_x, bq_tab);
    else
        gather_epilogue<TM, TN, WGM, WGN, BN, BWD, false>(g, acc, smem, tid, lane, wave, wm, wn, n0, bm, rowpix);
}

// Many filters in one launch: job j owns the blocks first_block[j] .. first_block[j+1]-1, one block per
// (tap, 64 output channels, 64 input channels) tile, transposed through LDS with 16-byte accesses on both
// sides where K and C are multiples of 8 (element by element otherwise).
__global__ void __launch_bounds__(256) transpose_filter_batched(const SagaFilterTransposeJob *__restrict__ jobs, int njobs)
{
    __shared__ half_t tile[64][72];
    int lo = 0, hi = njobs - 1;
    const int b = blockIdx.x;
    while(lo < hi) { // last job whose first block is <= b
        const int mid = (lo + hi + 1) >> 1;
        if(jobs[mid].first_block <= b)
            lo = mid;
        else
            hi = mid - 1;
    }
    const SagaFilterTransposeJob job = jobs[lo];
    const half_t *__restrict__ w = (const half_t *)job.w;
    half_t *__restrict__ wt = (half_t *)job.wt;
    const int K = job.K, C = job.C, RS = job.RS;
    const int tk = (K + 63) / 64, tc = (C + 63) / 64;
    int r = b - job.first_block;
    const int c0 = (r % tc) * 64;
    r /= tc;
    const int k0 = (r % tk) * 64, tap = r / tk;
    const int t = threadIdx.x;
    const bool vec = ((K | C) & 7) == 0 && (((uintptr_t)w | (uintptr_t)wt) & 15) == 0;
    if(vec) {
#pragma unroll
        for(int pass = 0; pass < 2; pass++) {
            const int row = pass * 32 + (t >> 3), col = (t & 7) * 8;
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if(k0 + row < K && c0 + col < C)
                v = *(const half8_t *)(w + ((int64_t)(k0 + row) * RS + tap) * C + c0 + col);
            *(half8_t *)&tile[row][col] = v;
        }
        __syncthreads();
#pragma unroll
        for(int pass = 0; pass < 2; pass++) {
            const int row = pass * 32 + (t >> 3), col = (t & 7) * 8; // row: input channel, col: first of 8 output channels
            if(c0 + row < C && k0 + col < K) {
                half8_t v;
#pragma unroll
                for(int e = 0; e < 8; e++)
                    v[e] = tile[col + e][row];
                *(half8_t *)(wt + ((int64_t)(c0 + row) * RS + tap) * K + k0 + col) = v;
            }
        }
    } else {
        for(int i = t; i < 64 * 64; i += 256) {
            const int c = c0 + (i >> 6), k = k0 + (i & 63);
            if(c < C && k < K)
                wt[((int64_t)c * RS + tap) * K + k] = w[((int64_t)k * RS + tap) * C + c];
        }
    }
}

// w (K, C, R, S logical; stored K,R,S,C) -> wT stored C,R,S,K
__global__ void __launch_bounds__(256) transpose_filter(const half_t *__restrict__ w, half_t *__restrict__ wt, int K, int C, int RS)
{
    const int64_t total = (int64_t)K * C * RS;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        // i enumerates the destination: (c, tap, k) with k fastest
        const int k = (int)(i % K);
        const int tap = (int)((i / K) % RS);
        const int c = (int)(i / ((int64_t)K * RS));
        wt[i] = w[((int64_t)k * RS + tap) * C + c];
    }
}


// ---------------------------------------------------------------- backward filter
//
// dw[k, tap, c] = sum_m dy[m, k] * x[pix(m, tap), c].  Both operands arrive with the
// reduction index m as the SLOW axis (rows of channels), while the MFMA wants, per lane,
// eight consecutive reduction elements of one row.  The tiles are therefore transposed on
// their way into LDS: each thread loads 16 bytes = 8 channels of one pixel and scatters
// them with eight 2-byte LDS writes into [channel][pixel] rows.  Channel ch of a tile
// is placed in LDS row (ch % 8) * NV + ch / 8 (NV = channel vectors per tile): with that
// permutation the 64 lanes of one write hit 64 different banks, and the epilogue simply
// undoes it when it writes the result.
// The reduction is split over `splits` blocks per output tile; every block writes an fp32
// partial tile to the workspace and a second kernel adds the partials in a fixed order
// (deterministic, no atomics) and applies alpha/beta.

struct FilterArgs {
    const half_t *x;
    const half_t *dy;
    float *partial;    // [splits][K][RSC]
    int M;             // N * P * Q
    int K, C, RSC;
    int H, W, P, Q, S;
    int pad, stride, dil;
    int ldx, ldy;
    int tiles_k, tiles_c;
    int splits, m_per_split; // m_per_split is a multiple of BK
};

template <int BM, int BN>
__global__ void __launch_bounds__(256) conv_bwd_filter_mfma(FilterArgs g)
{
    constexpr int NVA = BM / 8, NVB = BN / 8;           // channel vectors per tile
    constexpr int PA = 256 / NVA, PB = 256 / NVB;       // pixels covered per round
    constexpr int RA = BK / PA, RB = BK / PB;           // rounds per slice
    constexpr int WGM = BM >= 128 ? 2 : 1, WGN = 4 / WGM;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(RA >= 1 && RB >= 1 && TM >= 1 && TN >= 1, "tile");

    __shared__ __attribute__((aligned(16))) half_t As[2][BM * LDK];
    __shared__ __attribute__((aligned(16))) half_t Bs[2][BN * LDK];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int b = blockIdx.x;
    const int split = b % g.splits;
    b /= g.splits;
    const int tc = b % g.tiles_c, tk = b / g.tiles_c;
    const int k0 = tk * BM, j0 = tc * BN;
    const int m_begin = split * g.m_per_split;
    int m_end = m_begin + g.m_per_split;
    if(m_end > g.M)
        m_end = g.M;

    // A operand (dy): channel vector cva, pixel slots pa(j) = 2*ga + j  (RA == 2) or ga (RA == 1)
    const int cva = tid % NVA, ga = tid / NVA;
    const bool ka_ok = k0 + cva * 8 < g.K;
    // B operand (x): column vector -> fixed (tap, c) for this thread
    const int cvb = tid % NVB, gb = tid / NVB;
    const int col = j0 + cvb * 8;
    const bool cb_ok = col < g.RSC;
    const int tap = cb_ok ? col / g.C : 0;
    const int cc = cb_ok ? col - tap * g.C : 0;
    const int fr = tap / g.S, fs = tap - fr * g.S;
    const int offy = fr * g.dil - g.pad, offx = fs * g.dil - g.pad;

    // pixel coordinates of this thread's B rows, advanced incrementally by BK per slice
    int bn_[RB], by_[RB], bx_[RB];
#pragma unroll
    for(int j = 0; j < RB; j++) {
        const int pm = RB == 1 ? gb : gb * RB + j;
        const int m = m_begin + pm;
        const int mm = m < g.M ? m : 0;
        bx_[j] = mm % g.Q;
        const int t = mm / g.Q;
        by_[j] = t % g.P;
        bn_[j] = t / g.P;
    }

    half8_t ra[RA], rb[RB];
    const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    auto load_slice = [&](int ms) {
#pragma unroll
        for(int j = 0; j < RA; j++) {
            const int pm = RA == 1 ? ga : ga * RA + j;
            const int m = ms + pm;
            ra[j] = zero;
            if(ka_ok && m < m_end)
                ra[j] = *(const half8_t *)(g.dy + (int64_t)m * g.ldy + k0 + cva * 8);
        }
#pragma unroll
        for(int j = 0; j < RB; j++) {
            const int pm = RB == 1 ? gb : gb * RB + j;
            const int m = ms + pm;
            const int iy = by_[j] * g.stride + offy, ix = bx_[j] * g.stride + offx;
            rb[j] = zero;
            if(cb_ok && m < m_end && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W)
                rb[j] = *(const half8_t *)(g.x + (int64_t)((bn_[j] * g.H + iy) * g.W + ix) * g.ldx + cc);
        }
    };
    auto advance = [&]() {
#pragma unroll
        for(int j = 0; j < RB; j++) {
            bx_[j] += BK;
            while(bx_[j] >= g.Q) {
                bx_[j] -= g.Q;
                by_[j]++;
            }
            while(by_[j] >= g.P) {
                by_[j] -= g.P;
                bn_[j]++;
            }
        }
    };
    auto store_slice = [&](int st) {
#pragma unroll
        for(int j = 0; j < RA; j++) {
            const int pm = RA == 1 ? ga : ga * RA + j;
#pragma unroll
            for(int e = 0; e < 8; e++)
                As[st][(e * NVA + cva) * LDK + pm] = ra[j][e];
        }
#pragma unroll
        for(int j = 0; j < RB; j++) {
            const int pm = RB == 1 ? gb : gb * RB + j;
#pragma unroll
            for(int e = 0; e < 8; e++)
                Bs[st][(e * NVB + cvb) * LDK + pm] = rb[j][e];
        }
    };

    float16_t acc[TM][TN];
#pragma unroll
    for(int i = 0; i < TM; i++)
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][j][v] = 0.0f;

    const int wm = (wave / WGN) * WTM, wn = (wave % WGN) * WTN;
    const int frow = lane & 31, fk = (lane >> 5) * 8;
    const int KT = (m_end - m_begin + BK - 1) / BK;

    if(KT > 0) {
        load_slice(m_begin);
        store_slice(0);
    }
    __syncthreads();
    for(int kt = 0; kt < KT; kt++) {
        const int cur = kt & 1;
        if(kt + 1 < KT) {
            advance();
            load_slice(m_begin + (kt + 1) * BK);
        }
#pragma unroll
        for(int kk = 0; kk < BK; kk += 16) {
            half8_t fa[TM], fb[TN];
#pragma unroll
            for(int i = 0; i < TM; i++)
                fa[i] = *(const half8_t *)(&As[cur][(wm + i * 32 + frow) * LDK + kk + fk]);
#pragma unroll
            for(int j = 0; j < TN; j++)
                fb[j] = *(const half8_t *)(&Bs[cur][(wn + j * 32 + frow) * LDK + kk + fk]);
#pragma unroll
            for(int i = 0; i < TM; i++)
#pragma unroll
                for(int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if(kt + 1 < KT)
            store_slice(cur ^ 1);
        __syncthreads();
    }

    // epilogue: undo the row permutations, write the fp32 partial tile
    float *out = g.partial + (int64_t)split * g.K * g.RSC;
    const int ecol = lane & 31, erow = (lane >> 5) * 4;
#pragma unroll
    for(int i = 0; i < TM; i++) {
#pragma unroll
        for(int j = 0; j < TN; j++) {
            const int pb = wn + j * 32 + ecol;                 // permuted column
            const int cj = j0 + (pb % NVB) * 8 + pb / NVB;     // flat (tap, c) column
            if(cj >= g.RSC)
                continue;
#pragma unroll
            for(int v = 0; v < 16; v++) {
                const int pa = wm + i * 32 + (v >> 2) * 8 + erow + (v & 3);
                const int k = k0 + (pa % NVA) * 8 + pa / NVA;
                if(k < g.K)
                    out[(int64_t)k * g.RSC + cj] = acc[i][j][v];
            }
        }
    }
}

// ---------------------------------------------------------------- pipelined backward-filter
//
// Same GEMM as conv_bwd_filter_mfma (rows = output channels of dy, columns = flat (tap, c),
// reduction over pixels), but the tiles stay in their memory order in LDS - one row per pixel,
// channels contiguous - so they can be filled by buffer-load-to-LDS with STAGES-1 slices in
// flight, and the MFMA operands (8 consecutive PIXELS of one channel per lane) are produced
// by the transposing LDS read: within a group of 16 lanes, lane i element j of
// ds_read_b64_tr_b16 is element i%4 of the 8 bytes addressed by lane 4*j + i/4.  Pointing
// lane s at (pixel s/4, channels 4*(s%4)..+3) therefore hands lane i (channel i, pixels 0..3).
// The 16-byte granules of a row are XOR-swizzled with the pixel number so that the four
// pixel rows one such read touches fall into different banks.

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) short4_t *lds_short4_ptr;

__device__ __forceinline__ half8_t tr_read8(const char *lo, const char *hi)
{
    const short4_t a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)lo);
    const short4_t b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)hi);
    const short8_t v = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(half8_t, v);
}

// The same two reads as instructions of our own: addr = LDS byte address, LO / HI = immediate offsets.  The
// compiler does not know that they read LDS, which is the point - in front of a ds_read that it has emitted itself
// it waits for EVERY outstanding buffer_load ... lds whose target it cannot tell apart from the read's address (a
// stage picked at run time), the slice just requested included, and the loads of the pipelined kernel below are
// then never in flight while it multiplies.  The caller waits for the data (s_waitcnt lgkmcnt) before it uses it.
template <int LO, int HI> __device__ __forceinline__ half8_t tr_read8_raw(unsigned addr)
{
    short4_t a, b;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(a) : "v"(addr), "n"(LO) : "memory");
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(b) : "v"(addr), "n"(HI) : "memory");
    const short8_t v = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(half8_t, v);
}

template <int BM, int BN, int STAGES, int NW>
__global__ void __launch_bounds__(64 * NW) conv_bwd_filter_dma(FilterArgs g, unsigned x_bytes, unsigned dy_bytes)
{
    constexpr int GA = BM / 8, GB = BN / 8;             // 16-byte granules per LDS row
    constexpr int RPA = 64 / GA, RPB = 64 / GB;         // pixel rows one wave instruction fills
    constexpr int RA = BK / (NW * RPA), RB = BK / (NW * RPB);
    constexpr int ROWA = BM * 2, ROWB = BN * 2;
    constexpr int STAGE_BYTES = BK * (ROWA + ROWB);
    constexpr int WGM = NW == 16 ? 4 : (BM >= 128 ? 2 : 1), WGN = NW / WGM;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr unsigned OOB = 0x7fffff00u;
    static_assert(RA >= 1 && RB >= 1 && (GA == 8 || GA == 16 || GA == 32) && (GB == 8 || GB == 16 || GB == 32), "tile");

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // tiles are the fast index and every XCD gets a contiguous run of block ids, so the
    // blocks that read the same pixel range of x and dy (one split, all tiles) run on one
    // XCD at about the same time and share the range through its L2
    int b = xcd_remap(blockIdx.x, gridDim.x);
    const int ntiles = g.tiles_k * g.tiles_c;
    const int split = b / ntiles;
    b -= split * ntiles;
    const int tc = b % g.tiles_c, tk = b / g.tiles_c;
    const int k0 = tk * BM, j0 = tc * BN;
    const int m_begin = split * g.m_per_split;
    int m_end = m_begin + g.m_per_split;
    if(m_end > g.M)
        m_end = g.M;

    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc((void *)g.dy, 0, dy_bytes, 0x00020000);

    // A (dy): this lane fills physical granule lane % GA of pixel row pa0 (+ 4*RPA per round)
    const int pa0 = wave * RPA + lane / GA;
    const int swa = GA >= 16 ? (pa0 & 3) << 2 : ((pa0 >> 1) & 1) << 2;
    const int ka = k0 + (((lane % GA) ^ swa) << 3);
    const bool ka_ok = ka < g.K;
    // B (x): likewise; the logical granule fixes this lane's (tap, c)
    const int pb0 = wave * RPB + lane / GB;
    const int swb = GB >= 16 ? (pb0 & 3) << 2 : ((pb0 >> 1) & 1) << 2;
    const int col = j0 + (((lane % GB) ^ swb) << 3);
    const bool cb_ok = col < g.RSC;
    const int tap = cb_ok ? col / g.C : 0;
    const int cc = cb_ok ? col - tap * g.C : 0;
    const int fr = tap / g.S, fs = tap - fr * g.S;
    const int offy = fr * g.dil - g.pad, offx = fs * g.dil - g.pad;

    int bn_[RB], by_[RB], bx_[RB];
#pragma unroll
    for(int j = 0; j < RB; j++) {
        const int m = m_begin + pb0 + j * NW * RPB;
        const int mm = m < g.M ? m : 0;
        bx_[j] = mm % g.Q;
        const int t = mm / g.Q;
        by_[j] = t % g.P;
        bn_[j] = t / g.P;
    }
    int ms = m_begin; // first pixel of the next slice to be issued

    // one slice = RA + RB load instructions ("pieces"): piece p < RA is round p of the dy rows, the others are rounds
    // of the x rows; after the last piece of a slice the cursor moves on
    auto issue_piece = [&](int stage, int p) {
        char *sa = smem + stage * STAGE_BYTES;
        char *sb = sa + BK * ROWA;
        if(p < RA) {
            const int j = p;
            const int m = ms + pa0 + j * NW * RPA;
            const unsigned off = (ka_ok && m < m_end) ? (unsigned)((m * g.ldy + ka) * 2) : OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ry, (lds_ptr_t)(sa + (wave + NW * j) * 1024), 16, off, 0, 0, 0);
        } else {
            const int j = p - RA;
            const int m = ms + pb0 + j * NW * RPB;
            // (through locals: a captured array element passed directly makes the host pass drop the kernel)
            const int byj = by_[j], bxj = bx_[j], bnj = bn_[j];
            const int iy = byj * g.stride + offy, ix = bxj * g.stride + offx;
            const bool ok = cb_ok && m < m_end && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
            const unsigned off = ok ? (unsigned)((((bnj * g.H + iy) * g.W + ix) * g.ldx + cc) * 2) : OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(sb + (wave + NW * j) * 1024), 16, off, 0, 0, 0);
            bx_[j] += BK;
            while(bx_[j] >= g.Q) {
                bx_[j] -= g.Q;
                by_[j]++;
            }
            while(by_[j] >= g.P) {
                by_[j] -= g.P;
                bn_[j]++;
            }
        }
        if(p == RA + RB - 1)
            ms += BK;
    };
    auto issue = [&](int stage) {
#pragma unroll
        for(int p = 0; p < RA + RB; p++)
            issue_piece(stage, p);
    };

    float16_t acc[TM][TN];
#pragma unroll
    for(int i = 0; i < TM; i++)
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][j][v] = 0.0f;

    const int wm = (wave / WGN) * WTM, wn = (wave % WGN) * WTN;
    // transposing fragment reads: this lane addresses pixel fp (+4 for the upper half, +16 per
    // MFMA step) and channels fc .. fc+3 of a 32-channel tile
    const int fp = 8 * (lane >> 5) + ((lane & 15) >> 2);
    const int fc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    const int fswa = GA >= 16 ? (fp & 3) << 2 : ((fp >> 1) & 1) << 2;
    const int fswb = GB >= 16 ? (fp & 3) << 2 : ((fp >> 1) & 1) << 2;
    int foa[TM], fob[TN];
#pragma unroll
    for(int i = 0; i < TM; i++) {
        const int c = wm + i * 32 + fc;
        foa[i] = fp * ROWA + (((c >> 3) ^ fswa) << 4) + (c & 7) * 2;
    }
#pragma unroll
    for(int j = 0; j < TN; j++) {
        const int c = wn + j * 32 + fc;
        fob[j] = BK * ROWA + fp * ROWB + (((c >> 3) ^ fswb) << 4) + (c & 7) * 2;
    }

    const unsigned lds0 = (unsigned)(uintptr_t)(lds_ptr_t)smem;
    const int KT = (m_end - m_begin + BK - 1) / BK;
#pragma unroll
    for(int st = 0; st < STAGES - 1; st++)
        if(st < KT)
            issue(st);

    for(int kt = 0; kt < KT; kt++) {
        if(kt + STAGES - 2 < KT)
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((RA + RB) * (STAGES - 2)) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        const bool more = kt + STAGES - 1 < KT;
        const int nst = (kt + STAGES - 1) % STAGES;
        // the slice's fragments: all reads go out, then each 16-pixel step waits for its own (tr_read8_raw)
        const unsigned sbase = lds0 + (kt % STAGES) * STAGE_BYTES;
        static_assert(BK == 32, "two 16-pixel steps per slice");
        half8_t fa[2][TM], fb[2][TN];
#pragma unroll
        for(int i = 0; i < TM; i++) {
            fa[0][i] = tr_read8_raw<0, 4 * ROWA>(sbase + foa[i]);
        }
#pragma unroll
        for(int j = 0; j < TN; j++)
            fb[0][j] = tr_read8_raw<0, 4 * ROWB>(sbase + fob[j]);
#pragma unroll
        for(int i = 0; i < TM; i++)
            fa[1][i] = tr_read8_raw<16 * ROWA, 20 * ROWA>(sbase + foa[i]);
#pragma unroll
        for(int j = 0; j < TN; j++)
            fb[1][j] = tr_read8_raw<16 * ROWB, 20 * ROWB>(sbase + fob[j]);
        // The loads of the slice STAGES - 1 ahead go out between the multiplications: the address unit takes a
        // kilobyte in 16 cycles, and right behind the barrier every wavefront of the block would stand in line for
        // it with nothing running on the matrix units (0.4 us of a 1.3 us iteration on sixteen wavefronts).
        constexpr int NP = RA + RB, NQ = 2 * TM * TN;
#pragma unroll
        for(int q = 0; q < NQ; q++) {
            const int kk = q / (TM * TN), i = (q / TN) % TM, j = q % TN;
            if(q % (TM * TN) == 0) {
                if(kk == 0)
                    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(2 * (TM + TN)) : "memory");
                else
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                // (the multiplications must stay behind the wait: their operands pass through it)
#pragma unroll
                for(int ii = 0; ii < TM; ii++)
                    asm volatile("" : "+v"(fa[kk][ii]));
#pragma unroll
                for(int jj = 0; jj < TN; jj++)
                    asm volatile("" : "+v"(fb[kk][jj]));
            }
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kk][i], fb[kk][j], acc[i][j], 0, 0, 0);
#pragma unroll
            for(int p = 0; p < NP; p++)
                if(q == ((p + 1) * NQ) / (NP + 1)) {
                    __builtin_amdgcn_sched_barrier(0);
                    if(more)
                        issue_piece(nst, p);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    float *out = g.partial + (int64_t)split * g.K * g.RSC;
    const int ecol = lane & 31, erow = (lane >> 5) * 4;
#pragma unroll
    for(int i = 0; i < TM; i++) {
#pragma unroll
        for(int j = 0; j < TN; j++) {
            const int cj = j0 + wn + j * 32 + ecol;
            if(cj >= g.RSC)
                continue;
#pragma unroll
            for(int v = 0; v < 16; v++) {
                const int k = k0 + wm + i * 32 + (v >> 2) * 8 + erow + (v & 3);
                if(k < g.K)
                    out[(int64_t)k * g.RSC + cj] = acc[i][j][v];
            }
        }
    }
}

// Sum of the split partials for tensors whose rows need no re-pitching: 16 lanes cover 64
// consecutive elements with float4 loads, the 16 lane groups of a block take every 16th
// partial, and LDS combines the groups in a fixed order (deterministic).
__global__ void __launch_bounds__(256)
    filter_reduce_v4(const float *__restrict__ partial, half_t *__restrict__ dw, int64_t n, int splits, float alpha,
                     float beta)
{
    __shared__ float4_t red[16][16];
    const int ev = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int64_t e = ((int64_t)blockIdx.x * 16 + ev) * 4;
    float4_t s = {0, 0, 0, 0};
    if(e < n)
        for(int p = sl; p < splits; p += 16)
            s += *(const float4_t *)(partial + (int64_t)p * n + e);
    red[sl][ev] = s;
    __syncthreads();
    if(sl == 0 && e < n) {
#pragma unroll
        for(int q = 1; q < 16; q++)
            s += red[q][ev];
#pragma unroll
        for(int j = 0; j < 4; j++) {
            float v = alpha * s[j];
            if(beta != 0.0f)
                v += beta * (float)dw[e + j];
            dw[e + j] = (half_t)v;
        }
    }
}

// dw[row, c] = alpha * sum_p partial[p][row, c] + beta * dw ; rows = K*R*S, the partial rows are
// Cp wide (Cp >= C when the input channels were padded)
__global__ void __launch_bounds__(256)
    filter_reduce(const float *__restrict__ partial, half_t *__restrict__ dw, int64_t n, int C, int Cp, int splits,
                  float alpha, float beta)
{
    const int64_t np = n / C * Cp;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = i / C;
        const int64_t j = row * Cp + (i - row * C);
        float s = 0;
        for(int p = 0; p < splits; p++)
            s += partial[(int64_t)p * np + j];
        s *= alpha;
        if(beta != 0.0f)
            s += beta * (float)dw[i];
        dw[i] = (half_t)s;
    }
}

// Copies rows of C channels (pitch `sp`) into rows of Cp = multiple-of-8 channels, zero filled:
// gives odd channel counts (the 3-channel network input) the 16-byte vectors the MFMA kernels load.
__global__ void __launch_bounds__(256)
    pad_channels(const half_t *__restrict__ src, int64_t sp, int C, half_t *__restrict__ dst, int Cp, int64_t rows)
{
    const int groups = Cp / 8;
    const int64_t total = rows * groups;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / groups;
        const int c0 = (int)(i - r * groups) * 8;
        half8_t v;
#pragma unroll
        for(int e = 0; e < 8; e++)
            v[e] = (c0 + e < C) ? src[r * sp + c0 + e] : (half_t)0;
        *(half8_t *)(dst + r * Cp + c0) = v;
    }
}

struct FilterPlan {
    int bm, bn, tiles_k, tiles_c, splits, m_per_split;
};

// big_ok: the caller will run the pipelined kernel, the only one that has the large tiles
static FilterPlan plan_filter(const ConvGeom &g, bool big_ok = true, bool thin = false)
{
    FilterPlan p;
    const int RSC = g.R * g.S * g.C;
    const int64_t M = (int64_t)g.N * g.P * g.Q;
    p.bm = g.K > 64 ? 128 : 64; // 256x128 tiles were measured slower on every ResNet-50 layer
    p.bn = 128;
    // SAGA_HIP_FILTER_TILE=128 keeps the small tiles everywhere, =256 takes the large one wherever it fits
    static const char *env = getenv("SAGA_HIP_FILTER_TILE");
    static const int forced = env ? atoi(env) : 0;
    int target = 512; // two blocks per CU (three fit): measured best of 256 / 512 / 640 / 768 / 1024
    // 256x256 on sixteen wavefronts, one block per CU: half the LDS fill traffic per flop.  Measured
    // 25-35 % faster where the reduction per tile is long enough to pay for the smaller grid (3x3
    // filters, or 1x1 with >= 1024 input and >= 512 output channels), slower on the other 1x1 layers.
    const bool fits = big_ok && g.K > 128 && RSC > 128;
    const bool pays = RSC >= 1024 && (g.R * g.S > 1 || g.K >= 512);
    if(fits && forced != 128 && (pays || forced == 256)) {
        p.bm = p.bn = 256;
        target = 256;
    } else if(big_ok && g.K > 64 && g.K <= 128 && RSC >= 1024 && g.R * g.S > 1 && forced != 128) {
        p.bn = 256; // 128x256 on eight wavefronts, two blocks per CU
        target = 512;
    } else if(big_ok && g.K <= 64 && RSC >= 512 && g.R * g.S > 1 && forced != 128) {
        p.bn = 256; // 64x256 on four wavefronts with two stages, four blocks per CU (measured 17 % faster)
        target = 1024;
    } else if(thin && g.K <= 64 && RSC > 128 && RSC <= 256 && forced != 128) {
        p.bn = 256; // the stem: all 7 x 32 virtual channels in one tile, so dy (the large operand) is read once
        target = 1024;
    }
    p.tiles_k = (g.K + p.bm - 1) / p.bm;
    p.tiles_c = (RSC + p.bn - 1) / p.bn;
    const int tiles = p.tiles_k * p.tiles_c;
    // with one block per CU a grid just above the CU count would take two rounds: round down there
    int64_t want = p.bn == 256 ? target / tiles : (target + tiles - 1) / tiles;
    const int64_t maxs = (M + 255) / 256; // at least 256 pixels per split
    if(want > maxs)
        want = maxs;
    if(want < 1)
        want = 1;
    int64_t per = (M + want - 1) / want;
    per = (per + BK - 1) / BK * BK;
    p.m_per_split = (int)per;
    p.splits = (int)((M + per - 1) / per);
    return p;
}

static bool krsc_dense(const SagaTensorView *w)
{
    const int C = w->dims[1], R = w->dims[2], S = w->dims[3];
    if(C > 1 && w->strides[1] != 1)
        return false;
    if(S > 1 && w->strides[3] != C)
        return false;
    if(R > 1 && w->strides[2] != (int64_t)S * C)
        return false;
    if(w->dims[0] > 1 && w->strides[0] != (int64_t)R * S * C)
        return false;
    return true;
}

static int ilog2_exact(int v)
{
    int s = 0;
    while((1 << s) < v)
        s++;
    return (1 << s) == v ? s : -1;
}

// ---------------------------------------------------------------- thin inputs (C <= 4)
//
// A convolution over 1..4 input channels (the RGB stem) would spend a 32-wide reduction slice
// on the 3 channels of one tap.  Instead x is copied once into x4[N][H+2pad][Wp][4]
// (spatially zero-padded, 4 halves = 8 bytes per pixel); the 8 pixels x4[n][iy][ix .. ix+7]
// are then 32 contiguous halves holding the taps s = 0..7 of filter row r, so the same
// gather kernels run a "virtual" convolution with R taps of 32 channels each: pixel pitch 4,
// channel extent 32 (rows overlap), filter repacked to [K][R][s*4+c] with zeros for s >= S
// and c >= C.  ix = ox*stride is even for even strides, which keeps every 16-byte load aligned.

__global__ void __launch_bounds__(256)
    pad_thin(const half_t *__restrict__ x, int64_t sp, int C, int H, int W, int pad, half_t *__restrict__ x4, int Hp,
             int Wp, int64_t total)
{
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    // (total < 2^31, checked by thin_ok: 32-bit index arithmetic - the 64-bit divisions were most of this kernel)
    const unsigned tot = (unsigned)total, step = gridDim.x * blockDim.x;
    for(unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < tot; i += step) {
        const unsigned t = i / (unsigned)Wp;
        const int wp = (int)(i - t * (unsigned)Wp);
        const unsigned n = t / (unsigned)Hp;
        const int hp = (int)(t - n * (unsigned)Hp);
        const int h = hp - pad, w = wp - pad;
        h4 v = {0, 0, 0, 0};
        if(h >= 0 && h < H && w >= 0 && w < W) {
            const half_t *src = x + (((int64_t)n * H + h) * W + w) * sp;
            if(C == 3) {
                v[0] = src[0];
                v[1] = src[1];
                v[2] = src[2];
            } else {
                for(int c = 0; c < C; c++)
                    v[c] = src[c];
            }
        }
        *(h4 *)(x4 + (size_t)i * 4) = v;
    }
}

// The same copy for dense 3-channel rows whose byte length is a multiple of 16 (W * 6 bytes: the RGB stem): one
// block per padded row.  The source row comes into LDS through aligned 16-byte loads, every thread then builds
// two padded pixels (16 bytes, one store) from six halves of the LDS copy - instead of three 2-byte global loads
// and one 8-byte store per pixel.
__global__ void __launch_bounds__(128)
    pad_thin_rgb_rows(const half_t *__restrict__ x, int H, int W, int pad, half_t *__restrict__ x4, int Hp, int Wp)
{
    extern __shared__ __attribute__((aligned(16))) half_t row[];
    const int hp = blockIdx.x % Hp, n = blockIdx.x / Hp;
    const int h = hp - pad;
    const bool inside = h >= 0 && h < H;
    const int chunks = W * 6 / 16;
    if(inside) {
        const uint4_t *src = (const uint4_t *)(x + ((int64_t)n * H + h) * W * 3);
        for(int i = threadIdx.x; i < chunks; i += blockDim.x)
            ((uint4_t *)row)[i] = src[i];
    }
    __syncthreads();
    half_t *dst = x4 + ((int64_t)n * Hp + hp) * Wp * 4;
    for(int j = threadIdx.x; j < Wp / 2; j += blockDim.x) {
        half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for(int e = 0; e < 2; e++) {
            const int w = 2 * j + e - pad;
            if(inside && w >= 0 && w < W) {
                v[4 * e + 0] = row[3 * w + 0];
                v[4 * e + 1] = row[3 * w + 1];
                v[4 * e + 2] = row[3 * w + 2];
            }
        }
        *(half8_t *)(dst + 8 * j) = v;
    }
}

// wv[k][r][s*4 + c] = w[k][r][s][c] (s < S, c < C), 0 elsewhere; 32 halves per (k, r)
__global__ void __launch_bounds__(256)
    repack_thin_filter(const half_t *__restrict__ w, half_t *__restrict__ wv, int C, int S, int64_t total)
{
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int e = (int)(i & 31), s = e >> 2, c = e & 3;
        const int64_t kr = i >> 5;
        wv[i] = (s < S && c < C) ? w[(kr * S + s) * C + c] : (half_t)0;
    }
}

// dw[k][r][s][c] = alpha * sum_p partial[p][k][r][s*4 + c] + beta * dw
// 16 outputs per block, 16 threads per output that each add every 16th split (four loads in flight),
// then a fixed-order sum of the 16: hundreds of splits would otherwise be one long dependent chain.
__global__ void __launch_bounds__(256)
    thin_filter_reduce(const float *__restrict__ partial, half_t *__restrict__ dw, int64_t n, int C, int S, int splits,
                       float alpha, float beta)
{
    __shared__ float part[16][17];
    const int64_t np = n / (S * C) * 32;
    const int o = threadIdx.x & 15, q = threadIdx.x >> 4;
    const int64_t i = (int64_t)blockIdx.x * 16 + o;
    float acc = 0;
    if(i < n) {
        const int c = (int)(i % C);
        const int64_t t = i / C;
        const int s = (int)(t % S);
        const float *src = partial + (t / S) * 32 + s * 4 + c;
        int p = q;
        for(; p + 48 < splits; p += 64) {
            const float v0 = src[(int64_t)p * np], v1 = src[(int64_t)(p + 16) * np];
            const float v2 = src[(int64_t)(p + 32) * np], v3 = src[(int64_t)(p + 48) * np];
            acc += (v0 + v1) + (v2 + v3);
        }
        for(; p < splits; p += 16)
            acc += src[(int64_t)p * np];
    }
    part[q][o] = acc;
    __syncthreads();
    if(q == 0 && i < n) {
        for(int k = 1; k < 16; k++)
            acc += part[k][o];
        acc *= alpha;
        if(beta != 0.0f)
            acc += beta * (float)dw[i];
        dw[i] = (half_t)acc;
    }
}

static int num_cus()
{
    static int v = 0;
    if(v <= 0) {
        int d = 0;
        if(hipGetDevice(&d) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, d) != hipSuccess ||
           v <= 0)
            v = 256;
    }
    return v;
}

struct ThinGeom {
    int Hp, Wp;
    size_t x4_bytes, wv_bytes;
};

static void launch_pad_thin(const half_t *x, int64_t pitch, const ConvGeom &g, half_t *x4, const ThinGeom &tg, int64_t px,
                            hipStream_t st);

static bool thin_ok(const ConvGeom &g, ThinGeom *t)
{
    if(g.C > 4 || g.S > 8 || g.dil != 1 || g.stride < 2 || (g.stride & 1) || g.group != 1)
        return false;
    t->Hp = g.H + 2 * g.pad;
    t->Wp = (g.W + 2 * g.pad + 8 + 1) & ~1;
    const int64_t px = (int64_t)g.N * t->Hp * t->Wp;
    if(px * 8 >= 0x7fffff00)
        return false;
    t->x4_bytes = ((size_t)px * 8 + 255) & ~(size_t)255;
    t->wv_bytes = ((size_t)g.K * g.R * 32 * sizeof(half_t) + 255) & ~(size_t)255;
    return true;
}

// ---------------------------------------------------------------- thin inputs, whole image rows in LDS
//
// The "virtual" convolution of a thin input (above: x4[N][Hp][Wp][4], windows of 8 pixels = 32 halves per filter
// row) run through the gather kernel loads every output pixel's 64-byte window separately, and neighbouring
// windows overlap by 48 of their 64 bytes: the LDS fill is four times the input, a block lives for R short
// slices, and with two blocks per CU the loop is bound by the latency of those fills (RGB stem of ResNet-50:
// 264 us for 92 GFLOP and 520 MB).  Here a block owns TR whole output rows of one image (TR * Q <= 256 pixels),
// copies the (TR - 1) * stride + R padded input rows they read ONCE into LDS as they are, and an MFMA operand -
// 8 halves of pixel window (oy, ox), filter row r - is the 16 bytes at
//     (orow * stride + r) * row_bytes + ox * stride * 8 + 16 * (k / 8)
// of that copy: overlapping windows are overlapping reads.  The filter (64 output channels x R x 32 halves) stays
// in registers for the whole launch; blocks are persistent and walk the tiles grid-strided with two LDS buffers,
// the rows of the tile after next being requested while the current one is multiplied.  Order inside one
// iteration: multiply tile t - wait for everything outstanding (the rows of t + 1 and the stores of t - 1, both
// issued a whole multiplication ago; loads and stores retire through one in-order counter) - barrier - store
// tile t - request the rows of t + 2 into the buffer that t was read from.
constexpr int THIN_ROWS_DEPTH = 4; // tiles whose rows are in LDS or on their way
struct ThinRowsArgs {
    int TR;          // output rows per tile
    int tpi;         // tiles per image
    int ntiles;
    int npix;        // TR * Q
    int Hp;          // rows of the padded input per image
    int row_bytes;   // bytes per padded input row
    int chunks_row;  // 16-byte chunks per input row
    int chunks_tile; // chunks_row * input rows per tile
    int buf_bytes;   // one LDS buffer: a tile's rows, rounded up to the 1 KB a load instruction fills
    int epi_off;     // where the epilogue's LDS scratch starts, minus what gather_epilogue adds itself
};

// MODE: 0 plain (alpha, beta), 1 folded inference batch norm, 2 batch-norm statistics - one instantiation each, so
// that the register allocation of one epilogue does not pay for the others.
template <int R, int MODE> __global__ void __launch_bounds__(256, 2) conv_thin_rows(GatherArgs g, ThinRowsArgs t)
{
    if constexpr(MODE != 1)
        g.bn_s = nullptr;
    // (statistics: every lane keeps the running totals of one channel over the tiles its block walks, and the block
    // leaves ONE partial row at the end - no barrier or LDS round trip per tile, and a finalize step that adds a few
    // hundred rows instead of one per tile)
    float *const stats = MODE == 2 ? g.stats : nullptr;
    g.stats = nullptr;
    float run_s = 0.0f, run_q = 0.0f;
    if constexpr(MODE != 0)
        g.beta = 0.0f;
    constexpr int TM = 2, TN = 2, NLD_MAX = 8, D = THIN_ROWS_DEPTH;
    constexpr unsigned OOB = 0x7fffff00u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hi = lane >> 5;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void *)g.a, 0, g.a_bytes, 0x00020000);

    // the filter: fragment (r, kk, j) = halves 16*kk + 8*hi .. +8 of filter row r of output channel 32*j + lane%32
    half8_t fb[R][2][TN];
#pragma unroll
    for(int j = 0; j < TN; j++) {
        const int o = j * 32 + (lane & 31);
        const bool ok = o < g.Ngemm;
        const half_t *src = g.b + ((int64_t)(ok ? o : 0) * R) * 32 + hi * 8;
#pragma unroll
        for(int r = 0; r < R; r++)
#pragma unroll
            for(int kk = 0; kk < 2; kk++) {
                const half8_t v = *(const half8_t *)(src + r * 32 + kk * 16);
                const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
                fb[r][kk][j] = ok ? v : zero;
            }
    }
    // Chunk (q * 4 + wave) * 64 + lane of a tile's rows is this lane's share of load q; its place in the padded
    // input relative to the tile's first row is the same for every tile.  (Recomputed for every request rather
    // than kept: registers are what limits this kernel, and a value spilled here would be reloaded behind the
    // epilogue's stores.)  A wavefront issues my_nld loads per tile - those with at least one chunk of the tile.
    const int c0 = wave * 64 + lane;
    const int row0 = c0 / t.chunks_row, col0 = c0 - row0 * t.chunks_row;
    const int my_nld = t.chunks_tile > wave * 64 ? (t.chunks_tile - wave * 64 + 255) / 256 : 0;
    auto request = [&](int tile, int b) {
        const int n = tile / t.tpi;
        const int oy0 = (tile - n * t.tpi) * t.TR;
        const int base = (n * t.Hp + oy0 * g.stride) * t.row_bytes; // (the whole padded input is below 2 GB)
        char *dst = smem + b * t.buf_bytes + wave * 1024;
        // chunk c0 + 256 q: 256 chunks further on is rows256 rows and cols256 columns further on, with a carry
        const int rows256 = 256 / t.chunks_row, cols256 = 256 - rows256 * t.chunks_row;
        int row = row0, col = col0;
#pragma unroll
        for(int q = 0; q < NLD_MAX; q++)
            if(q < my_nld) {
                const unsigned off = c0 + 256 * q < t.chunks_tile ? (unsigned)(row * t.row_bytes + col * 16) : OOB;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(dst + q * 4096), 16, off, base, 0, 0);
                row += rows256;
                col += cols256;
                if(col >= t.chunks_row) {
                    col -= t.chunks_row;
                    row++;
                }
            }
    };
    // this lane's two pixels (row blocks i of the wavefront's 64) inside a tile, as byte offsets into the LDS copy
    int abase[TM];
#pragma unroll
    for(int i = 0; i < TM; i++) {
        const int p = wave * 64 + i * 32 + (lane & 31);
        const int pp = p < t.npix ? p : 0;
        const int orow = pp / g.OW;
        abase[i] = orow * g.stride * t.row_bytes + (pp - orow * g.OW) * g.stride * 8 + hi * 16;
    }
    char *epi = smem + t.epi_off;
    const int G = gridDim.x;

    // each die's blocks take neighbouring tiles, which share input rows: the die's L2 then fetches those rows once
    int tile = xcd_remap(blockIdx.x, G);
    const int first_tile = tile; // also the block's row in the statistics
#pragma unroll
    for(int d = 0; d < D; d++)
        if(tile + d * G < t.ntiles)
            request(tile + d * G, d);
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    int b = 0; // buffer of the current tile
    for(; tile < t.ntiles; tile += G) {
        const char *buf = smem + b * t.buf_bytes;
        float16_t acc[TM][TN];
#pragma unroll
        for(int i = 0; i < TM; i++)
#pragma unroll
            for(int j = 0; j < TN; j++)
#pragma unroll
                for(int v = 0; v < 16; v++)
                    acc[i][j][v] = 0.0f;
#pragma unroll
        for(int r = 0; r < R; r++) {
            half8_t fa[2][TM];
#pragma unroll
            for(int kk = 0; kk < 2; kk++)
#pragma unroll
                for(int i = 0; i < TM; i++)
                    fa[kk][i] = *(const half8_t *)(buf + abase[i] + r * t.row_bytes + kk * 32);
#pragma unroll
            for(int kk = 0; kk < 2; kk++)
#pragma unroll
                for(int i = 0; i < TM; i++)
#pragma unroll
                    for(int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[r][kk][j], fa[kk][i], acc[i][j], 0, 0, 0);
        }
        // The rows of the NEXT tile must have arrived before the barrier that lets everybody read them.  This
        // wavefront's memory operations retire in order, and behind those rows it has issued, per tile, NST stores
        // (the epilogue's, always all of them: BUFST) and its my_nld loads, for D - 2 tiles: those may stay in flight,
        // so neither the stores nor the later rows are waited for until they are two multiplications old.  Near the
        // end of the walk fewer operations are behind the rows, and the wait is for everything.
        constexpr int NST = TM * TN * 2;
        if(tile + (D - 1) * G < t.ntiles) {
            switch(my_nld) {
            case 0: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((0 + NST) * (D - 2)) : "memory"); break;
            case 1: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((1 + NST) * (D - 2)) : "memory"); break;
            case 2: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((2 + NST) * (D - 2)) : "memory"); break;
            case 3: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((3 + NST) * (D - 2)) : "memory"); break;
            case 4: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((4 + NST) * (D - 2)) : "memory"); break;
            case 5: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((5 + NST) * (D - 2)) : "memory"); break;
            case 6: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((6 + NST) * (D - 2)) : "memory"); break;
            case 7: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((7 + NST) * (D - 2)) : "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((8 + NST) * (D - 2)) : "memory"); break;
            }
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        asm volatile("s_barrier" ::: "memory");
        const int n = tile / t.tpi;
        const int oy0 = (tile - n * t.tpi) * t.TR;
        const int64_t pix0 = ((int64_t)n * g.OH + oy0) * g.OW;
        auto rowpix = [&](int mrow, bool &ok, int64_t &pix) {
            ok = mrow < t.npix && oy0 + mrow / g.OW < g.OH;
            pix = pix0 + (ok ? mrow : 0);
        };
        gather_epilogue<TM, TN, 4, 1, 64, false, true, true>(g, acc, epi, tid, lane, wave, wave * 64, 0, 0, tile, rowpix);
        if constexpr(MODE == 2) {
            bool okr[TM];
#pragma unroll
            for(int i = 0; i < TM; i++) {
                int64_t pix;
                rowpix(wave * 64 + i * 32 + (lane & 31), okr[i], pix);
            }
            float s0, q0;
            stats_lane_totals<TM, TN, true>(g.alpha, acc, okr, lane, s0, q0);
            run_s += s0;
            run_q += q0;
        }
        // every wavefront is past the barrier, so nobody reads this tile's buffer any more
        if(tile + D * G < t.ntiles)
            request(tile + D * G, b);
        b = b + 1 == D ? 0 : b + 1;
    }
    if constexpr(MODE == 2) {
        g.stats = stats;
        __syncthreads();
        stats_block_write<TN, 4, 1, 64>(g, epi + 32768, tid, lane, wave, 0, 0, first_tile, run_s, run_q);
    }
}

// ---------------------------------------------------------------- 3x3, 64 -> 64 channels, whole image rows in LDS
//
// The 3x3 layers with 64 input and 64 output channels over large images (ResNet-50's first stage, 56x56) have too
// little arithmetic per byte for the gather kernel's scheme - every output pixel's input is fetched into LDS nine
// times, once per tap, and a 256 x 64 tile leaves the matrix unit waiting for those fills (114 us for 59 GFLOP).
// Same idea as conv_thin_rows: a persistent block owns TR whole output rows of an image (TR * W <= 256 pixels),
// copies the TR + 2 input rows they read ONCE into LDS - pixel slots of 144 bytes (128 of data + 16 of padding, so
// that the 16-byte operand reads of 16 neighbouring pixels fall into 64 different banks), with a zero slot left
// and right and zero rows above / below the image, all by out-of-range load offsets - and an MFMA operand of tap
// (dr, ds) is the 16 bytes at ((orow + dr) * (W + 2) + ox + ds) * 144 + 16 * (k / 8): nine taps are nine
// immediate offsets on one address.  Eight wavefronts: four groups of 64 pixels x two halves of the output
// channels; a wavefront keeps its half of the filter (32 x 9 x 64 halves) in 144 registers for the whole launch.
// FLIP reads the taps in reverse order: backward data of such a layer is this convolution of dy with the
// transposed filter (C,R,S,K, which backward data keeps in its workspace anyway) mirrored.
struct Rows64Args {
    int H, W;
    int TR;          // output rows per tile
    int tpi;         // tiles per image
    int ntiles;
    int npix;        // TR * W
    int slots_row;   // W + 2 pixel slots per LDS row
    int chunks_tile; // (TR + 2) * slots_row * 9: 16-byte chunks of a tile's copy
    int buf_bytes;   // one LDS buffer (chunks_tile * 16 rounded up to the 1 KB a load instruction fills)
    int epi_off;     // where the epilogue's LDS scratch starts, minus what gather_epilogue adds itself
};

template <int MODE, bool FLIP, int WGM> __global__ void __launch_bounds__(128 * WGM, 4 / WGM) conv_rows64(GatherArgs g, Rows64Args t)
{
    float *const stats = MODE == 2 ? g.stats : nullptr;
    g.stats = nullptr;
    if constexpr(MODE != 1)
        g.bn_s = nullptr;
    else
        g.bn_flags &= SAGA_BN_RELU; // (no residual here: its registers would not fit beside the filter's)
    if constexpr(MODE != 0)
        g.beta = 0.0f;
    float run_s = 0.0f, run_q = 0.0f;
    constexpr int TM = 2, TN = 1, NLD_MAX = 10, SLOT = 144, NW = 2 * WGM;
    constexpr unsigned OOB = 0x7fffff00u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hi = lane >> 5;
    const int wmi = wave >> 1, cj = wave & 1; // pixel group, channel half
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void *)g.a, 0, g.a_bytes, 0x00020000);

    // this wavefront's half of the filter: fragment (tap, kk) = halves 16*kk + 8*hi .. +8 of that tap of output
    // channel 32*cj + lane%32
    half8_t fb[9][4];
    {
        const int o = cj * 32 + (lane & 31);
        const bool ok = o < g.Ngemm;
        const half_t *src = g.b + (int64_t)(ok ? o : 0) * 9 * 64 + hi * 8;
#pragma unroll
        for(int tp = 0; tp < 9; tp++)
#pragma unroll
            for(int kk = 0; kk < 4; kk++) {
                const half8_t v = *(const half8_t *)(src + (FLIP ? 8 - tp : tp) * 64 + kk * 16);
                const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
                fb[tp][kk] = ok ? v : zero;
            }
    }
    const int my_nld = t.chunks_tile > wave * 64 ? (t.chunks_tile - wave * 64 + NW * 64 - 1) / (NW * 64) : 0;
    // LDS chunk L = (q * 8 + wave) * 64 + lane of a tile's copy: pixel slot L / 9 (row r, column p of the padded
    // rows), chunk L % 9 of the slot (the ninth is padding).  It has a source - channels 8*(L%9).. of input pixel
    // (oy0 - 1 + r, p - 1) - unless that lies outside the image, and reads as zeros otherwise.
    auto request = [&](int tile, int b) {
        const int n = tile / t.tpi;
        const int oy0 = (tile - n * t.tpi) * t.TR;
        char *dst = smem + b * t.buf_bytes + wave * 1024;
#pragma unroll
        for(int q = 0; q < NLD_MAX; q++)
            if(q < my_nld) {
                const int L = (q * NW + wave) * 64 + lane;
                const int slot = L / 9, kpos = L - slot * 9;
                const int r = slot / t.slots_row, pcol = slot - r * t.slots_row;
                const int iy = oy0 - 1 + r, ix = pcol - 1;
                const bool ok = L < t.chunks_tile && kpos < 8 && ix >= 0 && ix < t.W && iy >= 0 && iy < t.H;
                const unsigned off = ok ? (unsigned)((((n * t.H + iy) * t.W + ix) * g.lda + kpos * 8) * 2) : OOB;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(dst + q * (NW * 1024)), 16, off, 0, 0, 0);
            }
    };
    // this lane's two pixels (row blocks i of the wavefront's 64) inside a tile: byte offset of the top left tap
    int abase[TM], prow[TM]; // prow: the pixel's output row inside the tile, or a row beyond every image
#pragma unroll
    for(int i = 0; i < TM; i++) {
        const int pp0 = wmi * 64 + i * 32 + (lane & 31);
        const int pp = pp0 < t.npix ? pp0 : 0;
        const int orow = pp / t.W;
        abase[i] = (orow * t.slots_row + (pp - orow * t.W)) * SLOT + hi * 16;
        prow[i] = pp0 < t.npix ? orow : 0x40000000;
    }
    char *epi = smem + t.epi_off;
    const int G = gridDim.x;
    int tile = xcd_remap(blockIdx.x, G);
    const int first_tile = tile;
    if(tile < t.ntiles)
        request(tile, 0);
    if(tile + G < t.ntiles)
        request(tile + G, 1);
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    int b = 0;
    for(; tile < t.ntiles; tile += G) {
        const char *buf = smem + b * t.buf_bytes;
        float16_t acc[TM][TN];
#pragma unroll
        for(int i = 0; i < TM; i++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][0][v] = 0.0f;
#pragma unroll
        for(int dr = 0; dr < 3; dr++)
#pragma unroll
            for(int ds = 0; ds < 3; ds++) {
                const int tapoff = (dr * t.slots_row + ds) * SLOT;
                half8_t fa[4][TM];
#pragma unroll
                for(int kk = 0; kk < 4; kk++)
#pragma unroll
                    for(int i = 0; i < TM; i++)
                        fa[kk][i] = *(const half8_t *)(buf + abase[i] + tapoff + kk * 32);
#pragma unroll
                for(int kk = 0; kk < 4; kk++)
#pragma unroll
                    for(int i = 0; i < TM; i++)
                        acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[dr * 3 + ds][kk], fa[kk][i], acc[i][0], 0, 0, 0);
            }
        // the next tile's rows (requested a whole multiplication ago) and the previous tile's stores
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        const int n = tile / t.tpi;
        const int oy0 = (tile - n * t.tpi) * t.TR;
        const int64_t pix0 = ((int64_t)n * t.H + oy0) * t.W;
        // (mrow is one of this lane's two rows: no division here, the epilogue's arithmetic is a large part of a tile)
        auto rowpix = [&](int mrow, bool &ok, int64_t &pix) {
            const int pr = ((mrow - wmi * 64) & 32) ? prow[1] : prow[0];
            ok = oy0 + pr < t.H;
            pix = pix0 + (ok ? mrow : 0);
        };
        gather_epilogue<TM, TN, WGM, 2, 64, false, true, true>(g, acc, epi, tid, lane, wave, wmi * 64, cj * 32, 0, tile, rowpix);
        if constexpr(MODE == 2) {
            bool okr[TM];
#pragma unroll
            for(int i = 0; i < TM; i++) {
                int64_t pix;
                rowpix(wmi * 64 + i * 32 + (lane & 31), okr[i], pix);
            }
            float s0, q0;
            stats_lane_totals<TM, TN, true>(g.alpha, acc, okr, lane, s0, q0);
            run_s += s0;
            run_q += q0;
        }
        // every wavefront is past the barrier, so nobody reads this tile's buffer any more
        if(tile + 2 * G < t.ntiles)
            request(tile + 2 * G, b);
        b ^= 1;
    }
    if constexpr(MODE == 2) {
        g.stats = stats;
        __syncthreads();
        stats_block_write<TN, WGM, 2, 64>(g, epi + WGM * 8192, tid, lane, wave, cj * 32, 0, first_tile, run_s, run_q);
    }
}

// s_waitcnt vmcnt(n) for a count known only at run time (the same for the whole wavefront)
__device__ __forceinline__ void wait_vmcnt(int n)
{
#define SAGA_VMCNT_CASE(k) case k: asm volatile("s_waitcnt vmcnt(" #k ")" ::: "memory"); break;
    switch(__builtin_amdgcn_readfirstlane(n)) {
        SAGA_VMCNT_CASE(1) SAGA_VMCNT_CASE(2) SAGA_VMCNT_CASE(3) SAGA_VMCNT_CASE(4) SAGA_VMCNT_CASE(5) SAGA_VMCNT_CASE(6)
        SAGA_VMCNT_CASE(7) SAGA_VMCNT_CASE(8) SAGA_VMCNT_CASE(9) SAGA_VMCNT_CASE(10) SAGA_VMCNT_CASE(11) SAGA_VMCNT_CASE(12)
        SAGA_VMCNT_CASE(13) SAGA_VMCNT_CASE(14) SAGA_VMCNT_CASE(15) SAGA_VMCNT_CASE(16) SAGA_VMCNT_CASE(17) SAGA_VMCNT_CASE(18)
        SAGA_VMCNT_CASE(19) SAGA_VMCNT_CASE(20) SAGA_VMCNT_CASE(21) SAGA_VMCNT_CASE(22) SAGA_VMCNT_CASE(23) SAGA_VMCNT_CASE(24)
        SAGA_VMCNT_CASE(25) SAGA_VMCNT_CASE(26) SAGA_VMCNT_CASE(27) SAGA_VMCNT_CASE(28) SAGA_VMCNT_CASE(29) SAGA_VMCNT_CASE(30)
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef SAGA_VMCNT_CASE
}

// Epilogue of conv_rows64_wide: a wavefront's 64 pixels x 64 channels.  alpha / beta, the folded batch norm
// (MODE 1, table at bnp), rounding to fp16 - and the stores go out as whole pixels: the accumulator layout gives a
// lane 16-byte pieces of 32 different pixels, i.e. 32 cache lines touched per store instruction; the pieces are
// exchanged through LDS (stg: this wavefront's kilobyte q at stg + 4096 * q, rows of 128 bytes with the 16-byte
// chunks XOR-swizzled by the row) so that a store instruction writes 8 whole pixels.  soff[it]: byte offset in the
// output of chunk lane%8 of pixel 8*it + lane/8 of the wavefront, or out of range.
template <int MODE>
__device__ __forceinline__ void rows64_wide_epilogue(const GatherArgs &g, float16_t (&acc)[2][2], const float *bnp, char *stg,
                                                     int lane, const bool (&okr)[2], const int64_t (&pix)[2],
                                                     const unsigned (&soff)[8])
{
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const int hi = lane >> 5;
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) {
            float f[16];
#pragma unroll
            for(int v = 0; v < 16; v++)
                f[v] = g.alpha * acc[i][j][v];
            if(g.beta != 0.0f) {
                float old[16];
                load_row32(g.out + pix[i] * g.ldo, okr[i], j * 32, g.Ngemm, hi, old);
#pragma unroll
                for(int v = 0; v < 16; v++)
                    f[v] += g.beta * old[v];
            }
            if constexpr(MODE == 1) {
#pragma unroll
                for(int q = 0; q < 4; q++) {
                    const int cl = j * 32 + 8 * q + 4 * hi;
                    const float4_t sc = *(const float4_t *)(bnp + cl), sh = *(const float4_t *)(bnp + 64 + cl);
#pragma unroll
                    for(int e = 0; e < 4; e++) {
                        float t = __builtin_fmaf(f[4 * q + e], sc[e], sh[e]);
                        if(g.bn_flags & SAGA_BN_RELU)
                            t = (t != t) ? t : fmaxf(t, 0.0f);
                        f[4 * q + e] = t;
                    }
                }
            }
            const int row = i * 32 + (lane & 31);
            char *srow = stg + (row >> 3) * 4096 + (row & 7) * 128;
#pragma unroll
            for(int q = 0; q < 2; q++) {
                const unsigned x0 = pack2(f[8 * q + 0], f[8 * q + 1]), x1 = pack2(f[8 * q + 2], f[8 * q + 3]);
                const unsigned y0 = pack2(f[8 * q + 4], f[8 * q + 5]), y1 = pack2(f[8 * q + 6], f[8 * q + 7]);
                const auto s0_ = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
                const auto s1_ = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
                const u4 o = {s0_[0], s1_[0], s0_[1], s1_[1]};
                const int chunk = 4 * j + 2 * q + hi;
                *(u4 *)(srow + ((chunk ^ (row & 7)) << 4)) = o;
            }
        }
    // LDS operations of one wavefront complete in order: its reads below see its writes above
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void *)g.out, 0, g.out_bytes, 0x00020000);
    const int r8 = lane >> 3, chunk = lane & 7;
#pragma unroll
    for(int it = 0; it < 8; it++) {
        const u4 o = *(const u4 *)(stg + it * 4096 + r8 * 128 + ((chunk ^ r8) << 4));
        const unsigned off = soff[it]; // (a local: see the loads)
        __builtin_amdgcn_raw_buffer_store_b128(o, ro, off, 0, 0);
    }
}

// the loads of one tile's rows (conv_rows64_wide)
struct Rows64Req {
    const char *img; // the tile's image
    unsigned base;   // byte offset of the tile's first input row inside it (may be negative: rows above the image)
    char *dst;       // this wavefront's first kilobyte of the tile's LDS buffer
};

// The same convolution with one wavefront per SIMD: four wavefronts, each with 64 pixels x ALL 64 output channels
// and the whole filter in registers (288 of the 512 a lone wavefront may use).  In conv_rows64 every matrix
// instruction needs a 16-byte LDS read of its own, which is exactly what a CU's LDS delivers while the matrix units
// run flat out - two pipelines that would both have to be 100 % busy; here one pixel operand feeds two
// instructions.  No other wavefront fills a SIMD's gaps any more, so the matrix phase is scheduled by hand (LDS
// reads one tap ahead, pinned between the matrix instructions: it then runs at the matrix unit's rate) and the
// rest of a tile's work is kept short:
// - the byte offsets of a lane's row loads are computed once (a tile's position is one scalar added to them, and
//   the rows above and below an image fall outside a buffer that covers just that image);
// - the rows go through THREE LDS buffers; the loads of the tile after the next are issued one at a time between
//   the matrix instructions, and the wait in front of a tile's barrier leaves them and the previous tile's stores
//   in flight;
// - the filter reaches the registers through LDS (fetched straight from memory a lane's fragments are 1152 bytes
//   from its neighbour's, 64 cache lines per load instruction, times four wavefronts: 10 us before the first tile);
// - the outputs are exchanged through LDS so that a store instruction writes whole pixels (rows64_wide_epilogue).
template <int MODE, bool FLIP> __global__ void __launch_bounds__(256, 1) conv_rows64_wide(GatherArgs g, Rows64Args t)
{
    float *const stats = MODE == 2 ? g.stats : nullptr;
    g.stats = nullptr;
    if constexpr(MODE != 1)
        g.bn_s = nullptr;
    else
        g.bn_flags &= SAGA_BN_RELU;
    if constexpr(MODE != 0)
        g.beta = 0.0f;
    float run_s = 0.0f, run_q = 0.0f;
    constexpr int TM = 2, TN = 2, NLD_MAX = 13, SLOT = 144, NW = 4;
    constexpr unsigned OOB = 0x7fffff00u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hi = lane >> 5;

    // LDS chunk L = (q * 4 + wave) * 64 + lane of a tile's copy: pixel slot L / 9 (row r, column p of the padded
    // rows), chunk L % 9 of the slot (the ninth is padding): channels 8*(L%9).. of the pixel p - 1 of row r of the
    // tile's TR + 2 input rows, as a byte offset from the tile's first input row (which may lie above the image).
    // Every wavefront issues the same nld loads per tile (a buffer is a whole number of 4 KB rounds).
    const int nld = t.buf_bytes >> 12; // NLD_MAX - 1 or NLD_MAX (the host's condition)
    unsigned roff[NLD_MAX];
    {
        // (from one load to the next L grows by 256 = 28 * 9 + 4: no division per load)
        const int L0 = wave * 64 + lane;
        int slot = L0 / 9, kpos = L0 - slot * 9;
        int r = slot / t.slots_row, pcol = slot - r * t.slots_row;
#pragma unroll
        for(int q = 0; q < NLD_MAX; q++) {
            const int ix = pcol - 1;
            const bool ok = slot * 9 + kpos < t.chunks_tile && kpos < 8 && ix >= 0 && ix < t.W;
            roff[q] = ok ? (unsigned)(((r * t.W + ix) * g.lda + kpos * 8) * 2) : OOB;
            kpos += 4;
            const int step = kpos >= 9 ? 29 : 28;
            kpos -= kpos >= 9 ? 9 : 0;
            slot += step;
            pcol += step;
#pragma unroll
            for(int w = 0; w < 3; w++) { // (slots_row >= 10: at most three rows further)
                const bool wrap = pcol >= t.slots_row;
                pcol -= wrap ? t.slots_row : 0;
                r += wrap ? 1 : 0;
            }
        }
    }
    const unsigned img_bytes = (unsigned)(t.H * t.W * g.lda * 2);
    const int row_bytes = t.W * g.lda * 2;
    // a tile's loads: rows outside the image are outside the buffer that covers just the image (a negative offset
    // is a huge unsigned one) and read as zeros
    // (a tile beyond the last one: every offset out of range - the loads are issued all the same, so that the count
    // of outstanding memory operations does not depend on it, and write zeros into a buffer that nobody reads)
    auto req_setup = [&](int tile, int buffer) {
        Rows64Req r;
        const bool real = tile < t.ntiles;
        const int tl = real ? tile : 0;
        const int n = tl / t.tpi;
        const int oy0 = (tl - n * t.tpi) * t.TR;
        r.img = (const char *)g.a + (int64_t)n * img_bytes;
        r.base = real ? (unsigned)((oy0 - 1) * row_bytes) : OOB;
        r.dst = smem + buffer * t.buf_bytes + wave * 1024;
        return r;
    };
    auto req_piece = [&](const Rows64Req &r, int q) {
        const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc((void *)r.img, 0, img_bytes, 0x00020000);
        // (the offset goes through a local: a captured array element passed directly makes the host pass drop the kernel)
        const unsigned off = roff[q];
        if(q < NLD_MAX - 1 || nld == NLD_MAX)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ri, (lds_ptr_t)(r.dst + q * (NW * 1024)), 16, off + r.base, 0, 0, 0);
    };
    // this lane's two pixels (row blocks i of the wavefront's 64) inside a tile: byte offset of the top left tap
    int abase[TM], prow[TM]; // prow: the pixel's output row inside the tile, or a row beyond every image
#pragma unroll
    for(int i = 0; i < TM; i++) {
        const int pp0 = wave * 64 + i * 32 + (lane & 31);
        const int pp = pp0 < t.npix ? pp0 : 0;
        const int orow = pp / t.W;
        abase[i] = (orow * t.slots_row + (pp - orow * t.W)) * SLOT + hi * 16;
        prow[i] = pp0 < t.npix ? orow : 0x40000000;
    }
    // the stores' side: store instruction it writes chunk lane%8 of pixel 8*it + lane/8 of the wavefront's 64
    int srow[8];       // that pixel's output row inside the tile, or a row beyond every image
    unsigned sconst[8]; // its byte offset from the tile's first output pixel
#pragma unroll
    for(int it = 0; it < 8; it++) {
        const int pp0 = wave * 64 + it * 8 + (lane >> 3);
        const bool ok = pp0 < t.npix && (lane & 7) * 8 < g.Ngemm;
        srow[it] = ok ? pp0 / t.W : 0x40000000;
        sconst[it] = (unsigned)((pp0 * g.ldo + (lane & 7) * 8) * 2);
    }
    char *epi = smem + t.epi_off;
    const int G = gridDim.x;
    int tile = xcd_remap(blockIdx.x, G);
    const int first_tile = tile;
    {
        const Rows64Req r0 = req_setup(tile, 0);
#pragma unroll
        for(int q = 0; q < NLD_MAX; q++)
            req_piece(r0, q);
    }
    // The filter, [channel][tap][64] in memory.  A lane's fragments lie 1152 bytes from its neighbour's, so loading
    // them straight into registers touches 64 cache lines per instruction (and four wavefronts do it): the block
    // copies the filter through LDS instead - whole kilobytes per load instruction, into the two buffers that are
    // still free, as rows of 73 sixteen-byte chunks (72 + 1 of padding: a fragment read then hits 64 different
    // banks) - and every wavefront picks its fragments there.  Channels beyond the filter's read as zeros.
    {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void *)g.b, 0, g.b_bytes, 0x00020000);
        char *stage = smem + t.buf_bytes + wave * 1024;
#pragma unroll
        for(int q = 0; q < 19; q++) { // 64 * 73 = 4672 chunks, 256 per round
            const int L = (q * NW + wave) * 64 + lane;
            const int row = L / 73, cpos = L - row * 73;
            const unsigned off = (cpos < 72 && row < (FLIP && g.b_krsc ? g.Cred : g.Ngemm) && row < 64) ? (unsigned)((row * 576 + cpos * 8) * 2) : OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(stage + q * (NW * 1024)), 16, off, 0, 0, 0);
        }
    }
    if constexpr(MODE == 1) // the folded norm's table: the same for every tile
        bnfold_table<64>(g, (float *)(epi + 32768), tid, 0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // fragment (tap, kk, j) = halves 16*kk + 8*hi .. +8 of that tap of output channel 32*j + lane%32
    half8_t fb[9][4][TN];
    if(FLIP && g.b_krsc) {
        // Backward data straight from the forward filter w[k][tap][c] (no transposed copy: a stand-alone call saves
        // the launch that makes one): a fragment is 8 consecutive k of one c, which is what the transposing LDS read
        // delivers - the lane points at row k = 16*kk + fp (the read's second half: + 4) and 4 columns of its tile.
        const int fp = 8 * (lane >> 5) + ((lane & 15) >> 2), fc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
        const unsigned src = (unsigned)(uintptr_t)(lds_ptr_t)(smem + t.buf_bytes) + fp * (73 * 16) + fc * 2;
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int tp = 0; tp < 9; tp++) {
#pragma unroll
                for(int kk = 0; kk < 4; kk++)
                    fb[tp][kk][j] = tr_read8_raw<0, 4 * 73 * 16>(src + kk * (16 * 73 * 16) + ((8 - tp) * 64 + j * 32) * 2);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                for(int kk = 0; kk < 4; kk++)
                    asm volatile("" : "+v"(fb[tp][kk][j]));
            }
    } else {
#pragma unroll
        for(int j = 0; j < TN; j++) {
            const char *src = smem + t.buf_bytes + (j * 32 + (lane & 31)) * (73 * 16) + hi * 16;
#pragma unroll
            for(int tp = 0; tp < 9; tp++)
#pragma unroll
                for(int kk = 0; kk < 4; kk++)
                    fb[tp][kk][j] = *(const half8_t *)(src + (FLIP ? 8 - tp : tp) * 128 + kk * 32);
        }
    }
    // (everybody has its fragments before the second tile's rows overwrite them)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const Rows64Req r1 = req_setup(tile + G, 1);
#pragma unroll
    for(int q = 0; q < NLD_MAX; q++)
        req_piece(r1, q);
    // (the first tile's rows arrived with the filter)
    constexpr int NST = TM * TN * 2; // the epilogue's stores per tile (always all of them: BUFST)
    int b = 0;      // buffer of the current tile; the next tile's is b + 1, the one after goes to b + 2 (mod 3)
    int behind = 0; // this wavefront's memory operations issued after the next tile's loads and before this tile's
    for(; tile < t.ntiles; tile += G) {
        const char *buf = smem + b * t.buf_bytes;
        // the rows of the tile after the next go out between this tile's multiplications, into the buffer that the
        // previous tile has left (every wavefront has passed that tile's barrier)
        const Rows64Req rq = req_setup(tile + 2 * G, b >= 1 ? b - 1 : 2);
        float16_t acc[TM][TN];
#pragma unroll
        for(int i = 0; i < TM; i++)
#pragma unroll
            for(int j = 0; j < TN; j++)
#pragma unroll
                for(int v = 0; v < 16; v++)
                    acc[i][j][v] = 0.0f;
        // one tap ahead: the reads of tap + 1 go out between the multiplications of tap, two per four matrix
        // instructions (the scheduling barriers pin LDS reads, loads and matrix instructions, other instructions
        // may move: left to itself the compiler issues each read right in front of its first use and waits for it)
        half8_t fa[2][4][TM];
#pragma unroll
        for(int kk = 0; kk < 4; kk++)
#pragma unroll
            for(int i = 0; i < TM; i++)
                fa[0][kk][i] = *(const half8_t *)(buf + abase[i] + kk * 32);
        __builtin_amdgcn_sched_barrier(0x6);
#pragma unroll
        for(int tp = 0; tp < 9; tp++) {
            const int tapoff = tp + 1 < 9 ? (((tp + 1) / 3) * t.slots_row + (tp + 1) % 3) * SLOT : 0;
#pragma unroll
            for(int kk = 0; kk < 4; kk++) {
                if(tp + 1 < 9) {
#pragma unroll
                    for(int i = 0; i < TM; i++)
                        fa[(tp + 1) & 1][kk][i] = *(const half8_t *)(buf + abase[i] + tapoff + kk * 32);
                }
                __builtin_amdgcn_sched_barrier(0x6);
#pragma unroll
                for(int i = 0; i < TM; i++)
#pragma unroll
                    for(int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[tp][kk][j], fa[tp & 1][kk][i], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0x6);
                // (a load every second or third group of four)
#pragma unroll
                for(int q = 0; q < NLD_MAX; q++)
                    if((q * 36) / NLD_MAX == tp * 4 + kk) {
                        req_piece(rq, q);
                        __builtin_amdgcn_sched_barrier(0x6);
                    }
            }
        }
        // The NEXT tile's rows must have arrived before the barrier that lets everybody read them.  Behind them this
        // wavefront has issued the previous tile's stores and this tile's loads: those may stay in flight.
        wait_vmcnt(behind + nld);
        asm volatile("s_barrier" ::: "memory");
        behind = NST;
        const int n = tile / t.tpi;
        const int oy0 = (tile - n * t.tpi) * t.TR;
        const int64_t pix0 = ((int64_t)n * t.H + oy0) * t.W;
        bool okr[TM];
        int64_t pix[TM];
#pragma unroll
        for(int i = 0; i < TM; i++) {
            okr[i] = oy0 + prow[i] < t.H;
            pix[i] = pix0 + (okr[i] ? wave * 64 + i * 32 + (lane & 31) : 0);
        }
        unsigned soff[8];
        const unsigned tile_off = (unsigned)(pix0 * g.ldo * 2); // (the output's bytes fit 31 bits: the host's condition)
#pragma unroll
        for(int it = 0; it < 8; it++)
            soff[it] = oy0 + srow[it] < t.H ? sconst[it] + tile_off : OOB;
        // (staged in this tile's buffer: every wavefront is past the barrier, so nobody reads it any more, and
        // the kilobytes a wavefront stages in are the ones that only its own later loads write)
        rows64_wide_epilogue<MODE>(g, acc, (const float *)(epi + 32768), smem + b * t.buf_bytes + wave * 1024, lane, okr, pix, soff);
        if constexpr(MODE == 2) {
            float s0, q0;
            stats_lane_totals<TM, TN, true>(g.alpha, acc, okr, lane, s0, q0);
            run_s += s0;
            run_q += q0;
        }
        b = b == 2 ? 0 : b + 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // (loads into this block's LDS may still be in flight)
    if constexpr(MODE == 2) {
        g.stats = stats;
        __syncthreads();
        stats_block_write<TN, 4, 1, 64>(g, epi + 32768, tid, lane, wave, 0, 0, first_tile, run_s, run_q);
    }
}

// ---------------------------------------------------------------- backward filter of those layers, whole image rows in LDS
//
// dw[k][tap][c] = sum over pixels of dy[p][k] * x[p + tap][c] for the 3x3, stride-1 layers with 64 input channels and
// at most 64 output channels.  conv_bwd_filter_dma treats the nine taps as nine column blocks of a GEMM: x goes
// from L2 to LDS nine times, dy three times (three column tiles), and the partial tiles of a thousand blocks are
// 50 MB to write and read back.  Here, as in conv_rows64_wide, a persistent block of four wavefronts (one per SIMD)
// walks tiles of TR whole image rows: the TR + 2 rows of x (144-byte pixel slots with zero borders, the same copy
// as conv_rows64_wide's) and the TR rows of dy (128-byte pixel rows, 16-byte granules XOR-swizzled as in
// conv_bwd_filter_dma) are copied ONCE per tile, the x operand of tap (dr, ds) is the same copy read (dr, ds) slots
// further on, and the whole 64 x 9 x 64 result stays in the block's registers for the launch: wavefront (mt, nt)
// holds output channels 32*mt.. x input channels 32*nt.. of all nine taps (144 accumulator registers), and one
// partial per BLOCK goes to the second pass (filter_reduce_v4: 256 partials instead of 1000).
// The reduction index of an MFMA is the pixel: operands come from the transposing LDS read (tr_read8_raw), 16
// pixels per step, one dy operand and nine x operands for nine instructions.  One wavefront per SIMD: the reads run
// three operands ahead of the multiplications that use them, in program order (they are instructions of our own,
// and the waits in front of the multiplications count them), and a tile's loads go out between the multiplications
// of the tile before.  NSTEPS = pixels of a tile / 16 (the host's condition: a whole number).
struct FilterRowsArgs {
    const half_t *x, *dy;
    float *partial;      // [block][K][9][64]
    int ldx, ldy, H, W, K;
    int TR, tpi, ntiles; // output rows per tile, tiles per image, tiles
    int slots_row;       // W + 2 pixel slots per LDS row of x
    int xchunks;         // (TR + 2) * slots_row * 9: 16-byte chunks of a tile's x copy
    int x_bytes, y_bytes; // one LDS buffer of each (whole rounds of the four wavefronts' loads)
};

template <int NSTEPS> __global__ void __launch_bounds__(256, 1) conv_bwd_filter_rows64(FilterRowsArgs t)
{
    constexpr int NW = 4, SLOT = 144, NLX = 13, NLY = (NSTEPS * 16 * 8 + 255) / 256;
    constexpr unsigned OOB = 0x7fffff00u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mt = wave >> 1, nt = wave & 1;
    const int npix = NSTEPS * 16;

    // x rows: as in conv_rows64_wide (chunk L = (q * 4 + wave) * 64 + lane: slot L / 9, chunk L % 9 of it)
    const int nlx = t.x_bytes >> 12;
    unsigned roffx[NLX];
    {
        const int L0 = wave * 64 + lane;
        int slot = L0 / 9, kpos = L0 - slot * 9;
        int r = slot / t.slots_row, pcol = slot - r * t.slots_row;
#pragma unroll
        for(int q = 0; q < NLX; q++) {
            const int ix = pcol - 1;
            const bool ok = slot * 9 + kpos < t.xchunks && kpos < 8 && ix >= 0 && ix < t.W;
            roffx[q] = ok ? (unsigned)(((r * t.W + ix) * t.ldx + kpos * 8) * 2) : OOB;
            kpos += 4;
            const int step = kpos >= 9 ? 29 : 28;
            kpos -= kpos >= 9 ? 9 : 0;
            slot += step;
            pcol += step;
#pragma unroll
            for(int w = 0; w < 3; w++) {
                const bool wrap = pcol >= t.slots_row;
                pcol -= wrap ? t.slots_row : 0;
                r += wrap ? 1 : 0;
            }
        }
    }
    // dy rows: chunk L: pixel L / 8 of the tile, physical granule L % 8 = logical granule ^ 4 * bit 1 of the pixel
    unsigned roffy[NLY];
#pragma unroll
    for(int q = 0; q < NLY; q++) {
        const int L = (q * NW + wave) * 64 + lane;
        const int pp = L >> 3, gran = (L & 7) ^ (((pp >> 1) & 1) << 2);
        roffy[q] = (pp < npix && gran * 8 < t.K) ? (unsigned)((pp * t.ldy + gran * 8) * 2) : OOB;
    }
    const unsigned ximg = (unsigned)(t.H * t.W * t.ldx * 2), yimg = (unsigned)(t.H * t.W * t.ldy * 2);
    char *const xbuf = smem, *const ybuf = smem + 2 * t.x_bytes;
    // piece p of a tile's loads: the first NLX are x, the others dy.  A tile beyond the last one: every offset out
    // of range (the loads are issued all the same and write zeros into a buffer that nobody reads)
    auto req_piece = [&](int tile, int b, int p) {
        const bool real = tile < t.ntiles;
        const int tl = real ? tile : 0;
        const int n = tl / t.tpi;
        const int oy0 = (tl - n * t.tpi) * t.TR;
        if(p < NLX) {
            const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)t.x + (int64_t)n * ximg), 0, ximg, 0x00020000);
            const unsigned base = real ? (unsigned)((oy0 - 1) * t.W * t.ldx * 2) : OOB;
            const unsigned off = roffx[p]; // (a local: a captured array element passed directly makes the host pass drop the kernel)
            if(p < NLX - 1 || nlx == NLX)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(xbuf + b * t.x_bytes + (p * NW + wave) * 1024), 16, off + base, 0, 0, 0);
        } else {
            const int q = p - NLX;
            const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)t.dy + (int64_t)n * yimg), 0, yimg, 0x00020000);
            const unsigned base = real ? (unsigned)(oy0 * t.W * t.ldy * 2) : OOB;
            const unsigned off = roffy[q];
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ry, (lds_ptr_t)(ybuf + b * t.y_bytes + (q * NW + wave) * 1024), 16, off + base, 0, 0, 0);
        }
    };
    // Operand addresses.  A transposing read hands lane i (channel i of 16, 4 pixels): the lane points at pixel fp
    // (the read's second half: fp + 4) of the 16-pixel step and at 4 channels of its 32-channel tile.
    const int fp = 8 * (lane >> 5) + ((lane & 15) >> 2);
    const int fc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    const unsigned lds0 = (unsigned)(uintptr_t)(lds_ptr_t)smem;
    const int ca = mt * 32 + fc, cb = nt * 32 + fc;
    // dy: pixel rows of 128 bytes (the swizzle term is the same for every step: steps are 16 pixels apart)
    const unsigned ya = (unsigned)(fp * 128 + (((ca >> 3) ^ (((fp >> 1) & 1) << 2)) << 4) + (ca & 7) * 2);
    // x: the slot of the lane's two pixels in step 0, and their columns (a step moves 16 pixels on, across row ends)
    const unsigned xc = (unsigned)((cb >> 3) * 16 + (cb & 7) * 2);
    const int r0lo = fp / t.W, c0lo = fp - r0lo * t.W, r0hi = (fp + 4) / t.W, c0hi = fp + 4 - r0hi * t.W;
    unsigned tapoff[9];
#pragma unroll
    for(int tp = 0; tp < 9; tp++)
        tapoff[tp] = (unsigned)(((tp / 3) * t.slots_row + tp % 3) * SLOT);

    float16_t acc[9];
#pragma unroll
    for(int tp = 0; tp < 9; tp++)
#pragma unroll
        for(int v = 0; v < 16; v++)
            acc[tp][v] = 0.0f;

    const int G = gridDim.x;
    int tile = xcd_remap(blockIdx.x, G);
#pragma unroll
    for(int p = 0; p < NLX + NLY; p++)
        req_piece(tile, 0, p);
    int b = 0;
    for(; tile < t.ntiles; tile += G) {
        // this tile's rows have arrived (everybody's: the barrier), and everybody is done with the other buffer
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        const unsigned xb = lds0 + b * t.x_bytes + xc, yb = lds0 + 2 * t.x_bytes + b * t.y_bytes + ya;
        int rlo = r0lo, clo = c0lo, rhi = r0hi, chi = c0hi; // the step's pixels: row inside the tile, column
        auto xaddr = [&](int r, int c) { return xb + (unsigned)((r * t.slots_row + c) * SLOT); };
        auto next_step = [&]() {
            clo += 16;
            const bool wl = clo >= t.W;
            clo -= wl ? t.W : 0;
            rlo += wl ? 1 : 0;
            chi += 16;
            const bool wh = chi >= t.W;
            chi -= wh ? t.W : 0;
            rhi += wh ? 1 : 0;
        };
        auto read_x = [&](unsigned alo, unsigned ahi, int tp) {
            short4_t lo, hi;
            asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(alo + tapoff[tp]) : "memory");
            asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(hi) : "v"(ahi + tapoff[tp]) : "memory");
            const short8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(half8_t, v);
        };
        // the pipeline of operand reads: item (step, -1) is the step's dy operand, (step, tp) its x operand of tap
        // tp; three x operands ahead of the multiplication that uses them
        half8_t fa[2], fb[2][9];
        unsigned alo = xaddr(rlo, clo), ahi = xaddr(rhi, chi);
        fa[0] = tr_read8_raw<0, 512>(yb);
        fb[0][0] = read_x(alo, ahi, 0);
        fb[0][1] = read_x(alo, ahi, 1);
        fb[0][2] = read_x(alo, ahi, 2);
#pragma unroll
        for(int st = 0; st < NSTEPS; st++) {
            const int cur = st & 1, nxt = cur ^ 1;
            unsigned nlo = alo, nhi = ahi;
#pragma unroll
            for(int tp = 0; tp < 9; tp++) {
                // issue: the x operand three taps on; at the end of a step the next step's dy operand and first x
                // operands (after the last step: the first step's again, never used - the waits count them)
                if(tp < 6) {
                    fb[cur][tp + 3] = read_x(alo, ahi, tp + 3);
                } else if(tp == 6) {
                    if(st + 1 < NSTEPS) {
                        next_step();
                        nlo = xaddr(rlo, clo);
                        nhi = xaddr(rhi, chi);
                    }
                    fa[nxt] = st + 1 < NSTEPS ? tr_read8_raw<0, 512>(yb + (st + 1) * 2048) : tr_read8_raw<0, 512>(yb);
                } else if(tp == 7) {
                    fb[nxt][0] = read_x(nlo, nhi, 0);
                } else {
                    fb[nxt][1] = read_x(nlo, nhi, 1);
                    fb[nxt][2] = read_x(nlo, nhi, 2);
                }
                // wait for this multiplication's operands: three items (two instructions each) were issued
                // behind them, four at the last tap
                if(tp == 8)
                    asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
                else
                    asm volatile("s_waitcnt lgkmcnt(6)" ::: "memory");
                asm volatile("" : "+v"(fa[cur]), "+v"(fb[cur][tp]));
                acc[tp] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[cur], fb[cur][tp], acc[tp], 0, 0, 0);
                // the next tile's loads: two per step, four multiplications apart, while there are any
                constexpr int NP = NLX + NLY;
                static_assert(2 * NSTEPS >= NP, "a step issues two of the next tile's loads");
                if((tp == 2 || tp == 6) && 2 * st + (tp == 6) < NP) {
                    __builtin_amdgcn_sched_barrier(0);
                    req_piece(tile + G, b ^ 1, 2 * st + (tp == 6));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            alo = nlo;
            ahi = nhi;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // (the reads that nobody uses)
        b ^= 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // (loads into this block's LDS may still be in flight)
    // the block's partial: acc[tp][v] = element (k = 32*mt + 8*(v/4) + 4*(lane/32) + v%4, tap tp, c = 32*nt + lane%32)
    float *out = t.partial + (int64_t)blockIdx.x * t.K * 576;
    const int ecol = nt * 32 + (lane & 31), erow = mt * 32 + (lane >> 5) * 4;
#pragma unroll
    for(int tp = 0; tp < 9; tp++)
#pragma unroll
        for(int v = 0; v < 16; v++) {
            const int k = erow + (v >> 2) * 8 + (v & 3);
            if(k < t.K)
                out[(int64_t)k * 576 + tp * 64 + ecol] = acc[tp][v];
        }
}

// Launches conv_rows64 if the geometry is its: returns false (and launches nothing) otherwise.  g: as for
// launch_gather, with a = the NHWC input (pixel pitch lda), b = [Ngemm][9][64].
// krsc: b is the untransposed forward filter (backward data only): only the kernel that can read it that way may run.
template <bool FLIP> static bool launch_rows64(GatherArgs &g, const CLInfo &lout, hipStream_t st, size_t stats_floats, int *rc, bool krsc = false)
{
    g.b_krsc = krsc ? 1 : 0;
    if(krsc && (g.Ngemm != 64 || g.Cred != 64))
        return false;
    static const bool off = getenv("SAGA_HIP_ROWS64") && atoi(getenv("SAGA_HIP_ROWS64")) == 0;
    if(off || g.R != 3 || g.S != 3 || g.Cred != 64 || g.Ngemm > 64 || g.Ngemm % 8 || g.stride != 1 || g.pad != 1 ||
       g.dil != 1 || g.IH != g.OH || g.IW != g.OW || g.OW < 8 || (g.bn_s && (g.bn_flags & SAGA_BN_ADD)) || g.bq_partial || !g.a_bytes || !g.b_bytes)
        return false;
    Rows64Args t;
    t.H = g.OH;
    t.W = g.OW;
    static const int wgm = getenv("SAGA_HIP_ROWS64_WGM") ? atoi(getenv("SAGA_HIP_ROWS64_WGM")) : 4;
    const int bm = wgm == 2 ? 128 : 256;
    if(t.W > bm)
        return false;
    t.TR = std::min(bm / t.W, t.H);
    t.tpi = (t.H + t.TR - 1) / t.TR;
    const int64_t nimg = (int64_t)g.M / ((int64_t)t.H * t.W);
    if(nimg * t.tpi > 0x7fffffff || nimg * t.tpi < 2 * num_cus()) // small problems: too few tiles to walk
        return false;
    t.ntiles = (int)(nimg * t.tpi);
    t.npix = t.TR * t.W;
    t.slots_row = t.W + 2;
    t.chunks_tile = (t.TR + 2) * t.slots_row * 9;
    t.buf_bytes = (t.chunks_tile * 16 + 1023) & ~1023;
    const int buf_narrow = t.buf_bytes;
    const int epi_back = wgm == 2 ? 16384 : 32768; // gather_epilogue's scratch sits this far behind its base
    const bool vec_ok = (lout.pitch & 7) == 0 && aligned16(g.out) && ((lout.rows - 1) * lout.pitch + g.Ngemm) * 2 < 0x7fffff00ll &&
                        (g.lda & 7) == 0 && aligned16(g.a);
    // one wavefront per SIMD with the whole filter in registers, where a block may have the LDS for three buffers
    static const bool wide_on = !(getenv("SAGA_HIP_ROWS64_WIDE") && atoi(getenv("SAGA_HIP_ROWS64_WIDE")) == 0);
    static const int lds_max = [] {
        int dev = 0, v = 0;
        if(hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess)
            return 64 * 1024;
        return std::min(v, 160 * 1024);
    }();
    t.buf_bytes = (t.chunks_tile * 16 + 4095) & ~4095; // (a whole number of rounds of the four wavefronts' loads)
    if(wide_on && wgm == 4 && vec_ok && t.chunks_tile <= 13 * 256 && t.chunks_tile > 11 * 256 && (int64_t)t.H * t.W * g.lda * 2 < 0x7fff0000ll) {
        const int epi_at = std::max(3 * t.buf_bytes, epi_back);
        t.epi_off = epi_at - epi_back;
        const int lds = epi_at + 4096;
        const int blocks = std::min(t.ntiles, num_cus());
        if(lds <= lds_max && !(g.stats && (size_t)blocks * g.Ngemm * 2 > stats_floats)) {
            static bool once = false;
            if(!once) {
                for(const void *k : {(const void *)conv_rows64_wide<0, FLIP>, (const void *)conv_rows64_wide<1, FLIP>,
                                     (const void *)conv_rows64_wide<2, FLIP>}) {
                    const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds_max);
                    if(e != hipSuccess) {
                        *rc = (int)e;
                        return true;
                    }
                }
                once = true;
            }
            g.classes = 1;
            g.no_stage = 1;
            g.nblk_n = 1;
            g.out_bytes = (unsigned)(((lout.rows - 1) * lout.pitch + g.Ngemm) * 2);
            g.stats_rows = blocks;
            if(g.bn_s)
                conv_rows64_wide<1, FLIP><<<blocks, 256, lds, st>>>(g, t);
            else if(g.stats)
                conv_rows64_wide<2, FLIP><<<blocks, 256, lds, st>>>(g, t);
            else
                conv_rows64_wide<0, FLIP><<<blocks, 256, lds, st>>>(g, t);
            *rc = 0;
            return true;
        }
    }
    if(krsc)
        return false;
    t.buf_bytes = buf_narrow;
    const int epi_at = std::max(2 * t.buf_bytes, epi_back);
    t.epi_off = epi_at - epi_back;
    const int lds = epi_at + 4096;
    const int blocks = std::min(t.ntiles, (wgm == 2 ? 2 : 1) * num_cus());
    if(!vec_ok || t.chunks_tile > 10 * (wgm == 2 ? 256 : 512) || lds > (wgm == 2 ? 76 : 150) * 1024 || (g.stats && (size_t)blocks * g.Ngemm * 2 > stats_floats))
        return false;
    static bool once = false;
    if(!once) {
        for(const void *k : {(const void *)conv_rows64<0, FLIP, 4>, (const void *)conv_rows64<1, FLIP, 4>,
                             (const void *)conv_rows64<2, FLIP, 4>, (const void *)conv_rows64<0, FLIP, 2>,
                             (const void *)conv_rows64<1, FLIP, 2>, (const void *)conv_rows64<2, FLIP, 2>}) {
            const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
            if(e != hipSuccess) {
                *rc = (int)e;
                return true;
            }
        }
        once = true;
    }
    g.classes = 1;
    g.no_stage = 1;
    g.nblk_n = 1;
    g.out_bytes = (unsigned)(((lout.rows - 1) * lout.pitch + g.Ngemm) * 2);
    g.stats_rows = blocks;
#define GO_ROWS64(W_)                                                        \
    do {                                                                     \
        if(g.bn_s)                                                           \
            conv_rows64<1, FLIP, W_><<<blocks, 128 * W_, lds, st>>>(g, t);    \
        else if(g.stats)                                                     \
            conv_rows64<2, FLIP, W_><<<blocks, 128 * W_, lds, st>>>(g, t);    \
        else                                                                 \
            conv_rows64<0, FLIP, W_><<<blocks, 128 * W_, lds, st>>>(g, t);    \
    } while(0)
    if(wgm == 2)
        GO_ROWS64(2);
    else
        GO_ROWS64(4);
#undef GO_ROWS64
    *rc = 0;
    return true;
}

static void launch_pad_thin(const half_t *x, int64_t pitch, const ConvGeom &g, half_t *x4, const ThinGeom &tg, int64_t px,
                            hipStream_t st)
{
    const int64_t blocks = (int64_t)g.N * tg.Hp;
    if(g.C == 3 && pitch == 3 && (g.W * 6) % 16 == 0 && aligned16(x) && tg.Wp % 2 == 0 && blocks < (1ll << 31) &&
       (size_t)g.W * 6 <= 48 * 1024)
        pad_thin_rgb_rows<<<(int)blocks, 128, (size_t)g.W * 6, st>>>(x, g.H, g.W, g.pad, x4, tg.Hp, tg.Wp);
    else
        pad_thin<<<grid_for(px, 256, 1 << 20), 256, 0, st>>>(x, pitch, g.C, g.H, g.W, g.pad, x4, tg.Hp, tg.Wp, px);
}

// out[row][0..C) = 0 for rows of pitch `pitch` elements (C and pitch multiples of 8, 16-byte aligned)
__global__ void __launch_bounds__(256) zero_rows(half_t *__restrict__ out, int64_t rows, int C, int64_t pitch)
{
    const int groups = C / 8;
    const int64_t total = rows * groups;
    const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / groups;
        *(half8_t *)(out + r * pitch + (i - r * groups) * 8) = z;
    }
}

// ---------------------------------------------------------------- 1x1, 64 -> 256 channels: a streaming kernel
//
// The 1x1 convolutions that widen 64 channels to 256 over large images (ResNet-50's first stage, 56x56: 103 MB in,
// 411 MB out at batch 256) are stores and little else: 64 multiply-adds per output.  Through the gather kernel a
// block lives for two slices of the reduction, and its prologue, its barriers and the drain of its stores are not
// hidden by the one other block of the CU: 132 - 145 us, 3.6 TB/s, where plain stores reach 6.9 TB/s.  Here the
// whole filter stays in registers and a WAVEFRONT, not a block, is the unit: it owns strips of 64 pixels and one half
// of the output channels (the two wavefronts of a pair copy the same strip, the second time from L2), copies a
// strip into its own LDS (144-byte pixel slots, as in conv_rows64), multiplies and stores - no barrier after the
// set-up, the next strip's copy in flight behind this strip's stores.  Eight wavefronts per CU, two per SIMD: one
// converts and stores while the other multiplies.
template <int MODE>
__device__ __forceinline__ void c64_epilogue(const GatherArgs &g, float16_t (&acc)[2][2], const float *bnp, char *stg, int lane,
                                             int c0, const bool (&okr)[2], const int64_t (&pix)[2], const unsigned (&soff)[8],
                                             float (&st)[16])
{
    // (rows64_wide_epilogue for channels c0 .. c0 + 63 of a wider output, this wavefront's kilobytes contiguous,
    // no beta, and the residual of the folded norm)
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const int hi = lane >> 5;
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) {
            float f[16];
#pragma unroll
            for(int v = 0; v < 16; v++)
                f[v] = acc[i][j][v];
            if(g.alpha != 1.0f) {
#pragma unroll
                for(int v = 0; v < 16; v++)
                    f[v] *= g.alpha;
            }
            if constexpr(MODE == 1) {
                float zz[16];
                if(g.bn_flags & SAGA_BN_ADD)
                    load_row32(g.z + pix[i] * g.ldz, okr[i], c0 + j * 32, g.Ngemm, hi, zz);
#pragma unroll
                for(int q = 0; q < 4; q++) {
                    const int cl = j * 32 + 8 * q + 4 * hi;
                    const float4_t sc = *(const float4_t *)(bnp + cl), sh = *(const float4_t *)(bnp + 64 + cl);
#pragma unroll
                    for(int e = 0; e < 4; e++) {
                        float t = __builtin_fmaf(f[4 * q + e], sc[e], sh[e]);
                        if(g.bn_flags & SAGA_BN_ADD)
                            t += zz[4 * q + e];
                        if(g.bn_flags & SAGA_BN_RELU)
                            t = (t != t) ? t : fmaxf(t, 0.0f);
                        f[4 * q + e] = t;
                    }
                }
            }
            const int row = i * 32 + (lane & 31);
            char *srow = stg + (row >> 3) * 1024 + (row & 7) * 128;
#pragma unroll
            for(int q = 0; q < 2; q++) {
                const unsigned x0 = pack2(f[8 * q + 0], f[8 * q + 1]), x1 = pack2(f[8 * q + 2], f[8 * q + 3]);
                const unsigned y0 = pack2(f[8 * q + 4], f[8 * q + 5]), y1 = pack2(f[8 * q + 6], f[8 * q + 7]);
                const auto s0_ = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
                const auto s1_ = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
                const u4 o = {s0_[0], s1_[0], s0_[1], s1_[1]};
                const int chunk = 4 * j + 2 * q + hi;
                *(u4 *)(srow + ((chunk ^ (row & 7)) << 4)) = o;
            }
        }
    // LDS operations of one wavefront complete in order: its reads below see its writes above
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void *)g.out, 0, g.out_bytes, 0x00020000);
    const int r8 = lane >> 3, chunk = lane & 7;
#pragma unroll
    for(int it = 0; it < 8; it++) {
        const u4 o = *(const u4 *)(stg + it * 1024 + r8 * 128 + ((chunk ^ r8) << 4));
        const unsigned off = soff[it]; // (a local: an element of a captured array passed directly makes the host pass drop the kernel)
        // (plain stores: with the non-temporal hint this kernel alone writes at 6.3 TB/s instead of 5.0, but inside a
        // network the next operation no longer finds the tail of the tensor in the last-level cache and the step as a
        // whole takes longer)
        __builtin_amdgcn_raw_buffer_store_b128(o, ro, off, 0, 0);
        if constexpr(MODE == 2) {
            // Statistics of the values as stored: here a lane holds 8 channels of ONE pixel, so sums over pixels are
            // sums in the lane's own registers (st: 8 sums, 8 sums of squares; a pixel past the tensor's end holds
            // zeros) and the lanes are added up once, at the end of the launch.
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for(int e = 0; e < 4; e++) {
                const unsigned w = o[e]; // (bit_cast of the element expression itself reads element 0 for every e)
                const h2 v = __builtin_bit_cast(h2, w);
                const float a = (float)v[0], b = (float)v[1];
                st[2 * e] += a;
                st[2 * e + 1] += b;
                st[8 + 2 * e] = __builtin_fmaf(a, a, st[8 + 2 * e]);
                st[8 + 2 * e + 1] = __builtin_fmaf(b, b, st[8 + 2 * e + 1]);
            }
        }
    }
}

constexpr int C64_BUF = 9216;                       // a strip in LDS: 64 pixel slots of 144 bytes
constexpr int C64_LDS = 8 * 2 * C64_BUF + 256 * 8;  // two strips per wavefront, the folded norm's table behind them

template <int MODE> __global__ void __launch_bounds__(512, 1) conv1x1_c64_n256(GatherArgs g, int nstrips)
{
    float *const stats = MODE == 2 ? g.stats : nullptr;
    g.stats = nullptr;
    if constexpr(MODE != 1)
        g.bn_s = nullptr;
    constexpr int SLOT = 144, NLD = 9, NST = 16;
    constexpr unsigned OOB = 0x7fffff00u;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hi = lane >> 5;
    const int half = wave & 1, slot = wave >> 1; // which half of the output channels, which of the block's four strips
    float *bnp = (float *)(smem + 8 * 2 * C64_BUF);

    // The filter, [256][64] halves: through LDS (whole kilobytes per load instruction, rows of 144 bytes so that a
    // fragment read hits 64 different banks), then this wavefront's 128 channels into registers.
    {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void *)g.b, 0, g.b_bytes, 0x00020000);
#pragma unroll
        for(int q = 0; q < 5; q++) { // 256 * 9 = 2304 chunks, 512 per round
            const int L = q * 512 + tid;
            const int row = L / 9, k = L - row * 9;
            const unsigned off = (k < 8 && row < 256) ? (unsigned)((row * 64 + k * 8) * 2) : OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(smem + (q * 8 + wave) * 1024), 16, off, 0, 0, 0);
        }
    }
    if constexpr(MODE == 1) {
#pragma unroll
        for(int cb = 0; cb < 4; cb++)
            bnfold_table<64>(g, bnp + cb * 128, tid, cb * 64);
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // fragment (cb, kk, j) = halves 16*kk + 8*hi .. +8 of output channel 128*half + 64*cb + 32*j + lane%32
    half8_t fb[2][4][2];
#pragma unroll
    for(int cb = 0; cb < 2; cb++)
#pragma unroll
        for(int j = 0; j < 2; j++) {
            const char *src = smem + (half * 128 + cb * 64 + j * 32 + (lane & 31)) * SLOT + hi * 16;
#pragma unroll
            for(int kk = 0; kk < 4; kk++)
                fb[cb][kk][j] = *(const half8_t *)(src + kk * 32);
        }
    // (everybody has its fragments before the first strips overwrite the staged filter)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // Chunk L = q * 64 + lane of a strip's copy: chunk L % 9 of pixel L / 9 (the ninth is the slot's padding), as a
    // byte offset from the strip's first pixel.  Pixels past the tensor's end are out of the buffer's range.
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void *)g.a, 0, g.a_bytes, 0x00020000);
    unsigned roff[NLD];
#pragma unroll
    for(int q = 0; q < NLD; q++) {
        const int L = q * 64 + lane;
        const int p = L / 9, k = L - p * 9;
        roff[q] = k < 8 ? (unsigned)((p * g.lda + k * 8) * 2) : OOB;
    }
    char *const mybuf = smem + wave * 2 * C64_BUF;
    auto request = [&](int strip, int b) {
        // (a strip beyond the last: every offset out of range - the loads are issued all the same, so that the count of
        // outstanding memory operations does not depend on it)
        const unsigned base = strip < nstrips ? (unsigned)strip * 64u * (unsigned)g.lda * 2u : OOB;
#pragma unroll
        for(int q = 0; q < NLD; q++) {
            const unsigned r = roff[q];
            const unsigned off = (r == OOB || base == OOB) ? OOB : r + base;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(mybuf + b * C64_BUF + q * 1024), 16, off, 0, 0, 0);
        }
    };
    // this lane's two pixels (row blocks i of the strip) as byte offsets into the copy
    unsigned abase[2];
#pragma unroll
    for(int i = 0; i < 2; i++)
        abase[i] = (unsigned)(uintptr_t)(lds_ptr_t)mybuf + (i * 32 + (lane & 31)) * SLOT + hi * 16;
    // the stores' side: store instruction it writes chunk lane%8 of pixel 8*it + lane/8 of the strip
    unsigned sconst[8];
#pragma unroll
    for(int it = 0; it < 8; it++)
        sconst[it] = (unsigned)(((it * 8 + (lane >> 3)) * g.ldo + half * 128 + (lane & 7) * 8) * 2);
    const int step = gridDim.x * 4;
    int strip = blockIdx.x * 4 + slot;
    float st[2][16];
#pragma unroll
    for(int cb = 0; cb < 2; cb++)
#pragma unroll
        for(int e = 0; e < 16; e++)
            st[cb][e] = 0.0f;
    request(strip, 0);
    int b = 0, behind = 0;
    for(; strip < nstrips; strip += step, b ^= 1) {
        // the next strip's copy goes out behind the previous strip's stores; then this strip's must have landed
        request(strip + step, b ^ 1);
        static_assert(NST + NLD == 25 && NLD == 9, "the waits below");
        if(behind)
            asm volatile("s_waitcnt vmcnt(25)" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
        behind = NST;
        typedef unsigned u4 __attribute__((ext_vector_type(4)));
        u4 fa[4][2];
#pragma unroll
        for(int kk = 0; kk < 4; kk++)
#pragma unroll
            for(int i = 0; i < 2; i++)
                asm volatile("ds_read_b128 %0, %1" : "=v"(fa[kk][i]) : "v"(abase[i] + b * C64_BUF + kk * 32) : "memory");
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[1][0]), "+v"(fa[1][1]), "+v"(fa[2][0]), "+v"(fa[2][1]),
                       "+v"(fa[3][0]), "+v"(fa[3][1])
                     :
                     : "memory");
        bool okr[2];
        int64_t pix[2];
#pragma unroll
        for(int i = 0; i < 2; i++) {
            const int64_t p = (int64_t)strip * 64 + i * 32 + (lane & 31);
            okr[i] = p < g.M;
            pix[i] = okr[i] ? p : 0;
        }
        const unsigned strip_off = (unsigned)strip * 64u * (unsigned)g.ldo * 2u; // (the output's bytes fit 31 bits: the host's condition)
#pragma unroll
        for(int cb = 0; cb < 2; cb++) {
            float16_t acc[2][2];
#pragma unroll
            for(int i = 0; i < 2; i++)
#pragma unroll
                for(int j = 0; j < 2; j++)
#pragma unroll
                    for(int v = 0; v < 16; v++)
                        acc[i][j][v] = 0.0f;
#pragma unroll
            for(int kk = 0; kk < 4; kk++)
#pragma unroll
                for(int i = 0; i < 2; i++)
#pragma unroll
                    for(int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[cb][kk][j], __builtin_bit_cast(half8_t, fa[kk][i]),
                                                                           acc[i][j], 0, 0, 0);
            unsigned soff[8];
#pragma unroll
            for(int it = 0; it < 8; it++)
                soff[it] = (int64_t)strip * 64 + it * 8 + (lane >> 3) < g.M ? sconst[it] + strip_off + cb * 128 : OOB;
            // (staged in this strip's own copy: its operands are in registers)
            c64_epilogue<MODE>(g, acc, bnp + (half * 2 + cb) * 128, mybuf + b * C64_BUF, lane, half * 128 + cb * 64, okr, pix, soff,
                               st[cb]);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // (copies into this block's LDS may still be in flight)
    if constexpr(MODE == 2) {
        // Lane (r8, chunk) of wavefront (slot, half) holds, per channel block cb, sums over its pixels for the channels
        // 128*half + 64*cb + 8*chunk ..+7: all of them to LDS, then one thread per channel adds its 32 partial sums
        // (4 wavefronts x 8 lanes) in a fixed order: one row of partial sums per block.
        float *red = (float *)smem; // [wave][cb][lane][16]
        __syncthreads();
#pragma unroll
        for(int cb = 0; cb < 2; cb++)
#pragma unroll
            for(int e = 0; e < 16; e += 4) {
                const float4_t v4 = {st[cb][e], st[cb][e + 1], st[cb][e + 2], st[cb][e + 3]};
                *(float4_t *)(red + ((wave * 2 + cb) * 64 + lane) * 16 + e) = v4;
            }
        __syncthreads();
        if(tid < 256) {
            const int ch = tid & 63, hf = tid >> 7, cb = (tid >> 6) & 1;
            float s_ = 0.0f, q_ = 0.0f;
            for(int sl = 0; sl < 4; sl++)
                for(int r8 = 0; r8 < 8; r8++) {
                    const float *src = red + (((sl * 2 + hf) * 2 + cb) * 64 + r8 * 8 + (ch >> 3)) * 16 + (ch & 7);
                    s_ += src[0];
                    q_ += src[8];
                }
            typedef float float2_t __attribute__((ext_vector_type(2)));
            const float2_t t = {s_, q_};
            *(float2_t *)(stats + ((int64_t)blockIdx.x * g.Ngemm + tid) * 2) = t;
        }
    }
}

// The launch of conv1x1_c64_n256, or false when the shape is not its (SAGA_HIP_C64_WIDE=0 switches it off, =2 takes
// it for small tensors too, where a CU gets less than eight strips per wavefront pair).
static bool launch_c64_wide(GatherArgs &g, const CLInfo &lout, hipStream_t st, size_t stats_floats, int *rc)
{
    static const int mode = getenv("SAGA_HIP_C64_WIDE") ? atoi(getenv("SAGA_HIP_C64_WIDE")) : 1; // 2: also where it does not pay
    const bool on = mode != 0;
    const int64_t out_bytes = ((lout.rows - 1) * lout.pitch + g.Ngemm) * 2;
    if(!on || g.R != 1 || g.S != 1 || g.stride != 1 || g.pad != 0 || g.Cred != 64 || g.Ngemm != 256 || g.beta != 0.0f ||
       (g.lda & 7) || (g.ldo & 7) || !aligned16(g.a) || !aligned16(g.b) || !aligned16(g.out) || !g.a_bytes || !g.b_bytes ||
       out_bytes >= 0x7fffff00 || (int64_t)g.M * g.lda * 2 >= 0x7fffff00 || g.M != lout.rows)
        return false;
    // (with a residual the gather kernel is faster, 196 - 211 us against 222 - 245 us on the same tensors: here the
    // residual's loads, issued behind the next strip's copy, are waited for in issue order and nothing overlaps;
    // =2 still takes it, so that the path stays tested)
    if(g.bn_s && (g.bn_flags & SAGA_BN_ADD) && (mode != 2 || (g.ldz & 7) || !aligned16(g.z)))
        return false;
    const int nstrips = (g.M + 63) / 64;
    const int blocks = std::min((nstrips + 3) / 4, num_cus());
    if((nstrips < 8 * num_cus() && mode != 2) || (g.stats && (size_t)blocks * g.Ngemm * 2 > stats_floats))
        return false;
    static bool once = false;
    if(!once) {
        for(const void *k : {(const void *)conv1x1_c64_n256<0>, (const void *)conv1x1_c64_n256<1>, (const void *)conv1x1_c64_n256<2>}) {
            const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, C64_LDS);
            if(e != hipSuccess) {
                *rc = (int)e;
                return true;
            }
        }
        once = true;
    }
    g.out_bytes = (unsigned)out_bytes;
    g.stats_rows = blocks;
    if(g.bn_s)
        conv1x1_c64_n256<1><<<blocks, 512, C64_LDS, st>>>(g, nstrips);
    else if(g.stats)
        conv1x1_c64_n256<2><<<blocks, 512, C64_LDS, st>>>(g, nstrips);
    else
        conv1x1_c64_n256<0><<<blocks, 512, C64_LDS, st>>>(g, nstrips);
    *rc = (int)hipGetLastError();
    return true;
}

static int dma_stages()
{
    static int v = -1;
    if(v < 0) {
        const char *e = getenv("SAGA_HIP_CONV_STAGES");
        v = e ? atoi(e) : 3; // 0 selects the register-staged kernel
    }
    return v;
}

static int tile_override()
{
    static int v = -2;
    if(v == -2) {
        const char *e = getenv("SAGA_HIP_CONV_TILE");
        v = e ? atoi(e) : -1;
    }
    return v;
}

template <bool BWD> static int launch_gather(GatherArgs &g, hipStream_t st)
{
    static const int no_stage = getenv("SAGA_HIP_NO_STAGED_STORES") ? 1 : 0;
    g.no_stage = no_stage;
    g.classes = 1;
    g.Mc = g.M;
    g.OHc = g.OH;
    g.OWc = g.OW;
    // the pipelined kernel keeps one validity bit per tap (of a residue class) in a 64-bit mask
    // and, backward, steps one input row / column per tap: dilation 1, stride 1 or a class split
    const int sdiv = BWD ? g.stride : 1;
    const bool fits = ((g.R + sdiv - 1) / sdiv) * ((g.S + sdiv - 1) / sdiv) <= 64 &&
                      (!BWD || (g.dil == 1 && g.stride <= 4));
    if(dma_stages() >= 2 && g.a_bytes && g.b_bytes && fits) {
        constexpr int ST = 3;
        int active = 1;
        if(BWD && g.stride > 1 && g.stride <= 4 && g.dil == 1) {
            g.classes = g.stride * g.stride;
            g.OHc = (g.OH + g.stride - 1) / g.stride;
            g.OWc = (g.OW + g.stride - 1) / g.stride;
            g.Mc = g.M / (g.OH * g.OW) * g.OHc * g.OWc;
            // classes that no tap reaches produce beta*out: nothing to do for beta == 1, one
            // coalesced fill for beta == 0 (a vectorisable output; otherwise they keep their blocks)
            const bool can_fill = (g.ldo & 7) == 0 && (g.Ngemm & 7) == 0 && ((uintptr_t)g.out & 15) == 0;
            // (linked to a batch norm's backward, every pixel's old value counts in the sums: beta == 1 keeps all classes)
            const bool drop = (g.beta == 1.0f && !g.bq_partial) || (g.beta == 0.0f && can_fill);
            active = 0;
            for(int c = 0; c < g.classes; c++) {
                const int r0 = ((c >> g.sshift) + g.pad) & (g.stride - 1), s0 = ((c & (g.stride - 1)) + g.pad) & (g.stride - 1);
                if(!drop || (r0 < g.R && s0 < g.S))
                    g.cls_ids[active++] = (unsigned char)c;
            }
            if(active < g.classes && g.beta == 0.0f)
                zero_rows<<<grid_for((int64_t)g.M * (g.Ngemm / 8), 256, 256 * 16), 256, 0, st>>>(g.out, g.M, g.Ngemm, g.ldo);
            if(active == 0)
                return 0;
        }
        // tile: 256x128 on eight wavefronts (64x64 each) unless there are too few output
        // channels to fill it; measured faster than 128x128 and than 256x256 on four or eight
        // wavefronts on nearly every ResNet-50 layer, and faster than the same tiles with
        // 64-wide reduction slices (which leave room for one block per CU only)
        int tile = tile_override();
        if(tile < 0) {
            // at most 64 output channels: 256x64 on four wavefronts, which then hold five load
            // instructions per eight MFMAs each - four more wavefronts take the loads over (5-8 % faster)
            tile = g.Ngemm <= 64 ? 13 : 5;
            // at most one block per CU: nothing else on the CU hides the time a wavefront spends
            // issuing its loads, so four extra wavefronts per block do the issuing (measured
            // 5-15 % faster on the 7x7-pixel layers of ResNet-50, slower once CUs hold two blocks)
            if(tile == 5 && (int64_t)((g.Mc + 255) / 256) * ((g.Ngemm + 127) / 128) * active <= 256)
                tile = 12;
        }
        // linked to a batch norm's backward: only the 256-row tiles carry the link
        if(g.bq_partial && tile != 5 && tile != 12 && tile != 13)
            tile = g.Ngemm <= 64 ? 13 : 5;
#define LAUNCH(BM, BN, WGM, WGN, BKT, PROD)                                                            \
    do {                                                                                               \
        if constexpr(BWD && BM == 256 && (PROD > 0 || BN == 128)) {                                     \
            if(g.bq_partial) {                                                                         \
                LAUNCH_(BM, BN, WGM, WGN, BKT, PROD, true);                                            \
                break;                                                                                 \
            }                                                                                          \
        }                                                                                              \
        LAUNCH_(BM, BN, WGM, WGN, BKT, PROD, false);                                                   \
    } while(0)
#define LAUNCH_(BM, BN, WGM, WGN, BKT, PROD, BQ)                                                       \
    do {                                                                                               \
        auto kern = conv_gather_gemm_dma<BM, BN, WGM, WGN, ST, BKT, BWD, PROD, BQ>;                     \
        constexpr int lds = ST * (BM + BN) * BKT * 2 + (BQ ? 3 * BN * 4 : 0);                          \
        static bool once = false;                                                                      \
        if(lds > 64 * 1024 && !once) {                                                                 \
            const hipError_t e__ = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds); \
            if(e__ != hipSuccess)                                                                      \
                return (int)e__;                                                                       \
            once = true;                                                                               \
        }                                                                                              \
        g.nblk_n = (g.Ngemm + BN - 1) / BN;                                                            \
        g.blocks_per_class = ((g.Mc + BM - 1) / BM) * g.nblk_n;                                        \
        g.nblocks = g.blocks_per_class * active;                                                       \
        g.nactive = active;                                                                            \
        g.stats_rows = ((g.Mc + BM - 1) / BM) * active;                                                \
        kern<<<g.nblocks, 64 * (WGM * WGN + PROD), lds, st>>>(g);                                      \
    } while(0)
        switch(tile) {
        case 2: LAUNCH(128, 128, 2, 2, 32, 0); break;
        case 5: LAUNCH(256, 128, 4, 2, 32, 0); break;
        case 12: LAUNCH(256, 128, 4, 2, 32, 4); break;
        case 13: LAUNCH(256, 64, 4, 1, 32, 4); break;
        default: LAUNCH(256, 64, 4, 1, 32, 0); break;
        }
#undef LAUNCH
#undef LAUNCH_
        SAGA_CHECK_LAUNCH();
        return 0;
    }
    if(g.stats || (!BWD && g.bn_s) || g.bq_partial)
        return SAGA_HIP_EUNSUPPORTED;
    // tile choice by output-channel count; M tiles are 128 or 256 rows
    if(g.Ngemm > 64) {
        constexpr int BM = 128, BN = 128;
        g.nblk_n = (g.Ngemm + BN - 1) / BN;
        g.nblocks = ((g.M + BM - 1) / BM) * g.nblk_n;
        conv_gather_gemm<BM, BN, 2, 2, BWD><<<g.nblocks, 256, 0, st>>>(g);
    } else {
        constexpr int BM = 256, BN = 64;
        g.nblk_n = (g.Ngemm + BN - 1) / BN;
        g.nblocks = ((g.M + BM - 1) / BM) * g.nblk_n;
        conv_gather_gemm<BM, BN, 4, 1, BWD><<<g.nblocks, 256, 0, st>>>(g);
    }
    SAGA_CHECK_LAUNCH();
    return 0;
}

static int round8(int v) { return (v + 7) & ~7; }

// *pad is set when the gathered tensor cannot be loaded in 16-byte channel vectors as it is
// (channel count, pitch or base address) and has to go through pad_channels first
static bool common_ok(const SagaTensorView *act_in, const SagaTensorView *w, const SagaTensorView *act_out,
                      const ConvGeom &g, CLInfo *li, CLInfo *lo, bool *pad = nullptr)
{
    if(act_in->dtype != SAGA_HALF || g.group != 1)
        return false;
    if(!as_channels_last(act_in, li) || !as_channels_last(act_out, lo) || !krsc_dense(w))
        return false;
    const bool odd = li->C % 8 || li->pitch % 8 || !aligned16(act_in->ptr) || !aligned16(w->ptr);
    if(odd && !pad)
        return false;
    if(pad)
        *pad = odd;
    // 32-bit element offsets inside the kernels
    const int64_t in_pitch = odd ? round8(li->C) : li->pitch;
    if(li->rows * in_pitch >= (int64_t)1 << 31 || lo->rows * lo->pitch >= (int64_t)1 << 31)
        return false;
    if((int64_t)g.K * g.R * g.S * g.C >= (int64_t)1 << 31)
        return false;
    return true;
}

// fills the batch-norm fold of a forward launch; false if the residual cannot be read in place
static bool set_bn(GatherArgs &a, const ConvBnFold *bn, const SagaTensorView *y, const CLInfo &ly)
{
    a.bn_s = nullptr;
    a.z = nullptr;
    a.ldz = 0;
    a.bn_flags = 0;
    a.bn_eps = 0;
    if(!bn)
        return true;
    a.bn_s = bn->s; a.bn_b = bn->b; a.bn_m = bn->m; a.bn_v = bn->v;
    a.bn_eps = bn->eps;
    a.bn_flags = bn->flags;
    if(bn->flags & SAGA_BN_ADD) {
        CLInfo lz;
        if(!bn->z || bn->z->dtype != SAGA_HALF || !same_dims(bn->z, y) || !as_channels_last(bn->z, &lz) || lz.rows != ly.rows)
            return false;
        // where the epilogue stores 16-byte vectors it also reads the residual in 16-byte vectors
        const bool vec = ly.pitch % 8 == 0 && y->dims[1] % 8 == 0 && aligned16(y->ptr);
        if(vec && (lz.pitch % 8 || !aligned16(bn->z->ptr)))
            return false;
        a.z = (const half_t *)bn->z->ptr;
        a.ldz = (int)lz.pitch;
    }
    return true;
}

} // namespace

// floats a linked backward-data launch may write: per residue class of the stride, one row per 128 pixels
size_t conv_mfma_bnbwd_floats(const ConvGeom &g)
{
    const int64_t Mc = (int64_t)g.N * ((g.H + g.stride - 1) / g.stride) * ((g.W + g.stride - 1) / g.stride);
    return (size_t)((Mc + 127) / 128) * g.stride * g.stride * g.C * 2;
}

// floats a forward launch may write into its statistics buffer: the smallest M tile is 128 rows
size_t conv_mfma_stats_floats(const ConvGeom &g)
{
    const int64_t M = (int64_t)g.N * g.P * g.Q;
    return (size_t)((M + 127) / 128) * g.K * 2;
}

size_t conv_mfma_workspace(int kind, const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                           const ConvGeom &g)
{
    if(x->dtype != SAGA_HALF)
        return 0;
    // room for channel-padded copies of x and w (taken whenever C is not a multiple of 8; a
    // misaligned pitch or base needs it too, so it is always reserved - it is small next to x)
    const size_t Cp = round8(g.C);
    const size_t xpad = ((size_t)g.N * g.H * g.W * Cp * sizeof(half_t) + 255) & ~(size_t)255;
    const size_t wpad = ((size_t)g.K * g.R * g.S * Cp * sizeof(half_t) + 255) & ~(size_t)255;
    ThinGeom tg;
    const bool thin = thin_ok(g, &tg);
    if(kind == SAGA_CONV_FWD)
        return std::max(xpad + wpad, thin ? tg.x4_bytes + tg.wv_bytes : 0) + 256;
    if(kind == SAGA_CONV_BWD_DATA)
        return (size_t)g.K * g.C * g.R * g.S * sizeof(half_t) + 256;
    if(kind == SAGA_CONV_BWD_FILTER) {
        ConvGeom gp = g;
        gp.C = (int)Cp;
        // the launcher falls back to the small tiles for tensors beyond the buffer-load range
        const FilterPlan p = plan_filter(gp), ps = plan_filter(gp, false);
        size_t need = xpad + (size_t)std::max(p.splits, ps.splits) * g.K * g.R * g.S * Cp * sizeof(float);
        if(thin) {
            ConvGeom gv = g;
            gv.C = 32;
            gv.S = 1;
            const FilterPlan pv = plan_filter(gv, true, true);
            need = std::max(need, tg.x4_bytes + (size_t)pv.splits * g.K * g.R * 32 * sizeof(float));
        }
        return need + 256;
    }
    return 0;
}

int conv_mfma_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y, const ConvGeom &g,
                  float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st, float *stats, size_t stats_floats,
                  int *stats_rows, const ConvBnFold *bn)
{
    if(bn && (stats || beta != 0.0f))
        return SAGA_HIP_EINVAL;
    if(stats && (beta != 0.0f || stats_floats < conv_mfma_stats_floats(g)))
        return SAGA_HIP_EINVAL;
    CLInfo lx, ly;
    bool pad = false;
    if(!common_ok(x, w, y, g, &lx, &ly, &pad))
        return SAGA_HIP_EUNSUPPORTED;
    ThinGeom tg;
    if(dma_stages() >= 2 && thin_ok(g, &tg) && ly.rows * ly.pitch < ((int64_t)1 << 31)) {
        if(!ws || ws_bytes < tg.x4_bytes + tg.wv_bytes || !aligned16(ws))
            return SAGA_HIP_EWORKSPACE;
        half_t *x4 = (half_t *)ws, *wv = (half_t *)((char *)ws + tg.x4_bytes);
        const int64_t px = (int64_t)g.N * tg.Hp * tg.Wp, wn = (int64_t)g.K * g.R * 32;
        launch_pad_thin((const half_t *)x->ptr, lx.pitch, g, x4, tg, px, st);
        repack_thin_filter<<<grid_for(wn, 256, 256 * 16), 256, 0, st>>>((const half_t *)w->ptr, wv, g.C, g.S, wn);
        GatherArgs a;
        a.a = x4;
        a.b = wv;
        a.out = (half_t *)y->ptr;
        a.M = (int)ly.rows;
        a.Ngemm = g.K;
        a.Cred = 32;
        a.IH = tg.Hp; a.IW = tg.Wp; a.OH = g.P; a.OW = g.Q;
        a.R = g.R; a.S = 1;
        a.pad = 0; a.stride = g.stride; a.dil = 1; a.sshift = 0;
        a.lda = 4;
        a.ldo = (int)ly.pitch;
        a.alpha = alpha; a.beta = beta;
        a.a_bytes = (unsigned)(px * 8);
        a.b_bytes = (unsigned)(wn * 2);
        a.stats = stats;
        a.bq_partial = nullptr;
        if(!set_bn(a, bn, y, ly))
            return SAGA_HIP_EUNSUPPORTED;
        // whole rows in LDS (conv_thin_rows): 7-row filters into at most 64 channels, output rows of at most 256 pixels
        static const bool rows_off = getenv("SAGA_HIP_THIN_ROWS") && atoi(getenv("SAGA_HIP_THIN_ROWS")) == 0;
        if(!rows_off && g.R == 7 && g.K <= 64 && g.Q <= 256) {
            ThinRowsArgs t;
            t.TR = 256 / g.Q;
            if(t.TR > g.P)
                t.TR = g.P;
            t.tpi = (g.P + t.TR - 1) / t.TR;
            t.ntiles = g.N * t.tpi;
            t.npix = t.TR * g.Q;
            t.Hp = tg.Hp;
            t.row_bytes = tg.Wp * 8;
            t.chunks_row = t.row_bytes / 16;
            t.chunks_tile = t.chunks_row * ((t.TR - 1) * g.stride + g.R);
            t.buf_bytes = (t.chunks_tile * 16 + 1023) & ~1023;
            const int epi_at = std::max(THIN_ROWS_DEPTH * t.buf_bytes, 32768); // gather_epilogue's scratch sits 32 KB behind its base
            t.epi_off = epi_at - 32768;
            const int lds = epi_at + 4096;
            const bool vec_ok = (ly.pitch & 7) == 0 && (g.K & 7) == 0 && aligned16(y->ptr) &&
                                ((ly.rows - 1) * ly.pitch + g.K) * 2 < 0x7fffff00ll;
            const bool fits = vec_ok && t.chunks_tile <= 8 * 256 && lds <= 76 * 1024 && t.row_bytes % 16 == 0 &&
                              (!stats || (size_t)std::min(t.ntiles, 2 * num_cus()) * g.K * 2 <= stats_floats) &&
                              // the last window of a row ends inside the row's copy
                              ((g.Q - 1) * g.stride + 8) * 8 <= t.row_bytes;
            if(fits) {
                static bool once = false;
                if(!once) {
                    for(const void *k : {(const void *)conv_thin_rows<7, 0>, (const void *)conv_thin_rows<7, 1>,
                                         (const void *)conv_thin_rows<7, 2>}) {
                        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 76 * 1024);
                        if(e != hipSuccess)
                            return (int)e;
                    }
                    once = true;
                }
                a.classes = 1;
                a.no_stage = 1;
                a.out_bytes = (unsigned)(((ly.rows - 1) * ly.pitch + g.K) * 2); // rows * pitch < 2^31 on this path
                a.nblk_n = 1;
                const int blocks = std::min(t.ntiles, 2 * num_cus());
                a.stats_rows = blocks;
                if(a.bn_s)
                    conv_thin_rows<7, 1><<<blocks, 256, lds, st>>>(a, t);
                else if(a.stats)
                    conv_thin_rows<7, 2><<<blocks, 256, lds, st>>>(a, t);
                else
                    conv_thin_rows<7, 0><<<blocks, 256, lds, st>>>(a, t);
                SAGA_CHECK_LAUNCH();
                if(stats_rows)
                    *stats_rows = a.stats_rows;
                return 0;
            }
        }
        const int rc = launch_gather<false>(a, st);
        if(stats_rows)
            *stats_rows = a.stats_rows;
        return rc;
    }
    GatherArgs a;
    a.a = (const half_t *)x->ptr;
    a.b = (const half_t *)w->ptr;
    a.Cred = g.C;
    a.lda = (int)lx.pitch;
    if(pad) {
        const int Cp = round8(g.C);
        const size_t xpad = ((size_t)lx.rows * Cp * sizeof(half_t) + 255) & ~(size_t)255;
        const size_t wpad = (size_t)g.K * g.R * g.S * Cp * sizeof(half_t);
        if(!ws || ws_bytes < xpad + wpad || !aligned16(ws))
            return SAGA_HIP_EWORKSPACE;
        half_t *xp = (half_t *)ws, *wp = (half_t *)((char *)ws + xpad);
        pad_channels<<<grid_for(lx.rows * (Cp / 8), 256, 256 * 16), 256, 0, st>>>((const half_t *)x->ptr, lx.pitch, g.C,
                                                                                 xp, Cp, lx.rows);
        pad_channels<<<grid_for((int64_t)g.K * g.R * g.S * (Cp / 8), 256, 256 * 16), 256, 0, st>>>(
            (const half_t *)w->ptr, g.C, g.C, wp, Cp, (int64_t)g.K * g.R * g.S);
        a.a = xp;
        a.b = wp;
        a.Cred = Cp;
        a.lda = Cp;
    }
    a.out = (half_t *)y->ptr;
    a.M = (int)ly.rows;
    a.Ngemm = g.K;
    a.IH = g.H; a.IW = g.W; a.OH = g.P; a.OW = g.Q;
    a.R = g.R; a.S = g.S;
    a.pad = g.pad; a.stride = g.stride; a.dil = g.dil; a.sshift = 0;
    a.ldo = (int)ly.pitch;
    a.alpha = alpha; a.beta = beta;
    {
        const int64_t ab = (pad ? lx.rows * (int64_t)a.lda : (lx.rows - 1) * lx.pitch + lx.C) * 2;
        const int64_t bb = (int64_t)g.K * g.R * g.S * a.Cred * 2;
        a.a_bytes = ab < 0x7fffff00 ? (unsigned)ab : 0;
        a.b_bytes = bb < 0x7fffff00 ? (unsigned)bb : 0;
    }
    a.stats = stats;
    a.bq_partial = nullptr;
    if(!set_bn(a, bn, y, ly))
        return SAGA_HIP_EUNSUPPORTED;
    int rc = 0;
    if(!(dma_stages() >= 2 && !pad && (launch_rows64<false>(a, ly, st, stats_floats, &rc) || launch_c64_wide(a, ly, st, stats_floats, &rc))))
        rc = launch_gather<false>(a, st);
    if(stats_rows)
        *stats_rows = a.stats_rows;
    return rc;
}

int conv_mfma_transpose_blocks(int K, int C, int RS) { return RS * ((K + 63) / 64) * ((C + 63) / 64); }

int conv_mfma_transpose_batched(const SagaFilterTransposeJob *jobs, int njobs, int total_blocks, hipStream_t st)
{
    transpose_filter_batched<<<total_blocks, 256, 0, st>>>(jobs, njobs);
    SAGA_CHECK_LAUNCH();
    return 0;
}

bool conv_mfma_bwd_data_ok(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx, const ConvGeom &g)
{
    CLInfo ldy, ldx;
    return common_ok(dy, w, dx, g, &ldy, &ldx) && ilog2_exact(g.stride) >= 0;
}

// Whether a backward-data launch of this geometry can carry a batch-norm backward link: the conditions on the
// convolution's own tensors (those on the norm's input are checked at the launch).  The size query and the
// launcher share it, so that a caller is never told to allocate partials for a launch that would be refused.
bool conv_mfma_bnbwd_link_ok(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx, const ConvGeom &g)
{
    CLInfo ldy, ldx;
    if(!common_ok(dy, w, dx, g, &ldy, &ldx) || ilog2_exact(g.stride) < 0)
        return false;
    const int64_t ab = ((ldy.rows - 1) * ldy.pitch + ldy.C) * 2, bb = (int64_t)g.K * g.R * g.S * g.C * 2;
    const bool kernel_ok = dma_stages() >= 2 && ab < 0x7fffff00 && bb < 0x7fffff00 && g.dil == 1 && g.stride <= 4 &&
                           ((g.R + g.stride - 1) / g.stride) * ((g.S + g.stride - 1) / g.stride) <= 64;
    const bool vec = ldx.pitch % 8 == 0 && g.C % 8 == 0 && aligned16(dx->ptr);
    return kernel_ok && vec;
}

// wt_ready: the filter already transposed to C,R,S,K (by transpose_filter or the batched kernel below);
// otherwise it is transposed into the workspace first
int conv_mfma_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                       const ConvGeom &g, float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st,
                       const void *wt_ready, const ConvBnBwdLink *link)
{
    CLInfo ldy, ldx, lbx;
    if(!common_ok(dy, w, dx, g, &ldy, &ldx))
        return SAGA_HIP_EUNSUPPORTED;
    const int sshift = ilog2_exact(g.stride);
    if(sshift < 0)
        return SAGA_HIP_EUNSUPPORTED;
    if(link) {
        // only the pipelined kernel's vector epilogue carries the link; checked before anything is launched
        if(!conv_mfma_bnbwd_link_ok(dy, w, dx, g) || !link->x || link->x->dtype != SAGA_HALF || !same_dims(link->x, dx) ||
           !as_channels_last(link->x, &lbx) || lbx.rows != ldx.rows || lbx.pitch % 8 || !aligned16(link->x->ptr) ||
           lbx.rows * lbx.pitch >= (int64_t)1 << 31 || link->x->ptr == dx->ptr)
            return SAGA_HIP_EUNSUPPORTED;
        if(!link->mean || !link->partial || (link->relu && (!link->s || !link->b || !link->invstd)))
            return SAGA_HIP_EINVAL;
        if(link->partial_floats < conv_mfma_bnbwd_floats(g))
            return SAGA_HIP_EWORKSPACE;
    }
    const half_t *wt = (const half_t *)wt_ready;
    // nobody has transposed the filter: the row-resident 3x3 kernel reads it as it is
    bool krsc = false;
    if(!wt && !link && dma_stages() >= 2 && aligned16(w->ptr)) {
        wt = (const half_t *)w->ptr;
        krsc = true;
    }
    if(!wt) {
        const size_t need = (size_t)g.K * g.C * g.R * g.S * sizeof(half_t);
        if(!ws || ws_bytes < need || !aligned16(ws))
            return SAGA_HIP_EWORKSPACE;
        const int64_t total = (int64_t)g.K * g.C * g.R * g.S;
        transpose_filter<<<grid_for(total, 256, 256 * 16), 256, 0, st>>>((const half_t *)w->ptr, (half_t *)ws, g.K, g.C,
                                                                        g.R * g.S);
        wt = (const half_t *)ws;
    } else if(!aligned16(wt)) {
        return SAGA_HIP_EINVAL;
    }
    GatherArgs a;
    a.a = (const half_t *)dy->ptr;
    a.b = wt;
    a.out = (half_t *)dx->ptr;
    a.M = (int)ldx.rows;
    a.Ngemm = g.C;
    a.Cred = g.K;
    a.IH = g.P; a.IW = g.Q; a.OH = g.H; a.OW = g.W;
    a.R = g.R; a.S = g.S;
    a.pad = g.pad; a.stride = g.stride; a.dil = g.dil; a.sshift = sshift;
    a.lda = (int)ldy.pitch;
    a.ldo = (int)ldx.pitch;
    a.alpha = alpha; a.beta = beta;
    {
        const int64_t ab = ((ldy.rows - 1) * ldy.pitch + ldy.C) * 2;
        const int64_t bb = (int64_t)g.K * g.R * g.S * g.C * 2;
        a.a_bytes = ab < 0x7fffff00 ? (unsigned)ab : 0;
        a.b_bytes = bb < 0x7fffff00 ? (unsigned)bb : 0;
    }
    a.stats = nullptr;
    a.bn_s = nullptr;
    a.bq_partial = nullptr;
    if(link) {
        a.bq_x = (const half_t *)link->x->ptr;
        a.bq_ldx = (int)lbx.pitch;
        a.bq_mean = link->mean; a.bq_s = link->s; a.bq_invstd = link->invstd; a.bq_b = link->b;
        a.bq_relu = link->relu ? 1 : 0;
        a.bq_partial = link->partial;
    }
    int rc = 0;
    if(krsc) {
        if(launch_rows64<true>(a, ldx, st, 0, &rc, true))
            return rc;
        // (not that kernel's geometry: the transposed copy after all)
        const size_t need = (size_t)g.K * g.C * g.R * g.S * sizeof(half_t);
        if(!ws || ws_bytes < need || !aligned16(ws))
            return SAGA_HIP_EWORKSPACE;
        const int64_t total = (int64_t)g.K * g.C * g.R * g.S;
        transpose_filter<<<grid_for(total, 256, 256 * 16), 256, 0, st>>>((const half_t *)w->ptr, (half_t *)ws, g.K, g.C,
                                                                        g.R * g.S);
        a.b = (const half_t *)ws;
        a.b_krsc = 0;
    }
    if(!(dma_stages() >= 2 && !link && launch_rows64<true>(a, ldx, st, 0, &rc)))
        rc = launch_gather<true>(a, st);
    if(link && link->partial_rows)
        *link->partial_rows = a.stats_rows;
    return rc;
}

int conv_mfma_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw,
                         const ConvGeom &g, float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st)
{
    CLInfo lx, ldy;
    bool pad = false;
    if(!common_ok(x, dw, dy, g, &lx, &ldy, &pad))
        return SAGA_HIP_EUNSUPPORTED;
    if(g.K % 8 || ldy.pitch % 8 || !aligned16(dy->ptr))
        return SAGA_HIP_EUNSUPPORTED;
    const int64_t n = (int64_t)g.K * g.R * g.S * g.C;
    ThinGeom tg;
    if(dma_stages() >= 2 && thin_ok(g, &tg)) {
        ConvGeom gv = g;
        gv.C = 32;
        gv.S = 1;
        const FilterPlan p = plan_filter(gv, true, true);
        const size_t need = tg.x4_bytes + (size_t)p.splits * g.K * g.R * 32 * sizeof(float);
        const int64_t yb = ((ldy.rows - 1) * ldy.pitch + ldy.C) * 2;
        if(!ws || ws_bytes < need || !aligned16(ws))
            return SAGA_HIP_EWORKSPACE;
        if(yb >= 0x7fffff00)
            return SAGA_HIP_EUNSUPPORTED;
        half_t *x4 = (half_t *)ws;
        const int64_t px = (int64_t)g.N * tg.Hp * tg.Wp;
        launch_pad_thin((const half_t *)x->ptr, lx.pitch, g, x4, tg, px, st);
        FilterArgs a;
        a.x = x4;
        a.ldx = 4;
        a.dy = (const half_t *)dy->ptr;
        a.partial = (float *)((char *)ws + tg.x4_bytes);
        a.M = (int)ldy.rows;
        a.K = g.K; a.C = 32; a.RSC = g.R * 32;
        a.H = tg.Hp; a.W = tg.Wp; a.P = g.P; a.Q = g.Q; a.S = 1;
        a.pad = 0; a.stride = g.stride; a.dil = 1;
        a.ldy = (int)ldy.pitch;
        a.tiles_k = p.tiles_k; a.tiles_c = p.tiles_c;
        a.splits = p.splits; a.m_per_split = p.m_per_split;
        const int blocks = p.tiles_k * p.tiles_c * p.splits;
        constexpr int ST = 3, FNW = 8;
        if(p.bm == 128)
            conv_bwd_filter_dma<128, 128, ST, FNW><<<blocks, 64 * FNW, ST * BK * 512, st>>>(a, (unsigned)(px * 8), (unsigned)yb);
        else if(p.bn == 256)
            conv_bwd_filter_dma<64, 256, 2, 4><<<blocks, 256, 2 * BK * 640, st>>>(a, (unsigned)(px * 8), (unsigned)yb);
        else
            conv_bwd_filter_dma<64, 128, ST, 4><<<blocks, 256, ST * BK * 384, st>>>(a, (unsigned)(px * 8), (unsigned)yb);
        SAGA_CHECK_LAUNCH();
        thin_filter_reduce<<<(int)((n + 15) / 16), 256, 0, st>>>(a.partial, (half_t *)dw->ptr, n, g.C, g.S, p.splits,
                                                                    alpha, beta);
        SAGA_CHECK_LAUNCH();
        return 0;
    }
    const int Cp = pad ? round8(g.C) : g.C;
    ConvGeom gp = g;
    gp.C = Cp;
    const int64_t xb = ((lx.rows - 1) * (int64_t)(pad ? Cp : lx.pitch) + Cp) * 2, yb = ((ldy.rows - 1) * ldy.pitch + ldy.C) * 2;
    const bool pipelined = dma_stages() >= 2 && xb < 0x7fffff00 && yb < 0x7fffff00;
    const FilterPlan p = plan_filter(gp, pipelined);
    const size_t xpad = pad ? (((size_t)lx.rows * Cp * sizeof(half_t) + 255) & ~(size_t)255) : 0;
    const size_t need = xpad + (size_t)p.splits * g.K * g.R * g.S * Cp * sizeof(float);
    if(!ws || ws_bytes < need || !aligned16(ws))
        return SAGA_HIP_EWORKSPACE;
    // the 3x3, stride-1 layers with 64 input channels over large images: whole image rows in LDS
    static const bool rows_on = !(getenv("SAGA_HIP_FILTER_ROWS64") && atoi(getenv("SAGA_HIP_FILTER_ROWS64")) == 0);
    if(rows_on && pipelined && !pad && g.R == 3 && g.S == 3 && g.stride == 1 && g.pad == 1 && g.dil == 1 && g.C == 64 && g.K <= 64 &&
       g.P == g.H && g.Q == g.W && g.W >= 16 && g.W <= 256 && (lx.pitch & 7) == 0 && aligned16(x->ptr)) {
        FilterRowsArgs t;
        int tr = std::min(256 / g.W, g.H);
        while(tr > 1 && (tr * g.W) % 16)
            tr--;
        const int nsteps = tr * g.W / 16;
        t.TR = tr;
        t.tpi = (g.H + tr - 1) / tr;
        const int64_t ntiles = (int64_t)g.N * t.tpi;
        t.slots_row = g.W + 2;
        t.xchunks = (tr + 2) * t.slots_row * 9;
        t.x_bytes = (t.xchunks * 16 + 4095) & ~4095;
        t.y_bytes = nsteps * 16 * 128;
        const int blocks = num_cus();
        const int lds = 2 * t.x_bytes + 2 * t.y_bytes;
        static const int lds_max = [] {
            int dev = 0, v = 0;
            if(hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess)
                return 64 * 1024;
            return v;
        }();
        if((tr * g.W) % 16 == 0 && (nsteps == 14 || nsteps == 16) && ntiles >= 2 * blocks && ntiles < 0x7fffffff &&
           (t.x_bytes >> 12) >= 12 && (t.x_bytes >> 12) <= 13 && (t.y_bytes & 4095) == 0 &&
           (int64_t)g.H * g.W * lx.pitch * 2 < 0x7fff0000ll && (int64_t)g.H * g.W * ldy.pitch * 2 < 0x7fff0000ll &&
           (size_t)blocks * n * sizeof(float) <= ws_bytes && lds <= lds_max) {
            t.x = (const half_t *)x->ptr;
            t.dy = (const half_t *)dy->ptr;
            t.partial = (float *)ws;
            t.ldx = (int)lx.pitch;
            t.ldy = (int)ldy.pitch;
            t.H = g.H;
            t.W = g.W;
            t.K = g.K;
            t.ntiles = (int)ntiles;
            auto kern = nsteps == 14 ? conv_bwd_filter_rows64<14> : conv_bwd_filter_rows64<16>;
            static bool once[2] = {false, false};
            if(!once[nsteps == 16]) {
                const hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_max);
                if(e != hipSuccess)
                    return (int)e;
                once[nsteps == 16] = true;
            }
            kern<<<blocks, 256, lds, st>>>(t);
            SAGA_CHECK_LAUNCH();
            filter_reduce_v4<<<(unsigned)((n / 4 + 15) / 16), 256, 0, st>>>(t.partial, (half_t *)dw->ptr, n, blocks, alpha, beta);
            SAGA_CHECK_LAUNCH();
            return 0;
        }
    }
    FilterArgs a;
    a.x = (const half_t *)x->ptr;
    a.ldx = (int)lx.pitch;
    if(pad) {
        half_t *xp = (half_t *)ws;
        pad_channels<<<grid_for(lx.rows * (Cp / 8), 256, 256 * 16), 256, 0, st>>>((const half_t *)x->ptr, lx.pitch, g.C,
                                                                                 xp, Cp, lx.rows);
        a.x = xp;
        a.ldx = Cp;
    }
    a.dy = (const half_t *)dy->ptr;
    a.partial = (float *)((char *)ws + xpad);
    a.M = (int)ldy.rows;
    a.K = g.K; a.C = Cp; a.RSC = g.R * g.S * Cp;
    a.H = g.H; a.W = g.W; a.P = g.P; a.Q = g.Q; a.S = g.S;
    a.pad = g.pad; a.stride = g.stride; a.dil = g.dil;
    a.ldy = (int)ldy.pitch;
    a.tiles_k = p.tiles_k; a.tiles_c = p.tiles_c;
    a.splits = p.splits; a.m_per_split = p.m_per_split;
    const int blocks = p.tiles_k * p.tiles_c * p.splits;
    if(pipelined) {
        constexpr int ST = 3, FNW = 8;
        if(p.bm == 256) {
            auto kern = conv_bwd_filter_dma<256, 256, ST, 16>;
            constexpr int lds = ST * BK * 1024;
            static bool once = false;
            if(!once) {
                const hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
                if(e != hipSuccess)
                    return (int)e;
                once = true;
            }
            kern<<<blocks, 1024, lds, st>>>(a, (unsigned)xb, (unsigned)yb);
        } else if(p.bm == 128 && p.bn == 256) {
            auto kern = conv_bwd_filter_dma<128, 256, ST, FNW>;
            constexpr int lds = ST * BK * 768;
            static bool once = false;
            if(!once) {
                const hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
                if(e != hipSuccess)
                    return (int)e;
                once = true;
            }
            kern<<<blocks, 64 * FNW, lds, st>>>(a, (unsigned)xb, (unsigned)yb);
        } else if(p.bm == 64 && p.bn == 256) {
            conv_bwd_filter_dma<64, 256, 2, 4><<<blocks, 256, 2 * BK * 640, st>>>(a, (unsigned)xb, (unsigned)yb);
        } else if(p.bm == 128)
            conv_bwd_filter_dma<128, 128, ST, FNW><<<blocks, 64 * FNW, ST * BK * 512, st>>>(a, (unsigned)xb, (unsigned)yb);
        else
            conv_bwd_filter_dma<64, 128, ST, 4><<<blocks, 256, ST * BK * 384, st>>>(a, (unsigned)xb, (unsigned)yb);
    } else if(p.bm == 128) {
        conv_bwd_filter_mfma<128, 128><<<blocks, 256, 0, st>>>(a);
    } else {
        conv_bwd_filter_mfma<64, 128><<<blocks, 256, 0, st>>>(a);
    }
    SAGA_CHECK_LAUNCH();
    if(Cp == g.C && n % 4 == 0 && aligned16(a.partial) && ((uintptr_t)dw->ptr & 7) == 0)
        filter_reduce_v4<<<(unsigned)((n / 4 + 15) / 16), 256, 0, st>>>(a.partial, (half_t *)dw->ptr, n, p.splits, alpha,
                                                                       beta);
    else
        filter_reduce<<<grid_for(n, 256, 256 * 8), 256, 0, st>>>(a.partial, (half_t *)dw->ptr, n, g.C, Cp, p.splits,
                                                                alpha, beta);
    SAGA_CHECK_LAUNCH();
    return 0;
}
