// Reindex kernels: permute, slice, broadcast (one gather formulation) and concat.
//
// ratchet's kernels for these ops move one scalar per thread and pay three integer divisions per element
// (ops/reindex/mod.rs:48-124, gpu/wgsl/kernel_builder.rs:198-221 in crates/ratchet-core/src).  Here the host folds the
// op into "dst[i0,i1,i2,i3] = src[base + i0*S0 + i1*S1 + i2*S2 + i3*S3]" with strides resolved at launch, picks the
// widest vector (16/8/4/2 bytes) that keeps every source and destination access aligned, and each thread moves whole
// vectors along the destination's last dimension with multiply-shift index math.  A permutation that moves the
// source's contiguous dimension is transposed in V x V blocks in registers when rows are whole 16-byte vectors, and
// through an LDS tile otherwise, so both the read and the write side stay coalesced.
#include "rt_arith.h"
#include "rt_internal.h"

namespace {

constexpr int BLOCK = 256;
constexpr int UNROLL = 2;                 // vectors per thread where more than one pays (concat, splat, repeated source dims): two before the first store (four were slower on the 21 MB concat: 9.4 -> 7.7 us)

struct GatherArgs {
    FastDiv d3, d2, d1;      // destination extents, d3 in vectors
    uint64_t base;           // source offset of dst[0,0,0,0], in vectors (elements for the splat kernel)
    uint64_t s[4];           // source strides per destination dim, in vectors (elements for the splat kernel)
    uint32_t nvec;           // destination vectors
    // Block order for a swap of two outer dims with short rows (K/V heads: [S, H, 80] -> [H, S, 80] in f16, 160-byte
    // rows): the source rows of neighbouring heads share 128-byte lines, and in destination order those heads are
    // 40 blocks apart, on another XCD, so every shared line is fetched twice (FETCH_SIZE 1.6x the tensor).  Hardware
    // block b runs on XCD b % 8; with rm_h > 0 an XCD's consecutive blocks take the same rows of rm_h consecutive
    // heads (rm_j blocks per head, a multiple of 8), and the second head finds the line in that XCD's L2.
    FastDiv rm_h;
    uint32_t rm_j;
};

__device__ __forceinline__ uint32_t gather_block(const GatherArgs& p) {
    uint32_t blk = blockIdx.x;
    if (p.rm_j) {
        const uint32_t xcd = blk & 7u;
        uint32_t jj, h;
        fd_divmod(blk >> 3, p.rm_h, jj, h);
        blk = h * p.rm_j + jj * 8u + xcd;
    }
    return blk;
}

// one VecT per thread-iteration; source contiguous along the destination's last dim (s[3] == 1)
// U vectors per thread: one for a large tensor whose destination vectors each have a source vector of their own
// (permute, slice: a wave that stores once and ends leaves HBM a more even stream; [32,4096,32,128] f16 heads swap
// 389 -> 347 us, 134 MB 37 -> 35 us, [1,4096,32,128] f16, 34 MB, 15.5 -> 14.2 us, [1,2048,32,128] f16, 17 MB, 8.4 -> 7.8 us),
// UNROLL for small ones (10 MB: 6.5 us against 6.9) and when a source dim is
// repeated (broadcast_to [1,1,4096,4096] -> [1,32,..]: 224 us against 250)
constexpr uint64_t GATHER_ONE_FROM_BYTES = 16ull << 20;
template <typename VecT, int U>
__global__ void __launch_bounds__(BLOCK) gather_vec_kernel(const VecT* __restrict__ x, VecT* __restrict__ y, GatherArgs p) {
    const uint32_t base = gather_block(p) * (BLOCK * U) + threadIdx.x;
    VecT r[U];
#pragma unroll
    for (int k = 0; k < U; k++) {
        const uint32_t v = base + k * BLOCK;
        if (v < p.nvec) {
            uint32_t row, i3, t, i2, i1, i0;
            fd_divmod(v, p.d3, row, i3);
            fd_divmod(row, p.d2, t, i2);
            fd_divmod(t, p.d1, i0, i1);
            r[k] = x[p.base + i0 * p.s[0] + i1 * p.s[1] + i2 * p.s[2] + i3 * p.s[3]];
        }
    }
#pragma unroll
    for (int k = 0; k < U; k++) {
        const uint32_t v = base + k * BLOCK;
        if (v < p.nvec) st_stream(y + v, r[k]);
    }
}

// source broadcast along the destination's last dim (s[3] == 0): load one element, replicate it through a VecT.
// Strides and base are in elements here; PER = elements per VecT.
template <typename ElemT, typename VecT>
__global__ void __launch_bounds__(BLOCK) gather_splat_kernel(const ElemT* __restrict__ x, VecT* __restrict__ y, GatherArgs p) {
    constexpr int PER = sizeof(VecT) / sizeof(ElemT);
    const uint32_t base = blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const uint32_t v = base + k * BLOCK;
        if (v < p.nvec) {
            uint32_t row, i3, t, i2, i1, i0;
            fd_divmod(v, p.d3, row, i3);
            fd_divmod(row, p.d2, t, i2);
            fd_divmod(t, p.d1, i0, i1);
            const ElemT e = x[p.base + i0 * p.s[0] + i1 * p.s[1] + i2 * p.s[2]];
            union { VecT v; ElemT e[PER]; } u;
#pragma unroll
            for (int q = 0; q < PER; q++) u.e[q] = e;
            st_stream(y + v, u.v);
        }
    }
}

// Tiled transpose for permutations that move the source's contiguous dimension.
// Destination dims: `q` is the one fed by the source's last dim; 3 is fed by source dim with stride sj.
// A block owns a TQ x TJ patch over (dst dim q, dst dim 3), 4096 elements; the two remaining dims are flattened into the
// block index.  The patch is square unless one side is short (channel-last images, [H,W,3] <-> [3,H,W]), where a
// 64 x 64 patch would be mostly empty.
constexpr int TILE_ELEMS = 4096;
struct TransposeArgs {
    uint32_t nq, n3;         // extents of dst dim q and dst dim 3
    uint64_t s3;             // source stride (elements) of the dim that becomes dst dim 3
    // dst dim 3 may stand for two dst dims merged (the destination is contiguous across them, the source is not): index j
    // of it lies at (j / inner) * s2 + (j % inner) * s3 in the source.  Plain: inner = 1, s2 = s3.  (tr_row; the kernels
    // that take whole-vector rows use s3 alone and are not launched on a merged dim.)
    FastDiv inner;
    uint64_t s2;
    uint64_t dq;             // destination stride (elements) of dim q
    FastDiv gx, gy;          // tile counts along dst dim q and dst dim 3 (blockIdx.x = (z * gy + ty) * gx + tx)
    FastDiv ob;              // extent of the second "other" dim (other dims = (oa, ob), ob fastest)
    uint64_t sa, sb;         // source strides of the other dims
    uint64_t da, db;         // destination strides of the other dims
};

__device__ __forceinline__ uint64_t tr_row(const TransposeArgs& p, uint32_t j) {
    uint32_t hi, lo;
    fd_divmod(j, p.inner, hi, lo);
    return (uint64_t)hi * p.s2 + (uint64_t)lo * p.s3;
}

template <typename ElemT, int TQ>
__global__ void __launch_bounds__(BLOCK) transpose_kernel(const ElemT* __restrict__ x, ElemT* __restrict__ y, TransposeArgs p) {
    constexpr int TJ = TILE_ELEMS / TQ;
    // the pitch is an odd number of 4-byte words: the column reads below touch every bank once
    __shared__ ElemT tile[TJ][TQ + (sizeof(ElemT) == 4 ? 1 : 2)];
    uint32_t oa, obi, bz, byx, by, bx;
    fd_divmod(blockIdx.x, p.gx, byx, bx);
    fd_divmod(byx, p.gy, bz, by);
    fd_divmod(bz, p.ob, oa, obi);
    const uint64_t src0 = oa * p.sa + obi * p.sb;
    const uint64_t dst0 = oa * p.da + obi * p.db;
    const uint32_t q0 = bx * TQ, j0 = by * TJ;                         // origin in (dst dim q, dst dim 3)
    // read: rows = dst-dim-3 index (source stride s3), columns = source's contiguous dim (dst dim q)
#pragma unroll 4
    for (uint32_t i = threadIdx.x; i < TILE_ELEMS; i += BLOCK) {
        const uint32_t r = i / TQ, c = i % TQ;
        const uint32_t j = j0 + r, q = q0 + c;
        if (j < p.n3 && q < p.nq) tile[r][c] = x[src0 + tr_row(p, j) + q];
    }
    __syncthreads();
    // write: rows = dst dim q, columns = dst dim 3 (contiguous in the destination)
#pragma unroll 4
    for (uint32_t i = threadIdx.x; i < TILE_ELEMS; i += BLOCK) {
        const uint32_t r = i / TJ, c = i % TJ;
        const uint32_t q = q0 + r, j = j0 + c;
        if (q < p.nq && j < p.n3) y[dst0 + (uint64_t)q * p.dq + j] = tile[c][r];
    }
}

// A short contiguous dim that changes sides: [.., J, C] -> [.., C, J] (interleaved channels to planes, TO_PLANES) and
// back, C = 2 .. 16 ([B,H,W,3] <-> [B,3,H,W]).  The interleaved side of a tile of PJ positions is one contiguous run of
// PJ * C elements, moved with 16-byte accesses; the planar side is C runs of PJ elements, 16-byte accesses too; in
// between the tile lies in LDS as [position][channel] with an odd pitch (C, or C + 1 for an even C: with the pitch of
// 4 or 16 channels every lane of the strided side would meet the same bank) and is read (or written) with that stride.
// The launcher checks that every run starts on a 16-byte boundary and is a whole number of vectors (J a multiple of the
// vector length, strides of the outer dims and of the planes too); PJ * C <= CH_TILE.
constexpr int CH_TILE = 4096;
struct ChannelArgs {
    uint32_t C, J, PJ;
    uint32_t P;              // LDS pitch: C | 1
    FastDiv cdiv;            // C
    FastDiv gj;              // tiles along J (blockIdx.x = (oa * ob + obi) * gj + tile)
    FastDiv ob;              // extent of the inner of the two outer dims
    uint64_t ia, ib;         // strides of the outer dims on the interleaved side
    uint64_t pa, pb, plane;  // strides of the outer dims and of a plane on the planar side
};

template <typename ElemT, bool TO_PLANES>
__global__ void __launch_bounds__(BLOCK) channels_kernel(const ElemT* __restrict__ x, ElemT* __restrict__ y, ChannelArgs p) {
    constexpr int VE = 16 / (int)sizeof(ElemT);
    constexpr int NV = CH_TILE / VE / BLOCK;                 // vectors per thread at most: 4 (32-bit), 2 (16-bit)
    __shared__ __attribute__((aligned(16))) ElemT tile[CH_TILE + CH_TILE / 4];       // PJ <= CH_TILE / 4 whenever C is even
    uint32_t z, tl, oa, obi;
    fd_divmod(blockIdx.x, p.gj, z, tl);
    fd_divmod(z, p.ob, oa, obi);
    const uint32_t j0 = tl * p.PJ;
    const uint32_t nj = p.J - j0 < p.PJ ? p.J - j0 : p.PJ;   // a multiple of VE
    const uint32_t nflat = nj * p.C / VE, nvp = nj / VE;     // vectors of the interleaved run, of one plane's run
    const uint32_t nplanar = nvp * p.C;
    const uint64_t inter0 = oa * p.ia + obi * p.ib + (uint64_t)j0 * p.C;
    const uint64_t planar0 = oa * p.pa + obi * p.pb + j0;
    // the VE elements of vector i of the interleaved run <-> LDS: they are consecutive channels, wrapping to the next position
    auto flat_to_lds = [&](uint32_t i, const Vec16<ElemT>& v) {
        uint32_t j, c;
        fd_divmod(i * VE, p.cdiv, j, c);
        uint32_t at = j * p.P + c;
#pragma unroll
        for (int e = 0; e < VE; e++) {
            tile[at] = v.e[e];
            const bool wrap = ++c == p.C;
            at += wrap ? 1 + p.P - p.C : 1;
            c = wrap ? 0 : c;
        }
    };
    auto lds_to_flat = [&](uint32_t i) -> Vec16<ElemT> {
        Vec16<ElemT> v;
        uint32_t j, c;
        fd_divmod(i * VE, p.cdiv, j, c);
        uint32_t at = j * p.P + c;
#pragma unroll
        for (int e = 0; e < VE; e++) {
            v.e[e] = tile[at];
            const bool wrap = ++c == p.C;
            at += wrap ? 1 + p.P - p.C : 1;
            c = wrap ? 0 : c;
        }
        return v;
    };
    if (TO_PLANES) {
        const v4u* src = reinterpret_cast<const v4u*>(x + inter0);
        Vec16<ElemT> in[NV];
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = threadIdx.x + k * BLOCK;
            in[k].u = ld_stream(src + (i < nflat ? i : 0));
        }
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = threadIdx.x + k * BLOCK;
            if (i < nflat) flat_to_lds(i, in[k]);
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = threadIdx.x + k * BLOCK;
            if (i < nplanar) {
                const uint32_t c = i / nvp, t = i - c * nvp;
                Vec16<ElemT> out;
#pragma unroll
                for (int e = 0; e < VE; e++) out.e[e] = tile[(t * VE + e) * p.P + c];
                st_stream(reinterpret_cast<v4u*>(y + planar0 + (uint64_t)c * p.plane) + t, out.u);
            }
        }
    } else {
        Vec16<ElemT> in[NV];
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = threadIdx.x + k * BLOCK;
            const uint32_t ii = i < nplanar ? i : 0;
            const uint32_t c = ii / nvp, t = ii - c * nvp;
            in[k].u = ld_stream(reinterpret_cast<const v4u*>(x + planar0 + (uint64_t)c * p.plane) + t);
        }
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = threadIdx.x + k * BLOCK;
            if (i < nplanar) {
                const uint32_t c = i / nvp, t = i - c * nvp;
#pragma unroll
                for (int e = 0; e < VE; e++) tile[(t * VE + e) * p.P + c] = in[k].e[e];
            }
        }
        __syncthreads();
        v4u* dst = reinterpret_cast<v4u*>(y + inter0);
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = threadIdx.x + k * BLOCK;
            if (i < nflat) st_stream(dst + i, lds_to_flat(i).u);
        }
    }
}

// The same 64 x 64 patch with the widest accesses each side allows: LW elements per load along the source's contiguous
// dim, SW elements per store along the destination's (each 1, 2, 4 or 8 elements and at most 16 bytes; the launcher
// checks that every row start and extent on that side is a multiple).  K^T of [B,H,1500,D] in 16 bits, whose destination
// rows of 1500 elements are whole 8-byte units but not whole 16-byte vectors: 16-byte loads, 8-byte stores.
// TQ other than 64 (80, 96, 128): the patch covers the whole of a short source row (head dims 72 to 128, K^T of
// [B,H,S,80] and [B,H,S,96]), where patches of 64 leave a second, mostly empty one (80 = 64 + 16: two patches for the
// work of 1.25); the 64 source rows of such a patch are one contiguous run.
template <typename ElemT, int LW, int SW, int TQ = 64>
__global__ void __launch_bounds__(BLOCK) transpose_wide_kernel(const ElemT* __restrict__ x, ElemT* __restrict__ y, TransposeArgs p) {
    constexpr int TJ = 64;
    static_assert(TQ % LW == 0 && TJ % SW == 0, "whole accesses per patch row");
    constexpr int PAD = sizeof(ElemT) == 4 ? 1 : 2;
    __shared__ ElemT tile[TJ][TQ + PAD];
    uint32_t oa, obi, bz, byx, by, bx;
    fd_divmod(blockIdx.x, p.gx, byx, bx);
    fd_divmod(byx, p.gy, bz, by);
    fd_divmod(bz, p.ob, oa, obi);
    const uint64_t src0 = oa * p.sa + obi * p.sb;
    const uint64_t dst0 = oa * p.da + obi * p.db;
    const uint32_t q0 = bx * TQ, j0 = by * TJ;
    struct alignas(LW * sizeof(ElemT)) LoadT { ElemT e[LW]; };
    struct alignas(SW * sizeof(ElemT)) StoreT { ElemT e[SW]; };
    constexpr int LOADS = TJ * (TQ / LW), STORES = TQ * (TJ / SW);              // accesses per patch
    constexpr int NL = (LOADS + BLOCK - 1) / BLOCK, NS = (STORES + BLOCK - 1) / BLOCK;
    LoadT in[NL] = {};
#pragma unroll
    for (int k = 0; k < NL; k++) {
        const uint32_t i = threadIdx.x + k * BLOCK;
        const uint32_t r = i / (TQ / LW), c = (i % (TQ / LW)) * LW;
        const uint32_t j = j0 + r, q = q0 + c;
        if ((LOADS % BLOCK == 0 || i < LOADS) && j < p.n3 && q < p.nq) in[k] = *reinterpret_cast<const LoadT*>(x + src0 + tr_row(p, j) + q);
    }
#pragma unroll
    for (int k = 0; k < NL; k++) {
        const uint32_t i = threadIdx.x + k * BLOCK;
        const uint32_t r = i / (TQ / LW), c = (i % (TQ / LW)) * LW;
        if (LOADS % BLOCK == 0 || i < LOADS) {
#pragma unroll
            for (int e = 0; e < LW; e++) tile[r][c + e] = in[k].e[e];
        }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < NS; k++) {
        const uint32_t i = threadIdx.x + k * BLOCK;
        const uint32_t r = i / (TJ / SW), c = (i % (TJ / SW)) * SW;
        const uint32_t q = q0 + r, j = j0 + c;
        if ((STORES % BLOCK == 0 || i < STORES) && q < p.nq && j < p.n3) {
            StoreT out;
#pragma unroll
            for (int e = 0; e < SW; e++) out.e[e] = tile[c + e][r];
            *reinterpret_cast<StoreT*>(y + dst0 + (uint64_t)q * p.dq + j) = out;
        }
    }
}

// The same permutations when every row on both sides is a whole number of aligned 16-byte vectors (the attention
// transposes: [B,H,T,D] -> [B,H,D,T], [B,T,H,D] -> [B,H,D,T]): no LDS.  A thread loads V rows of one 16-byte vector
// (V = 8 halves or 4 words: a V x V block), transposes the block in its registers and stores V vectors.  The 64 lanes of
// a wave are laid out as QB blocks along the source's contiguous dim by JB blocks along the destination's, so a load
// instruction reads JB runs of QB * 16 bytes and a store instruction writes QB runs of JB * 16 bytes; QB covers the
// whole source row when that is short (head dims up to 96 halves), which makes the source patch one contiguous run.
struct TransposeRegArgs {
    uint32_t nqb, njb;       // blocks of V elements along dst dim q / dst dim 3
    uint32_t QB, JB;         // blocks per wave along q / along j (QB * JB <= 64)
    FastDiv qb_div;          // lane -> (jb, qb)
    uint64_t s3;             // source stride (elements) of the dim that becomes dst dim 3
    uint64_t dq;             // destination stride (elements) of dim q
    FastDiv gx, gy;          // tile counts along q (QB blocks each) and along j (4 waves x JB blocks each)
    FastDiv ob;
    uint64_t sa, sb, da, db;
};

__device__ __forceinline__ void transpose_block(const v4u (&in)[8], v4u (&out)[8], uint16_t) {
    // out[k] holds element k of each of the 8 input rows: halves (2w, 2w+1) of out[k] come from in[2w], in[2w+1]
#pragma unroll
    for (int k = 0; k < 8; k++)
#pragma unroll
        for (int w = 0; w < 4; w++)
            out[k][w] = __builtin_amdgcn_perm(in[2 * w + 1][k / 2], in[2 * w][k / 2], (k & 1) ? 0x07060302u : 0x05040100u);
}
__device__ __forceinline__ void transpose_block(const v4u (&in)[4], v4u (&out)[4], uint32_t) {
#pragma unroll
    for (int k = 0; k < 4; k++)
#pragma unroll
        for (int w = 0; w < 4; w++) out[k][w] = in[w][k];
}

template <typename ElemT>
__global__ void __launch_bounds__(BLOCK) transpose_reg_kernel(const ElemT* __restrict__ x, ElemT* __restrict__ y, TransposeRegArgs p) {
    constexpr int V = 16 / sizeof(ElemT);
    uint32_t oa, obi, bz, byx, by, bx;
    fd_divmod(blockIdx.x, p.gx, byx, bx);
    fd_divmod(byx, p.gy, bz, by);
    fd_divmod(bz, p.ob, oa, obi);
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t jb, qb;
    fd_divmod(lane, p.qb_div, jb, qb);
    qb += bx * p.QB;
    const uint32_t jblk = (by * (BLOCK / 64) + wave) * p.JB + jb;
    if (jb >= p.JB || qb >= p.nqb || jblk >= p.njb) return;
    const ElemT* src = x + oa * p.sa + obi * p.sb + (uint64_t)jblk * V * p.s3 + (uint64_t)qb * V;
    ElemT* dst = y + oa * p.da + obi * p.db + (uint64_t)qb * V * p.dq + (uint64_t)jblk * V;
    v4u in[V], out[V];
#pragma unroll
    for (int i = 0; i < V; i++) in[i] = ld_stream(reinterpret_cast<const v4u*>(src + (uint64_t)i * p.s3));
    transpose_block(in, out, ElemT());
#pragma unroll
    for (int k = 0; k < V; k++) st_stream(reinterpret_cast<v4u*>(dst + (uint64_t)k * p.dq), out[k]);
}

// The same permutations through LDS with one 16-byte load and one 16-byte store per thread: a 512-thread block moves a
// patch of 64 (dst dim 3) x 8 vectors (dst dim q) = 8 KiB, whole 128-byte lines on both sides.  A thread loads one
// vector of a source row and writes its words to the tile (pitch 33 words: the column reads below touch every bank
// once); then it gathers the V elements of one destination vector from V consecutive tile rows and stores it.  A wave's
// store covers 8 (f16) or 4 (f32) destination rows with one full run of 128 / 256 bytes each.
constexpr int TV_BLOCK = 512;
template <typename ElemT>
__global__ void __launch_bounds__(TV_BLOCK) transpose_vec_kernel(const ElemT* __restrict__ x, ElemT* __restrict__ y, TransposeArgs p) {
    constexpr int V = 16 / sizeof(ElemT);            // elements per vector
    constexpr int TJ = 64, TQW = 32;                 // patch: 64 rows of 32 words (8 vectors)
    __shared__ uint32_t tile[TJ][TQW + 1];
    uint32_t oa, obi, bz, byx, by, bx;
    fd_divmod(blockIdx.x, p.gx, byx, bx);
    fd_divmod(byx, p.gy, bz, by);
    fd_divmod(bz, p.ob, oa, obi);
    const uint64_t src0 = oa * p.sa + obi * p.sb;
    const uint64_t dst0 = oa * p.da + obi * p.db;
    const uint32_t q0 = bx * (8 * V), j0 = by * TJ;
    {
        const uint32_t r = threadIdx.x >> 3, v = threadIdx.x & 7;
        const uint32_t j = j0 + r, q = q0 + v * V;
        if (j < p.n3 && q < p.nq) {
            const v4u in = ld_stream(reinterpret_cast<const v4u*>(x + src0 + (uint64_t)j * p.s3 + q));
#pragma unroll
            for (int w = 0; w < 4; w++) tile[r][v * 4 + w] = in[w];
        }
    }
    __syncthreads();
    const uint32_t d = threadIdx.x / (TJ / V), tv = threadIdx.x % (TJ / V);      // d: 0..63 (f16) or 0..31 (f32)
    const uint32_t q = q0 + d, j = j0 + tv * V;
    if (q < p.nq && j < p.n3) {
        v4u out;
        if (sizeof(ElemT) == 4) {
#pragma unroll
            for (int k = 0; k < 4; k++) out[k] = tile[tv * 4 + k][d];
        } else {
            const uint16_t* t16 = reinterpret_cast<const uint16_t*>(&tile[0][0]);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t lo = t16[(tv * 8 + 2 * k) * (2 * (TQW + 1)) + d];
                const uint32_t hi = t16[(tv * 8 + 2 * k + 1) * (2 * (TQW + 1)) + d];
                out[k] = lo | (hi << 16);
            }
        }
        st_stream(reinterpret_cast<v4u*>(y + dst0 + (uint64_t)q * p.dq + j), out);
    }
}

// Larger patches of the same scheme for large tensors: TJ source rows (elements along dst dim 3) x TQ elements along the
// source's contiguous dim, so a block reads TJ runs of TQ * sizeof(ElemT) bytes and writes TQ runs of TJ * sizeof(ElemT)
// bytes, several vectors per thread, all loads in flight before the tile is written.
template <typename ElemT, int TJ, int TQ>
__global__ void __launch_bounds__(TV_BLOCK) transpose_big_kernel(const ElemT* __restrict__ x, ElemT* __restrict__ y, TransposeArgs p) {
    constexpr int V = 16 / sizeof(ElemT);
    constexpr int TQW = TQ * (int)sizeof(ElemT) / 4;         // words per tile row
    constexpr int QV = TQ / V;                               // vectors per source run
    constexpr int JV = TJ / V;                               // vectors per destination run
    constexpr int NLD = TJ * QV / TV_BLOCK;                  // vectors per thread
    static_assert(TJ * QV % TV_BLOCK == 0 && NLD >= 1, "whole vectors per thread");
    __shared__ uint32_t tile[TJ][TQW + 1];
    uint32_t oa, obi, bz, byx, by, bx;
    fd_divmod(blockIdx.x, p.gx, byx, bx);
    fd_divmod(byx, p.gy, bz, by);
    fd_divmod(bz, p.ob, oa, obi);
    const uint64_t src0 = oa * p.sa + obi * p.sb;
    const uint64_t dst0 = oa * p.da + obi * p.db;
    const uint32_t q0 = bx * TQ, j0 = by * TJ;
    v4u in[NLD];
#pragma unroll
    for (int k = 0; k < NLD; k++) {
        const uint32_t t = threadIdx.x + k * TV_BLOCK;
        const uint32_t r = t / QV, v = t % QV;
        const uint32_t j = j0 + r, q = q0 + v * V;
        in[k] = v4u{0u, 0u, 0u, 0u};
        if (j < p.n3 && q < p.nq) in[k] = ld_stream(reinterpret_cast<const v4u*>(x + src0 + (uint64_t)j * p.s3 + q));
    }
#pragma unroll
    for (int k = 0; k < NLD; k++) {
        const uint32_t t = threadIdx.x + k * TV_BLOCK;
        const uint32_t r = t / QV, v = t % QV;
#pragma unroll
        for (int w = 0; w < 4; w++) tile[r][v * 4 + w] = in[k][w];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < NLD; k++) {
        const uint32_t t = threadIdx.x + k * TV_BLOCK;
        const uint32_t d = t / JV, tv = t % JV;
        const uint32_t q = q0 + d, j = j0 + tv * V;
        if (q < p.nq && j < p.n3) {
            v4u out;
            if (sizeof(ElemT) == 4) {
#pragma unroll
                for (int e = 0; e < 4; e++) out[e] = tile[tv * 4 + e][d];
            } else {
                const uint16_t* t16 = reinterpret_cast<const uint16_t*>(&tile[0][0]);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t lo = t16[(tv * 8 + 2 * e) * (2 * (TQW + 1)) + d];
                    const uint32_t hi = t16[(tv * 8 + 2 * e + 1) * (2 * (TQW + 1)) + d];
                    out[e] = lo | (hi << 16);
                }
            }
            st_stream(reinterpret_cast<v4u*>(y + dst0 + (uint64_t)q * p.dq + j), out);
        }
    }
}

// concat: input k is [a_dim, bv[k]] vectors, copied into dst rows of dst_sv vectors at column dst_ov[k]
struct ConcatArgs {
    const void* src[8];
    FastDiv bv[8];
    uint32_t dst_ov[8];
    uint32_t nvec[8];
    uint32_t dst_sv;
};

template <typename VecT, int U>
__global__ void __launch_bounds__(BLOCK) concat_kernel(VecT* __restrict__ y, ConcatArgs p) {
    const int k = blockIdx.y;
    const VecT* __restrict__ x = reinterpret_cast<const VecT*>(p.src[k]);
    const uint32_t nvec = p.nvec[k];
    const uint32_t base = blockIdx.x * (BLOCK * U) + threadIdx.x;
    if (blockIdx.x * (BLOCK * U) >= nvec) return;
    VecT r[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t v = base + u * BLOCK;
        if (v < nvec) r[u] = ld_stream(x + v);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t v = base + u * BLOCK;
        if (v < nvec) {
            uint32_t row, col;
            fd_divmod(v, p.bv[k], row, col);
            st_stream(y + ((uint64_t)row * p.dst_sv + p.dst_ov[k] + col), r[u]);
        }
    }
}

// The same copy walked in destination order, for short segments (x.slice(..rot).rope().cat(x.slice(rot..)) along the last
// dim: 64- and 96-byte pieces): a destination vector finds its input by its column, so the stores of a wave are one
// contiguous run and only the loads come in pieces.  (Walking the inputs instead leaves every store instruction with
// pieces: [4M,8] + [4M,8] f16 ran at 2.1 TB/s.)
struct ConcatRowsArgs {
    const void* src[8];
    uint32_t dst_ov[8];      // first destination column (in vectors) of input k; unused slots hold 0xffffffff
    uint32_t seg_v[8];       // vectors per row of input k
    FastDiv dst_sv;          // destination vectors per row
    uint64_t nvec;           // destination vectors
};

template <typename VecT>
__global__ void __launch_bounds__(BLOCK) concat_rows_kernel(VecT* __restrict__ y, ConcatRowsArgs p) {
    const uint64_t base = (uint64_t)blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
    VecT r[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const uint64_t v = base + (uint64_t)u * BLOCK;
        if (v < p.nvec) {
            uint32_t row, col;
            fd_divmod((uint32_t)v, p.dst_sv, row, col);
            // select chain instead of an index: the argument arrays stay in scalar registers
            const void* src = p.src[0];
            uint32_t seg = p.seg_v[0], ov = p.dst_ov[0];
#pragma unroll
            for (int j = 1; j < 8; j++)
                if (col >= p.dst_ov[j]) {
                    src = p.src[j];
                    seg = p.seg_v[j];
                    ov = p.dst_ov[j];
                }
            r[u] = ld_stream(reinterpret_cast<const VecT*>(src) + ((uint64_t)row * seg + (col - ov)));
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const uint64_t v = base + (uint64_t)u * BLOCK;
        if (v < p.nvec) st_stream(y + v, r[u]);
    }
}

// KV-cache append: blockIdx.y == 0 copies the filled prefix of the cache into dst, blockIdx.y == 1 writes the new rows
// into both the cache (at `offset`) and dst.  All quantities are in vectors of sizeof(VecT) bytes.
struct CacheArgs {
    FastDiv pv, sv;          // prefix / source vectors per outer row
    uint32_t cap_v, dst_v;   // cache / dst vectors per outer row
    uint32_t off_v;          // offset, in vectors, inside an outer row
    uint32_t n_prefix, n_src;
};

// (dst is written with streaming stores: [4,32,2048,80] f32 + one row 31.9 -> 26.3 us, [4,32,4096,96] f16 prefill 30.4 -> 27.2 us;
// streaming loads as well help the large appends and cost the small ones, 5.1 -> 6.7 us, and are not used)
template <typename VecT>
__global__ void __launch_bounds__(BLOCK) cache_kernel(VecT* __restrict__ cache, const VecT* __restrict__ src, VecT* __restrict__ dst,
                                                      CacheArgs p) {
    const uint32_t base = blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
    if (blockIdx.y == 0) {
        if (blockIdx.x * (BLOCK * UNROLL) >= p.n_prefix) return;
        VecT r[UNROLL];
        uint32_t row[UNROLL], col[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const uint32_t v = base + u * BLOCK;
            if (v < p.n_prefix) {
                fd_divmod(v, p.pv, row[u], col[u]);
                r[u] = cache[(uint64_t)row[u] * p.cap_v + col[u]];
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const uint32_t v = base + u * BLOCK;
            if (v < p.n_prefix) st_stream(dst + (uint64_t)row[u] * p.dst_v + col[u], r[u]);
        }
    } else {
        if (blockIdx.x * (BLOCK * UNROLL) >= p.n_src) return;
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const uint32_t v = base + u * BLOCK;
            if (v < p.n_src) {
                uint32_t row, col;
                fd_divmod(v, p.sv, row, col);
                const VecT val = src[v];
                cache[(uint64_t)row * p.cap_v + p.off_v + col] = val;
                st_stream(dst + (uint64_t)row * p.dst_v + p.off_v + col, val);
            }
        }
    }
}

// IndexSelect: dst[left, i, right] = src[left, indices[i], right].  One thread per vector of the `right` run; an index
// outside [0, src_dim) (the reference panics on it) yields a row of zeros rather than a wild read.
struct SelectArgs {
    FastDiv rv;              // vectors per `right` run
    FastDiv n_ids;
    uint32_t src_dim;
    uint32_t nvec;
};

template <typename VecT>
__global__ void __launch_bounds__(BLOCK) index_select_kernel(const VecT* __restrict__ src, const int32_t* __restrict__ indices,
                                                             VecT* __restrict__ dst, SelectArgs p) {
    const uint32_t v = blockIdx.x * BLOCK + threadIdx.x;
    if (v >= p.nvec) return;
    uint32_t row, col, left, i;
    fd_divmod(v, p.rv, row, col);
    fd_divmod(row, p.n_ids, left, i);
    const uint32_t idx = (uint32_t)indices[i];
    VecT val = {};
    if (idx < p.src_dim) val = src[((uint64_t)left * p.src_dim + idx) * p.rv.d + col];
    st_stream(dst + v, val);
}

// IndexSelect from a Q8_0 source (the embedding table of a quantized model): four signed bytes per packed word, one scale
// per 32 consecutive elements of the flat source; a thread expands one word: dst = float(int8) * scale, rounded once to
// the scale's type (f32 for Q8_0F, f16 for Q8_0H).
template <typename T>
__global__ void __launch_bounds__(BLOCK) index_select_q8_kernel(const uint32_t* __restrict__ packed, const T* __restrict__ scales,
                                                                const int32_t* __restrict__ indices, T* __restrict__ dst, SelectArgs p) {
    const uint32_t v = blockIdx.x * BLOCK + threadIdx.x;       // destination word index: 4 elements
    if (v >= p.nvec) return;
    uint32_t row, col, left, i;
    fd_divmod(v, p.rv, row, col);
    fd_divmod(row, p.n_ids, left, i);
    const uint32_t idx = (uint32_t)indices[i];
    T out[4];
#pragma unroll
    for (int j = 0; j < 4; j++) out[j] = Ar<T>::conv(0.0f);
    if (idx < p.src_dim) {
        const uint64_t w = ((uint64_t)left * p.src_dim + idx) * p.rv.d + col;          // source word
        const uint32_t q = packed[w];
        const float sc = Ar<T>::widen(scales[w >> 3]);
#pragma unroll
        for (int j = 0; j < 4; j++) out[j] = Ar<T>::conv((float)(int8_t)(q >> (8 * j)) * sc);
    }
    if (sizeof(T) == 4) {
        v4u o;
        __builtin_memcpy(&o, out, 16);
        st_stream(reinterpret_cast<v4u*>(dst) + v, o);
    } else {
        v2u o;
        __builtin_memcpy(&o, out, 8);
        st_stream(reinterpret_cast<v2u*>(dst) + v, o);
    }
}

// IndexWrite: a flat run of src copied into dst from a linear offset (bytes here)
__global__ void __launch_bounds__(BLOCK) index_write_vec_kernel(v4u* __restrict__ dst, const v4u* __restrict__ src, uint64_t nvec) {
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < nvec) dst[i] = ld_stream(src + i);
}
__global__ void __launch_bounds__(BLOCK) index_write_u16_kernel(uint16_t* __restrict__ dst, const uint16_t* __restrict__ src, uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

inline unsigned blocks_for(uint64_t items, uint64_t per_block) {
    const uint64_t b = (items + per_block - 1) / per_block;
    return (unsigned)(b ? b : 1);
}

inline void contiguous_strides(const uint32_t shape[4], uint64_t out[4]) {
    uint64_t s = 1;
    for (int i = 3; i >= 0; i--) { out[i] = s; s *= shape[i]; }
}

// Launches the gather dst[i] = src[base + sum i_k * S_k] (all in elements) choosing the widest usable vector.
// Rows that start or end off the vector grid (a slice to columns 3 .. 69): the destination is contiguous, so it is written
// as flat 16-byte vectors whatever the row length, and only the source is read element by element.  p.d3 divides by the
// whole last dim, p.s and p.base are in elements here.  [4,32,2048,80] sliced to columns 3 .. 69 in f16: 39.8 -> 21.3 us
// against element-wise stores, in f32 42.2 -> 27.7 us.
template <typename ET>
__global__ void __launch_bounds__(BLOCK) gather_flat_kernel(const ET* __restrict__ x, ET* __restrict__ y, GatherArgs p, uint64_t numel) {
    constexpr int VE = 16 / (int)sizeof(ET);
    const uint64_t f0 = ((uint64_t)blockIdx.x * BLOCK + threadIdx.x) * VE;
    if (f0 >= numel) return;
    uint32_t row, col, i0, i1, i2, t;
    fd_divmod((uint32_t)f0, p.d3, row, col);
    fd_divmod(row, p.d2, t, i2);
    fd_divmod(t, p.d1, i0, i1);
    uint64_t off = p.base + (uint64_t)i0 * p.s[0] + (uint64_t)i1 * p.s[1] + (uint64_t)i2 * p.s[2] + (uint64_t)col * p.s[3];
    const uint32_t d3 = p.d3.d;
    Vec16<ET> out;
#pragma unroll
    for (int e = 0; e < VE; e++) {
        out.e[e] = x[f0 + e < numel ? off : p.base];         // (nothing is read past the slice's last element)
        off += p.s[3];
        if (++col == d3 && e + 1 < VE) {                     // the next element starts a row
            col = 0;
            fd_divmod((uint32_t)f0 + e + 1, p.d3, row, t);
            fd_divmod(row, p.d2, t, i2);
            fd_divmod(t, p.d1, i0, i1);
            off = p.base + (uint64_t)i0 * p.s[0] + (uint64_t)i1 * p.s[1] + (uint64_t)i2 * p.s[2];
        }
    }
    if (f0 + VE <= numel) {
        st_stream(reinterpret_cast<v4u*>(y + f0), out.u);
    } else {
        for (int e = 0; e < VE && f0 + e < numel; e++) y[f0 + e] = out.e[e];
    }
}

int launch_gather(rt_device* dev, int eb, const void* x, void* y, const uint32_t dst_shape_in[4], const uint64_t S_in[4],
                  uint64_t base_elems, const char* who) {
    // Drop size-1 dims and merge neighbours that are contiguous on both sides (the destination always is): a slice of
    // the leading dim only, or a broadcast of whole rows, becomes one long row and gets the widest vectors.
    uint32_t dst_shape[4] = {1, 1, 1, 1};
    uint64_t S[4] = {0, 0, 0, 0};
    {
        uint64_t ext[4], st[4];
        int m = 0;
        for (int i = 0; i < 4; i++) {
            if (dst_shape_in[i] == 1) continue;
            if (m > 0 && st[m - 1] == S_in[i] * dst_shape_in[i] && ext[m - 1] * dst_shape_in[i] <= 0xffffffffull &&
                (S_in[i] != 0 || st[m - 1] == 0)) {
                ext[m - 1] *= dst_shape_in[i];
                st[m - 1] = S_in[i];
            } else {
                ext[m] = dst_shape_in[i];
                st[m] = S_in[i];
                m++;
            }
        }
        for (int i = 0; i < m; i++) {
            dst_shape[4 - m + i] = (uint32_t)ext[i];
            S[4 - m + i] = st[i];
        }
    }
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) n *= dst_shape[i];
    const uint64_t row_bytes = (uint64_t)dst_shape[3] * eb;
    const bool splat = (S[3] == 0 && dst_shape[3] > 1);
    // widest vector width (bytes) that divides the row, the strides and the base, with both pointers aligned
    int vb = 16;
    for (; vb > eb; vb >>= 1) {
        if (row_bytes % vb) continue;
        if (!rt_aligned(y, (size_t)vb)) continue;
        if (!splat) {
            if (!rt_aligned(x, (size_t)vb)) continue;
            if ((base_elems * eb) % vb) continue;
            bool ok = true;
            for (int i = 0; i < 3; i++)
                if (dst_shape[i] > 1 && (S[i] * eb) % vb) ok = false;
            if (!ok) continue;
        }
        break;
    }
    const bool contiguous_last = (S[3] == 1 || dst_shape[3] == 1);
    if (!contiguous_last && !splat) vb = eb;      // strided last dim that is not a broadcast: scalar gather
    const uint32_t per = (uint32_t)(vb / eb);
    const uint64_t nvec = n / per;
    RT_REQUIRE(nvec <= 0xffffffffull - (uint64_t)BLOCK * UNROLL, RT_ERR_SIZE, "%s: %llu vectors exceed the 32-bit index space",
               who, (unsigned long long)nvec);
    if (!splat && contiguous_last && vb == eb && eb < 16 && rt_aligned(y, 16) && n <= 0xfffffff0ull && n * (uint64_t)eb >= (1u << 20)) {
        // element-wise on both sides otherwise: flat vectors for the destination
        GatherArgs f;
        f.d3 = make_fastdiv(dst_shape[3]);
        f.d2 = make_fastdiv(dst_shape[2]);
        f.d1 = make_fastdiv(dst_shape[1]);
        f.base = base_elems;
        for (int i = 0; i < 4; i++) f.s[i] = dst_shape[i] > 1 ? S[i] : 0;
        f.nvec = 0;
        f.rm_h = make_fastdiv(1);
        f.rm_j = 0;
        const uint32_t ve = 16u / (uint32_t)eb;
        const unsigned fblocks = blocks_for((n + ve - 1) / ve, BLOCK);
        if (eb == 4) hipLaunchKernelGGL((gather_flat_kernel<uint32_t>), dim3(fblocks), dim3(BLOCK), 0, dev->stream, (const uint32_t*)x, (uint32_t*)y, f, n);
        else hipLaunchKernelGGL((gather_flat_kernel<uint16_t>), dim3(fblocks), dim3(BLOCK), 0, dev->stream, (const uint16_t*)x, (uint16_t*)y, f, n);
        RT_CHECK_LAUNCH(who);
        return RT_OK;
    }
    GatherArgs p;
    p.d3 = make_fastdiv(dst_shape[3] / per);
    p.d2 = make_fastdiv(dst_shape[2]);
    p.d1 = make_fastdiv(dst_shape[1]);
    p.nvec = (uint32_t)nvec;
    // vectors per thread of the vector kernel: see gather_vec_kernel
    bool repeats = false;
    for (int i = 0; i < 4; i++) repeats = repeats || (dst_shape[i] > 1 && S[i] == 0);
    const int per_thread = (splat || repeats || n * (uint64_t)eb < GATHER_ONE_FROM_BYTES) ? UNROLL : 1;
    const unsigned blocks = blocks_for(nvec, (uint64_t)BLOCK * per_thread);
    p.rm_h = make_fastdiv(1);
    p.rm_j = 0;
    if (!splat && dst_shape[1] > 1 && dst_shape[2] > 1 && S[1] != 0 && S[1] < S[2] && (row_bytes % 128) != 0) {
        // dim 1 lies closer together in the source than dim 2 and the rows do not fill whole lines
        const uint64_t slice_vec = (uint64_t)dst_shape[2] * dst_shape[3] / per;
        const uint64_t heads = (uint64_t)dst_shape[0] * dst_shape[1];
        if (slice_vec % (BLOCK * per_thread) == 0) {
            const uint64_t j = slice_vec / (BLOCK * per_thread);
            if (j % 8 == 0 && j * heads == blocks) {
                p.rm_h = make_fastdiv((uint32_t)heads);
                p.rm_j = (uint32_t)j;
            }
        }
    }
    if (splat) {
        p.base = base_elems;
        for (int i = 0; i < 4; i++) p.s[i] = S[i];
#define RT_SPLAT(ET, VT) \
    hipLaunchKernelGGL((gather_splat_kernel<ET, VT>), dim3(blocks), dim3(BLOCK), 0, dev->stream, (const ET*)x, (VT*)y, p)
        if (eb == 4) {
            if (vb == 16) RT_SPLAT(uint32_t, v4u);
            else if (vb == 8) RT_SPLAT(uint32_t, v2u);
            else RT_SPLAT(uint32_t, uint32_t);
        } else {
            if (vb == 16) RT_SPLAT(uint16_t, v4u);
            else if (vb == 8) RT_SPLAT(uint16_t, v2u);
            else if (vb == 4) RT_SPLAT(uint16_t, uint32_t);
            else RT_SPLAT(uint16_t, uint16_t);
        }
#undef RT_SPLAT
    } else {
        // convert to vector units; with per == 1 a strided last dim keeps its element stride
        p.base = base_elems / per;
        for (int i = 0; i < 3; i++) p.s[i] = (dst_shape[i] > 1) ? S[i] / per : 0;
        p.s[3] = (per > 1 || dst_shape[3] == 1) ? (dst_shape[3] == 1 ? 0 : 1) : S[3];
#define RT_GATHER(VT)                                                                                                                  \
    do {                                                                                                                               \
        if (per_thread == 1)                                                                                                           \
            hipLaunchKernelGGL((gather_vec_kernel<VT, 1>), dim3(blocks), dim3(BLOCK), 0, dev->stream, (const VT*)x, (VT*)y, p);       \
        else                                                                                                                           \
            hipLaunchKernelGGL((gather_vec_kernel<VT, UNROLL>), dim3(blocks), dim3(BLOCK), 0, dev->stream, (const VT*)x, (VT*)y, p);  \
    } while (0)
        if (vb == 16) RT_GATHER(v4u);
        else if (vb == 8) RT_GATHER(v2u);
        else if (vb == 4) RT_GATHER(uint32_t);
        else RT_GATHER(uint16_t);
#undef RT_GATHER
    }
    RT_CHECK_LAUNCH(who);
    return RT_OK;
}

int validate_common(int elem_bytes, const void* x, const void* y, const char* who) {
    RT_REQUIRE(elem_bytes == 2 || elem_bytes == 4, RT_ERR_ARG, "%s: elem_bytes must be 2 or 4, got %d", who, elem_bytes);
    RT_REQUIRE(x && y, RT_ERR_NULL_POINTER, "%s: NULL operand", who);
    RT_REQUIRE(rt_aligned(x, (size_t)elem_bytes) && rt_aligned(y, (size_t)elem_bytes), RT_ERR_ALIGN, "%s: misaligned pointer", who);
    return RT_OK;
}

}  // namespace

extern "C" {

int rt_permute(rt_device* dev, int elem_bytes, const void* x, void* y, const uint32_t src_shape[4], const uint32_t perm[4]) {
    RT_REQUIRE(src_shape && perm, RT_ERR_NULL_POINTER, "rt_permute: NULL shape or perm");
    bool seen[4] = {false, false, false, false};
    for (int i = 0; i < 4; i++) {
        RT_REQUIRE(perm[i] < 4 && !seen[perm[i]], RT_ERR_PERM, "rt_permute: [%u,%u,%u,%u] is not a permutation of 0..3", perm[0],
                   perm[1], perm[2], perm[3]);
        seen[perm[i]] = true;
    }
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) {
        RT_REQUIRE(src_shape[i] > 0, RT_ERR_SHAPE, "rt_permute: zero extent in dim %d", i);
        n *= src_shape[i];
    }
    RT_REQUIRE(n <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_permute: tensor too large");
    int rc = validate_common(elem_bytes, x, y, "rt_permute");
    if (rc) return rc;
    rc = rt_enter(dev);
    if (rc) return rc;

    uint64_t src_strides[4], S[4];
    uint32_t dst_shape[4];
    contiguous_strides(src_shape, src_strides);
    for (int i = 0; i < 4; i++) {
        dst_shape[i] = src_shape[perm[i]];           // permute.rs:53-56
        S[i] = src_strides[perm[i]];
    }
    // Does the source's contiguous run survive?  Drop size-1 dims from the question: they carry no data movement.
    if (S[3] == 1 || dst_shape[3] == 1) return launch_gather(dev, elem_bytes, x, y, dst_shape, S, 0, "rt_permute");

    // find the dst dim fed by the source's innermost non-trivial dim
    int q = -1;
    for (int i = 0; i < 3; i++)
        if (S[i] == 1 && dst_shape[i] > 1) q = i;
    if (q < 0) {
        // the source's last dim has extent 1, so "contiguous" is carried by a dim with stride > 1 everywhere: plain
        // strided gather is as good as it gets
        return launch_gather(dev, elem_bytes, x, y, dst_shape, S, 0, "rt_permute");
    }
    uint64_t dst_strides[4];
    contiguous_strides(dst_shape, dst_strides);
    int others[2], no = 0;
    for (int i = 0; i < 3; i++)
        if (i != q) others[no++] = i;
    {
        // a short contiguous dim that changes sides (channels): [.., J, C] -> [.., C, J] or back, in 16-byte accesses on both
        // sides.  [4,1024,1024,5] -> [4,5,1024,1024] f32 took 33 us with the scalar accesses of the LDS-tile kernel.
        const uint32_t VE = 16u / (uint32_t)elem_bytes;
        ChannelArgs c;
        bool fits = false, to_planes = false;
        uint32_t ea = 1, eb_ = 1;
        if (dst_shape[q] >= 2 && dst_shape[q] <= 16 && S[3] == dst_shape[q]) {
            // interleaved source: dst dim q is the channel, dst dim 3 (with dst dim 2 merged in when it continues the run) is J
            to_planes = true;
            c.C = dst_shape[q];
            uint64_t J = dst_shape[3];
            const bool merged = q != 2 && S[2] == S[3] * dst_shape[3];
            if (merged) J *= dst_shape[2];
            ea = dst_shape[others[0]];
            eb_ = merged ? 1 : dst_shape[others[1]];
            c.ia = S[others[0]];
            c.ib = merged ? 0 : S[others[1]];
            c.pa = dst_strides[others[0]];
            c.pb = merged ? 0 : dst_strides[others[1]];
            c.plane = dst_strides[q];
            fits = J <= 0xffffffffull;
            c.J = (uint32_t)J;
        } else if (q == 2 && dst_shape[3] >= 2 && dst_shape[3] <= 16) {
            // interleaved destination: dst dim 3 is the channel, dst dim 2 (with dst dim 1 merged in) is J
            c.C = dst_shape[3];
            uint64_t J = dst_shape[2];
            const bool merged = S[1] == dst_shape[2];
            if (merged) J *= dst_shape[1];
            ea = dst_shape[0];
            eb_ = merged ? 1 : dst_shape[1];
            c.ia = dst_strides[0];
            c.ib = merged ? 0 : dst_strides[1];
            c.pa = S[0];
            c.pb = merged ? 0 : S[1];
            c.plane = S[3];
            fits = J <= 0xffffffffull;
            c.J = (uint32_t)J;
        }
        if (fits && c.J % VE == 0 && c.ia % VE == 0 && c.ib % VE == 0 && c.pa % VE == 0 && c.pb % VE == 0 && c.plane % VE == 0 &&
            rt_aligned(x, 16) && rt_aligned(y, 16)) {
            c.PJ = c.C <= 4 ? 1024 : c.C <= 8 ? 512 : 256;   // PJ * C <= CH_TILE
            c.P = c.C | 1u;
            c.cdiv = make_fastdiv(c.C);
            const uint64_t gj = ((uint64_t)c.J + c.PJ - 1) / c.PJ;
            const uint64_t blocks = gj * ea * eb_;
            if (blocks <= 0x7fffffffull) {
                c.gj = make_fastdiv((uint32_t)gj);
                c.ob = make_fastdiv(eb_);
                const dim3 grid((unsigned)blocks), block(BLOCK);
                if (elem_bytes == 4) {
                    if (to_planes) hipLaunchKernelGGL((channels_kernel<uint32_t, true>), grid, block, 0, dev->stream, (const uint32_t*)x, (uint32_t*)y, c);
                    else hipLaunchKernelGGL((channels_kernel<uint32_t, false>), grid, block, 0, dev->stream, (const uint32_t*)x, (uint32_t*)y, c);
                } else {
                    if (to_planes) hipLaunchKernelGGL((channels_kernel<uint16_t, true>), grid, block, 0, dev->stream, (const uint16_t*)x, (uint16_t*)y, c);
                    else hipLaunchKernelGGL((channels_kernel<uint16_t, false>), grid, block, 0, dev->stream, (const uint16_t*)x, (uint16_t*)y, c);
                }
                RT_CHECK_LAUNCH("channels_kernel");
                return RT_OK;
            }
        }
    }
    // A short dst dim 3 (fewer than 64 elements) behind a dst dim 2 that is not the source's contiguous one: the two are
    // one contiguous run in the destination, so they are transposed against dim q as one dim whose source offset has two
    // levels ([8,32,512,80] -> perm (1,3,2,0) = [32,80,512,8]: rows of 8 elements became rows of 4096; 56 -> 11 us in f16, the reversal (3,2,1,0) of that shape 61 -> 12 us).
    bool merged23 = false;
    uint32_t inner23 = 1;
    uint64_t s_outer23 = 0;
    if (q != 2 && dst_shape[3] < 64 && dst_shape[2] > 1 && (uint64_t)dst_shape[2] * dst_shape[3] <= 0xffffffffull) {
        merged23 = true;
        inner23 = dst_shape[3];
        s_outer23 = S[2];
        const uint32_t d0 = dst_shape[0], d1 = dst_shape[1], d23 = dst_shape[2] * dst_shape[3];
        const uint64_t s0 = S[0], s1 = S[1], s3 = S[3];
        dst_shape[0] = 1; dst_shape[1] = d0; dst_shape[2] = d1; dst_shape[3] = d23;
        S[0] = 0; S[1] = s0; S[2] = s1; S[3] = s3;
        q += 1;
        contiguous_strides(dst_shape, dst_strides);
        no = 0;
        for (int i = 0; i < 3; i++)
            if (i != q) others[no++] = i;
    }
    {
        // The LDS patch kernel where it beats the register transpose below: tensors of 128 MB and more, where one store per
        // thread pays ([8,32,2048,128] f16: 48 -> 45 us; 32-bit ones in larger patches).  (Source rows of 65 to 128 elements
        // that are not 64 or 128 long, head dims 80 and 96, go to transpose_wide_kernel in one patch across the row: K^T of
        // [4,32,2048,80] f16 21.6 -> 17.7 us, of [4,32,4096,96] f16 45.2 -> 37.8 us, against 64-wide patches of this kernel.)
        const uint32_t V = 16u / (uint32_t)elem_bytes;
        uint64_t total = (uint64_t)elem_bytes;
        for (int i = 0; i < 4; i++) total *= dst_shape[i];
        const bool short_row = dst_shape[q] > 64 && dst_shape[q] <= 128 && dst_shape[q] % 64 != 0;    // one patch of transpose_wide_kernel across it
        // (16-bit rows that are not whole 128-byte lines on both sides: transpose_wide_kernel below, whose patches this
        // kernel's 128-byte runs, each across two lines there, do not beat: [1,8200,8200] f16 154 -> 97 us, [4,4104,4104]
        // 128 -> 87 us, [1,8192,8200] 82 -> 61 us; 32-bit ones gain nothing from it)
        const bool lines16 = elem_bytes == 4 || ((uint64_t)dst_shape[q] * elem_bytes % 128 == 0 && (uint64_t)dst_shape[3] * elem_bytes % 128 == 0);
        if (!merged23 && total >= (128ull << 20) && !short_row && lines16 && dst_shape[q] % V == 0 && dst_shape[3] % V == 0 &&
            S[3] % V == 0 && S[others[0]] % V == 0 && S[others[1]] % V == 0 && rt_aligned(x, 16) && rt_aligned(y, 16)) {
            TransposeArgs p;
            p.inner = make_fastdiv(1);
            p.s2 = S[3];
            p.nq = dst_shape[q];
            p.n3 = dst_shape[3];
            p.s3 = S[3];
            p.dq = dst_strides[q];
            p.ob = make_fastdiv(dst_shape[others[1]]);
            p.sa = S[others[0]];
            p.sb = S[others[1]];
            p.da = dst_strides[others[0]];
            p.db = dst_strides[others[1]];
            if (elem_bytes == 4 && total >= (128ull << 20)) {
                // 32-bit tensors of 128 MB and more: patches of 128 x 64 elements, 256-byte runs in, 512-byte runs out
                // ([2,4096,4096] 58.6 -> 47.9 us, [1,8192,8192] 137 -> 123 us, [16,2048,2048] 93.9 -> 87.5 us, [3,3000,5120]
                // 88 -> 79 us; 16-bit tensors gained nothing from patches of 128 x 128, 256 x 64 or 64 x 256)
                constexpr int TJ = 128, TQ = 64;
                const uint64_t gx = (p.nq + TQ - 1) / TQ, gy = (p.n3 + TJ - 1) / TJ;
                const uint64_t blocks = gx * gy * dst_shape[others[0]] * dst_shape[others[1]];
                RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_permute: %llu tiles exceed the grid limit", (unsigned long long)blocks);
                p.gx = make_fastdiv((uint32_t)gx);
                p.gy = make_fastdiv((uint32_t)gy);
                hipLaunchKernelGGL((transpose_big_kernel<uint32_t, TJ, TQ>), dim3((unsigned)blocks), dim3(TV_BLOCK), 0, dev->stream,
                                   (const uint32_t*)x, (uint32_t*)y, p);
                RT_CHECK_LAUNCH("transpose_big_kernel");
                return RT_OK;
            }
            const uint64_t gx = (p.nq + 8 * V - 1) / (8 * V), gy = (p.n3 + 63) / 64;
            const uint64_t blocks = gx * gy * dst_shape[others[0]] * dst_shape[others[1]];
            RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_permute: %llu tiles exceed the grid limit", (unsigned long long)blocks);
            p.gx = make_fastdiv((uint32_t)gx);
            p.gy = make_fastdiv((uint32_t)gy);
            if (elem_bytes == 4)
                hipLaunchKernelGGL((transpose_vec_kernel<uint32_t>), dim3((unsigned)blocks), dim3(TV_BLOCK), 0, dev->stream, (const uint32_t*)x,
                                   (uint32_t*)y, p);
            else
                hipLaunchKernelGGL((transpose_vec_kernel<uint16_t>), dim3((unsigned)blocks), dim3(TV_BLOCK), 0, dev->stream, (const uint16_t*)x,
                                   (uint16_t*)y, p);
            RT_CHECK_LAUNCH("transpose_vec_kernel");
            return RT_OK;
        }
    }
    {
        // whole aligned 16-byte vectors on both sides: the register transpose
        const uint32_t V = 16u / (uint32_t)elem_bytes;
        // (when one side is so short that its blocks cannot fill half a wave, the LDS tile below does better; so it does when
        // the rows of either side are not whole 128-byte lines, where every 128-byte run of the register kernel touches two
        // lines: [8,1500,1000] f32 34.7 -> 23.3 us, [4,2040,3080] f32 78 -> 54 us, [3,3000,5120] f16 63 -> 44 us, K^T of
        // [16,6,1500,64] f32 22.1 -> 20.8 us; on whole lines the two are within 5 % of each other)
        const bool whole_lines = (uint64_t)dst_shape[q] * elem_bytes % 128 == 0 && (uint64_t)dst_shape[3] * elem_bytes % 128 == 0;
        uint32_t qb = dst_shape[q] / V <= 12 ? dst_shape[q] / V : 8, jb = 64 / (qb ? qb : 1);
        if (jb > dst_shape[3] / V) jb = dst_shape[3] / V;
        if (!merged23 && dst_shape[q] % V == 0 && dst_shape[3] % V == 0 && rt_aligned(x, 16) && rt_aligned(y, 16) && qb * jb >= 32 && whole_lines) {
            TransposeRegArgs r;
            r.nqb = dst_shape[q] / V;
            r.njb = dst_shape[3] / V;
            r.QB = qb;
            r.JB = jb;
            r.qb_div = make_fastdiv(r.QB);
            r.s3 = S[3];
            r.dq = dst_strides[q];
            r.ob = make_fastdiv(dst_shape[others[1]]);
            r.sa = S[others[0]];
            r.sb = S[others[1]];
            r.da = dst_strides[others[0]];
            r.db = dst_strides[others[1]];
            const uint64_t gz = (uint64_t)dst_shape[others[0]] * dst_shape[others[1]];
            const uint64_t gx = (r.nqb + r.QB - 1) / r.QB, gy = (r.njb + (BLOCK / 64) * r.JB - 1) / ((BLOCK / 64) * r.JB);
            const uint64_t blocks = gx * gy * gz;
            RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_permute: %llu tiles exceed the grid limit", (unsigned long long)blocks);
            r.gx = make_fastdiv((uint32_t)gx);
            r.gy = make_fastdiv((uint32_t)gy);
            if (elem_bytes == 4) {
                hipLaunchKernelGGL((transpose_reg_kernel<uint32_t>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream,
                                   (const uint32_t*)x, (uint32_t*)y, r);
            } else {
                hipLaunchKernelGGL((transpose_reg_kernel<uint16_t>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream,
                                   (const uint16_t*)x, (uint16_t*)y, r);
            }
            RT_CHECK_LAUNCH("transpose_reg_kernel");
            return RT_OK;
        }
    }
    TransposeArgs p;
    p.nq = dst_shape[q];
    p.n3 = dst_shape[3];
    p.s3 = S[3];
    p.inner = make_fastdiv(inner23);
    p.s2 = merged23 ? s_outer23 : S[3];
    p.dq = dst_strides[q];
    p.ob = make_fastdiv(dst_shape[others[1]]);
    p.sa = S[others[0]];
    p.sb = S[others[1]];
    p.da = dst_strides[others[0]];
    p.db = dst_strides[others[1]];
    const uint64_t gz = (uint64_t)dst_shape[others[0]] * dst_shape[others[1]];
    const uint32_t tq = p.nq <= 8 ? 8 : p.nq <= 16 ? 16 : p.n3 <= 8 ? 512 : p.n3 <= 16 ? 256 : 64, tj = TILE_ELEMS / tq;
    if (tq == 64) {
        // square patches: the widest loads and stores that every row start and extent on each side is a multiple of
        auto width = [&](uint64_t extent, uint64_t s0, uint64_t s1, uint64_t s2, const void* base) -> int {
            int w = 16 / elem_bytes;
            while (w > 1 && (extent % w || s0 % w || s1 % w || s2 % w || !rt_aligned(base, (size_t)w * elem_bytes))) w >>= 1;
            return w;
        };
        int lw = width(p.nq, p.s3, p.sa, p.sb, x);
        while (lw > 1 && p.s2 % lw) lw >>= 1;
        const int sw = width(p.n3, p.dq, p.da, p.db, y);
        if (lw > 1 || sw > 1) {
            // a source row of 65 to 128 elements in whole vectors: one patch across it
            const int lw_max = 16 / elem_bytes;
            const uint32_t wtq = (lw == lw_max && p.nq > 64 && p.nq <= 128 && p.nq % 64 != 0) ? (p.nq <= 80 ? 80 : p.nq <= 96 ? 96 : 128) : 64;
            const uint64_t wgx = (p.nq + wtq - 1) / wtq, wgy = (p.n3 + 63) / 64;
            const uint64_t wblocks = wgx * wgy * gz;
            RT_REQUIRE(wblocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_permute: %llu tiles exceed the grid limit", (unsigned long long)wblocks);
            p.gx = make_fastdiv((uint32_t)wgx);
            p.gy = make_fastdiv((uint32_t)wgy);
#define RT_TW(E, LWC, SWC) \
    hipLaunchKernelGGL((transpose_wide_kernel<E, LWC, SWC>), dim3((unsigned)wblocks), dim3(BLOCK), 0, dev->stream, (const E*)x, (E*)y, p)
#define RT_TW_S(E, LWC)                   \
    do {                                  \
        if (sw == 1) RT_TW(E, LWC, 1);    \
        else if (sw == 2) RT_TW(E, LWC, 2); \
        else if (sw == 4 || sizeof(E) == 4) RT_TW(E, LWC, 4); \
        else RT_TW(E, LWC, (sizeof(E) == 4 ? 4 : 8)); \
    } while (0)
#define RT_TW_L(E)                        \
    do {                                  \
        if (lw == 1) RT_TW_S(E, 1);       \
        else if (lw == 2) RT_TW_S(E, 2);  \
        else if (lw == 4 || sizeof(E) == 4) RT_TW_S(E, 4); \
        else RT_TW_S(E, (sizeof(E) == 4 ? 4 : 8)); \
    } while (0)
#define RT_TW_Q(E, TQC)                                                                                                       \
    do {                                                                                                                      \
        constexpr int LWM = 16 / (int)sizeof(E);                                                                              \
        if (sw == 1) hipLaunchKernelGGL((transpose_wide_kernel<E, LWM, 1, TQC>), dim3((unsigned)wblocks), dim3(BLOCK), 0, dev->stream, (const E*)x, (E*)y, p); \
        else if (sw == 2) hipLaunchKernelGGL((transpose_wide_kernel<E, LWM, 2, TQC>), dim3((unsigned)wblocks), dim3(BLOCK), 0, dev->stream, (const E*)x, (E*)y, p); \
        else if (sw == 4 || sizeof(E) == 4) hipLaunchKernelGGL((transpose_wide_kernel<E, LWM, 4, TQC>), dim3((unsigned)wblocks), dim3(BLOCK), 0, dev->stream, (const E*)x, (E*)y, p); \
        else hipLaunchKernelGGL((transpose_wide_kernel<E, LWM, LWM, TQC>), dim3((unsigned)wblocks), dim3(BLOCK), 0, dev->stream, (const E*)x, (E*)y, p); \
    } while (0)
#define RT_TW_QS(E)                          \
    do {                                     \
        if (wtq == 80) RT_TW_Q(E, 80);       \
        else if (wtq == 96) RT_TW_Q(E, 96);  \
        else RT_TW_Q(E, 128);                \
    } while (0)
            if (wtq != 64) {
                if (elem_bytes == 4) RT_TW_QS(uint32_t);
                else RT_TW_QS(uint16_t);
            } else if (elem_bytes == 4) RT_TW_L(uint32_t);
            else RT_TW_L(uint16_t);
#undef RT_TW_QS
#undef RT_TW_Q
#undef RT_TW_L
#undef RT_TW_S
#undef RT_TW
            RT_CHECK_LAUNCH("transpose_wide_kernel");
            return RT_OK;
        }
    }
    const uint64_t gx = (p.nq + tq - 1) / tq, gy = (p.n3 + tj - 1) / tj;
    const uint64_t blocks = gx * gy * gz;
    RT_REQUIRE(blocks <= 0x7fffffffull, RT_ERR_SIZE, "rt_permute: %llu tiles exceed the grid limit", (unsigned long long)blocks);
    p.gx = make_fastdiv((uint32_t)gx);
    p.gy = make_fastdiv((uint32_t)gy);
#define RT_TR(E, TQ) hipLaunchKernelGGL((transpose_kernel<E, TQ>), dim3((unsigned)blocks), dim3(BLOCK), 0, dev->stream, (const E*)x, (E*)y, p)
#define RT_TR_E(E)                       \
    do {                                 \
        if (tq == 8) RT_TR(E, 8);        \
        else if (tq == 16) RT_TR(E, 16); \
        else if (tq == 64) RT_TR(E, 64); \
        else if (tq == 256) RT_TR(E, 256); \
        else RT_TR(E, 512);              \
    } while (0)
    if (elem_bytes == 4) RT_TR_E(uint32_t);
    else RT_TR_E(uint16_t);
#undef RT_TR_E
#undef RT_TR
    RT_CHECK_LAUNCH("transpose_kernel");
    return RT_OK;
}

int rt_slice(rt_device* dev, int elem_bytes, const void* x, void* y, const uint32_t src_shape[4], const uint32_t start[4],
             const uint32_t dst_shape[4]) {
    RT_REQUIRE(src_shape && start && dst_shape, RT_ERR_NULL_POINTER, "rt_slice: NULL shape");
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) {
        // slice.rs:38-51 asserts start <= end <= dim; the CPU path additionally asserts start < end (cpu/reindex.rs:103-105)
        RT_REQUIRE(dst_shape[i] > 0 && src_shape[i] > 0, RT_ERR_SHAPE, "rt_slice: empty range in dim %d", i);
        RT_REQUIRE((uint64_t)start[i] + dst_shape[i] <= src_shape[i], RT_ERR_SHAPE, "rt_slice: dim %d: %u + %u exceeds %u", i,
                   start[i], dst_shape[i], src_shape[i]);
        n *= src_shape[i];
    }
    RT_REQUIRE(n <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_slice: tensor too large");
    int rc = validate_common(elem_bytes, x, y, "rt_slice");
    if (rc) return rc;
    rc = rt_enter(dev);
    if (rc) return rc;
    uint64_t S[4], base = 0;
    contiguous_strides(src_shape, S);
    for (int i = 0; i < 4; i++) base += (uint64_t)start[i] * S[i];
    return launch_gather(dev, elem_bytes, x, y, dst_shape, S, base, "rt_slice");
}

int rt_broadcast(rt_device* dev, int elem_bytes, const void* x, void* y, const uint32_t src_shape[4], const uint32_t dst_shape[4]) {
    RT_REQUIRE(src_shape && dst_shape, RT_ERR_NULL_POINTER, "rt_broadcast: NULL shape");
    uint64_t n = 1;
    for (int i = 0; i < 4; i++) {
        RT_REQUIRE(src_shape[i] > 0 && dst_shape[i] > 0, RT_ERR_SHAPE, "rt_broadcast: zero extent in dim %d", i);
        // Broadcast::check_shapes (broadcast.rs:31-58)
        RT_REQUIRE(src_shape[i] == 1 || src_shape[i] == dst_shape[i], RT_ERR_SHAPE,
                   "rt_broadcast: source dimension %u cannot be broadcast to %u", src_shape[i], dst_shape[i]);
        n *= dst_shape[i];
    }
    RT_REQUIRE(n <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_broadcast: tensor too large");
    int rc = validate_common(elem_bytes, x, y, "rt_broadcast");
    if (rc) return rc;
    rc = rt_enter(dev);
    if (rc) return rc;
    uint64_t S[4];
    contiguous_strides(src_shape, S);
    for (int i = 0; i < 4; i++)
        if (src_shape[i] == 1) S[i] = 0;
    return launch_gather(dev, elem_bytes, x, y, dst_shape, S, 0, "rt_broadcast");
}

int rt_concat(rt_device* dev, int elem_bytes, int n_inputs, const void* const* xs, const uint32_t (*shapes)[4], int dim, void* y) {
    RT_REQUIRE(elem_bytes == 2 || elem_bytes == 4, RT_ERR_ARG, "rt_concat: elem_bytes must be 2 or 4, got %d", elem_bytes);
    // Concat::check_shapes (concat.rs:131-152)
    RT_REQUIRE(n_inputs >= 2 && n_inputs <= 8, RT_ERR_ARG, "rt_concat: %d inputs (2..8 supported)", n_inputs);
    RT_REQUIRE(dim >= 0 && dim < 4, RT_ERR_ARG, "rt_concat: dim %d out of range", dim);
    RT_REQUIRE(xs && shapes && y, RT_ERR_NULL_POINTER, "rt_concat: NULL argument");
    uint64_t a_dim = 1, block = 1, dst_dim = 0;
    for (int k = 0; k < n_inputs; k++) {
        RT_REQUIRE(xs[k], RT_ERR_NULL_POINTER, "rt_concat: input %d is NULL", k);
        RT_REQUIRE(rt_aligned(xs[k], (size_t)elem_bytes), RT_ERR_ALIGN, "rt_concat: input %d misaligned", k);
        for (int a = 0; a < 4; a++) {
            RT_REQUIRE(shapes[k][a] > 0, RT_ERR_SHAPE, "rt_concat: input %d has a zero extent", k);
            if (a != dim)
                RT_REQUIRE(shapes[k][a] == shapes[0][a], RT_ERR_SHAPE, "rt_concat: input %d differs from input 0 in dim %d", k, a);
        }
        dst_dim += shapes[k][dim];
    }
    RT_REQUIRE(rt_aligned(y, (size_t)elem_bytes), RT_ERR_ALIGN, "rt_concat: output misaligned");
    for (int a = 0; a < dim; a++) a_dim *= shapes[0][a];
    for (int a = dim + 1; a < 4; a++) block *= shapes[0][a];
    const uint64_t dst_s = block * dst_dim;
    RT_REQUIRE(a_dim * dst_s <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_concat: output too large");
    int rc = rt_enter(dev);
    if (rc) return rc;

    // widest vector that divides every segment length, every column offset and the destination row
    int vb = 16;
    for (; vb > elem_bytes; vb >>= 1) {
        bool ok = rt_aligned(y, (size_t)vb) && (dst_s * elem_bytes) % vb == 0;
        uint64_t off = 0;
        for (int k = 0; k < n_inputs && ok; k++) {
            const uint64_t b_dim = block * shapes[k][dim];
            ok = rt_aligned(xs[k], (size_t)vb) && (b_dim * elem_bytes) % vb == 0 && (off * elem_bytes) % vb == 0;
            off += b_dim;
        }
        if (ok) break;
    }
    const uint64_t per = (uint64_t)vb / elem_bytes;
    RT_REQUIRE(dst_s / per <= 0xffffffffull, RT_ERR_SIZE, "rt_concat: destination row too long");
    {
        // short segments: walk the destination
        uint64_t min_seg = ~0ull;
        for (int k = 0; k < n_inputs; k++)
            if (block * shapes[k][dim] < min_seg) min_seg = block * shapes[k][dim];
        const uint64_t total = a_dim * dst_s / per;
        if (min_seg * elem_bytes < 1024 && total <= 0xffffffffull) {
            ConcatRowsArgs r;
            uint64_t o = 0;
            for (int k = 0; k < 8; k++) {
                r.src[k] = k < n_inputs ? xs[k] : xs[0];
                r.dst_ov[k] = k < n_inputs ? (uint32_t)(o / per) : 0xffffffffu;
                r.seg_v[k] = k < n_inputs ? (uint32_t)(block * shapes[k][dim] / per) : 0;
                if (k < n_inputs) o += block * shapes[k][dim];
            }
            r.dst_sv = make_fastdiv((uint32_t)(dst_s / per));
            r.nvec = total;
            const dim3 grid(blocks_for(total, BLOCK * UNROLL));
            if (vb == 16) hipLaunchKernelGGL((concat_rows_kernel<v4u>), grid, dim3(BLOCK), 0, dev->stream, (v4u*)y, r);
            else if (vb == 8) hipLaunchKernelGGL((concat_rows_kernel<v2u>), grid, dim3(BLOCK), 0, dev->stream, (v2u*)y, r);
            else if (vb == 4) hipLaunchKernelGGL((concat_rows_kernel<uint32_t>), grid, dim3(BLOCK), 0, dev->stream, (uint32_t*)y, r);
            else hipLaunchKernelGGL((concat_rows_kernel<uint16_t>), grid, dim3(BLOCK), 0, dev->stream, (uint16_t*)y, r);
            RT_CHECK_LAUNCH("concat_rows_kernel");
            return RT_OK;
        }
    }
    ConcatArgs p;
    uint64_t off = 0, max_nvec = 0;
    p.dst_sv = (uint32_t)(dst_s / per);
    for (int k = 0; k < 8; k++) {
        if (k < n_inputs) {
            const uint64_t b_dim = block * shapes[k][dim];
            const uint64_t nvec = a_dim * b_dim / per;
            RT_REQUIRE(nvec <= 0xffffffffull - (uint64_t)BLOCK * UNROLL, RT_ERR_SIZE, "rt_concat: input %d too large", k);
            p.src[k] = xs[k];
            p.bv[k] = make_fastdiv((uint32_t)(b_dim / per));
            p.dst_ov[k] = (uint32_t)(off / per);
            p.nvec[k] = (uint32_t)nvec;
            if (nvec > max_nvec) max_nvec = nvec;
            off += b_dim;
        } else {
            p.src[k] = nullptr;
            p.bv[k] = make_fastdiv(1);
            p.dst_ov[k] = 0;
            p.nvec[k] = 0;
        }
    }
    // vectors per thread: one for outputs of 64 MiB and more (as in gather_vec_kernel: [1,8192,4096] x 3 f16 71.1 -> 64.0 us,
    // [1,8192,3072] x 2 36.9 -> 34.3 us), two below ([1,2048,2560] x 2: 8.9 us against 9.3)
    const bool one = (uint64_t)a_dim * dst_s * elem_bytes >= (64ull << 20);
    const dim3 grid(blocks_for(max_nvec, BLOCK * (one ? 1 : UNROLL)), (unsigned)n_inputs);
#define RT_CC(VT)                                                                                                   \
    do {                                                                                                            \
        if (one) hipLaunchKernelGGL((concat_kernel<VT, 1>), grid, dim3(BLOCK), 0, dev->stream, (VT*)y, p);          \
        else hipLaunchKernelGGL((concat_kernel<VT, UNROLL>), grid, dim3(BLOCK), 0, dev->stream, (VT*)y, p);         \
    } while (0)
    if (vb == 16) RT_CC(v4u);
    else if (vb == 8) RT_CC(v2u);
    else if (vb == 4) RT_CC(uint32_t);
    else RT_CC(uint16_t);
#undef RT_CC
    RT_CHECK_LAUNCH("concat_kernel");
    return RT_OK;
}

int rt_cache(rt_device* dev, int elem_bytes, void* cache, const uint32_t cache_shape[4], const void* source, const uint32_t source_shape[4],
             int dim, uint32_t offset, void* dst) {
    RT_REQUIRE(elem_bytes == 2 || elem_bytes == 4, RT_ERR_ARG, "rt_cache: elem_bytes must be 2 or 4, got %d", elem_bytes);
    RT_REQUIRE(dim >= 0 && dim < 4, RT_ERR_ARG, "rt_cache: dim %d out of range", dim);
    RT_REQUIRE(cache_shape && source_shape, RT_ERR_NULL_POINTER, "rt_cache: NULL shape");
    uint64_t outer = 1, inner = 1;
    for (int a = 0; a < 4; a++) {
        RT_REQUIRE(cache_shape[a] > 0 && source_shape[a] > 0, RT_ERR_SHAPE, "rt_cache: zero extent in dim %d", a);
        if (a != dim)
            RT_REQUIRE(cache_shape[a] == source_shape[a], RT_ERR_SHAPE, "rt_cache: source differs from the cache in dim %d", a);
        if (a < dim) outer *= cache_shape[a];
        if (a > dim) inner *= cache_shape[a];
    }
    const uint64_t cap = cache_shape[dim], s = source_shape[dim];
    // Cache::check_shapes (ops/cache.rs:125-128): offset <= cache extent; the write itself must also fit
    RT_REQUIRE(offset <= cap && (uint64_t)offset + s <= cap, RT_ERR_SHAPE, "rt_cache: offset %u + %llu rows exceed the cache's %llu", offset,
               (unsigned long long)s, (unsigned long long)cap);
    RT_REQUIRE(cache && source && dst, RT_ERR_NULL_POINTER, "rt_cache: NULL operand");
    RT_REQUIRE(rt_aligned(cache, (size_t)elem_bytes) && rt_aligned(source, (size_t)elem_bytes) && rt_aligned(dst, (size_t)elem_bytes),
               RT_ERR_ALIGN, "rt_cache: misaligned pointer");
    RT_REQUIRE(outer * cap * inner <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_cache: cache too large");
    int rc = rt_enter(dev);
    if (rc) return rc;
    const uint64_t pre_b = (uint64_t)offset * inner * elem_bytes, src_b = s * inner * elem_bytes, cap_b = cap * inner * elem_bytes,
                   dst_b = ((uint64_t)offset + s) * inner * elem_bytes;
    int vb = 16;
    for (; vb > elem_bytes; vb >>= 1)
        if (pre_b % vb == 0 && src_b % vb == 0 && cap_b % vb == 0 && dst_b % vb == 0 && rt_aligned(cache, (size_t)vb) &&
            rt_aligned(source, (size_t)vb) && rt_aligned(dst, (size_t)vb))
            break;
    CacheArgs p;
    const uint64_t n_prefix = outer * pre_b / vb, n_src = outer * src_b / vb;
    RT_REQUIRE(n_prefix <= 0xffffffffull - (uint64_t)BLOCK * UNROLL && n_src <= 0xffffffffull - (uint64_t)BLOCK * UNROLL &&
                   cap_b / vb <= 0xffffffffull,
               RT_ERR_SIZE, "rt_cache: tensor too large for 32-bit vector indices");
    p.pv = make_fastdiv((uint32_t)(pre_b / vb ? pre_b / vb : 1));
    p.sv = make_fastdiv((uint32_t)(src_b / vb));
    p.cap_v = (uint32_t)(cap_b / vb);
    p.dst_v = (uint32_t)(dst_b / vb);
    p.off_v = (uint32_t)(pre_b / vb);
    p.n_prefix = (uint32_t)n_prefix;
    p.n_src = (uint32_t)n_src;
    const dim3 grid(blocks_for(n_prefix > n_src ? n_prefix : n_src, BLOCK * UNROLL), 2);
    if (vb == 16) hipLaunchKernelGGL((cache_kernel<v4u>), grid, dim3(BLOCK), 0, dev->stream, (v4u*)cache, (const v4u*)source, (v4u*)dst, p);
    else if (vb == 8) hipLaunchKernelGGL((cache_kernel<v2u>), grid, dim3(BLOCK), 0, dev->stream, (v2u*)cache, (const v2u*)source, (v2u*)dst, p);
    else if (vb == 4)
        hipLaunchKernelGGL((cache_kernel<uint32_t>), grid, dim3(BLOCK), 0, dev->stream, (uint32_t*)cache, (const uint32_t*)source, (uint32_t*)dst, p);
    else
        hipLaunchKernelGGL((cache_kernel<uint16_t>), grid, dim3(BLOCK), 0, dev->stream, (uint16_t*)cache, (const uint16_t*)source, (uint16_t*)dst, p);
    RT_CHECK_LAUNCH("cache_kernel");
    return RT_OK;
}

int rt_index_select(rt_device* dev, int elem_bytes, const void* src, const uint32_t src_shape[4], const int32_t* indices,
                    uint32_t n_indices, int dim, void* dst) {
    RT_REQUIRE(elem_bytes == 2 || elem_bytes == 4, RT_ERR_ARG, "rt_index_select: elem_bytes must be 2 or 4, got %d", elem_bytes);
    RT_REQUIRE(dim >= 0 && dim < 4, RT_ERR_ARG, "rt_index_select: dim %d out of range", dim);
    RT_REQUIRE(src_shape, RT_ERR_NULL_POINTER, "rt_index_select: NULL shape");
    RT_REQUIRE(n_indices > 0, RT_ERR_SHAPE, "rt_index_select: no indices");
    uint64_t left = 1, right = 1;
    for (int a = 0; a < 4; a++) {
        RT_REQUIRE(src_shape[a] > 0, RT_ERR_SHAPE, "rt_index_select: zero extent in dim %d", a);
        if (a < dim) left *= src_shape[a];
        if (a > dim) right *= src_shape[a];
    }
    RT_REQUIRE(left * src_shape[dim] * right <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_index_select: source too large");
    RT_REQUIRE(src && indices && dst, RT_ERR_NULL_POINTER, "rt_index_select: NULL operand");
    RT_REQUIRE(rt_aligned(src, (size_t)elem_bytes) && rt_aligned(dst, (size_t)elem_bytes) && rt_aligned(indices, 4), RT_ERR_ALIGN,
               "rt_index_select: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    const uint64_t run_b = right * elem_bytes;
    int vb = 16;
    for (; vb > elem_bytes; vb >>= 1)
        if (run_b % vb == 0 && rt_aligned(src, (size_t)vb) && rt_aligned(dst, (size_t)vb)) break;
    const uint64_t nvec = left * n_indices * (run_b / vb);
    RT_REQUIRE(nvec <= 0xffffffffull - BLOCK && left * n_indices <= 0xffffffffull && run_b / vb <= 0xffffffffull, RT_ERR_SIZE,
               "rt_index_select: output too large for 32-bit vector indices");
    SelectArgs p;
    p.rv = make_fastdiv((uint32_t)(run_b / vb));
    p.n_ids = make_fastdiv(n_indices);
    p.src_dim = src_shape[dim];
    p.nvec = (uint32_t)nvec;
    const dim3 grid(blocks_for(nvec, BLOCK)), block(BLOCK);
    if (vb == 16) hipLaunchKernelGGL((index_select_kernel<v4u>), grid, block, 0, dev->stream, (const v4u*)src, indices, (v4u*)dst, p);
    else if (vb == 8) hipLaunchKernelGGL((index_select_kernel<v2u>), grid, block, 0, dev->stream, (const v2u*)src, indices, (v2u*)dst, p);
    else if (vb == 4) hipLaunchKernelGGL((index_select_kernel<uint32_t>), grid, block, 0, dev->stream, (const uint32_t*)src, indices, (uint32_t*)dst, p);
    else hipLaunchKernelGGL((index_select_kernel<uint16_t>), grid, block, 0, dev->stream, (const uint16_t*)src, indices, (uint16_t*)dst, p);
    RT_CHECK_LAUNCH("index_select_kernel");
    return RT_OK;
}

int rt_index_select_q8_0(rt_device* dev, int scale_dt, const uint32_t* packed, const void* scales, const uint32_t src_shape[4],
                         const int32_t* indices, uint32_t n_indices, int dim, void* dst) {
    RT_REQUIRE(scale_dt == RT_F32 || scale_dt == RT_F16, RT_ERR_DTYPE, "rt_index_select_q8_0: scale dtype %d is not F32 (Q8_0F) / F16 (Q8_0H)",
               scale_dt);
    RT_REQUIRE(dim >= 0 && dim < 4, RT_ERR_ARG, "rt_index_select_q8_0: dim %d out of range", dim);
    RT_REQUIRE(src_shape, RT_ERR_NULL_POINTER, "rt_index_select_q8_0: NULL shape");
    RT_REQUIRE(n_indices > 0, RT_ERR_SHAPE, "rt_index_select_q8_0: no indices");
    uint64_t left = 1, right = 1;
    for (int a = 0; a < 4; a++) {
        RT_REQUIRE(src_shape[a] > 0, RT_ERR_SHAPE, "rt_index_select_q8_0: zero extent in dim %d", a);
        if (a < dim) left *= src_shape[a];
        if (a > dim) right *= src_shape[a];
    }
    const uint64_t numel = left * src_shape[dim] * right;
    RT_REQUIRE(numel <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_index_select_q8_0: source too large");
    // quantize_inner's own conditions (quant.rs:20-21) and the kernel's word granularity (ops/select.rs:144-161)
    RT_REQUIRE(numel % 32 == 0 && right % 4 == 0, RT_ERR_SHAPE,
               "rt_index_select_q8_0: %llu elements / runs of %llu: the source must be whole groups of 32 and the runs whole words of 4",
               (unsigned long long)numel, (unsigned long long)right);
    RT_REQUIRE(packed && scales && indices && dst, RT_ERR_NULL_POINTER, "rt_index_select_q8_0: NULL operand");
    const size_t ob = scale_dt == RT_F32 ? 16 : 8;
    RT_REQUIRE(rt_aligned(packed, 4) && rt_aligned(scales, (size_t)rt_dt_bytes(scale_dt)) && rt_aligned(indices, 4) && rt_aligned(dst, ob),
               RT_ERR_ALIGN, "rt_index_select_q8_0: misaligned pointer (the destination must be aligned to four elements)");
    int rc = rt_enter(dev);
    if (rc) return rc;
    const uint64_t nvec = left * n_indices * (right / 4);
    RT_REQUIRE(nvec <= 0xffffffffull - BLOCK && left * n_indices <= 0xffffffffull, RT_ERR_SIZE,
               "rt_index_select_q8_0: output too large for 32-bit word indices");
    SelectArgs p;
    p.rv = make_fastdiv((uint32_t)(right / 4));
    p.n_ids = make_fastdiv(n_indices);
    p.src_dim = src_shape[dim];
    p.nvec = (uint32_t)nvec;
    const dim3 grid(blocks_for(nvec, BLOCK)), block(BLOCK);
    if (scale_dt == RT_F32) hipLaunchKernelGGL((index_select_q8_kernel<float>), grid, block, 0, dev->stream, packed, (const float*)scales, indices, (float*)dst, p);
    else hipLaunchKernelGGL((index_select_q8_kernel<half_t>), grid, block, 0, dev->stream, packed, (const half_t*)scales, indices, (half_t*)dst, p);
    RT_CHECK_LAUNCH("index_select_q8_kernel");
    return RT_OK;
}

int rt_index_write(rt_device* dev, int elem_bytes, void* dst, const uint32_t dst_shape[4], const void* src, uint64_t src_numel,
                   const uint32_t write_start[4]) {
    RT_REQUIRE(elem_bytes == 2 || elem_bytes == 4, RT_ERR_ARG, "rt_index_write: elem_bytes must be 2 or 4, got %d", elem_bytes);
    RT_REQUIRE(dst_shape && write_start, RT_ERR_NULL_POINTER, "rt_index_write: NULL shape");
    uint64_t numel = 1, off = 0;
    for (int a = 0; a < 4; a++) {
        RT_REQUIRE(dst_shape[a] > 0, RT_ERR_SHAPE, "rt_index_write: zero extent in dim %d", a);
        RT_REQUIRE(write_start[a] < dst_shape[a], RT_ERR_SHAPE, "rt_index_write: write_start[%d] = %u outside extent %u", a, write_start[a],
                   dst_shape[a]);
        off = off * dst_shape[a] + write_start[a];
        numel *= dst_shape[a];
        RT_REQUIRE(numel <= RT_MAX_NUMEL, RT_ERR_SIZE, "rt_index_write: destination too large");
    }
    // the reference's kernel writes D[offset + i] for i < src_numel with no bound (ops/index_write.rs:96-104)
    RT_REQUIRE(src_numel <= numel && off + src_numel <= numel, RT_ERR_SHAPE, "rt_index_write: %llu elements from offset %llu leave the destination",
               (unsigned long long)src_numel, (unsigned long long)off);
    if (src_numel == 0) return dev ? RT_OK : rt_fail(RT_ERR_NULL_DEVICE, "rt_device is NULL");
    RT_REQUIRE(dst && src, RT_ERR_NULL_POINTER, "rt_index_write: NULL operand");
    RT_REQUIRE(rt_aligned(dst, (size_t)elem_bytes) && rt_aligned(src, (size_t)elem_bytes), RT_ERR_ALIGN, "rt_index_write: misaligned pointer");
    int rc = rt_enter(dev);
    if (rc) return rc;
    unsigned char* d = static_cast<unsigned char*>(dst) + off * elem_bytes;
    const uint64_t bytes = src_numel * elem_bytes;
    if (rt_aligned(d, 16) && rt_aligned(src, 16) && bytes % 16 == 0) {
        hipLaunchKernelGGL(index_write_vec_kernel, dim3(blocks_for(bytes / 16, BLOCK)), dim3(BLOCK), 0, dev->stream, (v4u*)d, (const v4u*)src,
                           bytes / 16);
    } else {
        hipLaunchKernelGGL(index_write_u16_kernel, dim3(blocks_for(bytes / 2, BLOCK)), dim3(BLOCK), 0, dev->stream, (uint16_t*)d,
                           (const uint16_t*)src, bytes / 2);
    }
    RT_CHECK_LAUNCH("index_write kernel");
    return RT_OK;
}

}  // extern "C"
