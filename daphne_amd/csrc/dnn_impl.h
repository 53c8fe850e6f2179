// DNN inference kernels for DenseMatrix<float|double> (one NCHW image per matrix row):
// Conv2D forward (im2col-free implicit GEMM on MFMA), MaxPool forward, BiasAdd, BatchNorm
// inference, Softmax. Instantiated per value type by dnn_f32.hip / dnn_f64.hip.
//
// Arithmetic follows the reference's CPU kernels (paths relative to
// src/runtime/local/kernels/): Conv2DForward.h:77-140, Pooling.cpp:28-107 + Pooling.h:33-58,
// BiasAdd.h:34-52, BatchNorm2DTestForward.h:77-101, Softmax.h:22-58; the entry points stand in
// for the CUDA wrappers in kernels/CUDA/{Convolution,Pooling,BiasAdd,BatchNorm,Softmax}.cpp.
//
// Conv2D as a GEMM without materialising im2col:
//     out_n[f][pixel] = sum_k W[f][k] * patch[k][pixel],   k = (c, h, w), pixel = (n, p, q)
// The filter matrix (F x K, K contiguous) is the row operand; the patch matrix is never built:
// each workgroup gathers its BK x BN slice from the NCHW input into LDS, with consecutive lanes
// on consecutive output pixels so that both the gather and the final store are contiguous along q.
// When the convolution has a border, the input is first copied into a workspace with the zeros
// written out: the gather then needs no bounds checks, and with a table k -> offset no divisions,
// which leaves one scalar add and one load per gathered element. Pixels of all images form one long N dimension, so a
// tile may span image boundaries and small images still fill the 128-pixel tile.
//
// Images of at least a few hundred output pixels take conv2d_resident_kernel instead: the padded image sits in LDS
// (in stages of channels when it is large), the border is written while it is copied in, and the waves contract
// over K without a barrier, gathering patch values straight from LDS.
#pragma once

#include "gemm_impl.h"

#include <limits>
#include <type_traits>

namespace dh_dnn {

using dh_gemm::Mfma;
using dh_gemm::relu_of;
using dh_gemm::TileLayout;
using dh_gemm::TileMover;

struct ConvArgs {
    const void *xpad;    // input with the zero border materialised: N x C x Hp x Wp
    const void *wpack;   // filter matrix padded with zeros to Fpad x Kpad
    const int *ktab;     // k = (c, hy, hx) -> c*Hp*Wp + hy*Wp + hx, Kpad entries (zero beyond K)
    const void *bias;
    void *res;
    unsigned F, K, Kpad, P, Q, sh, sw, Wp;
    unsigned CHpWp;      // elements of one padded image
    unsigned relu;       // 1: max(0, .) after the bias, as ewBinaryObjSca(MAX, ., 0) computes it
    unsigned Qo, PQo;    // POOL: width and size of the pooled output plane
    size_t pixels;       // N*P*Q; POOL: 4*N*PQo, the window positions of a pooled pixel being four consecutive "pixels"
};


// Table of patch offsets and the zero-padded filter matrix, so that the main loop has neither divisions
// nor bounds checks on the filter side.
template <typename T>
__global__ __launch_bounds__(256) void conv_prep_kernel(int *tab, T *wpack, const T *filter, unsigned F, unsigned Fpad,
                                                        unsigned K, unsigned Kpad, unsigned HpWp, unsigned Wp,
                                                        unsigned Hf, unsigned Wf, unsigned stage_channels = ~0u,
                                                        unsigned scale = 1, unsigned pixel_stride = 0) {
    // stage_channels: offsets count from the first channel of the LDS stage a channel belongs to (all channels in one
    // stage by default); scale: 1 for offsets in elements, sizeof(T) for offsets in bytes.
    // pixel_stride != 0: the LDS stage holds its channels interleaved - element (y, x, c) at (y Wp + x) pixel_stride + c -
    // and k runs through a stage's taps with the stage's channels innermost: k = stage KG + tap stage_channels + c
    // (the channel count is a multiple of stage_channels), so that consecutive k are consecutive addresses.
    const unsigned t = blockIdx.x * 256 + threadIdx.x, nt = gridDim.x * 256;
    const unsigned HfWf = Hf * Wf, KG = stage_channels * HfWf; // KG only used with pixel_stride != 0
    for (unsigned k = t; k < Kpad; k += nt) {
        int off = 0;
        if (k < K) {
            if (pixel_stride != 0) {
                const unsigned kk = k % KG, tap = kk / stage_channels, c = kk % stage_channels;
                off = static_cast<int>((((tap / Wf) * Wp + tap % Wf) * pixel_stride + c) * scale);
            } else {
                const unsigned c = k / HfWf, hw = k % HfWf;
                off = static_cast<int>(((c % stage_channels) * HpWp + (hw / Wf) * Wp + hw % Wf) * scale);
            }
        }
        tab[k] = off;
    }
    const size_t total = static_cast<size_t>(Fpad) * Kpad;
    for (size_t i = t; i < total; i += nt) {
        const unsigned f = static_cast<unsigned>(i / Kpad), k = static_cast<unsigned>(i % Kpad);
        unsigned src = k;
        if (pixel_stride != 0 && k < K) {
            const unsigned stage = k / KG, kk = k % KG;
            src = (stage * stage_channels + kk % stage_channels) * HfWf + kk / stage_channels;
        }
        wpack[i] = (f < F && k < K) ? filter[static_cast<size_t>(f) * K + src] : T(0);
    }
}

// Copies the images into a buffer with the zero border of Padding.h:11-22 written out, one thread per
// padded element (consecutive threads along a padded row).
template <typename T>
__global__ __launch_bounds__(256) void conv_pad_kernel(T *xpad, const T *x, size_t total, unsigned H, unsigned W,
                                                       unsigned Hp, unsigned Wp, unsigned ph, unsigned pw) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total)
        return;
    size_t plane;
    unsigned r;
    const unsigned HpWp = Hp * Wp;
    if (total <= 0xffffffffull) {
        plane = static_cast<unsigned>(i) / HpWp;
        r = static_cast<unsigned>(i) % HpWp;
    } else {
        plane = i / HpWp;
        r = static_cast<unsigned>(i % HpWp);
    }
    const unsigned y = r / Wp - ph, x_ = r % Wp - pw; // wraps to a huge value inside the border
    xpad[i] = (y < H && x_ < W) ? x[plane * H * W + static_cast<size_t>(y) * W + x_] : T(0);
}

// POOL: the 2 x 2 / stride 2 maximum of the (biased, optionally rectified) convolution as maxPoolForward computes it
// (running maximum from zero over the window in row order, Pooling.cpp:77-105). The tile's pixel index then counts
// window positions, four to a pooled pixel, so that a window's values sit in four neighbouring lanes at the end.
template <typename T, int BM, int BN, int BK, int WN, bool POOL = false>
__global__ __launch_bounds__(64 * WN) void conv2d_kernel(ConvArgs g) {
    using M = Mfma<T>;
    static_assert(!POOL || (M::NT % 4 == 0 && BN % 4 == 0), "a window's four positions stay in one block of pixels");
    constexpr int THREADS = 64 * WN;
    constexpr int TN = BN / WN;
    constexpr int FM = BM / M::MT, FN = TN / M::NT;
    static_assert(BM % M::MT == 0 && TN % M::NT == 0 && BK % M::KT == 0, "tile shape");
    static_assert(THREADS % BN == 0 && BK % (THREADS / BN) == 0 && BN % 64 == 0, "gather mapping");
    constexpr int VEC = 16 / sizeof(T);
    constexpr int KPL = BK / (64 / M::ROWS); // k values per lane and tile
    static_assert(KPL % VEC == 0, "fragment reads are whole 16-byte vectors");
    using LA = TileLayout<T, BM, BK, true>;  // filter tile [f][k]
    using LB = TileLayout<T, BN, BK, false>; // patch tile  [k][pixel]
    __shared__ __attribute__((aligned(16))) T lds_a[2][LA::ELEMS];
    __shared__ __attribute__((aligned(16))) T lds_b[2][LB::ELEMS];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const size_t pix0 = static_cast<size_t>(blockIdx.x) * BN;
    const unsigned f0 = blockIdx.y * BM;
    const unsigned PQ = POOL ? 4 * g.PQo : g.P * g.Q; // "pixels" per image
    const bool small = g.pixels <= 0xffffffffull; // 32-bit divisions suffice (uniform)

    // Gather mapping: thread -> one pixel of the tile and a group of KPT consecutive k. The k group is the
    // same for a whole wave (BN is a multiple of 64) and kept in a scalar register, so the table entries
    // come by scalar loads and every gather load is "uniform base + per-lane 32-bit offset".
    constexpr int KG = THREADS / BN;
    constexpr int KPT = BK / KG;
    const int gj = tid % BN, gkg = __builtin_amdgcn_readfirstlane(tid / BN);
    // pixels past the end repeat the last one; their results are dropped by the epilogue
    const size_t gpix = pix0 + gj < g.pixels ? pix0 + gj : g.pixels - 1;
    size_t img0;
    unsigned img, pq;
    if (small) {
        img0 = static_cast<unsigned>(pix0) / PQ;
        img = static_cast<unsigned>(gpix) / PQ;
        pq = static_cast<unsigned>(gpix) % PQ;
    } else {
        img0 = pix0 / PQ;
        img = static_cast<unsigned>(gpix / PQ);
        pq = static_cast<unsigned>(gpix % PQ);
    }
    unsigned p, q;
    if constexpr (POOL) {
        const unsigned po = pq / 4, wpos = pq % 4;
        p = 2 * (po / g.Qo) + wpos / 2;
        q = 2 * (po % g.Qo) + wpos % 2;
    } else {
        p = pq / g.Q;
        q = pq % g.Q;
    }
    const char *xblk = reinterpret_cast<const char *>(static_cast<const T *>(g.xpad) + img0 * g.CHpWp);
    // byte offset of this pixel's window origin from the block's first image (the host checks the range)
    const unsigned voff = static_cast<unsigned>(((img - static_cast<unsigned>(img0)) * g.CHpWp + p * g.sh * g.Wp + q * g.sw) *
                                                sizeof(T));
    const int *tab = g.ktab + gkg * KPT;

    // filter tile: whole 16-byte vectors of the padded matrix
    constexpr int VPR = BK / VEC, NVEC = BM * VPR, APT = (NVEC + THREADS - 1) / THREADS;
    const T *wrow[APT];
    int a_lds[APT];
#pragma unroll
    for (int i = 0; i < APT; i++) {
        const int v = tid + i * THREADS;
        const int o = (v / VPR) % BM, iv = v % VPR;
        wrow[i] = static_cast<const T *>(g.wpack) + static_cast<size_t>(f0 + o) * g.Kpad + iv * VEC;
        a_lds[i] = LA::at(o, iv * VEC);
    }

    T ga[APT][VEC], gb[KPT];
    auto fetch = [&](unsigned k0) {
#pragma unroll
        for (int i = 0; i < APT; i++)
            if ((NVEC % THREADS == 0) || (tid + i * THREADS < NVEC))
                dh_load_vec<T, VEC>(wrow[i] + k0, ga[i]);
        int off[KPT];
#pragma unroll
        for (int i = 0; i < KPT; i++)
            off[i] = tab[k0 + i];
        if (k0 + BK <= g.K) {
#pragma unroll
            for (int i = 0; i < KPT; i++)
                gb[i] = *reinterpret_cast<const T *>(xblk + static_cast<ptrdiff_t>(off[i]) * static_cast<ptrdiff_t>(sizeof(T)) + voff);
        } else {
            // last tile: k beyond K contributes nothing, whatever the image holds there
#pragma unroll
            for (int i = 0; i < KPT; i++) {
                const T v = *reinterpret_cast<const T *>(xblk + static_cast<ptrdiff_t>(off[i]) * static_cast<ptrdiff_t>(sizeof(T)) + voff);
                gb[i] = (k0 + gkg * KPT + i < g.K) ? v : T(0);
            }
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < APT; i++)
            if ((NVEC % THREADS == 0) || (tid + i * THREADS < NVEC))
                dh_store_vec<T, VEC>(lds_a[buf] + a_lds[i], ga[i]);
#pragma unroll
        for (int i = 0; i < KPT; i++)
            lds_b[buf][LB::at(gj, gkg * KPT + i)] = gb[i];
    };

    typename M::acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
            acc[i][j] = M::zero();

    const int frag_row = lane % M::ROWS, frag_k = lane / M::ROWS;
    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (unsigned k0 = 0; k0 < g.K; k0 += BK) {
        const bool more = k0 + BK < g.K;
        if (more)
            fetch(k0 + BK);
        const T *la = lds_a[buf];
        const T *lb = lds_b[buf];
        // The k index an MFMA step assigns to a lane group is free as long as both operands agree:
        // lane group h takes the KPL consecutive values k = h*KPL .. h*KPL+KPL-1 of the tile, one per
        // step, so the filter fragment (contiguous along k in LDS) is read with 16-byte loads.
        T fa[FM][KPL], fb[FN][KPL];
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int v = 0; v < KPL; v += VEC) {
                T t[VEC];
                dh_load_vec<T, VEC>(la + LA::at(i * M::MT + frag_row, frag_k * KPL + v), t);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    fa[i][v + e] = t[e];
            }
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int s_ = 0; s_ < KPL; s_++)
                fb[j][s_] = lb[LB::at(wave * TN + j * M::NT + frag_row, frag_k * KPL + s_)];
#pragma unroll
        for (int s_ = 0; s_ < KPL; s_++)
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++)
                    acc[i][j] = M::mma(fa[i][s_], fb[j][s_], acc[i][j]);
        if (more)
            stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    // out[img][f][pq]: lanes along pixels -> contiguous stores
    T *out = static_cast<T *>(g.res);
    const T *bias = static_cast<const T *>(g.bias);
    // this lane's bias values first: loaded inside the store loop, every one of them would wait behind the
    // previous store (the compiler cannot rule out that res and bias overlap)
    T bv[FM][M::ACC];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int v = 0; v < M::ACC; v++) {
            const size_t f = f0 + i * M::MT + M::row(lane, v);
            bv[i][v] = (bias && f < g.F) ? bias[f] : T(0);
        }
#pragma unroll
    for (int j = 0; j < FN; j++) {
        const size_t pix = pix0 + wave * TN + j * M::NT + M::col(lane);
        const bool live = pix < g.pixels; // POOL: the same for the four lanes of a window
        size_t oimg, opq;
        if (small) {
            oimg = static_cast<unsigned>(live ? pix : 0) / PQ;
            opq = static_cast<unsigned>(live ? pix : 0) % PQ;
        } else {
            oimg = (live ? pix : 0) / PQ;
            opq = (live ? pix : 0) % PQ;
        }
        if constexpr (POOL) {
            T *obase = out + oimg * g.F * g.PQo + opq / 4;
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int v = 0; v < M::ACC; v++) {
                    const size_t f = f0 + i * M::MT + M::row(lane, v);
                    T o = acc[i][j][v] + bv[i][v];
                    o = g.relu ? relu_of(o) : o;
                    // the window's values in row order, from the four lanes of the quad
                    const T w0 = dh_dpp<0x00>(o), w1 = dh_dpp<0x55>(o), w2 = dh_dpp<0xAA>(o), w3 = dh_dpp<0xFF>(o);
                    T m = T(0);
                    m = (m < w0) ? w0 : m;
                    m = (m < w1) ? w1 : m;
                    m = (m < w2) ? w2 : m;
                    m = (m < w3) ? w3 : m;
                    if (live && lane % 4 == 0 && f < g.F)
                        obase[f * g.PQo] = m;
                }
        } else if (live) {
            T *obase = out + oimg * g.F * PQ + opq;
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int v = 0; v < M::ACC; v++) {
                    const size_t f = f0 + i * M::MT + M::row(lane, v);
                    if (f < g.F) {
                        const T o = acc[i][j][v] + bv[i][v];
                        obase[f * PQ] = g.relu ? relu_of(o) : o;
                    }
                }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Convolution with the image resident in LDS. One workgroup of 8 waves takes one image (all of its channels,
// with the zero border written out while it is copied in), 16 * MFW filters and up to `chunk` output pixels, and
// runs the whole K = C * Hf * Wf contraction without a barrier: every wave owns one block of 16 filters and NF
// blocks of 16 pixels as accumulators of the 16x16x4 matrix instruction, reads its filter fragment from the
// padded filter matrix in global memory (a 16-byte vector per lane, one block of K ahead) and gathers the
// patch fragment straight from the LDS image at "pixel offset + table[k]".
// ---------------------------------------------------------------------------------------
struct ConvResidentArgs {
    const void *x;     // N x C x H x W
    const void *wpack; // filter matrix padded with zeros to Fpad x Kpad
    const int *ktab;   // k -> byte offset of tap (c, hy, hx) from the start of its channel stage in LDS (0 beyond K)
    const void *bias;
    void *res;
    unsigned C, H, W, Hp, Wp, ph, pw, Q, sh, sw, F, Kpad, HpWp, PQ, chunk;
    unsigned CG, KG;   // channels per stage of the LDS image and their share of K (a multiple of the K block)
    unsigned N, NI;    // images in all, images per workgroup (their pixels form one pixel range)
    unsigned relu;     // 1: max(0, .) after the bias
    unsigned Qo, PQo;  // POOL: width and size of the pooled output plane (PQ, Q stay those of the convolution)
    unsigned lds_bias; // byte offset of the workgroup's bias values in LDS (behind the image stage)
};

// Copies one image (C x H x W at x) into LDS as C x Hp x Wp with the zero border of Padding.h:11-22 written out,
// by the nt threads of a workgroup. A thread keeps its position(s) inside the padded plane and walks the
// channels, so the divisions are done once; planes of fewer than nt elements are taken by several groups of
// threads side by side.
template <typename T, int UN>
__device__ __forceinline__ void conv_stage_frame(T *frame, const T *x, unsigned C, unsigned H, unsigned W, unsigned Wp,
                                                 unsigned ph, unsigned pw, unsigned HpWp, unsigned frame_elems, int tid,
                                                 unsigned nt) {
    constexpr int VEC = 16 / sizeof(T);
    const unsigned HW = H * W;
    if (ph == 0 && pw == 0 && frame_elems % VEC == 0 && reinterpret_cast<size_t>(x) % 16 == 0) {
        // no border: the frame is the image, copied with 16-byte vectors, four loads of a thread in flight at once
        constexpr int UV = 4;
        const unsigned nvec = frame_elems / VEC;
        for (unsigned v0 = tid; v0 < nvec; v0 += nt * UV) {
            T t[UV][VEC];
#pragma unroll
            for (int u = 0; u < UV; u++) {
                const unsigned v = v0 + u * nt;
                dh_load_vec_stream<T, VEC>(x + static_cast<size_t>(v < nvec ? v : v0) * VEC, t[u]);
            }
#pragma unroll
            for (int u = 0; u < UV; u++)
                if (v0 + u * nt < nvec)
                    dh_store_vec<T, VEC>(frame + static_cast<size_t>(v0 + u * nt) * VEC, t[u]);
        }
        return;
    }
    const bool narrow = HpWp < nt;
    const unsigned groups = narrow ? nt / HpWp : 1;
    const unsigned grp = narrow ? tid / HpWp : 0;
    if (grp >= groups)
        return;
    for (unsigned r = narrow ? tid % HpWp : tid; r < HpWp; r += nt) {
        const unsigned y = r / Wp - ph, xx = r % Wp - pw; // wraps to a huge value inside the border
        const bool in = y < H && xx < W;
        const unsigned src = in ? y * W + xx : 0; // 32-bit offsets from the image: one register per load in flight
        T *dst = frame + r;
        // batches of UN channels: all loads of a batch are issued (unconditionally, from clamped addresses) before
        // the first value is stored; lanes on the border load the image's first element and store zeros
        for (unsigned c0 = grp; c0 < C; c0 += groups * UN) {
            T v[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const unsigned c = c0 + u * groups;
                v[u] = __builtin_nontemporal_load(x + (src + (c < C ? c : c0) * HW));
            }
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const unsigned c = c0 + u * groups;
                if (c < C)
                    dst[c * HpWp] = in ? v[u] : T(0);
            }
        }
    }
}

// The same with the channels interleaved: element (y, x, c) of the padded image at (y Wp + x) PS + c, PS = C + one
// vector. A thread takes VEC consecutive channels of one position: its loads are coalesced per channel plane
// (consecutive lanes, consecutive positions) and its one vector store lands PS elements from its neighbour's - with the
// odd vector of padding in PS, the 16 lanes that LDS serves together reach all banks.
template <typename T, int UB>
__device__ __forceinline__ void conv_stage_frame_interleaved(T *frame, const T *x, unsigned C, unsigned H, unsigned W, unsigned Wp,
                                                             unsigned ph, unsigned pw, unsigned HpWp, unsigned PS, int tid,
                                                             unsigned nt) {
    constexpr int VEC = 16 / sizeof(T);
    const unsigned HW = H * W, total = HpWp * (C / VEC);
    for (unsigned e0 = tid; e0 < total; e0 += nt * UB) {
        T v[UB][VEC];
        unsigned dst[UB];
        bool in[UB];
#pragma unroll
        for (int u = 0; u < UB; u++) {
            const unsigned e = e0 + u * nt < total ? e0 + u * nt : e0;
            const unsigned cv = e / HpWp, r = e % HpWp;
            const unsigned y = r / Wp - ph, xx = r % Wp - pw; // wraps to a huge value inside the border
            in[u] = y < H && xx < W;
            const unsigned src = (in[u] ? y * W + xx : 0) + cv * VEC * HW;
            dst[u] = r * PS + cv * VEC;
#pragma unroll
            for (int q = 0; q < VEC; q++)
                v[u][q] = __builtin_nontemporal_load(x + (src + q * HW));
        }
#pragma unroll
        for (int u = 0; u < UB; u++) {
            if (e0 + u * nt < total) {
                if (!in[u]) {
#pragma unroll
                    for (int q = 0; q < VEC; q++)
                        v[u][q] = T(0);
                }
                dh_store_vec<T, VEC>(frame + dst[u], v[u]);
            }
        }
    }
}

// POOL: the result is the 2 x 2 / stride 2 maximum of the (biased, optionally rectified) convolution, as maxPoolForward
// computes it (running maximum from zero over the window in row order, Pooling.cpp:77-105). The pixel index that
// workgroups and waves divide among themselves then counts window positions, four to a pooled pixel, so that a
// window's values end up in four neighbouring lanes.
// CI: the LDS image holds its channels interleaved (conv_stage_frame_interleaved; the stage's channel count is a
// multiple of 4 VEC, and k runs taps-outer / channels-inner, see conv_prep_kernel): the VEC values of k that a lane
// feeds into VEC consecutive matrix instructions are consecutive channels at one tap, one 16-byte LDS read.
template <typename T, int MFW, int NF, bool POOL, bool CI = false>
__global__ __launch_bounds__(512, (CI && NF <= 7 && sizeof(T) == 4) ? 4 : 1) void conv2d_resident_kernel(ConvResidentArgs g) {
    using M = dh_gemm::Mfma16<T>;
    constexpr int VEC = 16 / sizeof(T), NPARTS = 8 / MFW;
    extern __shared__ __attribute__((aligned(16))) unsigned char conv_lds[];
    int *ktab = reinterpret_cast<int *>(conv_lds);               // Kpad entries: a multiple of 16 bytes
    T *frame = reinterpret_cast<T *>(conv_lds + g.Kpad * sizeof(int));
    T *bias_l = reinterpret_cast<T *>(conv_lds + g.lds_bias); // the workgroup's 16 MFW bias values, behind the image
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const unsigned img = blockIdx.x * g.NI, f0 = blockIdx.y * (16 * MFW), px0 = blockIdx.z * g.chunk;
    const unsigned nimg = (g.N - img < g.NI) ? g.N - img : g.NI; // images of this workgroup
    const unsigned PQv = POOL ? 4 * g.PQo : g.PQ, PQout = POOL ? g.PQo : g.PQ; // "pixels" and results per image
    const unsigned PS = CI ? g.CG + VEC : 1;                     // CI: elements from a position to the next
    const unsigned npix = nimg * PQv, stage_elems = CI ? g.HpWp * PS : g.CG * g.HpWp;

    // the offset table: its first 2048 entries are asked for now and put into LDS after the first image stage has
    // been copied in, so that both sets of loads are on their way together
    constexpr int KTR = 4;
    int ktreg[KTR];
#pragma unroll
    for (int i = 0; i < KTR; i++) {
        const unsigned k = tid + i * 512;
        ktreg[i] = g.ktab[k < g.Kpad ? k : 0];
    }

    const int mf = wave % MFW, part = wave / MFW;
    const int li = lane % 16, lk = lane / 16;
    // this lane's pixel in each of the wave's pixel blocks; blocks past the image end are skipped (uniform)
    int pixoff[NF], outoff[NF];
    int nfv = 0;
#pragma unroll
    for (int j = 0; j < NF; j++) {
        const unsigned first = px0 + (j * NPARTS + part) * 16; // blocks dealt round-robin: the waves' counts differ by at most one
        const unsigned px = first + li;
        const bool ok = px < npix; // POOL: the same for the four lanes of a window
        const unsigned il = ok ? px / PQv : 0, pq = ok ? px % PQv : 0; // image of the workgroup, pixel in it
        unsigned pp, qq, po = pq;
        if constexpr (POOL) {
            po = pq / 4;
            pp = 2 * (po / g.Qo) + (pq % 4) / 2;
            qq = 2 * (po % g.Qo) + (pq % 4) % 2;
        } else {
            pp = pq / g.Q;
            qq = pq % g.Q;
        }
        pixoff[j] = static_cast<int>(il * stage_elems + (pp * g.sh * g.Wp + qq * g.sw) * PS);
        outoff[j] = ok ? static_cast<int>(il * g.F * PQout + po) : -1;
        if (first < npix)
            nfv = j + 1;
    }
    typename M::acc_t acc[NF];
#pragma unroll
    for (int j = 0; j < NF; j++)
        acc[j] = typename M::acc_t{0, 0, 0, 0};

    const T *wrow = static_cast<const T *>(g.wpack) + static_cast<size_t>(f0 + mf * 16 + li) * g.Kpad + lk * VEC;
    const int *ktl = ktab + lk * VEC; // byte offsets from the start of a channel's stage (conv_prep_kernel)
    const char *frame_b = reinterpret_cast<const char *>(frame);
#pragma unroll
    for (int j = 0; j < NF; j++)
        pixoff[j] *= static_cast<int>(sizeof(T));
    // The contraction, for a number of pixel blocks fixed at compile time: no branch inside the loop body. A wave
    // with fewer blocks than NF - 1 computes all NF (the spare ones gather pixel 0 and are never stored).
    // Every ordinary vector instruction and every LDS read that a SIMD issues takes about one pass out of its matrix
    // pipe (a 16x16x4 instruction is 8 passes), so the loop is written to issue as few as it can beside the matrix
    // instructions: per instruction one gather and one address add. The table holds ready byte offsets; the patch
    // values alternate between two register sets from step to step and the filter values / table entries between
    // two sets from block to block (both counts are even), so that nothing is copied from register to register.
    // One block = 4 * VEC values of k = VEC steps: (a_c, kt_c) are the block's filter values and table entries, those
    // of the block after it are fetched into (a_n, kt_n).
    auto kblock = [&](auto nv_tag, T(&a_c)[VEC], int(&kt_c)[VEC], T(&a_n)[VEC], int(&kt_n)[VEC], T(&b_even)[NF], T(&b_odd)[NF],
                      unsigned kn) {
        constexpr int NV = decltype(nv_tag)::value;
        static_assert(VEC % 2 == 0, "the two sets of patch registers alternate from step to step");
        dh_load_vec<T, VEC>(wrow + kn, a_n);
#pragma unroll
        for (int s_ = 0; s_ < VEC; s_++)
            kt_n[s_] = ktl[kn + s_];
#pragma unroll
        for (int s_ = 0; s_ < VEC; s_++) {
            // the patch values of the following step are on their way while this step's matrix instructions run
            const int kt_after = (s_ + 1 < VEC) ? kt_c[s_ + 1] : kt_n[0];
            __builtin_amdgcn_sched_barrier(0); // a gather must not sink to its use in the next step
            if (s_ % 2 == 0) {
#pragma unroll
                for (int j = 0; j < NV; j++)
                    b_odd[j] = *reinterpret_cast<const T *>(frame_b + (pixoff[j] + kt_after));
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < NV; j++)
                    acc[j] = M::mma(a_c[s_], b_even[j], acc[j]);
            } else {
#pragma unroll
                for (int j = 0; j < NV; j++)
                    b_even[j] = *reinterpret_cast<const T *>(frame_b + (pixoff[j] + kt_after));
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < NV; j++)
                    acc[j] = M::mma(a_c[s_], b_odd[j], acc[j]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // k_begin .. k_end: this stage's share of K; its blocks are taken two to a turn of the loop, a last odd one alone
    auto contract = [&](auto nv_tag, unsigned k_begin, unsigned k_end) {
        constexpr int NV = decltype(nv_tag)::value;
        constexpr unsigned KB = 4 * VEC;
        T a0[VEC], a1[VEC], b_even[NF], b_odd[NF];
        int kt0[VEC], kt1[VEC];
        dh_load_vec<T, VEC>(wrow + k_begin, a0);
#pragma unroll
        for (int s_ = 0; s_ < VEC; s_++)
            kt0[s_] = ktl[k_begin + s_];
#pragma unroll
        for (int j = 0; j < NV; j++)
            b_even[j] = *reinterpret_cast<const T *>(frame_b + (pixoff[j] + kt0[0]));
        unsigned k0 = k_begin;
        for (; k0 + 2 * KB <= k_end; k0 += 2 * KB) {
            // the block after the second one of this turn (the stage's last turn fetches a block of its own again)
            const unsigned kn = (k0 + 2 * KB < k_end) ? k0 + 2 * KB : k0;
            kblock(nv_tag, a0, kt0, a1, kt1, b_even, b_odd, k0 + KB);
            kblock(nv_tag, a1, kt1, a0, kt0, b_even, b_odd, kn);
        }
        if (k0 < k_end)
            kblock(nv_tag, a0, kt0, a1, kt1, b_even, b_odd, k0);
    };
    // CI: a block's patch values are one vector read per pixel block, asked for right after the matrix instructions
    // that used the previous block's vector in the same registers: per VEC matrix instructions one read and one
    // address addition (measured on a loop of nothing else: 87 % of the pipe's peak against 78 % with a 4-byte read
    // and an addition per instruction).
    typedef T patch_t __attribute__((ext_vector_type(VEC)));
    auto contract_ci = [&](auto nv_tag, unsigned k_begin, unsigned k_end) {
        constexpr int NV = decltype(nv_tag)::value;
        constexpr unsigned KB = 4 * VEC;
        T a0[VEC], a1[VEC];
        patch_t b[NF];
        dh_load_vec<T, VEC>(wrow + k_begin, a0);
        {
            const int kt = ktl[k_begin];
#pragma unroll
            for (int j = 0; j < NV; j++)
                b[j] = *reinterpret_cast<const patch_t *>(frame_b + (pixoff[j] + kt));
        }
        auto block = [&](T(&a_c)[VEC], T(&a_n)[VEC], unsigned kn) {
            dh_load_vec<T, VEC>(wrow + kn, a_n);
            const int kt_n = ktl[kn];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NV; j++) {
#pragma unroll
                for (int s_ = 0; s_ < VEC; s_++)
                    acc[j] = M::mma(a_c[s_], b[j][s_], acc[j]);
                __builtin_amdgcn_sched_barrier(0);
                b[j] = *reinterpret_cast<const patch_t *>(frame_b + (pixoff[j] + kt_n));
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        unsigned k0 = k_begin;
        for (; k0 + 2 * KB <= k_end; k0 += 2 * KB) {
            const unsigned kn = (k0 + 2 * KB < k_end) ? k0 + 2 * KB : k0; // the last turn fetches a block of its own again
            block(a0, a1, k0 + KB);
            block(a1, a0, kn);
        }
        if (k0 < k_end)
            block(a0, a1, k0);
    };
    // The image goes through LDS in stages of CG channels (all of them when they fit); the accumulators stay.
    const T *ximg = static_cast<const T *>(g.x) + static_cast<size_t>(img) * g.C * g.H * g.W;
    for (unsigned c0 = 0, k_begin = 0; c0 < g.C; c0 += g.CG, k_begin += g.KG) {
        const unsigned cg = (g.C - c0 < g.CG) ? g.C - c0 : g.CG;
        const unsigned k_end = (c0 + g.CG < g.C) ? k_begin + g.KG : g.Kpad;
        if (c0)
            __syncthreads(); // every wave is done with the previous stage
        for (unsigned il = 0; il < nimg; il++) {
            const T *xs = ximg + (static_cast<size_t>(il) * g.C + c0) * g.H * g.W;
            if constexpr (CI)
                conv_stage_frame_interleaved<T, 6>(frame + il * stage_elems, xs, cg, g.H, g.W, g.Wp, g.ph, g.pw, g.HpWp, PS, tid, 512);
            else
                conv_stage_frame<T, 8>(frame + il * stage_elems, xs, cg, g.H, g.W, g.Wp, g.ph, g.pw, g.HpWp, cg * g.HpWp, tid, 512);
        }
        if (c0 == 0) {
#pragma unroll
            for (int i = 0; i < KTR; i++)
                if (static_cast<unsigned>(tid + i * 512) < g.Kpad)
                    ktab[tid + i * 512] = ktreg[i];
            for (unsigned k = tid + KTR * 512; k < g.Kpad; k += 512)
                ktab[k] = g.ktab[k];
            // the bias comes in with the image: the epilogue, which a wave reaches with nothing else to do, then waits
            // for an LDS read instead of a trip to memory
            if (tid < 16 * MFW) {
                const T *bias = static_cast<const T *>(g.bias);
                bias_l[tid] = (bias && f0 + tid < g.F) ? bias[f0 + tid] : T(0);
            }
        }
        __syncthreads();
        if constexpr (CI) {
            if (nfv == NF - 1)
                contract_ci(std::integral_constant<int, NF - 1>{}, k_begin, k_end);
            else if (nfv > 0)
                contract_ci(std::integral_constant<int, NF>{}, k_begin, k_end);
        } else {
            if (nfv == NF - 1)
                contract(std::integral_constant<int, NF - 1>{}, k_begin, k_end);
            else if (nfv > 0)
                contract(std::integral_constant<int, NF>{}, k_begin, k_end);
        }
    }

    T *out = static_cast<T *>(g.res) + static_cast<size_t>(img) * g.F * PQout;
    T bv[4];
#pragma unroll
    for (int v = 0; v < 4; v++)
        bv[v] = bias_l[mf * 16 + M::row(lane, v)];
    if constexpr (POOL) {
#pragma unroll
        for (int j = 0; j < NF; j++) {
            if (j < nfv) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const unsigned f = f0 + mf * 16 + M::row(lane, v);
                    T o = acc[j][v] + bv[v];
                    o = g.relu ? relu_of(o) : o;
                    // the window's values in row order, from the four lanes of the quad
                    const T w0 = dh_dpp<0x00>(o), w1 = dh_dpp<0x55>(o), w2 = dh_dpp<0xAA>(o), w3 = dh_dpp<0xFF>(o);
                    T m = T(0);
                    m = (m < w0) ? w0 : m;
                    m = (m < w1) ? w1 : m;
                    m = (m < w2) ? w2 : m;
                    m = (m < w3) ? w3 : m;
                    if (outoff[j] >= 0 && lane % 4 == 0 && f < g.F)
                        out[static_cast<size_t>(f) * PQout + outoff[j]] = m;
                }
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < NF; j++) {
            if (j < nfv && outoff[j] >= 0) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const unsigned f = f0 + mf * 16 + M::row(lane, v);
                    if (f < g.F) {
                        const T o = acc[j][v] + bv[v];
                        out[static_cast<size_t>(f) * g.PQ + outoff[j]] = g.relu ? relu_of(o) : o;
                    }
                }
            }
        }
    }
}

template <typename T, int MFW, int NF, bool POOL = false, bool CI = false>
static inline dh_status conv2d_resident_launch(dh_ctx *ctx, const ConvResidentArgs &g, dim3 grid, size_t lds) {
    // dynamic LDS beyond 64 KiB has to be asked for, per kernel and device (the call is cheap next to the kernel)
    if (lds > 65536) {
        DH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&conv2d_resident_kernel<T, MFW, NF, POOL, CI>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    }
    hipLaunchKernelGGL((conv2d_resident_kernel<T, MFW, NF, POOL, CI>), grid, dim3(512), lds, ctx->stream, g);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// One input channel, a filter of 3 x 3 or 5 x 5, stride 1 (the first layer of a CNN on grey images): K = Hf Wf is too
// short for the matrix cores to pay - what such a layer costs is the store of F planes per image. Here a thread takes
// a 2 x 2 quad of output pixels: the (Hf + 1) x (Wf + 1) patch under it sits in registers, the weights are the same
// for all lanes (scalar loads into scalar registers, the multiply-add takes them from there), and consecutive threads
// own consecutive quads, so that each filter's results leave as whole runs of a plane - pooled (POOL: one value per
// quad, the running maximum from zero over the window in row order, Pooling.cpp:77-105) or as the four pixels.
// A result is bias + the chain fma(w[k], x[k], .) over k = hy Wf + hx from zero, the same for every epilogue.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float dh_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double dh_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }

struct ConvDirectArgs {
    unsigned N, H, W, ph, pw, P2, Q2, F; // P2, Q2: quads down and across (P / 2, Q / 2)
    unsigned relu;
    size_t quads;                        // N * P2 * Q2
};

template <typename T, int HF, int WF, bool POOL>
__global__ __launch_bounds__(256) void conv2d_direct_kernel(const T *__restrict__ xin, const T *__restrict__ w,
                                                            const T *__restrict__ bias, T *__restrict__ res, ConvDirectArgs g) {
    // (the pointers are parameters of their own and do not alias: only then do the weights take the scalar path)
    constexpr int FB = 4; // filters at a time: 16 accumulators beside the patch
    const size_t quad = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (quad >= g.quads)
        return;
    const unsigned per_img = g.P2 * g.Q2;
    const unsigned n = static_cast<unsigned>(quad / per_img), pq = static_cast<unsigned>(quad % per_img);
    const unsigned p2 = pq / g.Q2, q2 = pq % g.Q2;
    const T *img = xin + static_cast<size_t>(n) * g.H * g.W;
    T x[HF + 1][WF + 1];
#pragma unroll
    for (int a = 0; a < HF + 1; a++)
#pragma unroll
        for (int b = 0; b < WF + 1; b++) {
            const unsigned y = 2 * p2 + a - g.ph, xx = 2 * q2 + b - g.pw; // wraps to a huge value inside the border
            const bool in = y < g.H && xx < g.W;
            const T v = img[in ? y * g.W + xx : 0];
            x[a][b] = in ? v : T(0);
        }
    const unsigned P = 2 * g.P2, Q = 2 * g.Q2;
    T *out = res + static_cast<size_t>(n) * g.F * (POOL ? per_img : P * Q);
    for (unsigned f0 = 0; f0 < g.F; f0 += FB) {
        T acc[FB][4];
#pragma unroll
        for (int j = 0; j < FB; j++) {
            const T *wf = w + static_cast<size_t>(f0 + j < g.F ? f0 + j : f0) * (HF * WF); // the same address in all lanes
            acc[j][0] = acc[j][1] = acc[j][2] = acc[j][3] = T(0);
#pragma unroll
            for (int hy = 0; hy < HF; hy++)
#pragma unroll
                for (int hx = 0; hx < WF; hx++) {
                    const T wk = wf[hy * WF + hx];
                    acc[j][0] = dh_fma(wk, x[hy][hx], acc[j][0]);
                    acc[j][1] = dh_fma(wk, x[hy][hx + 1], acc[j][1]);
                    acc[j][2] = dh_fma(wk, x[hy + 1][hx], acc[j][2]);
                    acc[j][3] = dh_fma(wk, x[hy + 1][hx + 1], acc[j][3]);
                }
        }
#pragma unroll
        for (int j = 0; j < FB; j++) {
            const unsigned f = f0 + j;
            if (f < g.F) {
                const T bv = bias ? bias[f] : T(0);
                T o[4];
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    o[v] = acc[j][v] + bv;
                    // (a running maximum that starts from zero gives the same bits with and without the rectifier
                    // before it: negative values, zeros of either sign and NaNs never replace the maximum)
                    if constexpr (!POOL)
                        o[v] = g.relu ? relu_of(o[v]) : o[v];
                }
                if constexpr (POOL) {
                    T m = T(0);
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        m = (m < o[v]) ? o[v] : m;
                    out[static_cast<size_t>(f) * per_img + pq] = m;
                } else {
                    T *plane = out + static_cast<size_t>(f) * P * Q + (2 * p2) * Q + 2 * q2;
                    plane[0] = o[0];
                    plane[1] = o[1];
                    plane[Q] = o[2];
                    plane[Q + 1] = o[3];
                }
            }
        }
    }
}

template <typename T>
dh_status maxpool_forward(dh_ctx *ctx, T *res, size_t *res_h, size_t *res_w, const T *data, size_t N, size_t C,
                          size_t H, size_t W, size_t ph, size_t pw, size_t sh, size_t sw, size_t padh, size_t padw);

// epilogue: DH_EPILOGUE_RELU and / or DH_EPILOGUE_MAXPOOL_2X2, applied to the biased convolution in that order; the
// results are those of the separate operators (conv2dForward, ewBinaryObjSca(MAX, ., 0), maxPoolForward 2 x 2 / 2),
// bit for bit. With pooling, res is N x F * (P / 2) * (Q / 2) and res_h / res_w are the pooled extents.
template <typename T>
dh_status conv2d_forward(dh_ctx *ctx, T *res, size_t *res_h, size_t *res_w, const T *data, const T *filter,
                         size_t filter_rows, size_t filter_cols, const T *bias, size_t N, size_t C, size_t H,
                         size_t W, size_t Hf, size_t Wf, size_t sh, size_t sw, size_t ph, size_t pw,
                         unsigned epilogue = 0) {
    DH_REQUIRE_CTX(ctx);
    if (epilogue & ~(DH_EPILOGUE_RELU | DH_EPILOGUE_MAXPOOL_2X2))
        return dh_fail(DH_ERR_INVALID_ARG, "Convolution: unknown epilogue flags %#x", epilogue);
    const bool relu = (epilogue & DH_EPILOGUE_RELU) != 0, pool = (epilogue & DH_EPILOGUE_MAXPOOL_2X2) != 0;
    const size_t F = filter_rows;
    if (filter_rows * filter_cols != F * C * Hf * Wf)
        // kernels/CUDA/Convolution.cpp:32-39
        return dh_fail(DH_ERR_INVALID_ARG,
                       "Convolution kernel dimension mismatch: expected %zu elements [%zux%zux%zux%zu] but got %zu.",
                       F * C * Hf * Wf, F, C, Hf, Wf, filter_rows * filter_cols);
    if (sh == 0 || sw == 0 || H + 2 * ph < Hf || W + 2 * pw < Wf)
        return dh_fail(DH_ERR_INVALID_ARG, "Convolution: filter %zux%zu does not fit the padded image %zux%zu",
                       Hf, Wf, H + 2 * ph, W + 2 * pw);
    const size_t P = (H + 2 * ph - Hf) / sh + 1, Q = (W + 2 * pw - Wf) / sw + 1; // Padding.h:6-9
    if (pool && (P < 2 || Q < 2))
        return dh_fail(DH_ERR_INVALID_ARG, "Pooling: window 2x2 does not fit the padded image %zux%zu", P, Q);
    const size_t Po = pool ? (P - 2) / 2 + 1 : P, Qo = pool ? (Q - 2) / 2 + 1 : Q; // Pooling.cpp:38-39
    if (res_h)
        *res_h = Po;
    if (res_w)
        *res_w = Qo;
    const size_t pixels = N * P * Q;
    if (pixels == 0 || F == 0)
        return DH_OK;
    // One channel, 3 x 3 or 5 x 5, stride 1, even output extents: a thread per 2 x 2 quad of output pixels on the ordinary
    // ALUs (1 -> 32 channels, 5 x 5 on 28 x 28, batch 4096, with ReLU and pooling: 0.153 ms in the tiled kernel below).
    // As everywhere in this function the choice does not look at the epilogue.
    if (C == 1 && sh == 1 && sw == 1 && Hf == Wf && (Hf == 3 || Hf == 5) && P % 2 == 0 && Q % 2 == 0 && N < (size_t(1) << 31) &&
        H * W < (size_t(1) << 31) && F < (size_t(1) << 31) && N * (P / 2) * (Q / 2) < (size_t(1) << 39)) {
        ConvDirectArgs d{};
        d.N = static_cast<unsigned>(N);
        d.H = static_cast<unsigned>(H);
        d.W = static_cast<unsigned>(W);
        d.ph = static_cast<unsigned>(ph);
        d.pw = static_cast<unsigned>(pw);
        d.P2 = static_cast<unsigned>(P / 2);
        d.Q2 = static_cast<unsigned>(Q / 2);
        d.F = static_cast<unsigned>(F);
        d.relu = relu;
        d.quads = N * (P / 2) * (Q / 2);
        const dim3 dgrid(static_cast<unsigned>(dh_ceil_div(d.quads, static_cast<size_t>(256))));
        if (Hf == 5) {
            if (pool)
                hipLaunchKernelGGL((conv2d_direct_kernel<T, 5, 5, true>), dgrid, dim3(256), 0, ctx->stream, data, filter, bias, res, d);
            else
                hipLaunchKernelGGL((conv2d_direct_kernel<T, 5, 5, false>), dgrid, dim3(256), 0, ctx->stream, data, filter, bias, res, d);
        } else {
            if (pool)
                hipLaunchKernelGGL((conv2d_direct_kernel<T, 3, 3, true>), dgrid, dim3(256), 0, ctx->stream, data, filter, bias, res, d);
            else
                hipLaunchKernelGGL((conv2d_direct_kernel<T, 3, 3, false>), dgrid, dim3(256), 0, ctx->stream, data, filter, bias, res, d);
        }
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    constexpr int BK = dh_gemm::GemmBK<T>::value;
    constexpr int BN = 128;
    const size_t Hp = H + 2 * ph, Wp = W + 2 * pw, K = C * Hf * Wf;
    // a workgroup addresses its pixels with 32-bit byte offsets from its first image
    const size_t tile_px = pool ? 4 * Po * Qo : P * Q; // "pixels" per image as the tiled kernel counts them
    const size_t images_per_tile = (BN + tile_px - 2) / tile_px + 1;
    if (C * Hp * Wp * images_per_tile * sizeof(T) >= (size_t(1) << 32) || K >= (size_t(1) << 31) ||
        P * Q >= (size_t(1) << 31) || N >= (size_t(1) << 31) || F >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Convolution: image or filter extents exceed the 32-bit addressing of a tile");
    {
        // Image resident in LDS: the padded image and the offset table must fit, and every wave should own at
        // least three blocks of 16 pixels (smaller images leave the waves idle; they take the tiled kernel below).
        const int mfw = F <= 16 ? 1 : (F <= 32 ? 2 : 4);
        const size_t parts = 8 / mfw;
        const size_t kpad = dh_ceil_div(K, BK) * BK;
        const size_t plane_bytes = Hp * Wp * sizeof(T);
        // LDS for the images of a stage so that three workgroups fit a CU (160 KiB) beside their offset tables
        const size_t budget = kpad * sizeof(int) + 16 * 1024 < 52 * 1024 ? 52 * 1024 - kpad * sizeof(int) : 16 * 1024;
        // Channels per stage for `imgs` images per workgroup: all of them if that fits the budget, else the fewest
        // equal stages that do and whose share of K is a whole number of K blocks; failing that, all channels in
        // one stage as long as LDS holds them at all (one workgroup per CU). 0: nothing fits.
        auto channels_per_stage = [&](size_t imgs) -> size_t {
            if (imgs * C * plane_bytes <= budget)
                return C;
            for (size_t stages = dh_ceil_div(imgs * C * plane_bytes, budget); stages <= C; stages++) {
                const size_t per = dh_ceil_div(C, stages);
                if ((per * Hf * Wf) % BK == 0 && imgs * per * plane_bytes <= budget)
                    return per;
            }
            return imgs * C * plane_bytes + kpad * sizeof(int) <= 150 * 1024 ? C : 0;
        };
        // images per workgroup: one if that gives every wave six blocks of 16 pixels, else as many as do (at most 16)
        size_t ni = dh_ceil_div(6 * parts * 16, P * Q);
        if (ni > 16)
            ni = 16;
        if (ni > N)
            ni = N;
        size_t cg = channels_per_stage(ni);
        while (cg == 0 && ni > 1)
            cg = channels_per_stage(--ni);
        const size_t blocks16 = dh_ceil_div(ni * P * Q, 16);
        size_t lds = kpad * sizeof(int) + ni * cg * plane_bytes;
        const size_t fgroups = dh_ceil_div(F, static_cast<size_t>(16 * mfw));
        const size_t chunks = dh_ceil_div(blocks16, parts * 13);            // at most 13 blocks per wave
        const size_t nf = dh_ceil_div(blocks16, parts * chunks);            // spread evenly over the chunks
        const size_t chunk = parts * nf * 16;
        const size_t igroups = dh_ceil_div(N, ni);
        // Channels interleaved in LDS (one vector read per VEC matrix instructions): the stage's channels must come in
        // whole groups of 4 VEC, every stage must have the same number, and the wider image (a vector of padding per
        // position) must not cost a workgroup per CU.
        constexpr size_t vec = 16 / sizeof(T);
        bool ci = cg != 0 && cg % (4 * vec) == 0 && C % cg == 0 && mfw > 1;
        if (ci) {
            const size_t lds_ci = kpad * sizeof(int) + ni * Hp * Wp * (cg + vec) * sizeof(T);
            if (lds_ci > 150 * 1024 || (lds <= 80 * 1024 && lds_ci > 80 * 1024) || (lds <= 52 * 1024 && lds_ci > 53 * 1024))
                ci = false;
            else
                lds = lds_ci;
        }
        const size_t lds_bias = lds; // a whole number of elements: the table is whole K blocks of ints
        lds += 16 * mfw * sizeof(T);
        // One workgroup per CU (more than 80 KiB of LDS) has nothing to cover its loading phase and its LDS
        // latencies with: taken only when a wave has at least six blocks of matrix instructions per step.
        // With K < 32 (one or two K blocks) the output stores dominate, and the tiled kernel below writes longer
        // runs: 1 -> 32 channels, 5 x 5 on 28 x 28 takes 0.16 ms there and 0.28 ms here.
        // (One thread per pixel on the ordinary ALUs, weights broadcast from LDS, was tried for that layer as well:
        // 0.15 ms, bound by the LDS reads of the weights; four pixels per thread to share them: 0.20 ms.)
        // The choice does not look at the epilogue: the two kernels add up a result's terms in different orders, and
        // a call with an epilogue has to give the bits of the plain call.
        if (cg != 0 && lds <= 150 * 1024 && (lds <= 80 * 1024 || nf >= 6) && blocks16 >= 3 * parts && K >= 32 && fgroups < 65536 &&
            chunks < 65536) {
            const size_t fpad = fgroups * 16 * mfw;
            const size_t tab_bytes = dh_ceil_div(kpad * sizeof(int), 256) * 256;
            void *wsv = nullptr;
            dh_status st = dh_workspace(ctx, tab_bytes + fpad * kpad * sizeof(T), &wsv);
            if (st != DH_OK)
                return st;
            int *tab = static_cast<int *>(wsv);
            T *wpack = reinterpret_cast<T *>(static_cast<char *>(wsv) + tab_bytes);
            size_t pg = dh_ceil_div(fpad * kpad, 256);
            if (pg > 1024)
                pg = 1024;
            hipLaunchKernelGGL((conv_prep_kernel<T>), dim3(static_cast<unsigned>(pg)), dim3(256), 0, ctx->stream, tab, wpack,
                               filter, static_cast<unsigned>(F), static_cast<unsigned>(fpad), static_cast<unsigned>(K),
                               static_cast<unsigned>(kpad), static_cast<unsigned>(Hp * Wp), static_cast<unsigned>(Wp),
                               static_cast<unsigned>(Hf), static_cast<unsigned>(Wf), static_cast<unsigned>(cg),
                               static_cast<unsigned>(sizeof(T)), static_cast<unsigned>(ci ? cg + vec : 0));
            DH_CHECK_LAUNCH();
            ConvResidentArgs r{};
            r.x = data;
            r.wpack = wpack;
            r.ktab = tab;
            r.bias = bias;
            r.res = res;
            r.C = static_cast<unsigned>(C);
            r.H = static_cast<unsigned>(H);
            r.W = static_cast<unsigned>(W);
            r.Hp = static_cast<unsigned>(Hp);
            r.Wp = static_cast<unsigned>(Wp);
            r.ph = static_cast<unsigned>(ph);
            r.pw = static_cast<unsigned>(pw);
            r.Q = static_cast<unsigned>(Q);
            r.sh = static_cast<unsigned>(sh);
            r.sw = static_cast<unsigned>(sw);
            r.F = static_cast<unsigned>(F);
            r.Kpad = static_cast<unsigned>(kpad);
            r.HpWp = static_cast<unsigned>(Hp * Wp);
            r.CG = static_cast<unsigned>(cg);
            r.KG = static_cast<unsigned>(cg * Hf * Wf);
            r.N = static_cast<unsigned>(N);
            r.NI = static_cast<unsigned>(ni);
            r.PQ = static_cast<unsigned>(P * Q);
            r.chunk = static_cast<unsigned>(chunk);
            r.relu = relu;
            r.lds_bias = static_cast<unsigned>(lds_bias);
            r.Qo = static_cast<unsigned>(Qo);
            r.PQo = static_cast<unsigned>(Po * Qo);
            if (pool) {
                // the same division of work over the window positions, four to a pooled pixel (fewer than P * Q where P or Q is odd)
                const size_t pblocks = dh_ceil_div(ni * 4 * Po * Qo, 16);
                const size_t pchunks = dh_ceil_div(pblocks, parts * 13);
                const size_t np = dh_ceil_div(pblocks, parts * pchunks);
                r.chunk = static_cast<unsigned>(parts * np * 16);
                const dim3 pgrid(static_cast<unsigned>(igroups), static_cast<unsigned>(fgroups), static_cast<unsigned>(pchunks));
#define DH_CONV_POOL(MFW_)                                                                         \
    (np <= 4 ? conv2d_resident_launch<T, MFW_, 4, true>(ctx, r, pgrid, lds)                        \
             : (np <= 7 ? conv2d_resident_launch<T, MFW_, 7, true>(ctx, r, pgrid, lds)             \
                        : (np <= 10 ? conv2d_resident_launch<T, MFW_, 10, true>(ctx, r, pgrid, lds) \
                                    : conv2d_resident_launch<T, MFW_, 13, true>(ctx, r, pgrid, lds))))
#define DH_CONV_POOL_CI(MFW_)                                                                      \
    (np <= 4 ? conv2d_resident_launch<T, MFW_, 4, true, true>(ctx, r, pgrid, lds)                  \
             : (np <= 7 ? conv2d_resident_launch<T, MFW_, 7, true, true>(ctx, r, pgrid, lds)       \
                        : (np <= 10 ? conv2d_resident_launch<T, MFW_, 10, true, true>(ctx, r, pgrid, lds) \
                                    : conv2d_resident_launch<T, MFW_, 13, true, true>(ctx, r, pgrid, lds))))
                if (ci)
                    return mfw == 2 ? DH_CONV_POOL_CI(2) : DH_CONV_POOL_CI(4);
#undef DH_CONV_POOL_CI
                return mfw == 1 ? DH_CONV_POOL(1) : (mfw == 2 ? DH_CONV_POOL(2) : DH_CONV_POOL(4));
#undef DH_CONV_POOL
            }
            const dim3 grid(static_cast<unsigned>(igroups), static_cast<unsigned>(fgroups), static_cast<unsigned>(chunks));
#define DH_CONV_RES(MFW_)                                                                          \
    (nf <= 4 ? conv2d_resident_launch<T, MFW_, 4>(ctx, r, grid, lds)                               \
             : (nf <= 7 ? conv2d_resident_launch<T, MFW_, 7>(ctx, r, grid, lds)                    \
                        : (nf <= 10 ? conv2d_resident_launch<T, MFW_, 10>(ctx, r, grid, lds)       \
                                    : conv2d_resident_launch<T, MFW_, 13>(ctx, r, grid, lds))))
#define DH_CONV_RES_CI(MFW_)                                                                       \
    (nf <= 4 ? conv2d_resident_launch<T, MFW_, 4, false, true>(ctx, r, grid, lds)                  \
             : (nf <= 7 ? conv2d_resident_launch<T, MFW_, 7, false, true>(ctx, r, grid, lds)       \
                        : (nf <= 10 ? conv2d_resident_launch<T, MFW_, 10, false, true>(ctx, r, grid, lds) \
                                    : conv2d_resident_launch<T, MFW_, 13, false, true>(ctx, r, grid, lds))))
            if (ci)
                return mfw == 2 ? DH_CONV_RES_CI(2) : DH_CONV_RES_CI(4);
#undef DH_CONV_RES_CI
            return mfw == 1 ? DH_CONV_RES(1) : (mfw == 2 ? DH_CONV_RES(2) : DH_CONV_RES(4));
#undef DH_CONV_RES
        }
    }
    const size_t vpixels = pool ? 4 * N * Po * Qo : pixels; // the tile's pixel index counts window positions with pooling
    const size_t gx = dh_ceil_div(vpixels, BN);
    if (gx >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Convolution: too many output pixels for one launch");
    const int BM = F <= 32 ? 32 : 64;
    const unsigned gy = static_cast<unsigned>(dh_ceil_div(F, BM));
    const size_t Kpad = dh_ceil_div(K, BK) * BK, Fpad = static_cast<size_t>(gy) * BM;
    const bool padded = ph != 0 || pw != 0;

    // workspace: offset table | packed filter | padded images
    const size_t tab_bytes = dh_ceil_div(Kpad * sizeof(int), 256) * 256;
    const size_t w_bytes = dh_ceil_div(Fpad * Kpad * sizeof(T), 256) * 256;
    const size_t x_elems = padded ? N * C * Hp * Wp : 0;
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, tab_bytes + w_bytes + x_elems * sizeof(T), &wsv);
    if (st != DH_OK)
        return st;
    char *ws = static_cast<char *>(wsv);
    int *tab = reinterpret_cast<int *>(ws);
    T *wpack = reinterpret_cast<T *>(ws + tab_bytes);
    T *xpad = reinterpret_cast<T *>(ws + tab_bytes + w_bytes);
    size_t pg = dh_ceil_div(Fpad * Kpad, 256);
    if (pg > 1024)
        pg = 1024;
    hipLaunchKernelGGL((conv_prep_kernel<T>), dim3(static_cast<unsigned>(pg)), dim3(256), 0, ctx->stream, tab, wpack, filter,
                       static_cast<unsigned>(F), static_cast<unsigned>(Fpad), static_cast<unsigned>(K),
                       static_cast<unsigned>(Kpad), static_cast<unsigned>(Hp * Wp), static_cast<unsigned>(Wp),
                       static_cast<unsigned>(Hf), static_cast<unsigned>(Wf));
    DH_CHECK_LAUNCH();
    if (padded) {
        const size_t blocks = dh_ceil_div(x_elems, 256);
        if (blocks >= (size_t(1) << 31))
            return dh_fail(DH_ERR_RUNTIME, "Convolution: input too large for one launch");
        hipLaunchKernelGGL((conv_pad_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ctx->stream, xpad, data,
                           x_elems, static_cast<unsigned>(H), static_cast<unsigned>(W), static_cast<unsigned>(Hp),
                           static_cast<unsigned>(Wp), static_cast<unsigned>(ph), static_cast<unsigned>(pw));
        DH_CHECK_LAUNCH();
    }

    ConvArgs g{};
    g.xpad = padded ? xpad : data;
    g.wpack = wpack;
    g.ktab = tab;
    g.bias = bias;
    g.res = res;
    g.F = static_cast<unsigned>(F);
    g.K = static_cast<unsigned>(K);
    g.Kpad = static_cast<unsigned>(Kpad);
    g.P = static_cast<unsigned>(P);
    g.Q = static_cast<unsigned>(Q);
    g.sh = static_cast<unsigned>(sh);
    g.sw = static_cast<unsigned>(sw);
    g.Wp = static_cast<unsigned>(Wp);
    g.CHpWp = static_cast<unsigned>(C * Hp * Wp);
    g.relu = relu;
    g.Qo = static_cast<unsigned>(Qo);
    g.PQo = static_cast<unsigned>(Po * Qo);
    g.pixels = vpixels;
    const dim3 grid(static_cast<unsigned>(gx), gy);
    if (pool) {
        if (BM == 32)
            hipLaunchKernelGGL((conv2d_kernel<T, 32, BN, BK, 4, true>), grid, dim3(256), 0, ctx->stream, g);
        else
            hipLaunchKernelGGL((conv2d_kernel<T, 64, BN, BK, 4, true>), grid, dim3(256), 0, ctx->stream, g);
    } else if (BM == 32) {
        hipLaunchKernelGGL((conv2d_kernel<T, 32, BN, BK, 4>), grid, dim3(256), 0, ctx->stream, g);
    } else {
        hipLaunchKernelGGL((conv2d_kernel<T, 64, BN, BK, 4>), grid, dim3(256), 0, ctx->stream, g);
    }
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// MaxPool forward. One thread per output; consecutive threads on consecutive q.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void maxpool_kernel(T *res, const T *data, size_t total, unsigned planes_dummy,
                                                      unsigned H, unsigned W, unsigned P, unsigned Q, unsigned ph,
                                                      unsigned pw, unsigned sh, unsigned sw, unsigned padh,
                                                      unsigned padw) {
    const unsigned PQ = P * Q, HW = H * W;
    const bool small = total <= 0xffffffffull; // 32-bit divisions suffice (uniform)
    for (size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * 256) {
        size_t plane;
        unsigned pq;
        if (small) {
            plane = static_cast<unsigned>(idx) / PQ;
            pq = static_cast<unsigned>(idx) % PQ;
        } else {
            plane = idx / PQ;
            pq = static_cast<unsigned>(idx % PQ);
        }
        const unsigned p = pq / Q, q = pq % Q;
        const T *in = data + plane * HW;
        // window in image coordinates, clipped at the border (Pooling.cpp:77,89,102); the padding
        // ring holds zeros, and the output starts at zero anyway (Pooling.cpp:57, Pooling.h:46-54)
        const int y_lo = static_cast<int>(p * sh) - static_cast<int>(padh);
        const int x_lo = static_cast<int>(q * sw) - static_cast<int>(padw);
        const int y0 = y_lo < 0 ? 0 : y_lo, x0 = x_lo < 0 ? 0 : x_lo;
        int y1 = y_lo + static_cast<int>(ph), x1 = x_lo + static_cast<int>(pw);
        if (y1 > static_cast<int>(H))
            y1 = H;
        if (x1 > static_cast<int>(W))
            x1 = W;
        T m = T(0);
        for (int y = y0; y < y1; y++)
            for (int x = x0; x < x1; x++) {
                const T v = in[static_cast<unsigned>(y) * W + static_cast<unsigned>(x)];
                m = (m < v) ? v : m; // std::max(m, v)
            }
        res[idx] = m;
    }
}

// Pooling over small planes, `ppb` whole planes per workgroup: the planes are contiguous in memory, so
// the workgroup copies them into LDS with 16-byte loads (batches of four per thread, all issued before
// the first LDS store) and then gathers every window from LDS; the outputs of the planes are contiguous
// as well and go out coalesced. Window clipping and arithmetic are those of maxpool_kernel /
// avgpool_kernel. The host picks ppb so that a workgroup's first element is 16-byte aligned.
// TWO: the window is 2 x 2 with stride 2, no padding, H and W even: two 2-value reads per output, arithmetic of
// maxpool2x2_kernel.
template <typename T, bool AVG, bool TWO = false>
__global__ __launch_bounds__(256) void pool_planes_kernel(T *res, const T *data, size_t planes, unsigned ppb, unsigned H,
                                                          unsigned W, unsigned P, unsigned Q, unsigned ph, unsigned pw,
                                                          unsigned sh, unsigned sw, unsigned padh, unsigned padw, T plen) {
#pragma clang fp contract(off)
    extern __shared__ __attribute__((aligned(16))) unsigned char pool_lds[];
    T *tile = reinterpret_cast<T *>(pool_lds);
    constexpr int VEC = 16 / sizeof(T);
    const unsigned tid = threadIdx.x;
    const size_t first = static_cast<size_t>(blockIdx.x) * ppb;
    const size_t left = planes - first;
    const unsigned here = left < ppb ? static_cast<unsigned>(left) : ppb;
    const unsigned HW = H * W, PQ = P * Q;
    const unsigned n_in = here * HW, nvec = n_in / VEC;
    const T *src = data + first * HW;
    for (unsigned v0 = 0; v0 < nvec; v0 += 256 * 4) {
        T r[4][VEC];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const unsigned i = v0 + tid + 256 * k;
            dh_load_vec_stream<T, VEC>(src + static_cast<size_t>(i < nvec ? i : nvec - 1) * VEC, r[k]);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const unsigned i = v0 + tid + 256 * k;
            if (i < nvec)
                dh_store_vec<T, VEC>(tile + static_cast<size_t>(i) * VEC, r[k]);
        }
    }
    for (unsigned i = nvec * VEC + tid; i < n_in; i += 256)
        tile[i] = src[i];
    __syncthreads();
    const unsigned n_out = here * PQ;
    T *dst = res + first * PQ;
    if (!TWO && PQ <= 256) {
        // a thread keeps its place in the result plane and walks the planes: the window's extent is worked out once
        const unsigned groups = 256 / PQ, grp = tid / PQ, pq = tid % PQ;
        if (grp >= groups)
            return;
        const unsigned p = pq / Q, q = pq % Q;
        const int y_lo = static_cast<int>(p * sh) - static_cast<int>(padh);
        const int x_lo = static_cast<int>(q * sw) - static_cast<int>(padw);
        const int y0 = y_lo < 0 ? 0 : y_lo, x0 = x_lo < 0 ? 0 : x_lo;
        int y1 = y_lo + static_cast<int>(ph), x1 = x_lo + static_cast<int>(pw);
        if (y1 > static_cast<int>(H))
            y1 = H;
        if (x1 > static_cast<int>(W))
            x1 = W;
        for (unsigned plane = grp; plane < here; plane += groups) {
            const T *in = tile + plane * HW;
            T acc = T(0);
            for (int y = y0; y < y1; y++) {
                if constexpr (AVG) {
                    T s_ = T(0);
                    for (int x = x0; x < x1; x++)
                        s_ = s_ + in[static_cast<unsigned>(y) * W + static_cast<unsigned>(x)];
                    const T scaled = s_ * plen;
                    acc = scaled + acc;
                } else {
                    for (int x = x0; x < x1; x++) {
                        const T v = in[static_cast<unsigned>(y) * W + static_cast<unsigned>(x)];
                        acc = (acc < v) ? v : acc; // std::max(acc, v)
                    }
                }
            }
            dst[plane * PQ + pq] = acc;
        }
        return;
    }
    for (unsigned o = tid; o < n_out; o += 256) {
        const unsigned plane = o / PQ, pq = o % PQ;
        const unsigned p = pq / Q, q = pq % Q;
        const T *in = tile + plane * HW;
        if constexpr (TWO) {
            typedef T pair_t __attribute__((ext_vector_type(2)));
            const T *w = in + 2 * p * W + 2 * q; // an even offset: the pair is aligned
            const pair_t a = *reinterpret_cast<const pair_t *>(w), b = *reinterpret_cast<const pair_t *>(w + W);
            if constexpr (AVG) {
                const T s0 = (T(0) + a[0]) + a[1];
                const T s1 = (T(0) + b[0]) + b[1];
                const T r0 = s0 * T(0.25) + T(0);
                dst[o] = s1 * T(0.25) + r0;
            } else {
                T m = T(0);
                m = (m < a[0]) ? a[0] : m;
                m = (m < a[1]) ? a[1] : m;
                m = (m < b[0]) ? b[0] : m;
                m = (m < b[1]) ? b[1] : m;
                dst[o] = m;
            }
            continue;
        }
        const int y_lo = static_cast<int>(p * sh) - static_cast<int>(padh);
        const int x_lo = static_cast<int>(q * sw) - static_cast<int>(padw);
        const int y0 = y_lo < 0 ? 0 : y_lo, x0 = x_lo < 0 ? 0 : x_lo;
        int y1 = y_lo + static_cast<int>(ph), x1 = x_lo + static_cast<int>(pw);
        if (y1 > static_cast<int>(H))
            y1 = H;
        if (x1 > static_cast<int>(W))
            x1 = W;
        T acc = T(0);
        for (int y = y0; y < y1; y++) {
            if constexpr (AVG) {
                T s = T(0);
                for (int x = x0; x < x1; x++)
                    s = s + in[static_cast<unsigned>(y) * W + static_cast<unsigned>(x)];
                const T scaled = s * plen;
                acc = scaled + acc;
            } else {
                for (int x = x0; x < x1; x++) {
                    const T v = in[static_cast<unsigned>(y) * W + static_cast<unsigned>(x)];
                    acc = (acc < v) ? v : acc; // std::max(acc, v)
                }
            }
        }
        dst[o] = acc;
    }
}

// Planes per workgroup for pool_planes_kernel: about 16 KB of input and a plane count whose elements
// fill whole 16-byte vectors, so that every workgroup starts on a vector boundary. 0: the planes are
// too large for this kernel or the input is not aligned.
template <typename T> inline unsigned pool_planes_per_block(const T *data, size_t HW, size_t planes) {
    constexpr size_t VEC = 16 / sizeof(T);
    const size_t target = (16 * 1024) / sizeof(T);
    if (HW == 0 || HW > target || !dh_aligned(data, 16))
        return 0;
    size_t unit = VEC; // smallest plane count with unit * HW % VEC == 0
    while (unit > 1 && ((unit / 2) * HW) % VEC == 0)
        unit /= 2;
    size_t ppb = target / HW;
    if (ppb >= unit)
        ppb -= ppb % unit;
    else if (planes > ppb)
        return 0;
    // small inputs: more workgroups before more planes per workgroup
    while (ppb >= 2 * unit && (ppb / 2) % unit == 0 && dh_ceil_div(planes, ppb) < 2048)
        ppb /= 2;
    return static_cast<unsigned>(ppb);
}

// Non-overlapping 2x2 windows (stride 2, no padding, even H and W): the tensor is a flat list of row
// pairs [R][2][W] -> [R][W/2]. Each thread loads VI consecutive values of both rows of a pair and
// writes VI/2 outputs, all as single vector accesses.
template <typename T, int VI, bool AVG = false>
__global__ __launch_bounds__(256) void maxpool2x2_kernel(T *res, const T *data, size_t items, unsigned W,
                                                         unsigned wvecs) {
#pragma clang fp contract(off)
    const size_t item = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (item >= items)
        return;
    size_t r;
    unsigned j;
    if (items <= 0xffffffffull) {
        r = static_cast<unsigned>(item) / wvecs;
        j = static_cast<unsigned>(item) % wvecs;
    } else {
        r = item / wvecs;
        j = static_cast<unsigned>(item % wvecs);
    }
    const T *in = data + r * 2 * W + static_cast<size_t>(j) * VI;
    T a[VI], b[VI], o[VI / 2];
    {
        typedef T in_vec __attribute__((ext_vector_type(VI)));
        const in_vec va = __builtin_nontemporal_load(reinterpret_cast<const in_vec *>(in));
        const in_vec vb = __builtin_nontemporal_load(reinterpret_cast<const in_vec *>(in + W));
#pragma unroll
        for (int i = 0; i < VI; i++) {
            a[i] = va[i];
            b[i] = vb[i];
        }
    }
#pragma unroll
    for (int i = 0; i < VI / 2; i++) {
        // window order of Pooling.cpp:77-105 with the accumulator starting at zero
        if constexpr (AVG) {
            // per window row: sum from zero, scale by 1/4, add to the running result (Pooling.h:34-40)
            const T s0 = (T(0) + a[2 * i]) + a[2 * i + 1];
            const T s1 = (T(0) + b[2 * i]) + b[2 * i + 1];
            const T r0 = s0 * T(0.25) + T(0);
            o[i] = s1 * T(0.25) + r0;
        } else {
            T m = T(0);
            m = (m < a[2 * i]) ? a[2 * i] : m;
            m = (m < a[2 * i + 1]) ? a[2 * i + 1] : m;
            m = (m < b[2 * i]) ? b[2 * i] : m;
            m = (m < b[2 * i + 1]) ? b[2 * i + 1] : m;
            o[i] = m;
        }
    }
    T *out = res + r * (W / 2) + static_cast<size_t>(j) * (VI / 2);
    if constexpr (VI / 2 == 1) {
        *out = o[0];
    } else {
        typedef T half_vec __attribute__((ext_vector_type(VI / 2)));
        half_vec t;
#pragma unroll
        for (int i = 0; i < VI / 2; i++)
            t[i] = o[i];
        *reinterpret_cast<half_vec *>(out) = t;
    }
}

template <typename T> __global__ __launch_bounds__(256) void fill_kernel(T *p, size_t n, T v) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * 256)
        p[i] = v;
}

template <typename T>
dh_status maxpool_forward(dh_ctx *ctx, T *res, size_t *res_h, size_t *res_w, const T *data, size_t N, size_t C,
                          size_t H, size_t W, size_t ph, size_t pw, size_t sh, size_t sw, size_t padh, size_t padw) {
    DH_REQUIRE_CTX(ctx);
    if (sh == 0 || sw == 0 || H + 2 * padh < ph || W + 2 * padw < pw)
        return dh_fail(DH_ERR_INVALID_ARG, "Pooling: window %zux%zu does not fit the padded image %zux%zu", ph, pw,
                       H + 2 * padh, W + 2 * padw);
    // Pooling.cpp:38-39: P is derived with stride_w and Q with stride_h.
    const size_t P = (H + 2 * padh - ph) / sw + 1, Q = (W + 2 * padw - pw) / sh + 1;
    if (res_h)
        *res_h = P;
    if (res_w)
        *res_w = Q;
    const size_t total = N * C * P * Q;
    if (total == 0)
        return DH_OK;
    if (H * W >= (size_t(1) << 31) || P * Q >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Pooling: image extents exceed 2^31 elements");
    size_t grid = dh_ceil_div(total, 256);
    const size_t cap = size_t(1) << 30; // one output per thread; the loop only matters beyond 2^38 outputs
    if (grid > cap)
        grid = cap;
    constexpr int VI = 16 / sizeof(T);
    const bool pairs = ph == 2 && pw == 2 && sh == 2 && sw == 2 && padh == 0 && padw == 0 && H % 2 == 0 && W % 2 == 0 &&
                       total < (size_t(1) << 39);
    // rows of less than 128 bytes go through LDS even where they are whole vectors: measured 14 x 14 doubles
    const bool short_rows = W * sizeof(T) < 128;
    if (pairs && !short_rows && W % VI == 0 && dh_aligned(data, 16) && dh_aligned(res, 8)) {
        const size_t items = N * C * P * (W / VI);
        hipLaunchKernelGGL((maxpool2x2_kernel<T, VI>), dim3(static_cast<unsigned>(dh_ceil_div(items, 256))), dim3(256), 0,
                           ctx->stream, res, data, items, static_cast<unsigned>(W), static_cast<unsigned>(W / VI));
    } else if (const unsigned ppb2 = pairs ? pool_planes_per_block(data, H * W, N * C) : 0;
               ppb2 != 0 && dh_ceil_div(N * C, ppb2) < (size_t(1) << 31) && ppb2 * P * Q < (size_t(1) << 31)) {
        // rows that are no whole number of 16-byte vectors (14 x 14 floats): the planes are contiguous, so a workgroup
        // copies a run of them into LDS with 16-byte loads and gathers the windows there
        hipLaunchKernelGGL((pool_planes_kernel<T, false, true>), dim3(static_cast<unsigned>(dh_ceil_div(N * C, ppb2))), dim3(256),
                           ppb2 * H * W * sizeof(T), ctx->stream, res, data, N * C, ppb2, static_cast<unsigned>(H),
                           static_cast<unsigned>(W), static_cast<unsigned>(P), static_cast<unsigned>(Q), 2u, 2u, 2u, 2u, 0u, 0u, T(0));
    } else if (pairs && VI > 2 && dh_aligned(data, 8)) {
        // rows of an even number of floats that is not a multiple of four: 8-byte loads, one output per thread
        const size_t items = N * C * P * (W / 2);
        hipLaunchKernelGGL((maxpool2x2_kernel<T, 2>), dim3(static_cast<unsigned>(dh_ceil_div(items, 256))), dim3(256), 0,
                           ctx->stream, res, data, items, static_cast<unsigned>(W), static_cast<unsigned>(W / 2));
    } else if (P == 1 && Q == 1 && W == 1) {
        // Pooling.cpp:57-66: this quick path folds the window into numeric_limits::max(), so that
        // value is what the CPU kernel returns for every output.
        hipLaunchKernelGGL((fill_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, res, total,
                           std::numeric_limits<T>::max());
    } else if (const unsigned ppb = pool_planes_per_block(data, H * W, N * C);
               ppb != 0 && dh_ceil_div(N * C, ppb) < (size_t(1) << 31) && ppb * P * Q < (size_t(1) << 31)) {
        hipLaunchKernelGGL((pool_planes_kernel<T, false>), dim3(static_cast<unsigned>(dh_ceil_div(N * C, ppb))), dim3(256),
                           ppb * H * W * sizeof(T), ctx->stream, res, data, N * C, ppb, static_cast<unsigned>(H),
                           static_cast<unsigned>(W), static_cast<unsigned>(P), static_cast<unsigned>(Q),
                           static_cast<unsigned>(ph), static_cast<unsigned>(pw), static_cast<unsigned>(sh),
                           static_cast<unsigned>(sw), static_cast<unsigned>(padh), static_cast<unsigned>(padw), T(0));
    } else {
        hipLaunchKernelGGL((maxpool_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, res, data,
                           total, 0u, static_cast<unsigned>(H), static_cast<unsigned>(W), static_cast<unsigned>(P),
                           static_cast<unsigned>(Q), static_cast<unsigned>(ph), static_cast<unsigned>(pw),
                           static_cast<unsigned>(sh), static_cast<unsigned>(sw), static_cast<unsigned>(padh),
                           static_cast<unsigned>(padw));
    }
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// AvgPool forward with the CPU kernel's arithmetic (Pooling.cpp:28-107, Pooling.h:33-44): per window
// row the values are summed left to right, the row sum is scaled by 1 / (pool_h * pool_w) - the full
// window, padding included - and added to the running result, rounding after each step.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void avgpool_kernel(T *res, const T *data, size_t total, unsigned H, unsigned W,
                                                      unsigned P, unsigned Q, unsigned ph, unsigned pw, unsigned sh,
                                                      unsigned sw, unsigned padh, unsigned padw, T plen, int quick) {
#pragma clang fp contract(off)
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total)
        return;
    const unsigned PQ = P * Q, HW = H * W;
    size_t plane;
    unsigned pq;
    if (total <= 0xffffffffull) {
        plane = static_cast<unsigned>(idx) / PQ;
        pq = static_cast<unsigned>(idx) % PQ;
    } else {
        plane = idx / PQ;
        pq = static_cast<unsigned>(idx % PQ);
    }
    const unsigned p = pq / Q, q = pq % Q;
    const T *in = data + plane * HW;
    int y0, y1, x0, x1;
    if (quick) {
        // Pooling.cpp:57-66: one output per plane of a one-column image: the first min(pool_h, H) values
        y0 = 0;
        y1 = static_cast<int>(ph < H ? ph : H);
        x0 = 0;
        x1 = 1;
    } else {
        const int y_lo = static_cast<int>(p * sh) - static_cast<int>(padh);
        const int x_lo = static_cast<int>(q * sw) - static_cast<int>(padw);
        y0 = y_lo < 0 ? 0 : y_lo;
        x0 = x_lo < 0 ? 0 : x_lo;
        y1 = y_lo + static_cast<int>(ph);
        x1 = x_lo + static_cast<int>(pw);
        if (y1 > static_cast<int>(H))
            y1 = H;
        if (x1 > static_cast<int>(W))
            x1 = W;
    }
    T acc = T(0);
    for (int y = y0; y < y1; y++) {
        T s = T(0);
        for (int x = x0; x < x1; x++)
            s = s + in[static_cast<unsigned>(y) * W + static_cast<unsigned>(x)];
        const T scaled = s * plen;
        acc = scaled + acc;
    }
    res[idx] = acc;
}

template <typename T>
dh_status avgpool_forward(dh_ctx *ctx, T *res, size_t *res_h, size_t *res_w, const T *data, size_t N, size_t C,
                          size_t H, size_t W, size_t ph, size_t pw, size_t sh, size_t sw, size_t padh, size_t padw) {
    DH_REQUIRE_CTX(ctx);
    if (sh == 0 || sw == 0 || ph == 0 || pw == 0 || H + 2 * padh < ph || W + 2 * padw < pw)
        return dh_fail(DH_ERR_INVALID_ARG, "Pooling: window %zux%zu does not fit the padded image %zux%zu", ph, pw,
                       H + 2 * padh, W + 2 * padw);
    // Pooling.cpp:38-39: P is derived with stride_w and Q with stride_h.
    const size_t P = (H + 2 * padh - ph) / sw + 1, Q = (W + 2 * padw - pw) / sh + 1;
    if (res_h)
        *res_h = P;
    if (res_w)
        *res_w = Q;
    const size_t total = N * C * P * Q;
    if (total == 0)
        return DH_OK;
    if (H * W >= (size_t(1) << 31) || P * Q >= (size_t(1) << 31) || dh_ceil_div(total, 256) >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Pooling: image extents exceed 2^31 elements");
    constexpr int VI = 16 / sizeof(T);
    const bool pairs = ph == 2 && pw == 2 && sh == 2 && sw == 2 && padh == 0 && padw == 0 && H % 2 == 0 && W % 2 == 0 &&
                       total < (size_t(1) << 39);
    const bool short_rows = W * sizeof(T) < 128; // as in maxpool_forward
    if (pairs && !short_rows && W % VI == 0 && dh_aligned(data, 16) && dh_aligned(res, 8)) {
        const size_t items = N * C * P * (W / VI);
        hipLaunchKernelGGL((maxpool2x2_kernel<T, VI, true>), dim3(static_cast<unsigned>(dh_ceil_div(items, 256))), dim3(256),
                           0, ctx->stream, res, data, items, static_cast<unsigned>(W), static_cast<unsigned>(W / VI));
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    if (const unsigned ppb2 = pairs ? pool_planes_per_block(data, H * W, N * C) : 0;
        ppb2 != 0 && dh_ceil_div(N * C, ppb2) < (size_t(1) << 31) && ppb2 * P * Q < (size_t(1) << 31)) {
        hipLaunchKernelGGL((pool_planes_kernel<T, true, true>), dim3(static_cast<unsigned>(dh_ceil_div(N * C, ppb2))), dim3(256),
                           ppb2 * H * W * sizeof(T), ctx->stream, res, data, N * C, ppb2, static_cast<unsigned>(H),
                           static_cast<unsigned>(W), static_cast<unsigned>(P), static_cast<unsigned>(Q), 2u, 2u, 2u, 2u, 0u, 0u, T(0.25));
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    if (pairs && VI > 2 && dh_aligned(data, 8)) {
        const size_t items = N * C * P * (W / 2);
        hipLaunchKernelGGL((maxpool2x2_kernel<T, 2, true>), dim3(static_cast<unsigned>(dh_ceil_div(items, 256))), dim3(256), 0,
                           ctx->stream, res, data, items, static_cast<unsigned>(W), static_cast<unsigned>(W / 2));
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    const T plen = T(1) / static_cast<T>(pw * ph); // Pooling.cpp:50
    const bool quick = P == 1 && Q == 1 && W == 1;
    if (const unsigned ppb = quick ? 0 : pool_planes_per_block(data, H * W, N * C);
        ppb != 0 && dh_ceil_div(N * C, ppb) < (size_t(1) << 31) && ppb * P * Q < (size_t(1) << 31)) {
        hipLaunchKernelGGL((pool_planes_kernel<T, true>), dim3(static_cast<unsigned>(dh_ceil_div(N * C, ppb))), dim3(256),
                           ppb * H * W * sizeof(T), ctx->stream, res, data, N * C, ppb, static_cast<unsigned>(H),
                           static_cast<unsigned>(W), static_cast<unsigned>(P), static_cast<unsigned>(Q),
                           static_cast<unsigned>(ph), static_cast<unsigned>(pw), static_cast<unsigned>(sh),
                           static_cast<unsigned>(sw), static_cast<unsigned>(padh), static_cast<unsigned>(padw), plen);
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    hipLaunchKernelGGL((avgpool_kernel<T>), dim3(static_cast<unsigned>(dh_ceil_div(total, 256))), dim3(256), 0, ctx->stream,
                       res, data, total, static_cast<unsigned>(H), static_cast<unsigned>(W), static_cast<unsigned>(P),
                       static_cast<unsigned>(Q), static_cast<unsigned>(ph), static_cast<unsigned>(pw),
                       static_cast<unsigned>(sh), static_cast<unsigned>(sw), static_cast<unsigned>(padh),
                       static_cast<unsigned>(padw), plen, quick ? 1 : 0);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// Per-channel streaming ops: BiasAdd and BatchNorm inference. The matrix is viewed as
// (rows * C) x HW: every view row has one channel, so the statistics are fetched once per row.
// ---------------------------------------------------------------------------------------
template <typename T, int VEC, bool BATCHNORM>
__global__ __launch_bounds__(256) void channel_kernel(T *res, const T *data, size_t vrows, size_t hw_vecs, unsigned C,
                                                      const T *a0 /* bias | gamma */, const T *beta, const T *mean,
                                                      const T *var, T eps) {
    const size_t HW = hw_vecs * VEC;
    for (size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x; cv < hw_vecs;
         cv += static_cast<size_t>(gridDim.y) * blockDim.x) {
        for (size_t r = static_cast<size_t>(blockIdx.x) * blockDim.y + threadIdx.y; r < vrows;
             r += static_cast<size_t>(gridDim.x) * blockDim.y) {
            const unsigned ch = static_cast<unsigned>(r % C);
            T x[VEC];
            dh_load_vec<T, VEC>(data + r * HW + cv * VEC, x);
            T o[VEC];
            if constexpr (BATCHNORM) {
                // BatchNorm2DTestForward.h:96-97, same operation order
                const T sd = sizeof(T) == 4 ? sqrtf(var[ch] + eps) : sqrt(var[ch] + eps);
                const T g = a0[ch], b = beta[ch], mu = mean[ch];
#pragma unroll
                for (int i = 0; i < VEC; i++) {
                    const T x_hat = (x[i] - mu) / sd;
                    o[i] = g * x_hat + b;
                }
            } else {
                const T b = a0[ch];
#pragma unroll
                for (int i = 0; i < VEC; i++)
                    o[i] = x[i] + b;
            }
            dh_store_vec_stream<T, VEC>(res + r * HW + cv * VEC, o);
        }
    }
}

template <typename T, bool BATCHNORM>
static inline dh_status channel_launch(dh_ctx *ctx, T *res, const T *data, size_t vrows, size_t HW, size_t C,
                                       const T *a0, const T *beta, const T *mean, const T *var, T eps) {
    if (vrows == 0 || HW == 0)
        return DH_OK;
    constexpr int V = 16 / sizeof(T);
    const bool vec_ok = (HW % V == 0) && dh_aligned(res, 16) && dh_aligned(data, 16);
    const size_t cvecs = vec_ok ? HW / V : HW;
    unsigned tx = 1;
    while (tx < 256 && tx < cvecs)
        tx <<= 1;
    const unsigned ty = 256 / tx;
    size_t gy = dh_ceil_div(cvecs, tx);
    if (gy > 1024)
        gy = 1024;
    size_t gx = dh_ceil_div(vrows, ty);
    size_t cap = static_cast<size_t>(ctx->num_cus) * 32 / gy;
    if (cap < 1)
        cap = 1;
    if (gx > cap)
        gx = cap;
    const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy)), block(tx, ty);
    if (vec_ok)
        hipLaunchKernelGGL((channel_kernel<T, V, BATCHNORM>), grid, block, 0, ctx->stream, res, data, vrows, cvecs,
                           static_cast<unsigned>(C), a0, beta, mean, var, eps);
    else
        hipLaunchKernelGGL((channel_kernel<T, 1, BATCHNORM>), grid, block, 0, ctx->stream, res, data, vrows, cvecs,
                           static_cast<unsigned>(C), a0, beta, mean, var, eps);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T>
dh_status bias_add(dh_ctx *ctx, T *res, const T *data, size_t rows, size_t cols, const T *bias, size_t num_bias) {
    DH_REQUIRE_CTX(ctx);
    if (num_bias == 0 || cols % num_bias != 0 || num_bias >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "BiasAdd: %zu columns cannot be split into %zu channels", cols, num_bias);
    return channel_launch<T, false>(ctx, res, data, rows * num_bias, cols / num_bias, num_bias, bias, nullptr, nullptr,
                                    nullptr, T(0));
}

template <typename T>
dh_status batchnorm_inference(dh_ctx *ctx, T *res, const T *data, size_t rows, size_t cols, const T *gamma,
                              const T *beta, const T *mean, const T *var, size_t channels, T eps, int stat_index) {
    DH_REQUIRE_CTX(ctx);
    if (stat_index == 1) {
        // statistics indexed by the image (row) like the reference's CPU loop
        if (rows >= (size_t(1) << 31))
            return dh_fail(DH_ERR_RUNTIME, "BatchNorm: too many rows");
        return channel_launch<T, true>(ctx, res, data, rows, cols, rows ? rows : 1, gamma, beta, mean, var, eps);
    }
    if (stat_index != 0)
        return dh_fail(DH_ERR_RUNTIME, "BatchNorm: stat_index must be 0 (channel) or 1 (row)");
    if (channels == 0 || cols % channels != 0 || channels >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "BatchNorm: %zu columns cannot be split into %zu channels", cols, channels);
    return channel_launch<T, true>(ctx, res, data, rows * channels, cols / channels, channels, gamma, beta, mean, var,
                                   eps);
}

// ---------------------------------------------------------------------------------------
// Softmax: G lanes per row; max, exp and sum, scale (Softmax.h:36-52).
// ---------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ T dev_exp(T a);
template <> __device__ __forceinline__ float dev_exp<float>(float a) { return expf(a); }
template <> __device__ __forceinline__ double dev_exp<double>(double a) { return exp(a); }

template <typename T>
__global__ __launch_bounds__(256) void softmax_kernel(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,
                                                      size_t ld, int G) {
    const int lane = threadIdx.x % G;
    const size_t rpb = 256 / G;
    for (size_t r = static_cast<size_t>(blockIdx.x) * rpb + threadIdx.x / G; r < rows;
         r += static_cast<size_t>(gridDim.x) * rpb) {
        const T *in = arg + r * ld;
        T *out = res + r * ld_res;
        // max: NaN anywhere in the row ends up in every output through the sum, as on the CPU
        T mx = -std::numeric_limits<T>::infinity();
        for (size_t c = lane; c < cols; c += G) {
            const T v = in[c];
            mx = (mx < v) ? v : mx;
        }
        dh_butterfly(G, [&](auto peer) {
            const T o = peer(mx);
            mx = (mx < o) ? o : mx;
        });
        const T first = in[0];
        if (first != first)
            mx = first;
        T sum = T(0);
        for (size_t c = lane; c < cols; c += G) {
            const T e = dev_exp<T>(in[c] - mx);
            out[c] = e;
            sum += e;
        }
        dh_butterfly(G, [&](auto peer) { sum += peer(sum); });
        const T inv = T(1) / sum;
        for (size_t c = lane; c < cols; c += G)
            out[c] *= inv;
    }
}

// Rows of up to KEEP * G values stay in registers: one read and one write of the row, one-shot grid. Same
// per-lane order and shuffle trees as softmax_kernel, so both give the same bits.
template <typename T, int KEEP>
__global__ __launch_bounds__(256) void softmax_reg_kernel(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,
                                                          size_t ld, int G) {
    constexpr int RPG = 4; // rows per lane group, all loaded before any arithmetic
    const int lane = threadIdx.x % G;
    const size_t rpb = 256 / G;
    const size_t r0 = static_cast<size_t>(blockIdx.x) * rpb * RPG + threadIdx.x / G;
    T x[RPG][KEEP];
#pragma unroll
    for (int j = 0; j < RPG; j++) {
        const size_t r = r0 + j * rpb;
#pragma unroll
        for (int k = 0; k < KEEP; k++) {
            const size_t c = lane + static_cast<size_t>(k) * G;
            x[j][k] = (r < rows && c < cols) ? arg[r * ld + c] : -std::numeric_limits<T>::infinity();
        }
    }
#pragma unroll
    for (int j = 0; j < RPG; j++) {
        const size_t r = r0 + j * rpb; // uniform over the lane group
        T mx = -std::numeric_limits<T>::infinity();
#pragma unroll
        for (int k = 0; k < KEEP; k++)
            mx = (mx < x[j][k]) ? x[j][k] : mx; // columns past the end hold -inf
        dh_butterfly(G, [&](auto peer) {
            const T o = peer(mx);
            mx = (mx < o) ? o : mx;
        });
        const T first = __shfl(x[j][0], (threadIdx.x % DH_WAVE) - lane, DH_WAVE); // lane 0 of the group holds column 0
        if (first != first)
            mx = first;
        T sum = T(0);
#pragma unroll
        for (int k = 0; k < KEEP; k++) {
            const size_t c = lane + static_cast<size_t>(k) * G;
            if (c < cols) {
                x[j][k] = dev_exp<T>(x[j][k] - mx);
                sum += x[j][k];
            }
        }
        dh_butterfly(G, [&](auto peer) { sum += peer(sum); });
        const T inv = T(1) / sum;
        if (r < rows) {
#pragma unroll
            for (int k = 0; k < KEEP; k++) {
                const size_t c = lane + static_cast<size_t>(k) * G;
                if (c < cols)
                    res[r * ld_res + c] = x[j][k] * inv;
            }
        }
    }
}

// Short rows that are no multiple of 8 values (10 classes, say) waste most lanes of a lane group and give every
// wavefront load a few dozen scattered bytes. For contiguous matrices of such rows a workgroup copies 256 rows into
// LDS with whole 16-byte vectors, every thread then handles one row there (sequential max, exp and sum as the
// reference, Softmax.h:36-52), and the rows leave again as whole vectors.
template <typename T, int RPT>
__global__ __launch_bounds__(256) void softmax_lds_kernel(T *res, const T *arg, size_t rows, unsigned cols) {
    constexpr int VEC = 16 / sizeof(T), UN = 4;
    constexpr unsigned ROWS = 256 * RPT; // rows per workgroup, RPT per thread
    extern __shared__ __attribute__((aligned(16))) unsigned char softmax_lds[];
    T *buf = reinterpret_cast<T *>(softmax_lds); // ROWS rows x cols
    const unsigned tid = threadIdx.x;
    const size_t r0 = static_cast<size_t>(blockIdx.x) * ROWS;
    const unsigned nrows = rows - r0 < ROWS ? static_cast<unsigned>(rows - r0) : ROWS;
    const unsigned n = nrows * cols, nvec = n / VEC;
    const T *src = arg + r0 * cols; // 16-byte aligned: a multiple of 256 * cols values per workgroup
    T *dst = res + r0 * cols;
    for (unsigned v0 = tid; v0 < nvec; v0 += 256 * UN) {
        T t[UN][VEC];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const unsigned v = v0 + u * 256;
            dh_load_vec_stream<T, VEC>(src + static_cast<size_t>(v < nvec ? v : v0) * VEC, t[u]);
        }
#pragma unroll
        for (int u = 0; u < UN; u++)
            if (v0 + u * 256 < nvec)
                dh_store_vec<T, VEC>(buf + static_cast<size_t>(v0 + u * 256) * VEC, t[u]);
    }
    if (tid < n - nvec * VEC)
        buf[nvec * VEC + tid] = src[nvec * VEC + tid];
    __syncthreads();
#pragma unroll
    for (int q = 0; q < RPT; q++) {
        const unsigned rl = tid + 256 * q;
        if (rl >= nrows)
            break;
        T *row = buf + rl * cols;
        // max: NaN anywhere in the row ends up in every output through the sum, as on the CPU
        T mx = -std::numeric_limits<T>::infinity();
        for (unsigned c = 0; c < cols; c++) {
            const T v = row[c];
            mx = (mx < v) ? v : mx;
        }
        const T first = row[0];
        if (first != first)
            mx = first;
        T sum = T(0);
        for (unsigned c = 0; c < cols; c++) {
            const T e = dev_exp<T>(row[c] - mx);
            row[c] = e;
            sum += e;
        }
        const T inv = T(1) / sum;
        for (unsigned c = 0; c < cols; c++)
            row[c] *= inv;
    }
    __syncthreads();
    for (unsigned v = tid; v < nvec; v += 256) {
        T t[VEC];
        dh_load_vec<T, VEC>(buf + static_cast<size_t>(v) * VEC, t);
        dh_store_vec_stream<T, VEC>(dst + static_cast<size_t>(v) * VEC, t);
    }
    if (tid < n - nvec * VEC)
        dst[nvec * VEC + tid] = buf[nvec * VEC + tid];
}

template <typename T>
dh_status softmax(dh_ctx *ctx, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols || ld_res < cols)
        return dh_fail(DH_ERR_RUNTIME, "Softmax - a leading dimension is smaller than the column count");
    if (rows == 0 || cols == 0)
        return DH_OK;
    if (cols <= 32 && cols % 8 != 0 && ld == cols && ld_res == cols && dh_aligned(arg, 16) && dh_aligned(res, 16) &&
        rows >= 1024 && dh_ceil_div(rows, static_cast<size_t>(256)) < (size_t(1) << 31)) {
        // two rows a thread where that keeps a workgroup's LDS at 20 KB and still leaves two workgroups per CU: 1M x 10
        // floats 15.4 -> 12.6 us (40 KB of LDS for the same in double: slower)
        if (512 * cols * sizeof(T) <= 20480 && rows >= (size_t(1) << 18))
            hipLaunchKernelGGL((softmax_lds_kernel<T, 2>), dim3(static_cast<unsigned>(dh_ceil_div(rows, static_cast<size_t>(512)))), dim3(256),
                               512 * cols * sizeof(T), ctx->stream, res, arg, rows, static_cast<unsigned>(cols));
        else
            hipLaunchKernelGGL((softmax_lds_kernel<T, 1>), dim3(static_cast<unsigned>(dh_ceil_div(rows, static_cast<size_t>(256)))),
                               dim3(256), 256 * cols * sizeof(T), ctx->stream, res, arg, rows, static_cast<unsigned>(cols));
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    int G = 1;
    while (G < 64 && static_cast<size_t>(G) < cols)
        G <<= 1;
    const size_t oneshot = dh_ceil_div(rows, 256 / G);
    if (cols <= static_cast<size_t>(G) * 4 && oneshot < (size_t(1) << 31)) {
        const dim3 grid(static_cast<unsigned>(dh_ceil_div(oneshot, 4))); // four rows per lane group
        if (cols <= static_cast<size_t>(G))
            hipLaunchKernelGGL((softmax_reg_kernel<T, 1>), grid, dim3(256), 0, ctx->stream, res, ld_res, arg, rows, cols, ld, G);
        else
            hipLaunchKernelGGL((softmax_reg_kernel<T, 4>), grid, dim3(256), 0, ctx->stream, res, ld_res, arg, rows, cols, ld, G);
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    size_t grid = oneshot;
    const size_t cap = static_cast<size_t>(ctx->num_cus) * 16;
    if (grid > cap)
        grid = cap;
    hipLaunchKernelGGL((softmax_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, res, ld_res,
                       arg, rows, cols, ld, G);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

} // namespace dh_dnn
