// Scatterbrain-local attention forward for gfx950.
//
// Kernels:
//   sb_kfeat_kernel   : workgroups take one of two roles.  Key role, per (batch, head, range of
//                       64-key chunks): positive random features of the keys (projection on fp32
//                       MFMA, wavefront max reductions, exp), written to HBM once, plus the partial
//                       K'^T V / sum K' reductions with an online rescale to the running maximum.
//                       Query role (small problems only): the features of 64 queries.
//   sb_combine_kernel : merges the partial reductions of one (batch, head) (large problems; on small
//                       ones extra workgroups of the band kernel's launch do it).
//   sblocal_fwd_kernel: per (batch, head, 64-query tile, part of the band): query features in
//                       registers, then for each 32-key tile of its share of the band Q K^T and
//                       Q' K'^T on MFMA (transposed, so that every lane owns one query),
//                       band/length masking, online softmax with the low-rank overlap subtracted,
//                       P V on MFMA; key tiles are double-buffered through LDS.  With one part the
//                       epilogue adds the global low-rank term and writes out / log-normaliser;
//                       with several parts (small problems, to fill the chip) each part writes an
//                       un-normalised partial and sb_merge_kernel finishes the job: it merges the
//                       parts and adds the global low-rank term.
//
// Layout of an MFMA 16x16 result in a lane (r = lane%16, g = lane/16): element i is
// C[4g+i][r].  All products are formed "transposed" (rows = keys / features / value dims,
// columns = queries) so that r indexes the lane's query and the four register elements index
// consecutive keys/features -- which is exactly the operand layout the next product needs.
#include "common.h"
#include <hip/hip_ext.h>
#include <math.h>
#include <type_traits>
#include <atomic>

namespace flyhip {

constexpr int CH = 64;     // keys per feature chunk (granularity of the key-side stabiliser)
constexpr int TK = 32;     // keys per tile of the fused band kernel
constexpr int TQ = 64;     // queries per workgroup of the fused band kernel
constexpr int NT = 256;    // threads per workgroup (4 waves)
constexpr int NSTAT = 5;   // per-query statistics of a partial: m, ze, zp, qk1, lsq+kmax

// Optional phase timestamps of the fused kernel (a development build, -DFLY_PROFILE, reads them
// back through flyhip_prof_read); compiled out of the shipped library.
#ifdef FLY_PROFILE
__device__ long long g_prof[16384 * 8];
#define FLY_PROF(slot)                                                                                   \
    do {                                                                                                 \
        if (threadIdx.x == 0) {                                                                          \
            const int wg_ = blockIdx.x;                                                                  \
            if (wg_ < 16384) g_prof[wg_ * 8 + (slot)] = wall_clock64();                                  \
        }                                                                                                \
    } while (0)
// (shader-clock stamps inside one iteration of the band kernel's key loop)
__device__ long long g_prof2[16384 * 16];
#define FLY_PROF2(cond, slot)                                                                            \
    do {                                                                                                 \
        if ((cond) && threadIdx.x == 0 && blockIdx.x < 16384) g_prof2[blockIdx.x * 16 + (slot)] = __builtin_readcyclecounter(); \
    } while (0)
// (the same for waves 0 and 4 of a workgroup: slots 0..7 and 8..15)
#define FLY_PROF3(cond, slot)                                                                            \
    do {                                                                                                 \
        if ((cond) && (threadIdx.x & 0x1bf) == 0 && blockIdx.x < 16384)                                  \
            g_prof2[blockIdx.x * 16 + (threadIdx.x >> 8) * 8 + (slot)] = __builtin_readcyclecounter();   \
    } while (0)
// (the key pass has its own table: its grid is two-dimensional)
__device__ long long g_prof_k[4096 * 8];
#define FLY_PROFK(slot)                                                                                  \
    do {                                                                                                 \
        if (threadIdx.x == 0) {                                                                          \
            const int wg_ = blockIdx.y * gridDim.x + blockIdx.x;                                         \
            if (wg_ < 4096) g_prof_k[wg_ * 8 + (slot)] = wall_clock64();                                 \
        }                                                                                                \
    } while (0)
#else
#define FLY_PROF(slot)
#define FLY_PROF2(cond, slot)
#define FLY_PROF3(cond, slot)
#define FLY_PROFK(slot)
#endif

struct KvArgs {
    const void* k; const void* v; const float* proj; const int64_t* lens;
    void* kfeat; float* chunk_scale; float* kv_part; float* part_max;
    int B, H, S, mh_valid, n_chunks, n_split;
    long k_sb, k_sh, k_ss, v_sb, v_sh, v_ss;
    float temp;
    // optional query side: features of the queries and their log-scales, for the band kernel
    const void* q; float* qfeat; float* q_lsq;
    int T;
    long q_sb, q_sh, q_ss;
    int q_tiles;                    // query-role workgroups per (batch, head), after the n_split key-role ones
    void* vt;                       // bf16 inputs: V per 32-key tile, transposed ([d][k-slot]) for the band kernel's P V
    // float path with operand images only: the element type of q, k, v in memory (0 float, 1 bfloat16, 2 float16)
    int in_code = 0;
};

struct FwdArgs {
    const void* q; const void* k; const void* v; const float* proj;
    const void* kfeat; const float* chunk_scale; const float* kv; const float* ksum; const float* kmax;
    const float* qfeat; const float* q_lsq; const void* vt; const void* kvt;
    // several parts per query tile: the partial reductions of the key pass, merged by extra
    // workgroups of the band kernel's launch (ids >= band_wgs) into kv / ksum / kmax for the merge kernel
    const float* kv_part; const float* part_max; int n_split, band_wgs, cmb_wpb;    // cmb_wpb: combine workgroups per (batch, head)
    const int64_t* lens; void* out; float* log_norm; float* part_ws;
    int B, H, T, S, mh_valid, lc, n_chunks, n_parts;
    long q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss;
    float temp;
    // block-sparse support instead of a band (blocks of 16 x 16 or 32 x 32; the fp32 kernel's LIST variant): per (head,
    // 64-query tile) the 32-key tiles its block-rows touch -- tl_ptr (H * tiles + 1), tl_inner (tile per entry),
    // tl_blk (4 per entry: for queries 16 w .. 16 w + 15 of the tile bit 0 / bit 1 = keys 0..15 / 16..31 of the entry's
    // tile are on the support)
    const int32_t* tl_ptr; const int32_t* tl_inner; const int32_t* tl_blk;
    // optional: per head the query tiles in the order they should start (longest list first); an entry
    // -1 - tile marks a tile that is left to the workgroups walking long lists in parts
    const int32_t* tl_order;
    // long lists: tl_heavy (n_heavy entries head * tiles + tile) names the query tiles whose lists are walked
    // in n_parts parts: the first B * n_heavy * n_parts workgroups of the launch (rounded up to a multiple of the
    // XCD count) take one (batch, heavy entry, part) each and write a partial for the merge kernel.  They form
    // the query features themselves (part 0 leaves them in qfeat), take kmax from the combined reductions, and
    // index partials / query features by batch * n_heavy + entry.
    const int32_t* tl_heavy; int n_heavy;
    int n_xcd;                      // dies the dispatcher deals workgroup ids to (set at launch)
    // dropout of the exact weights (sblocal_attention.py:119: dropout(exp(QK - ln)); the normaliser sees no dropout):
    // drop_thresh = 0 means none; pair (query i of (batch, head) bh, key s) is kept iff
    // drop_keep(drop_row_hash(drop_seed, bh T + i), s, drop_thresh), kept weights times drop_scale (bf16-piece kernel)
    uint32_t drop_seed, drop_thresh; float drop_scale;
    // block-sparse support on operand images only: the element type of q and out in memory (0 float, 1 bfloat16, 2 float16)
    int io_code = 0;
};

// ROWS x W tile of a (seq, W) matrix, moved global -> registers -> LDS in two steps so that all of
// a thread's loads are in flight together (and, in the band kernel, fly during the MFMAs of the
// previous tile).  Row indices are clamped to `last_row`: rows past the end re-read the last valid
// row, which callers mask, so the loads need no branches and never leave the tensor.
template <int ROWS, int W>
struct RowTile {
    static constexpr int V4 = W / 4, N = (ROWS * V4 + NT - 1) / NT;
    floatx4 r[N];
    template <typename T>
    __device__ __forceinline__ void fetch(const T* src, long row_stride, int row0, int last_row, int tid) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = tid + NT * j, row = idx / V4, c4 = idx % V4;
            if (N * NT == ROWS * V4 || idx < ROWS * V4)
                r[j] = load4_f32(src + (long)min(row0 + row, last_row) * row_stride + 4 * c4);
        }
    }
    // byte offsets of this thread's pieces inside a tile whose rows all exist (computed once); with
    // them a fetch is one load per piece from a wave-uniform tile base, no address arithmetic
    template <typename T>
    __device__ __forceinline__ void offsets(uint32_t (&off)[N], long row_stride, int tid) const {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = tid + NT * j, row = idx / V4, c4 = idx % V4;
            off[j] = (uint32_t)((row * row_stride + 4 * c4) * (long)sizeof(T));
        }
    }
    template <typename T>
    __device__ __forceinline__ void fetch_fast(const T* tile_base, const uint32_t (&off)[N], int tid) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = tid + NT * j;
            if (N * NT == ROWS * V4 || idx < ROWS * V4)
                r[j] = load4_f32(reinterpret_cast<const T*>(reinterpret_cast<const char*>(tile_base) + off[j]));
        }
    }
    template <int LD>
    __device__ __forceinline__ void stash(float* dst, int tid, float scale = 1.0f) const {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = tid + NT * j, row = idx / V4, c4 = idx % V4;
            if (N * NT == ROWS * V4 || idx < ROWS * V4)
                *reinterpret_cast<floatx4*>(dst + row * LD + 4 * c4) = r[j] * scale;
        }
    }
};

// a value as the bfloat16 kernels see it: rounded to bf16.  Every product of a feature -- the overlap inside the band,
// K'^T V, sum K', q'.sum K', the global low-rank term -- must use the same rounded value, or the band's low-rank part and
// the global term no longer cancel to more than three digits.
__device__ __forceinline__ float bf16_round(float x) { return bf16_to_f32(f32_to_bf16(x)); }
__device__ __forceinline__ floatx4 bf16_round(floatx4 x) {
    floatx4 r = {bf16_round(x[0]), bf16_round(x[1]), bf16_round(x[2]), bf16_round(x[3])};
    return r;
}

// every value of the rows a RowTile holds -> the sum of its two bf16 pieces (head and rounded rest)
template <int ROWS, int W>
__device__ __forceinline__ void round_to_pieces2(RowTile<ROWS, W>& t) {
#pragma unroll
    for (int j = 0; j < RowTile<ROWS, W>::N; ++j) {
        uint2 h, l;
        split2_4(t.r[j], h, l);
        t.r[j] = floatx4{__uint_as_float(h.x << 16) + __uint_as_float(l.x << 16),
                         __uint_as_float(h.x & 0xffff0000u) + __uint_as_float(l.x & 0xffff0000u),
                         __uint_as_float(h.y << 16) + __uint_as_float(l.y << 16),
                         __uint_as_float(h.y & 0xffff0000u) + __uint_as_float(l.y & 0xffff0000u)};
    }
}

// K'^T V for the global low-rank term on the bf16 matrix pipe.  stash_pieces3: the rows a RowTile holds -> three bf16
// pieces in LDS ([h | m | l], M * 2 COLS bytes apart; rows of 2 COLS bytes in natural element order, 16-byte chunks
// swizzled): exact to fp32.  lowrank_pieces: lacc^T[d][query] += sum_f KV[f][d] q'[query][f] from those pieces, read
// transposed (k = feature), and the query features in two pieces (exact: they are rounded to 17 bits where they are
// formed); lane's k-slots of step ks are features 32 ks + 4 g + j and 32 ks + 16 + 4 g + j, as the overlap product
// holds them.  Five piece products, everything above 2^-24: the term cancels against the band's own low-rank part.
template <int M, int COLS>
__device__ __forceinline__ void stash_pieces3(const RowTile<M, COLS>& t, char* dst, int tid) {
    constexpr int V4 = COLS / 4, ROWB = 2 * COLS, PIECE = M * ROWB;
    static_assert(COLS >= 32, "the chunk swizzle needs rows of four chunks or more");
#pragma unroll
    for (int j = 0; j < RowTile<M, COLS>::N; ++j) {
        const int idx = tid + NT * j, row = idx / V4, c4 = idx % V4;
        if (RowTile<M, COLS>::N * NT == M * V4 || idx < M * V4) {
            uint2 h, m, l;
            split3_4(t.r[j], h, m, l);
            char* d = dst + row * ROWB + x3_swz(row, c4 >> 1, ROWB) * 16 + 8 * (c4 & 1);
            *reinterpret_cast<uint2*>(d) = h;
            *reinterpret_cast<uint2*>(d + PIECE) = m;
            *reinterpret_cast<uint2*>(d + 2 * PIECE) = l;
        }
    }
}
template <int M, int COLS, int NDB>
__device__ __forceinline__ void lowrank_pieces(const char* kvp, const uintx4 (&qh)[M / 32], const uintx4 (&ql)[M / 32],
                                               floatx4 (&lacc)[NDB], int r16, int g) {
    constexpr int ROWB = 2 * COLS, PIECE = M * ROWB;
    const int tr_row = 4 * g + (r16 >> 2), cb = r16 & 3;
#pragma unroll
    for (int ks = 0; ks < M / 32; ++ks)
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            const int row = 32 * ks + tr_row;
            const char* p = kvp + row * ROWB + x3_swz(row, 2 * db + (cb >> 1), ROWB) * 16 + 8 * (cb & 1);
            const uintx4 kh = lds_read_tr8(p, p + 16 * ROWB), km = lds_read_tr8(p + PIECE, p + PIECE + 16 * ROWB);
            const uintx4 kl = lds_read_tr8(p + 2 * PIECE, p + 2 * PIECE + 16 * ROWB);
            lacc[db] = mma_bf16(kl, qh[ks], lacc[db]);
            lacc[db] = mma_bf16(km, ql[ks], lacc[db]);
            lacc[db] = mma_bf16(km, qh[ks], lacc[db]);
            lacc[db] = mma_bf16(kh, ql[ks], lacc[db]);
            lacc[db] = mma_bf16(kh, qh[ks], lacc[db]);
        }
}

// projection matrix (MH, E) -> LDS rows of E+4 floats, scaled by sqrt(t)
template <int E, int MH>
__device__ __forceinline__ void load_proj(float* Ps, const float* proj, float scale, int tid) {
    RowTile<MH, E> t;
    t.fetch(proj, E, 0, MH - 1, tid);
    t.template stash<E + 4>(Ps, tid, scale);
}

// projection matrix (MH, E) times `scale` -> three bf16 pieces in LDS ([h | m | l], MH * 2 E bytes apart; rows of 2 E
// bytes with position 32 ks + 8 g + 4 h + i <- element 32 ks + 16 h + 4 g + i, the k-slot order of an operand that
// is split from fragments of elements 16 c + 4 g + i; 16-byte chunks swizzled): exact to fp32
template <int E, int MH>
__device__ __forceinline__ void load_proj_pieces(char* Pp, const float* proj, float scale, int tid) {
    constexpr int CH8 = E / 8, ROWB = 2 * E, PIECE = MH * ROWB;
    for (int idx = tid; idx < MH * CH8; idx += NT) {
        const int row = idx / CH8, cch = idx % CH8, ks = cch >> 2, gq = cch & 3;
        const float* sp = proj + (long)row * E + 32 * ks + 4 * gq;
        uintx4 h, m, l;
        split3(*reinterpret_cast<const floatx4*>(sp) * scale, *reinterpret_cast<const floatx4*>(sp + 16) * scale, h, m, l);
        char* d = Pp + row * ROWB + x3_swz(row, cch, ROWB) * 16;
        *reinterpret_cast<uintx4*>(d) = h;
        *reinterpret_cast<uintx4*>(d + PIECE) = m;
        *reinterpret_cast<uintx4*>(d + 2 * PIECE) = l;
    }
}

// KV = sum_s exp(part_max_s - kmax) KV_s, same for Ksum, of one (batch, head) by `wpb` workgroups
// (this is number `ci` of them; the output elements are dealt to their threads round-robin), the
// weights staged in LDS (`wgt`, n_split floats) so that the loads over s are independent and stay
// in flight together
constexpr int MAX_SPLIT = 1024;
#ifndef FLY_CMB_BATCH
#define FLY_CMB_BATCH 25
#endif
constexpr int CMB_BATCH = FLY_CMB_BATCH;     // partial reductions whose loads a combining thread keeps in flight together
__device__ __forceinline__ void sb_combine_body(float* wgt, const float* kv_part, const float* part_max, float* kv,
                                                float* ksum, float* kmax_out, uint16_t* kvt, int bh, int ci, int wpb,
                                                int n_split, int M, int D) {
    const int nthr = blockDim.x;
    const int per = M * (D + 1);
    float kmax = -INFINITY;
    for (int s = 0; s < n_split; ++s) kmax = fmaxf(kmax, part_max[(long)bh * n_split + s]);
    for (int s = threadIdx.x; s < n_split; s += nthr) {
        const float pm = part_max[(long)bh * n_split + s];
        // same expression as the band kernel's chunk weight, so that both sides of the
        // "global minus band" low-rank difference carry bit-identical factors
        wgt[s] = (pm == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((pm - kmax) * 1.4426950408889634f);
    }
    __syncthreads();
    if (ci == 0 && threadIdx.x == 0) kmax_out[bh] = (kmax == -INFINITY) ? 0.f : kmax;
    // Threads walk a partial in its storage order, four consecutive floats each (16-byte loads, coalesced
    // over the splits), in batches of CMB_BATCH splits whose loads are all in flight together: the partials come
    // from memory, and one round trip per split would make this the longest job of the launch.  The K'^T V
    // part is in accumulator order: offset ((tile*64 + lane)*4 + i) holds element (r, d) of tile (r/16, d/16)
    // with lane = 16*((r%16)/4) + d%16 and i = r%4.
    const int per4 = per / 4;                                   // M (D + 1) is a multiple of 4
    for (int q4 = ci * nthr + threadIdx.x; q4 < per4; q4 += wpb * nthr) {
        const floatx4* src = reinterpret_cast<const floatx4*>(kv_part + (long)bh * n_split * per) + q4;
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int s0 = 0; s0 < n_split; s0 += CMB_BATCH) {
            floatx4 pv[CMB_BATCH];
#pragma unroll
            for (int u = 0; u < CMB_BATCH; ++u) pv[u] = src[(long)min(s0 + u, n_split - 1) * per4];
#pragma unroll
            for (int u = 0; u < CMB_BATCH; ++u)
                if (s0 + u < n_split) acc += wgt[s0 + u] * pv[u];
        }
        const int idx = 4 * q4;
        if (idx < M * D) {
            const int lane = (idx >> 2) & 63, tile = idx >> 8;
            const int db_n = D >> 4, rb = tile / db_n, db = tile % db_n;
            const int r0 = 16 * rb + 4 * (lane >> 4), d = 16 * db + (lane & 15);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = r0 + i;
                kv[(long)bh * M * D + r * D + d] = acc[i];
                if (kvt) {      // bf16 copy for the bf16 band kernel: [d][slot], feature r in the k-slot order of its MFMA
                    const int c = r >> 4, slot = 32 * (c >> 1) + 8 * ((r >> 2) & 3) + 4 * (c & 1) + (r & 3);
                    // two pieces, M D elements apart: the term cancels against the band's low-rank part, and one bf16
                    // (three digits) of it would show in the result
                    const uint16_t hi = f32_to_bf16(acc[i]);
                    kvt[(long)bh * 2 * M * D + d * M + slot] = hi;
                    kvt[(long)bh * 2 * M * D + (long)M * D + d * M + slot] = f32_to_bf16(acc[i] - bf16_to_f32(hi));
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) ksum[(long)bh * M + idx - M * D + i] = acc[i];
        }
    }
}

__global__ __launch_bounds__(NT) void sb_combine_kernel(const float* kv_part, const float* part_max, float* kv,
                                                        float* ksum, float* kmax_out, uint16_t* kvt, int n_split,
                                                        int M, int D) {
    __shared__ float wgt[MAX_SPLIT];
    sb_combine_body(wgt, kv_part, part_max, kv, ksum, kmax_out, kvt, blockIdx.y, blockIdx.x, gridDim.x, n_split, M, D);
}

// The band kernels' view of the same maximum when the combine shares their launch (several parts per
// query tile): every wave reduces the partial maxima itself.
__device__ __forceinline__ float split_kmax(const float* part_max, int bh, int n_split) {
    float pm = -INFINITY;
    for (int s = threadIdx.x & 63; s < n_split; s += 64) pm = fmaxf(pm, part_max[(long)bh * n_split + s]);
    pm = wave_max(pm);
    return pm == -INFINITY ? 0.f : pm;
}

// ---------------------------------------------------------------------------------------
// key features + partial K'^T V
// ---------------------------------------------------------------------------------------
// One block of 16 features (block fbp of the [positive | negative] feature row; the lane holds
// features 16 fbp + 4g + i) of one key goes to the feature scratch.  float inputs: fp32, natural
// feature order.  bfloat16 inputs: bf16, in the order the 16x16x32 MFMA of the band kernel consumes
// (position 32 ks + 8 g + j holds feature 32 ks + 16 (j / 4) + 4 g + j % 4, so that a lane's eight
// k-slots are 16 contiguous bytes and the query features need no shuffle either).
template <typename T>
__device__ __forceinline__ void store_feat(void* kfeat, long row, int M, int fbp, int g, floatx4 f) {
    if (sizeof(T) == 4) {
        *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(kfeat) + row * M + 16 * fbp + 4 * g) = f;
    } else {
        uint2 u;
        u.x = pack_bf16x2(f[0], f[1]);
        u.y = pack_bf16x2(f[2], f[3]);
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(kfeat) + row * M + 32 * (fbp >> 1) + 8 * g + 4 * (fbp & 1)) = u;
    }
}

// stores of data that the next launch reads (tile images, partial results)
#if !defined(FLY_PLAIN_STORES)
// write-through to memory (device scope): nothing of it is left dirty in the L2 when the kernel ends (the
// write-back of megabytes of dirty lines at the end of a launch is time nothing overlaps), and a workgroup
// on another XCD that reads the line for the first time in its launch finds the data in memory
template <typename V>
__device__ __forceinline__ void store16_wt(V val, V* ptr) {
    static_assert(sizeof(V) == 16, "16-byte pieces");
    // (the wait states keep a following VALU write away from the data registers, which a store of more than
    // eight bytes reads a little after it issues; the compiler does that for its own stores)
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(ptr), "v"(val) : "memory");
}
#define FLY_STORE(val, ptr) store16_wt((val), (ptr))
#elif defined(FLY_NT_STORES)
#define FLY_STORE(val, ptr) __builtin_nontemporal_store((val), (ptr))
#else
#define FLY_STORE(val, ptr) (*(ptr) = (val))
#endif

// ---------------------------------------------------------------------------------------
// fp32 inputs on the bf16 matrix pipe: operands as sums of bf16 pieces
// ---------------------------------------------------------------------------------------
// The band kernel for float inputs forms its three products on v_mfma_f32_16x16x32_bf16 (16 times the
// rate of the fp32 MFMA) from operands split into bf16 pieces, x = hi + lo (+ a third piece), with
// fp32 accumulation.  Products of bf16 pairs are exact in fp32, so a product that takes every pair of
// pieces above the fp32 rounding level is as accurate as the fp32 MFMA:
//   features : q', k' are ROUNDED TO 16 SIGNIFICANT BITS where they are formed (key pass), two pieces
//              represent them exactly, and all four piece products are taken: the overlap q'.k' of the
//              band is then the exact product of the same numbers whose sums over all keys the global
//              low-rank term uses (also formed from the rounded features), so the "all keys minus the
//              band" difference cancels as well as it does in fp32 arithmetic.  The rounding itself
//              perturbs a feature by 2^-17 relative, consistently everywhere.
//   scores   : q, k in two pieces, three products (the lo.lo product, 2^-16 relative, is dropped: an
//              error in an exponent, not in a difference).
//   P V      : probabilities in three pieces (exact), values in X3_VP pieces: two (V rounded to 16 bits, five products;
//              K'^T V of the key pass multiplies the same rounded V) or three (exact, six products).
// The key pass leaves every 32-key tile as an image of what the band kernel wants in LDS: in the
// feature / operand scratch, per tile, [K hi][K lo][V^T h][V^T m]([V^T l]) (the "kv image") and
// [K' hi][K' lo] (the "feature image"); rows of K and K' in the k-slot order of the MFMA, V
// transposed to [d][key slot], and the 16-byte chunks of every row XOR-swizzled so that the
// fragment reads of 8 consecutive rows fall into different LDS banks without padding.
// bf16 pieces of V in the images: two carry 16 significant bits of V -- every product that involves V (P V in the band
// kernel, K'^T V in the key pass) then uses the same rounded V, so the cancellation between the band's low-rank part and
// the global term is untouched and the result moves by at most 2^-17 |V| -- three are exact to fp32 and cost a sixth more
// matrix and LDS work per tile.
#ifndef FLY_X3_VP
#define FLY_X3_VP 2
#endif
constexpr int X3_VP = FLY_X3_VP;
static_assert(X3_VP == 2 || X3_VP == 3, "two or three pieces");
template <int E, int D, int M>
struct X3Tile {
    static constexpr int K_ROW = 2 * E, F_ROW = 2 * M, V_ROW = 2 * TK;           // bytes per row
    static constexpr int K_PIECE = TK * K_ROW, F_PIECE = TK * F_ROW, V_PIECE = D * V_ROW;
    static constexpr int KV_BYTES = 2 * K_PIECE + X3_VP * V_PIECE;                // per tile, operand scratch
    static constexpr int F_BYTES = 2 * F_PIECE;                                   // per tile, feature scratch
    static constexpr int BYTES = KV_BYTES + F_BYTES;                              // one LDS stage
};
// 64 rows x W floats in LDS (row stride LD floats) -> the two-piece images of the two 32-row tiles:
// position 32ks + 8g + 4h + i of a row <- element 32ks + 16h + 4g + i (the k-slot order of the MFMA)
template <int W, int LD>
__device__ __forceinline__ void x3_emit_rows(const float* src, char* tile0, long tile_stride, int piece_bytes, int tid) {
    constexpr int CH8 = W / 8, ROWB = 2 * W, TOT = CH * CH8;
#pragma unroll
    for (int j = 0; j < (TOT + NT - 1) / NT; ++j) {
        const int idx = tid + NT * j;
        if (TOT % NT == 0 || idx < TOT) {
            const int row64 = idx / CH8, cch = idx % CH8, ks = cch >> 2, gq = cch & 3, row = row64 & (TK - 1);
            const float* sp = src + row64 * LD + 32 * ks + 4 * gq;
            uintx4 hi, lo;
            split2(*reinterpret_cast<const floatx4*>(sp), *reinterpret_cast<const floatx4*>(sp + 16), hi, lo);
            char* dst = tile0 + (row64 / TK) * tile_stride + row * ROWB + x3_swz(row, cch, ROWB) * 16;
            *reinterpret_cast<uintx4*>(dst) = hi;
            *reinterpret_cast<uintx4*>(dst + piece_bytes) = lo;
        }
    }
}
// 64 keys x D floats in LDS -> the three-piece transposed images [d][key slot] of the two 32-key tiles:
// slot 8g + j of a tile <- key 16 (j / 4) + 4 g + j % 4 (the order in which score tiles leave the probabilities)
// (with `gtile0` the same pieces also go to global memory, tiles `gtile_stride` bytes apart, write-through)
template <int D, int LD>
__device__ __forceinline__ void x3_emit_vt(const float* src, char* tile0, long tile_stride, int tid,
                                           char* gtile0 = nullptr, long gtile_stride = 0) {
    constexpr int TOT = 2 * D * 4, PIECE = D * 2 * TK;
#pragma unroll
    for (int j = 0; j < (TOT + NT - 1) / NT; ++j) {
        const int idx = tid + NT * j;
        if (TOT % NT == 0 || idx < TOT) {
            const int tile = idx / (4 * D), rem = idx % (4 * D), d = rem >> 2, gq = rem & 3;
            const float* col = src + (TK * tile + 4 * gq) * LD + d;
            const floatx4 x0 = {col[0], col[LD], col[2 * LD], col[3 * LD]};
            const floatx4 x1 = {col[16 * LD], col[17 * LD], col[18 * LD], col[19 * LD]};
            uintx4 h, m, l;
            if (X3_VP == 3) split3(x0, x1, h, m, l); else split2(x0, x1, h, m);
            char* dst = tile0 + tile * tile_stride + d * (2 * TK) + x3_swz(d, gq, 2 * TK) * 16;
            *reinterpret_cast<uintx4*>(dst) = h;
            *reinterpret_cast<uintx4*>(dst + PIECE) = m;
            if (X3_VP == 3) *reinterpret_cast<uintx4*>(dst + 2 * PIECE) = l;
            if (gtile0) {
                char* gd = gtile0 + tile * gtile_stride + d * (2 * TK) + x3_swz(d, gq, 2 * TK) * 16;
                FLY_STORE(h, reinterpret_cast<uintx4*>(gd));
                FLY_STORE(m, reinterpret_cast<uintx4*>(gd + PIECE));
                if (X3_VP == 3) FLY_STORE(l, reinterpret_cast<uintx4*>(gd + 2 * PIECE));
            }
        }
    }
}

// two waves per SIMD (two workgroups per CU) where the register budget allows it without spilling
constexpr int kfeat_waves(int E, int M) { return (E <= 64 && M <= 128) ? 2 : 1; }

template <typename T, int E, int D, int M, bool X3 = false>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(kfeat_waves(E, M), kfeat_waves(E, M))))
void sb_kfeat_kernel(KvArgs a) {
    static_assert(!X3 || sizeof(T) == 4, "piece images are for float inputs");
    typedef X3Tile<E, D, M> TL;
    constexpr int MH = M / 2, LDK = E + 4, LDV = D + 4, LDF = M + 4;
    constexpr int FB = MH / 16, EC = E / 16, DB = D / 16;
    constexpr int RB = (M / 16 + 3) / 4;         // K'^T V row blocks per wave
    constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
    extern __shared__ __attribute__((aligned(128))) float smem[];
    float* Ks = smem;                             // 64-key K tile
    float* Vs = Ks + CH * LDK;                    // 64-key V tile
    float* Fs = Vs + CH * LDV;                    // features of the current chunk
    float* red = Fs + CH * LDF;                   // 4 wave maxima

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H, sp = blockIdx.x;
    // projection fragments (A side: row = feature 16fb + r16, k = 16cc + 4g + j) come straight from
    // global memory: the matrix is small and stays in the L1/L2 caches
    const float* pp = a.proj + r16 * E + 4 * g;

    FLY_PROFK(0);
    if (sp >= a.n_split) {
        // Query role (workgroups past the key splits, present when the caller asks for query
        // features): q' = exp(+-sqrt(t) P q - max) of 64 queries, one per lane column, with the
        // per-query log-scale lsq = -t|q|^2/2 + max - log(2 mh)/2.  Lane (r16, g) ends with features
        // 16c + 4g + i of query 16w + r16, the B-side operand layout of the band kernel.
        const int iq = (sp - a.n_split) * TQ + 16 * w + r16;
        const T* qrow = reinterpret_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh + (long)min(iq, a.T - 1) * a.q_ss;
        floatx4 qr[EC];
        float sq = 0.f;
#pragma unroll
        for (int c = 0; c < EC; ++c) {
            qr[c] = load4_f32(qrow + 16 * c + 4 * g);
            sq += qr[c][0] * qr[c][0] + qr[c][1] * qr[c][1] + qr[c][2] * qr[c][2] + qr[c][3] * qr[c][3];
        }
        const float diag_q = 0.5f * a.temp * group_sum(sq);
        const float st = sqrtf(a.temp);
        floatx4 qf[FB];
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) qf[fb] = Frag<float>::zero();
#pragma unroll
        for (int c = 0; c < EC; ++c) {                      // the FB accumulation chains advance together
            floatx4 pa[FB];
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) pa[fb] = *reinterpret_cast<const floatx4*>(pp + 16 * fb * E + 16 * c) * st;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int fb = 0; fb < FB; ++fb)
                    qf[fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[fb][j], qr[c][j], qf[fb], 0, 0, 0);
        }
        float qmax = 0.f;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (16 * fb + 4 * g + i < a.mh_valid) qmax = fmaxf(qmax, fabsf(qf[fb][i]));
        qmax = group_max(qmax);
        if (iq < a.T) {
            float* dst = a.qfeat + ((long)bh * a.T + iq) * M;
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                floatx4 fp, fn;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool ok = 16 * fb + 4 * g + i < a.mh_valid;
                    fp[i] = ok ? __expf(qf[fb][i] - qmax) : 0.f;
                    fn[i] = ok ? __expf(-qf[fb][i] - qmax) : 0.f;
                }
                if (X3) { fp = quant16(fp); fn = quant16(fn); }
                if (sizeof(T) == 2) { fp = bf16_round(fp); fn = bf16_round(fn); }
                *reinterpret_cast<floatx4*>(dst + 16 * fb + 4 * g) = fp;
                *reinterpret_cast<floatx4*>(dst + MH + 16 * fb + 4 * g) = fn;
            }
            if (g == 0) a.q_lsq[(long)bh * a.T + iq] = -diag_q + qmax - 0.5f * __logf(2.0f * a.mh_valid);
        }
        FLY_PROFK(6);
        return;
    }

    const T* kptr = reinterpret_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh;
    const T* vptr = reinterpret_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half2 = 0.5f * __log2f(2.0f * a.mh_valid);      // base-2 from here on

    const int per = (a.n_chunks + a.n_split - 1) / a.n_split;
    const int c0 = sp * per, c1 = min(a.n_chunks, c0 + per);
    RowTile<CH, E> kt;
    RowTile<CH, D> vt;
    if (c0 < c1) {
        kt.fetch(kptr, a.k_ss, c0 * CH, a.S - 1, tid);
        vt.fetch(vptr, a.v_ss, c0 * CH, a.S - 1, tid);
    }
    const float pscale = sqrtf(a.temp) * LOG2E;                      // projections come out in base-2 units
    if (c0 < c1) {
        kt.template stash<LDK>(Ks, tid);
        if (X3 && X3_VP == 2) round_to_pieces2(vt);      // K'^T V multiplies the V the band kernel sees: its two pieces
        vt.template stash<LDV>(Vs, tid);
    }
    __syncthreads();

    FLY_PROFK(1);
    floatx4 kvacc[RB][DB];
#pragma unroll
    for (int x = 0; x < RB; ++x)
#pragma unroll
        for (int db = 0; db < DB; ++db) kvacc[x][db] = Frag<float>::zero();
    floatx4 ksp[FB], ksn[FB];                    // running sums of this lane's key column of K'
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) { ksp[fb] = Frag<float>::zero(); ksn[fb] = Frag<float>::zero(); }
    float run_max = -INFINITY;                   // base-2 running maximum of the chunk stabilisers

    for (int c = c0; c < c1; ++c) {
        const int s_base = c * CH;
        if (sizeof(T) == 2 && a.vt) {
            // the chunk's V, as two 32-key tiles [d][slot] with slot 8g+j = key 16(j/4) + 4g + j%4: the
            // k-slot order of the band kernel's P V product, so that it can copy 16-byte pieces
            uint16_t* vt = reinterpret_cast<uint16_t*>(a.vt) + ((long)bh * a.n_chunks + c) * (CH * D);
#pragma unroll
            for (int j = 0; j < CH * D / 8 / NT; ++j) {
                const int ci = tid + NT * j, tile = ci / (D * 4), rem = ci % (D * 4), d = rem / 4, c8 = rem % 4;
                const float* col = Vs + (32 * tile + 4 * c8) * LDV + d;          // key 4 c8 of the tile, dim d
                const uint4 u = make_uint4(pack_bf16x2(col[0], col[LDV]), pack_bf16x2(col[2 * LDV], col[3 * LDV]),
                                           pack_bf16x2(col[16 * LDV], col[17 * LDV]), pack_bf16x2(col[18 * LDV], col[19 * LDV]));
                *reinterpret_cast<uint4*>(vt + tile * (D * 32) + d * 32 + 8 * c8) = u;
            }
        }
        if (c + 1 < c1) {                        // next chunk's K and V fly during this chunk's work
            kt.fetch(kptr, a.k_ss, s_base + CH, a.S - 1, tid);
            vt.fetch(vptr, a.v_ss, s_base + CH, a.S - 1, tid);
        }
        char* kv_img = nullptr;
        char* f_img = nullptr;
        if (X3) {
            // the chunk's two 32-key tiles as the band kernel wants them in LDS: K in two bf16 pieces, V transposed in three
            kv_img = reinterpret_cast<char*>(a.vt) + ((long)bh * a.n_chunks + c) * (2 * (long)TL::KV_BYTES);
            f_img = reinterpret_cast<char*>(a.kfeat) + ((long)bh * a.n_chunks + c) * (2 * (long)TL::F_BYTES);
            x3_emit_rows<E, LDK>(Ks, kv_img, TL::KV_BYTES, TL::K_PIECE, tid);
            x3_emit_vt<D, LDV>(Vs, kv_img + 2 * TL::K_PIECE, TL::KV_BYTES, tid);
        }
        FLY_PROFK(2);
        // projection of this wave's 16 keys, all feature blocks advancing together:
        // dd[fb][i] = log2(e) * (sqrt(t) P)[16fb+4g+i] . k[16w+r16]
        floatx4 kb[EC];
        float sq = 0.f;
#pragma unroll
        for (int cc = 0; cc < EC; ++cc) {
            kb[cc] = *reinterpret_cast<const floatx4*>(Ks + (16 * w + r16) * LDK + 16 * cc + 4 * g);
            sq += kb[cc][0] * kb[cc][0] + kb[cc][1] * kb[cc][1] + kb[cc][2] * kb[cc][2] + kb[cc][3] * kb[cc][3];
            kb[cc] *= pscale;                    // the key operand carries sqrt(t) log2(e)
        }
        const float diag2 = 0.5f * a.temp * LOG2E * group_sum(sq);
        floatx4 dd[FB];
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) dd[fb] = Frag<float>::zero();
#pragma unroll
        for (int cc = 0; cc < EC; ++cc) {
            floatx4 pa[FB];
#pragma unroll
            for (int fb = 0; fb < FB; ++fb)
                pa[fb] = *reinterpret_cast<const floatx4*>(pp + 16 * fb * E + 16 * cc);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int fb = 0; fb < FB; ++fb)
                    dd[fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[fb][j], kb[cc][j], dd[fb], 0, 0, 0);
        }
        float amax = 0.f;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (16 * fb + 4 * g + i < a.mh_valid) amax = fmaxf(amax, fabsf(dd[fb][i]));
        amax = group_max(amax);
        const bool kvalid = (s_base + 16 * w + r16) < len;
        float cs = kvalid ? (amax - diag2 - lnm_half2) : -INFINITY;
        cs = wave_max(cs);
        if (lane == 0) red[w] = cs;
        __syncthreads();
        const float lmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float new_max = fmaxf(run_max, lmax);
        const long frow_g = (long)bh * a.n_chunks * CH + s_base + 16 * w + r16;      // this lane's key row
        if (new_max == -INFINITY) {   // no valid key yet (workgroup-uniform): features are zero
            if (X3) {
                for (int idx = tid; idx < 2 * TL::F_BYTES / 16; idx += NT)
                    reinterpret_cast<uintx4*>(f_img)[idx] = uintx4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                if (X3) break;
                store_feat<T>(a.kfeat, frow_g, M, fb, g, Frag<float>::zero());
                store_feat<T>(a.kfeat, frow_g, M, FB + fb, g, Frag<float>::zero());
            }
            if (tid == 0) a.chunk_scale[(long)bh * a.n_chunks + c] = 0.f;
        } else {
            const float rescale = (run_max == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(run_max - new_max);
            run_max = new_max;
#pragma unroll
            for (int x = 0; x < RB; ++x)
#pragma unroll
                for (int db = 0; db < DB; ++db) kvacc[x][db] *= rescale;
            const float off = -diag2 - lnm_half2 - new_max;
            float* frow_s = Fs + (16 * w + r16) * LDF;
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                floatx4 fp, fn;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool ok = kvalid && (16 * fb + 4 * g + i < a.mh_valid);
                    fp[i] = ok ? __builtin_amdgcn_exp2f(dd[fb][i] + off) : 0.f;
                    fn[i] = ok ? __builtin_amdgcn_exp2f(-dd[fb][i] + off) : 0.f;
                }
                if (X3) { fp = quant16(fp); fn = quant16(fn); }     // every later use sees the rounded features
                if (sizeof(T) == 2) { fp = bf16_round(fp); fn = bf16_round(fn); }
                ksp[fb] = ksp[fb] * rescale + fp;
                ksn[fb] = ksn[fb] * rescale + fn;
                *reinterpret_cast<floatx4*>(frow_s + 16 * fb + 4 * g) = fp;
                *reinterpret_cast<floatx4*>(frow_s + MH + 16 * fb + 4 * g) = fn;
                if (!X3) {
                    store_feat<T>(a.kfeat, frow_g, M, fb, g, fp);
                    store_feat<T>(a.kfeat, frow_g, M, FB + fb, g, fn);
                }
            }
            if (tid == 0) a.chunk_scale[(long)bh * a.n_chunks + c] = new_max * LN2;    // stored in natural-log units
            __syncthreads();
            FLY_PROFK(3);
            if (X3) x3_emit_rows<M, LDF>(Fs, f_img, TL::F_BYTES, TL::F_PIECE, tid);
            FLY_PROFK(4);
            // KV[r][d] += sum_keys F[key][r] V[key][d]; lane ends with KV[16rb+4g+i][16db+r16]
#pragma unroll
            for (int kk = 0; kk < CH / 16; ++kk) {
                floatx4 vb[DB];
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int j = 0; j < 4; ++j) vb[db][j] = Vs[(16 * kk + 4 * g + j) * LDV + 16 * db + r16];
#pragma unroll
                for (int x = 0; x < RB; ++x) {
                    const int rb = w + 4 * x;
                    if (rb < M / 16) {
                        floatx4 fa;
#pragma unroll
                        for (int j = 0; j < 4; ++j) fa[j] = Fs[(16 * kk + 4 * g + j) * LDF + 16 * rb + r16];
#pragma unroll
                        for (int j = 0; j < 4; ++j)
#pragma unroll
                            for (int db = 0; db < DB; ++db)
                                kvacc[x][db] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[j], vb[db][j], kvacc[x][db], 0, 0, 0);
                    }
                }
            }
        }
        FLY_PROFK(5);
        __syncthreads();                          // everyone is done with this chunk's tiles
        if (c + 1 < c1) {
            kt.template stash<LDK>(Ks, tid);
            if (X3 && X3_VP == 2) round_to_pieces2(vt);      // K'^T V multiplies the V the band kernel sees: its two pieces
            vt.template stash<LDV>(Vs, tid);
        }
        __syncthreads();                          // next tile visible; Fs and red free again
    }

    // partial K'^T V in accumulator order (tile (rb, db) -> 64 lanes x 4 floats): 16-byte stores,
    // the combine role undoes the order
    float* part = a.kv_part + ((long)bh * a.n_split + sp) * (M * (D + 1));
#pragma unroll
    for (int x = 0; x < RB; ++x) {
        const int rb = w + 4 * x;
        if (rb < M / 16) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
                *reinterpret_cast<floatx4*>(part + ((rb * DB + db) * 64 + lane) * 4) = kvacc[x][db];
        }
    }
    // column sums of K': over the 16 key lanes of a wave (DPP), then over the 4 waves (LDS)
    float* ks_lds = Fs;                           // 4 x M floats
#pragma unroll
    for (int fb = 0; fb < FB; ++fb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float p = row16_sum(ksp[fb][i]), n = row16_sum(ksn[fb][i]);
            if (r16 == 0) {
                ks_lds[w * M + 16 * fb + 4 * g + i] = p;
                ks_lds[w * M + MH + 16 * fb + 4 * g + i] = n;
            }
        }
    __syncthreads();
    if (tid < M) part[M * D + tid] = (ks_lds[tid] + ks_lds[M + tid]) + (ks_lds[2 * M + tid] + ks_lds[3 * M + tid]);
    if (tid == 0) a.part_max[(long)bh * a.n_split + sp] = run_max * LN2;
    FLY_PROFK(6);
}

// ---------------------------------------------------------------------------------------
// key pass for float inputs with both products on the bf16 matrix pipe (tile images built in LDS)
// ---------------------------------------------------------------------------------------
// The outputs of sb_kfeat_kernel<float, .., X3 = true> -- tile images, chunk scales, partial K'^T V / sum K' --
// with the images assembled in LDS, where they double as MFMA operands:
//   projection : dd[feature][key] = (sqrt(t) log2e P) . k with P in three bf16 pieces (exact) as the row
//                operand and the K image (two pieces) as the column operand, five piece products; a lane
//                ends with four features of its key, as in sb_kfeat_kernel
//   features   : exp2, rounded to 17 bits, written as two pieces into the feature image (16-byte writes:
//                the lane's blocks 2p, 2p+1 are the eight k-slots of one chunk)
//   K'^T V     : rows = feature positions of the image (transposing LDS reads hand a lane one feature
//                column of four key rows), columns = value dims from the V^T image, five piece products;
//                the partial leaves in the natural feature order the combine step expects
// One chunk of 64 keys = two tile images = 2 * X3Tile::BYTES of LDS, copied to global memory in 16-byte
// pieces.  Instantiated where that fits next to the fp32 V chunk and the projection image (E <= 64, m <= 128).
// TIN: the element type of q, k and v in memory (float, or a 2-byte type widened as it is loaded: its values are exact
// in two bf16 pieces at most).
template <int E, int D, int M, typename TIN = float>
__global__ __launch_bounds__(NT) void sb_kfeat_x3_kernel(KvArgs a) {
    typedef X3Tile<E, D, M> TL;
    constexpr int MH = M / 2, FB = MH / 16, EC = E / 16, DB = D / 16, KS = E / 32, FS = M / 32;
    constexpr int LDV = D + 4, P_ROW = 2 * E, P_PIECE = MH * P_ROW;
    constexpr int NBLK = M / 16, RB = (NBLK + 3) / 4;      // K'^T V row blocks (of feature positions) per wave
    constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
    extern __shared__ __attribute__((aligned(128))) float smem[];
    char* img = reinterpret_cast<char*>(smem);                         // two tile images
    float* Vs = reinterpret_cast<float*>(img + 2 * TL::BYTES);         // fp32 V chunk (for the transposition)
    char* Pimg = reinterpret_cast<char*>(Vs + CH * LDV);               // projection rows, three pieces
    float* diag = reinterpret_cast<float*>(Pimg + 3 * P_PIECE);        // t log2e |k|^2 / 2 per key
    float* red = diag + CH;                                            // 4 wave maxima

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H, sp = blockIdx.x;
    FLY_PROFK(0);
    if (sp >= a.n_split) {
        // Query role: the features of 64 queries, rounded to 17 bits, and their log-scales (see sb_kfeat_kernel)
        const float* pp = a.proj + r16 * E + 4 * g;
        const int iq = (sp - a.n_split) * TQ + 16 * w + r16;
        const TIN* qrow = reinterpret_cast<const TIN*>(a.q) + b * a.q_sb + h * a.q_sh + (long)min(iq, a.T - 1) * a.q_ss;
        floatx4 qr[EC];
        float sq = 0.f;
#pragma unroll
        for (int c = 0; c < EC; ++c) {
            qr[c] = load4_f32(qrow + 16 * c + 4 * g);
            sq += qr[c][0] * qr[c][0] + qr[c][1] * qr[c][1] + qr[c][2] * qr[c][2] + qr[c][3] * qr[c][3];
        }
        const float diag_q = 0.5f * a.temp * group_sum(sq);
        const float st = sqrtf(a.temp);
        floatx4 pa[EC][FB];
#pragma unroll
        for (int c = 0; c < EC; ++c)
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) pa[c][fb] = *reinterpret_cast<const floatx4*>(pp + 16 * fb * E + 16 * c) * st;
        floatx4 qf[FB];
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) qf[fb] = Frag<float>::zero();
#pragma unroll
        for (int c = 0; c < EC; ++c)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int fb = 0; fb < FB; ++fb)
                    qf[fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[c][fb][j], qr[c][j], qf[fb], 0, 0, 0);
        float qmax = 0.f;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (16 * fb + 4 * g + i < a.mh_valid) qmax = fmaxf(qmax, fabsf(qf[fb][i]));
        qmax = group_max(qmax);
        if (iq < a.T) {
            float* dst = a.qfeat + ((long)bh * a.T + iq) * M;
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                floatx4 fp, fn;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool ok = 16 * fb + 4 * g + i < a.mh_valid;
                    fp[i] = ok ? quant16(__expf(qf[fb][i] - qmax)) : 0.f;
                    fn[i] = ok ? quant16(__expf(-qf[fb][i] - qmax)) : 0.f;
                }
                FLY_STORE(fp, reinterpret_cast<floatx4*>(dst + 16 * fb + 4 * g));
                FLY_STORE(fn, reinterpret_cast<floatx4*>(dst + MH + 16 * fb + 4 * g));
            }
            if (g == 0) a.q_lsq[(long)bh * a.T + iq] = -diag_q + qmax - 0.5f * __logf(2.0f * a.mh_valid);
        }
        FLY_PROFK(6);
        return;
    }

    const TIN* kptr = reinterpret_cast<const TIN*>(a.k) + b * a.k_sb + h * a.k_sh;
    const TIN* vptr = reinterpret_cast<const TIN*>(a.v) + b * a.v_sb + h * a.v_sh;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half2 = 0.5f * __log2f(2.0f * a.mh_valid);
    const int per = (a.n_chunks + a.n_split - 1) / a.n_split;
    const int c0 = sp * per, c1 = min(a.n_chunks, c0 + per);
    // K is fetched in the pattern of its image: piece j of a thread is 16-byte chunk idx % (E / 8) of key row
    // idx / (E / 8), i.e. elements 32 ks + 4 gq + i and 32 ks + 16 + 4 gq + i -- two quads from global memory
    constexpr int KCH8 = E / 8, KTOT = CH * KCH8, KNJ = (KTOT + NT - 1) / NT;
    static_assert(KTOT % NT == 0 && NT % KCH8 == 0, "whole key rows per pass of the workgroup");
    floatx4 kq0[KNJ], kq1[KNJ];
    auto fetch_k = [&](int s_base) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < KNJ; ++j) {
            const int idx = tid + NT * j, row64 = idx / KCH8, cch = idx % KCH8;
            const TIN* sp_ = kptr + (long)min(s_base + row64, a.S - 1) * a.k_ss + 32 * (cch >> 2) + 4 * (cch & 3);
            kq0[j] = load4_f32(sp_);
            kq1[j] = load4_f32(sp_ + 16);
        }
    };
    RowTile<CH, D> vt;
    if (c0 < c1) {
        fetch_k(c0 * CH);
        vt.fetch(vptr, a.v_ss, c0 * CH, a.S - 1, tid);
    }
    // projection rows scaled by sqrt(t) log2e, as three bf16 pieces in the k-slot order of the K image
    {
        const float pscale = sqrtf(a.temp) * LOG2E;
        constexpr int CH8 = E / 8, TOT = MH * CH8;
#pragma unroll
        for (int j = 0; j < (TOT + NT - 1) / NT; ++j) {
            const int idx = tid + NT * j;
            if (TOT % NT == 0 || idx < TOT) {
                const int row = idx / CH8, cch = idx % CH8, ks = cch >> 2, gq = cch & 3;
                const float* sp_ = a.proj + (long)row * E + 32 * ks + 4 * gq;
                uintx4 ph, pm, pl;
                split3(*reinterpret_cast<const floatx4*>(sp_) * pscale, *reinterpret_cast<const floatx4*>(sp_ + 16) * pscale, ph, pm, pl);
                char* dst = Pimg + row * P_ROW + x3_swz(row, cch, P_ROW) * 16;
                *reinterpret_cast<uintx4*>(dst) = ph;
                *reinterpret_cast<uintx4*>(dst + P_PIECE) = pm;
                *reinterpret_cast<uintx4*>(dst + 2 * P_PIECE) = pl;
            }
        }
    }
    // a chunk in registers -> K image (two pieces, into LDS and, write-through, into global memory: the stores drain
    // while the projection runs) and |k|^2 per key; V as fp32 rows for the transposition
    auto stash = [&](int c) __attribute__((always_inline)) {
        char* kv_g = reinterpret_cast<char*>(a.vt) + ((long)bh * a.n_chunks + c) * (2 * (long)TL::KV_BYTES);
#pragma unroll
        for (int j = 0; j < KNJ; ++j) {
            const int idx = tid + NT * j, row64 = idx / KCH8, cch = idx % KCH8, row = row64 & (TK - 1);
            const floatx4 x = kq0[j], y = kq1[j];
            float sq = x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3] + y[0] * y[0] + y[1] * y[1] + y[2] * y[2] + y[3] * y[3];
#pragma unroll
            for (int off = 1; off < KCH8; off <<= 1) sq += __shfl_xor(sq, off);    // the lanes of one key row
            if (cch == 0) diag[row64] = 0.5f * a.temp * LOG2E * sq;
            uintx4 khi, klo;
            split2(x, y, khi, klo);
            const int o = row * TL::K_ROW + x3_swz(row, cch, TL::K_ROW) * 16;
            char* dst = img + (row64 / TK) * TL::BYTES + o;
            *reinterpret_cast<uintx4*>(dst) = khi;
            *reinterpret_cast<uintx4*>(dst + TL::K_PIECE) = klo;
            char* gd = kv_g + (row64 / TK) * (long)TL::KV_BYTES + o;
            FLY_STORE(khi, reinterpret_cast<uintx4*>(gd));
            FLY_STORE(klo, reinterpret_cast<uintx4*>(gd + TL::K_PIECE));
        }
        vt.template stash<LDV>(Vs, tid);
    };
    if (c0 < c1) stash(c0);
    __syncthreads();
    FLY_PROFK(1);

    floatx4 kvacc[RB][DB + 1];          // column block DB: the products with a column of ones = the sums of the features
#pragma unroll
    for (int x = 0; x < RB; ++x)
#pragma unroll
        for (int db = 0; db <= DB; ++db) kvacc[x][db] = Frag<float>::zero();
    float run_max = -INFINITY;
    const int tile_w = w >> 1, row_w = 16 * (w & 1) + r16;              // this lane's key: tile and row inside it
    // the projection fragments of this lane stay in registers for all chunks (one workgroup per compute unit: the
    // register file is not what limits this kernel)
    uintx4 pf[KS][FB][3];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
            const char* pp_ = Pimg + (16 * fb + r16) * P_ROW + x3_swz(r16, 4 * ks + g, P_ROW) * 16;
#pragma unroll
            for (int pc = 0; pc < 3; ++pc) pf[ks][fb][pc] = *reinterpret_cast<const uintx4*>(pp_ + pc * P_PIECE);
        }

    for (int c = c0; c < c1; ++c) {
        const int s_base = c * CH;
        if (c + 1 < c1) {
            fetch_k(s_base + CH);
            vt.fetch(vptr, a.v_ss, s_base + CH, a.S - 1, tid);
        }
        // projection of this wave's 16 keys: five piece products per step (the K image is complete: stash() wrote it)
        floatx4 dd[FB];
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) dd[fb] = Frag<float>::zero();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const char* kp = img + tile_w * TL::BYTES + row_w * TL::K_ROW + x3_swz(row_w, 4 * ks + g, TL::K_ROW) * 16;
            const uintx4 kh = *reinterpret_cast<const uintx4*>(kp), kl = *reinterpret_cast<const uintx4*>(kp + TL::K_PIECE);
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                const uintx4 ph = pf[ks][fb][0], pm = pf[ks][fb][1], pl = pf[ks][fb][2];
                floatx4 d_ = dd[fb];
                d_ = mma_bf16(pl, kh, d_);
                d_ = mma_bf16(pm, kl, d_);
                d_ = mma_bf16(ph, kl, d_);
                d_ = mma_bf16(pm, kh, d_);
                d_ = mma_bf16(ph, kh, d_);
                dd[fb] = d_;
            }
        }
        // V^T image from Vs (LDS and global memory), in the shadow of the projection; K'^T V below is its first reader
        {
            char* kv_g = reinterpret_cast<char*>(a.vt) + ((long)bh * a.n_chunks + c) * (2 * (long)TL::KV_BYTES);
            x3_emit_vt<D, LDV>(Vs, img + 2 * TL::K_PIECE, TL::BYTES, tid, kv_g + 2 * TL::K_PIECE, TL::KV_BYTES);
        }
        FLY_PROFK(2);
        const float diag2 = diag[16 * w + r16];
        float amax = 0.f;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (16 * fb + 4 * g + i < a.mh_valid) amax = fmaxf(amax, fabsf(dd[fb][i]));
        amax = group_max(amax);
        const bool kvalid = (s_base + 16 * w + r16) < len;
        float cs = kvalid ? (amax - diag2 - lnm_half2) : -INFINITY;
        cs = row16_max(cs);                                // (amax is already the maximum over the four lane groups)
        if (lane == 0) red[w] = cs;
        __syncthreads();
        const float lmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float new_max = fmaxf(run_max, lmax);
        const bool live = new_max != -INFINITY;            // workgroup-uniform: some valid key so far
        const float rescale = (run_max == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(run_max - new_max);
        if (live) run_max = new_max;
        const float off = -diag2 - lnm_half2 - new_max;
        floatx4 fblk[2 * FB];                              // the lane's features: blocks of the [positive | negative] row
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = live && kvalid && (16 * fb + 4 * g + i < a.mh_valid);
                fblk[fb][i] = ok ? quant16(__builtin_amdgcn_exp2f(dd[fb][i] + off)) : 0.f;
                fblk[FB + fb][i] = ok ? quant16(__builtin_amdgcn_exp2f(-dd[fb][i] + off)) : 0.f;
            }
        }
        {
            char* frow = img + tile_w * TL::BYTES + TL::KV_BYTES + row_w * TL::F_ROW;
#pragma unroll
            for (int p_ = 0; p_ < FS; ++p_) {
                uintx4 fh, fl;
                split2(fblk[2 * p_], fblk[2 * p_ + 1], fh, fl);
                char* dst = frow + x3_swz(row_w, 4 * p_ + g, TL::F_ROW) * 16;
                *reinterpret_cast<uintx4*>(dst) = fh;
                *reinterpret_cast<uintx4*>(dst + TL::F_PIECE) = fl;
            }
        }
        if (tid == 0) a.chunk_scale[(long)bh * a.n_chunks + c] = live ? new_max * LN2 : 0.f;
        __syncthreads();                                   // images complete
        FLY_PROFK(3);
        // feature images -> global memory, 16-byte pieces in thread order
        {
            char* f_g = reinterpret_cast<char*>(a.kfeat) + ((long)bh * a.n_chunks + c) * (2 * (long)TL::F_BYTES);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int j = 0; j < (TL::F_BYTES / 16 + NT - 1) / NT; ++j) {
                    const int idx = tid + NT * j;
                    if (TL::F_BYTES / 16 % NT == 0 || idx < TL::F_BYTES / 16)
                        FLY_STORE(reinterpret_cast<const uintx4*>(img + t * TL::BYTES + TL::KV_BYTES)[idx], reinterpret_cast<uintx4*>(f_g + t * TL::F_BYTES) + idx);
                }
            }
        }
        FLY_PROFK(4);
        // K'^T V: rows = feature positions 16 blk + r16, k = keys of a tile (transposing reads of the feature
        // image), columns = value dims (V^T image rows); five piece products
        if (live) {
#pragma unroll
            for (int x = 0; x < RB; ++x)
#pragma unroll
                for (int db = 0; db <= DB; ++db) kvacc[x][db] *= rescale;
            const uintx4 ones = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};     // bf16 1.0 in every k-slot
            typedef __attribute__((address_space(3))) shortx4 lds_s4;
            typedef unsigned int uintx2_t __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const char* ti = img + t * TL::BYTES;
                uintx4 vh[DB], vm[DB], vl[DB];
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const char* vp = ti + 2 * TL::K_PIECE + (16 * db + r16) * TL::V_ROW + x3_swz(r16, g, TL::V_ROW) * 16;
                    vh[db] = *reinterpret_cast<const uintx4*>(vp);
                    vm[db] = *reinterpret_cast<const uintx4*>(vp + TL::V_PIECE);
                    if (X3_VP == 3) vl[db] = *reinterpret_cast<const uintx4*>(vp + 2 * TL::V_PIECE);
                }
#pragma unroll
                for (int x = 0; x < RB; ++x) {
                    const int blk = w + 4 * x;
                    if (blk < NBLK) {
                        // lane (r16, g) points at key rows 4g + r16/4 and 16 + 4g + r16/4, position quad 16 blk + 4 (r16 % 4)
                        const int pos = 16 * blk + 4 * (r16 & 3), cch = pos >> 3, sub = (pos & 4) * 2;
                        const int row_lo = 4 * g + (r16 >> 2), row_hi = 16 + row_lo;
                        const char* flo_ = ti + TL::KV_BYTES + row_lo * TL::F_ROW + x3_swz(row_lo, cch, TL::F_ROW) * 16 + sub;
                        const char* fhi_ = ti + TL::KV_BYTES + row_hi * TL::F_ROW + x3_swz(row_hi, cch, TL::F_ROW) * 16 + sub;
                        uintx4 fh, fl;
                        {
                            const uintx2_t a0 = __builtin_bit_cast(uintx2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)flo_));
                            const uintx2_t a1 = __builtin_bit_cast(uintx2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)fhi_));
                            const uintx2_t b0 = __builtin_bit_cast(uintx2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(flo_ + TL::F_PIECE)));
                            const uintx2_t b1 = __builtin_bit_cast(uintx2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(fhi_ + TL::F_PIECE)));
                            fh = uintx4{a0[0], a0[1], a1[0], a1[1]};
                            fl = uintx4{b0[0], b0[1], b1[0], b1[1]};
                        }
#pragma unroll
                        for (int db = 0; db < DB; ++db) {
                            floatx4 o = kvacc[x][db];
                            o = mma_bf16(fl, vm[db], o);
                            if (X3_VP == 3) o = mma_bf16(fh, vl[db], o);
                            o = mma_bf16(fl, vh[db], o);
                            o = mma_bf16(fh, vm[db], o);
                            o = mma_bf16(fh, vh[db], o);
                            kvacc[x][db] = o;
                        }
                        kvacc[x][DB] = mma_bf16(fh, ones, mma_bf16(fl, ones, kvacc[x][DB]));
                    }
                }
            }
        }
        FLY_PROFK(5);
        if (c + 1 < c1) {
            __syncthreads();                               // everyone is done with the images
            stash(c + 1);
            __syncthreads();
        }
    }

    // partial K'^T V in the combine step's order: tile (rb, db) -> 64 lanes x 4 floats with element
    // (feature 16 rb + 4 g'' + i, dim 16 db + r16) at lane 16 g'' + r16.  This lane's accumulator row 4g + i of
    // position block blk is feature 32 (blk / 2) + 16 (g % 2) + 8 (blk % 2) + 4 (g / 2) + i.
    float* part = a.kv_part + ((long)bh * a.n_split + sp) * (M * (D + 1));
#pragma unroll
    for (int x = 0; x < RB; ++x) {
        const int blk = w + 4 * x;
        if (blk < NBLK) {
            const int rb = 2 * (blk >> 1) + (g & 1), g2 = 2 * (blk & 1) + (g >> 1);
#pragma unroll
            for (int db = 0; db < DB; ++db)
                FLY_STORE(kvacc[x][db], reinterpret_cast<floatx4*>(part + ((rb * DB + db) * 64 + 16 * g2 + r16) * 4));
            // every column of the ones block holds the sum over the keys of the row's feature: features 16 rb + 4 g2 + i
            if (r16 == 0) FLY_STORE(kvacc[x][DB], reinterpret_cast<floatx4*>(part + M * D + 16 * rb + 4 * g2));
        }
    }
    if (tid == 0) a.part_max[(long)bh * a.n_split + sp] = run_max * LN2;
    FLY_PROFK(6);
}

// ---------------------------------------------------------------------------------------
// fused band kernel for bfloat16 inputs
// ---------------------------------------------------------------------------------------
// Same algorithm and the same transposed formulation as sblocal_fwd_kernel, with the three
// contractions of the key loop (and the global low-rank term) on v_mfma_f32_16x16x32_bf16: a
// lane (r = lane%16, g = lane/16) supplies eight consecutive k-slots 8g..8g+7 of row / column r,
// 16 contiguous bytes, and receives D[4g+i][r].  The k-slot order of every product is chosen so
// that the operands exist without shuffles:
//   scores   K q      : slot = head-dim index, K rows and q rows as they are in memory
//   overlap  K' q'    : slot 8g+j of step ks = feature 32ks + 16(j/4) + 4g + j%4 -- the order in which
//                       the fp32 projection leaves the query features in a lane, and in which the
//                       key pass stores the bf16 key features
//   P V               : slot 8g+j = key 16(j/4) + 4g + j%4 of the 32-key tile -- the order in which the
//                       score tiles leave the probabilities in a lane; the key pass leaves V in HBM
//                       per 32-key tile already transposed, [d][slot]
// q and k are bf16 already, so the scores are as exact as on the fp32 path (the softmax scale is
// applied to the fp32 result, not to an operand); key features, probabilities and K'^T V are
// rounded to bf16 for their products.  The query projection sqrt(t) P q also runs on the bf16 MFMA
// without losing precision: q is bf16 already and P is split into a bf16 head and a bf16 remainder
// (two MFMAs per step; the split represents P to 2^-17).

// ROWS x W tile of 2-byte elements, global -> registers -> LDS (rows clamped like RowTile)

template <int ROWS, int W, int NT>
struct Tile16 {
    static constexpr int C8 = W / 8, N = (ROWS * C8 + NT - 1) / NT;
    uintx4 r[N];
    // the same with a wave-uniform tile base and per-thread byte offsets computed once (all rows exist)
    __device__ __forceinline__ void offsets(uint32_t (&off)[N], long row_stride, int tid) const {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = (tid + NT * j) % (ROWS * C8), row = idx / C8, c8 = idx % C8;
            off[j] = (uint32_t)((row * row_stride + 8 * c8) * 2);
        }
    }
    __device__ __forceinline__ void fetch_at(const uint16_t* tile_base, const uint32_t (&off)[N]) {
#pragma unroll
        for (int j = 0; j < N; ++j)
            r[j] = *reinterpret_cast<const uintx4*>(reinterpret_cast<const char*>(tile_base) + off[j]);
    }
    // (a tile with fewer pieces than threads wraps around: every thread loads and stores, see TileKV16)
    __device__ __forceinline__ void fetch(const uint16_t* src, long row_stride, int row0, int last_row, int tid) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = (tid + NT * j) % (ROWS * C8), row = idx / C8, c8 = idx % C8;
            r[j] = *reinterpret_cast<const uintx4*>(src + (long)min(row0 + row, last_row) * row_stride + 8 * c8);
        }
    }
    template <int LD>
    __device__ __forceinline__ void stash(uint16_t* dst, int tid) const {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = (tid + NT * j) % (ROWS * C8), row = idx / C8, c8 = idx % C8;
            *reinterpret_cast<uintx4*>(dst + row * LD + 8 * c8) = r[j];
        }
    }
};

// The K tile (TK rows of E, row-major) and the V tile (D rows of TK, contiguous) of one step as ONE
// list of 16-byte pieces dealt to the threads round-robin, so that every thread issues the same
// number of loads whatever it holds (whole waves hold K or V pieces: both piece counts are
// multiples of 64).  Addresses are a wave-uniform tile base plus a per-thread byte offset computed
// once: the key loop then contains no vector address arithmetic, whose temporaries the register
// allocator likes to place in the registers of the previous fetch, behind a full wait.  The K tile
// that runs past the last key row uses a second, clamped set of offsets.  A list shorter than the
// workgroup wraps around: the surplus threads repeat pieces (same data to the same LDS address).
template <int E, int D, int NT>
struct TileKV16 {
    static constexpr int KC = TK * E / 8, VC = D * TK / 8, TOT = KC + VC, N = (TOT + NT - 1) / NT;
    static_assert(KC % 64 == 0 && VC % 64 == 0, "whole waves hold K or V pieces");
    uintx4 r[N];
    struct Plan {
        uint32_t off[N], off_last[N];        // byte offsets from the tile base (off_last: K rows clamped)
        int lds[N];                          // element offset in the K region or the V region of a stage
        bool is_k[N];                        // wave-uniform
    };
    template <int LDK, int LDT>
    static __device__ __forceinline__ void plan(Plan& p, long k_stride, int rows_in_last_tile, int tid) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = (tid + NT * j) % TOT, vi = idx - KC;
            p.is_k[j] = __builtin_amdgcn_readfirstlane(idx < KC);
            const int row = idx / (E / 8), c8 = idx % (E / 8);
            p.off[j] = p.is_k[j] ? (uint32_t)((row * k_stride + 8 * c8) * 2) : (uint32_t)(16 * vi);
            p.off_last[j] = p.is_k[j] ? (uint32_t)((min(row, rows_in_last_tile - 1) * k_stride + 8 * c8) * 2) : (uint32_t)(16 * vi);
            p.lds[j] = p.is_k[j] ? row * LDK + 8 * c8 : (vi / (TK / 8)) * LDT + 8 * (vi % (TK / 8));
        }
    }
    __device__ __forceinline__ void fetch(const Plan& p, const uint16_t* k_tile, const uint16_t* v_tile, bool last_tile) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const char* base = reinterpret_cast<const char*>(p.is_k[j] ? k_tile : v_tile);      // scalar select
            r[j] = *reinterpret_cast<const uintx4*>(base + (last_tile ? p.off_last[j] : p.off[j]));
        }
    }
    __device__ __forceinline__ void stash(const Plan& p, uint16_t* kdst, uint16_t* vdst) const {
#pragma unroll
        for (int j = 0; j < N; ++j) *reinterpret_cast<uintx4*>((p.is_k[j] ? kdst : vdst) + p.lds[j]) = r[j];
    }
};


#ifndef FLY_TWO_PIECE_MAX
#define FLY_TWO_PIECE_MAX 128      // most features for which the bf16 band kernels carry the two-piece path (at 256 the
                                   // 32-queries-per-wave kernel has no registers left for it: +13 % on every input)
#endif
// bf16 band kernels: the probabilities p = e - (q'.k') beta go to the P V product as bf16, 2^-9 of their size.  Where
// the features approximate the exact weights that size is the size of the weights; where they do not (unscaled inputs,
// few features) the band's low-rank part can be hundreds of times the exact mass for some queries, cancels against the
// sums over all keys only in the result, and its rounding would show in the output at 2^-9 times that ratio.  Once the
// low-rank mass a lane has gathered on its keys of the band exceeds three times their exact mass, the wave hands P over
// in two pieces (head and rest, 2^-17) for that tile: one more pass of the tile's P V products, taken by no tile of
// well-conditioned inputs (for them the two masses are about equal), and what passes in one piece is bounded by four
// times the exact mass, i.e. by the normaliser.  Both masses in units of 2^m_run.
__device__ __forceinline__ bool second_piece_wanted(float lowrank_mass_so_far, float exact_mass_so_far) {
    return __builtin_amdgcn_ballot_w64(lowrank_mass_so_far > 3.f * exact_mass_so_far) != 0;
}
// what two floats lose when they are packed into the bf16 pair `head`, as a bf16 pair
__device__ __forceinline__ uint32_t pack_rest(float a, float b, uint32_t head) {
    return pack_bf16x2(a - __uint_as_float(head << 16), b - __uint_as_float(head & 0xffff0000u));
}

template <int E, int M> constexpr size_t fwd_bf16_smem() {
    constexpr size_t stage = (size_t)TK * (E + 8) + (size_t)TK * (M + 8) + (size_t)E * (TK + 8);   // 2-byte elements
    constexpr size_t tiles = 2 * stage * 2;
    constexpr size_t proj = (size_t)2 * (M / 2) * (E + 8) * 2;      // bf16 head and remainder of the projection
    constexpr size_t lowrank = (size_t)E * (M + 8) * 2;
    constexpr size_t need = tiles > proj ? (tiles > lowrank ? tiles : lowrank) : (proj > lowrank ? proj : lowrank);
    return need;
}

// A workgroup is NW waves of 16 queries each: more waves share every key tile, which divides the
// L2 -> CU traffic (the limit of this kernel: 24 KiB per 32-key tile at E = D = 64, m = 256).
constexpr int BF16_WAVES = 8;

template <int E, int D, int M, bool SPLIT, int NW>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2, 2))) void sblocal_fwd_bf16_kernel(FwdArgs a) {
    static_assert(TK == 32, "the P V product takes one 32-key tile per MFMA step");
    constexpr int NT = 64 * NW, TQ = 16 * NW;          // shadow the 4-wave constants of the fp32 kernels
    constexpr int TQ64 = 64;                           // queries per tile of the partial workspace / merge
    typedef bf16_t T;
    constexpr bool TWO_PIECE = M <= FLY_TWO_PIECE_MAX;
    constexpr int MH = M / 2, FB = MH / 16, EC = E / 16, DB = D / 16, KB = TK / 16;
    constexpr int LDK = E + 8, LDF = M + 8, LDT = TK + 8, LDKV = M + 8;   // LDS row strides in elements
    constexpr int STAGE = TK * LDK + TK * LDF + D * LDT;                  // elements per stage
    extern __shared__ __attribute__((aligned(128))) float smem[];
    uint16_t* lds = reinterpret_cast<uint16_t*>(smem);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    if (SPLIT && (int)blockIdx.x >= a.band_wgs) {       // combine role, see sblocal_fwd_kernel
        const int ci = blockIdx.x - a.band_wgs;
        sb_combine_body(smem, a.kv_part, a.part_max, const_cast<float*>(a.kv), const_cast<float*>(a.ksum),
                        const_cast<float*>(a.kmax), nullptr, ci / a.cmb_wpb, ci % a.cmb_wpb, a.cmb_wpb, a.n_split, M, D);
        return;
    }
    const int n_qt = (a.T + TQ - 1) / TQ;
    const int n_items = a.B * a.H * n_qt * a.n_parts;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // see sblocal_fwd_kernel
    if (item >= n_items) return;                       // workgroup-uniform
    const int part = item % a.n_parts;
    const int qt = (item / a.n_parts) % n_qt;
    const int bh = item / (a.n_parts * n_qt), b = bh / a.H, h = bh % a.H;
    const int q0 = qt * TQ;
    const int iq = q0 + 16 * w + r16;
    const bool qvalid = iq < a.T;
    const uint16_t* qptr = reinterpret_cast<const uint16_t*>(a.q) + b * a.q_sb + h * a.q_sh;
    const uint16_t* kptr = reinterpret_cast<const uint16_t*>(a.k) + b * a.k_sb + h * a.k_sh;
    const uint16_t* vtp = reinterpret_cast<const uint16_t*>(a.vt) + (long)bh * a.n_chunks * CH * D;   // [tile][d][slot]
    const uint16_t* fptr = reinterpret_cast<const uint16_t*>(a.kfeat) + (long)bh * a.n_chunks * CH * M;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half = 0.5f * __logf(2.0f * a.mh_valid);
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi
    constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;

    FLY_PROF(0);
    // this workgroup's share of the band, in 32-key tiles (as in sblocal_fwd_kernel)
    const int q_last = min(q0 + TQ - 1, a.T - 1);
    const int lo = max(0, q0 - lc_lo);
    const int hi = min(len, q_last + lc_hi);
    int kt_lo = lo / TK;
    int kt_hi = (hi > lo) ? (hi + TK - 1) / TK : kt_lo;
    if (SPLIT) {
        // an even split: the first (tiles % parts) parts take one tile more
        const int nt = kt_hi - kt_lo, base = nt / a.n_parts, extra = nt % a.n_parts;
        const int first = kt_lo + part * base + min(part, extra);
        kt_lo = first;
        kt_hi = first + base + (part < extra ? 1 : 0);
    }
    constexpr bool lowrank_here = !SPLIT;              // with several parts the merge kernel adds the low-rank term

    // Key tiles travel global -> registers -> LDS.  A tile is requested two iterations before it is
    // used (one iteration of work is shorter than the latency of the loads under load), so two
    // register sets alternate and the key loop is unrolled by two.
    struct TileRegs {
        TileKV16<E, D, NT> kv;        // K rows, and V already transposed by the key pass: D rows of 32 k-slots
        Tile16<TK, M, NT> f;
    };
    // the chunk log-scales of this workgroup's share of the band sit in LDS behind the tile stages
    // (the host sizes the region): a load of them inside the loop would have to be waited for at
    // the start of a step, and the memory counter retires in order -- behind it the tile prefetch
    float* cs_lds = reinterpret_cast<float*>(reinterpret_cast<char*>(smem) + fwd_bf16_smem<E, M>());
    const int c_lo = kt_lo * TK / CH;
    {
        const int n_cs = kt_hi > kt_lo ? (kt_hi - 1) * TK / CH - c_lo + 1 : 0;
        const float* csg = a.chunk_scale + (long)bh * a.n_chunks + c_lo;
        for (int i = tid; i < n_cs; i += NT) cs_lds[i] = csg[i];
    }
    constexpr int LOADS = TileKV16<E, D, NT>::N + Tile16<TK, M, NT>::N;     // vector loads of one fetch, per thread
    typename TileKV16<E, D, NT>::Plan kvp;
    const int last_tile = (a.S - 1) / TK;                 // the only K tile whose rows may not all exist
    TileKV16<E, D, NT>::template plan<LDK, LDT>(kvp, a.k_ss, a.S - last_tile * TK, tid);
    uint32_t foff[Tile16<TK, M, NT>::N];
    Tile16<TK, M, NT>().offsets(foff, M, tid);
    auto fetch = [&](TileRegs& r, int kt) __attribute__((always_inline)) {
        const int ktc = min(kt, last_tile);               // (tiles past the keys are never used; stay in bounds)
        r.kv.fetch(kvp, kptr + (long)ktc * TK * a.k_ss, vtp + (long)kt * (D * TK), ktc == last_tile);
        r.f.fetch_at(fptr + (long)kt * TK * M, foff);
    };
    auto stash = [&](const TileRegs& r, int stage) __attribute__((always_inline)) {
        uint16_t* dst = lds + stage * STAGE;
        r.kv.stash(kvp, dst, dst + TK * (LDK + LDF));
        r.f.template stash<LDF>(dst + TK * LDK, tid);
    };
    TileRegs ra, rb;
    // (clamped tile indices: the loads are unconditional so that the register sets are plain values)
    fetch(ra, min(kt_lo, max(kt_hi - 1, 0)));
    fetch(rb, min(kt_lo + 1, max(kt_hi - 1, 0)));
    const float kmax = SPLIT ? split_kmax(a.part_max, bh, a.n_split) : a.kmax[bh];

    // score operand: the query row as it is in memory
    const uint16_t* qrow = qptr + (long)min(iq, a.T - 1) * a.q_ss;
    uint4 qb[E / 32];
#pragma unroll
    for (int ks = 0; ks < E / 32; ++ks) qb[ks] = *reinterpret_cast<const uint4*>(qrow + 32 * ks + 8 * g);

    // query features in fp32: qf[c][i] = feature 16c + 4g + i of the [positive | negative] row
    floatx4 qf[2 * FB];
    float lsq;
    if (SPLIT) {
        const long qr_ = (long)bh * a.T + min(iq, a.T - 1);
#pragma unroll
        for (int c = 0; c < 2 * FB; ++c) qf[c] = *reinterpret_cast<const floatx4*>(a.qfeat + qr_ * M + 16 * c + 4 * g);
        lsq = a.q_lsq[qr_];
    } else {
        // |q|^2 from the score operand (lane g holds elements 32ks + 8g .. + 7 of its query row)
        float sq = 0.f;
#pragma unroll
        for (int ks = 0; ks < E / 32; ++ks) {
            const uint32_t wds[4] = {qb[ks].x, qb[ks].y, qb[ks].z, qb[ks].w};
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const float lo = __uint_as_float(wds[x] << 16), hi = __uint_as_float(wds[x] & 0xffff0000u);
                sq += lo * lo + hi * hi;
            }
        }
        const float diag_q = 0.5f * a.temp * group_sum(sq);
        // sqrt(t) P as bf16 head + bf16 remainder, rows of E + 8 elements
        uint16_t* Phi = lds;
        uint16_t* Plo = lds + MH * LDK;
        const float pscale = sqrtf(a.temp);
        for (int idx = tid; idx < MH * E / 4; idx += NT) {
            const int f = idx / (E / 4), c4 = idx % (E / 4);
            const floatx4 x = *reinterpret_cast<const floatx4*>(a.proj + (long)f * E + 4 * c4) * pscale;
            floatx4 rem;
            uint16_t hb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                hb[i] = f32_to_bf16(x[i]);
                rem[i] = x[i] - bf16_to_f32(hb[i]);
            }
            *reinterpret_cast<uint2*>(Phi + f * LDK + 4 * c4) = make_uint2(hb[0] | ((uint32_t)hb[1] << 16), hb[2] | ((uint32_t)hb[3] << 16));
            *reinterpret_cast<uint2*>(Plo + f * LDK + 4 * c4) = make_uint2(pack_bf16x2(rem[0], rem[1]), pack_bf16x2(rem[2], rem[3]));
        }
        __syncthreads();
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) qf[fb] = Frag<float>::zero();
#pragma unroll
        for (int ks = 0; ks < E / 32; ++ks)
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                const int off = (16 * fb + r16) * LDK + 32 * ks + 8 * g;
                qf[fb] = mma_bf16(*reinterpret_cast<const uint4*>(Phi + off), qb[ks], qf[fb]);
                qf[fb] = mma_bf16(*reinterpret_cast<const uint4*>(Plo + off), qb[ks], qf[fb]);
            }
        float qmax = 0.f;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (16 * fb + 4 * g + i < a.mh_valid) qmax = fmaxf(qmax, fabsf(qf[fb][i]));
        qmax = group_max(qmax);
        lsq = -diag_q + qmax - lnm_half;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
            const floatx4 dd = qf[fb];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float keep = (16 * fb + 4 * g + i < a.mh_valid) ? 1.f : 0.f;
                qf[fb][i] = keep * bf16_round(__builtin_amdgcn_exp2f((dd[i] - qmax) * LOG2E));
                qf[FB + fb][i] = keep * bf16_round(__builtin_amdgcn_exp2f((-dd[i] - qmax) * LOG2E));
            }
        }
        __syncthreads();                 // the projection rows are dead; the tile buffers may overwrite them
    }
    FLY_PROF(1);
    // normaliser of the global low-rank term, from the features as the overlap product sees them (bf16 values)
    float qk1 = 0.f;
    if (lowrank_here) {
#pragma unroll
        for (int c = 0; c < 2 * FB; ++c) {
            const floatx4 ks = *reinterpret_cast<const floatx4*>(a.ksum + (long)bh * M + 16 * c + 4 * g);
            qk1 += qf[c][0] * ks[0] + qf[c][1] * ks[1] + qf[c][2] * ks[2] + qf[c][3] * ks[3];
        }
        qk1 = group_sum(qk1);
    }
    // overlap operand: two 16-feature blocks make the eight k-slots of one MFMA step
    uint4 qfb[M / 32];
#pragma unroll
    for (int ks = 0; ks < M / 32; ++ks)
        qfb[ks] = make_uint4(pack_bf16x2(qf[2 * ks][0], qf[2 * ks][1]), pack_bf16x2(qf[2 * ks][2], qf[2 * ks][3]),
                             pack_bf16x2(qf[2 * ks + 1][0], qf[2 * ks + 1][1]), pack_bf16x2(qf[2 * ks + 1][2], qf[2 * ks + 1][3]));

    const float sc = a.temp * LOG2E;             // scores leave the MFMA unscaled; exponents are base 2
    const float c0 = (lsq + kmax) * LOG2E;       // base-2 log-scale of the global low-rank term
    float m_run = c0;
    float ze = 0.f, zp = 0.f;
    floatx4 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = Frag<float>::zero();
    const int qw0 = q0 + 16 * w;
    const int smin = max(iq - lc_lo, 0);
    const unsigned span = qvalid ? (unsigned)max(min(iq + lc_hi, len) - smin, 0) : 0u;

    stash(ra, 0);                          // (unconditional like every fetch and stash: see the key loop)
    __syncthreads();

    // One key tile takes two phases: scores (LDS fragment reads and the two score MFMA products) and
    // softmax (the arithmetic on the scores and P V).  The first phase loads the LDS and matrix
    // pipes, the second the vector ALU; the waves of a workgroup pass them in lock step if left
    // alone, so the upper half of the waves runs half a tile behind the lower half: while one half
    // reads fragments and multiplies, the other half does its softmax arithmetic.  A wave's scores
    // and V fragments of a tile stay in registers between the two phases.
    floatx4 s1[KB], s2[KB];
    uint4 vf[DB];
    auto touches = [&](int kt) __attribute__((always_inline)) {      // wave-uniform: does the tile touch the band of any of the wave's queries?
        const int s_base = kt * TK;
        return !(s_base + TK - 1 - qw0 < -lc_lo || s_base - (qw0 + 15) >= lc_hi || s_base >= len);
    };
    auto score_phase = [&](int kt, int stage) __attribute__((always_inline)) {
        if (!touches(kt)) return;
        const uint16_t* Ks = lds + stage * STAGE;
        const uint16_t* Fs = Ks + TK * LDK;
        const uint16_t* Vt = Fs + TK * LDF;
        // fragments are requested from LDS in batches ahead of the MFMAs that use them (the scheduling
        // barriers keep the loads from sinking to their uses, where each would wait alone); the feature
        // fragments come in two batches to stay inside the register budget
        constexpr int FS = M / 32, FH = FS > 4 ? FS / 2 : FS;
        uint4 kf[E / 32][KB], ff[FH][KB];
#pragma unroll
        for (int ks = 0; ks < E / 32; ++ks)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
                kf[ks][kb] = *reinterpret_cast<const uint4*>(Ks + (16 * kb + r16) * LDK + 32 * ks + 8 * g);
#pragma unroll
        for (int ks = 0; ks < FH; ++ks)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
                ff[ks][kb] = *reinterpret_cast<const uint4*>(Fs + (16 * kb + r16) * LDF + 32 * ks + 8 * g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) { s1[kb] = Frag<float>::zero(); s2[kb] = Frag<float>::zero(); }
#pragma unroll
        for (int ks = 0; ks < E / 32; ++ks)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) s1[kb] = mma_bf16(kf[ks][kb], qb[ks], s1[kb]);
#pragma unroll
        for (int ks = 0; ks < FH; ++ks)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) s2[kb] = mma_bf16(ff[ks][kb], qfb[ks], s2[kb]);
        if (FH < FS) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = FH; ks < FS; ++ks)
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
                    ff[ks - FH][kb] = *reinterpret_cast<const uint4*>(Fs + (16 * kb + r16) * LDF + 32 * ks + 8 * g);
#pragma unroll
            for (int db = 0; db < DB; ++db) vf[db] = *reinterpret_cast<const uint4*>(Vt + (16 * db + r16) * LDT + 8 * g);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = FH; ks < FS; ++ks)
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s2[kb] = mma_bf16(ff[ks - FH][kb], qfb[ks], s2[kb]);
        } else {
#pragma unroll
            for (int db = 0; db < DB; ++db) vf[db] = *reinterpret_cast<const uint4*>(Vt + (16 * db + r16) * LDT + 8 * g);
        }
    };
    auto soft_phase = [&](int kt, float cscale) __attribute__((always_inline)) {
        if (!touches(kt)) return;
        const int s_base = kt * TK;
        const float wc = __builtin_amdgcn_exp2f((cscale - kmax) * LOG2E);
        // lane holds the raw scores q.k of query iq against keys s_base + 16kb + 4g + i (the softmax
        // scale enters through one fma per exponent).  Tiles that lie inside the band of all 16
        // queries of the wave -- most of them -- skip the masks.
        const bool inside = s_base >= max(qw0 + 15 - lc_lo, 0) && s_base + TK <= min(qw0 + lc_hi, len) && qw0 + 15 < a.T;
        floatx4 p[KB];
        float ovs = 0.f;
        auto soft = [&](auto masked_t) __attribute__((always_inline)) {
            constexpr bool MASKED = decltype(masked_t)::value;
            bool ok[KB][4];
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int s = s_base + 16 * kb + 4 * g + i;
                    ok[kb][i] = !MASKED || (unsigned)(s - smin) < span;
                    mx = fmaxf(mx, ok[kb][i] ? s1[kb][i] : -INFINITY);
                }
            mx = group_max(mx) * sc;                               // sc > 0
            // (the reference exponent is raised only when a tile exceeds it by more than 2^8)
            if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.f) != 0) {      // wave-uniform
                const float m_new = fmaxf(m_run, mx);
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                m_run = m_new;
                ze *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
            }
            const float beta = wc * __builtin_amdgcn_exp2f(c0 - m_run);      // scale of the overlap term
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float e = ok[kb][i] ? __builtin_amdgcn_exp2f(__builtin_fmaf(s1[kb][i], sc, -m_run)) : 0.f;
                    const float ov = ok[kb][i] ? s2[kb][i] : 0.f;
                    ze += e;
                    ovs += ov;
                    p[kb][i] = e - ov * beta;
                }
        };
        if (inside) soft(std::false_type{}); else soft(std::true_type{});
        // (see second_piece_wanted: where the band's low-rank part dwarfs the exact weights the probabilities go to
        //  the matrix pipe in two bf16 pieces)
        zp += ovs * wc;
        const bool two = TWO_PIECE && second_piece_wanted(zp * __builtin_amdgcn_exp2f(c0 - m_run), ze);
        // O^T[d][query] += sum_keys V[key][d] p[key][query]: one MFMA step per 16 value dims
        const uint4 pb = make_uint4(pack_bf16x2(p[0][0], p[0][1]), pack_bf16x2(p[0][2], p[0][3]),
                                    pack_bf16x2(p[1][0], p[1][1]), pack_bf16x2(p[1][2], p[1][3]));
#pragma unroll
        for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db], pb, oacc[db]);
        if (two) {                                               // wave-uniform
            const uint4 pl = make_uint4(pack_rest(p[0][0], p[0][1], pb.x), pack_rest(p[0][2], p[0][3], pb.y),
                                        pack_rest(p[1][0], p[1][1], pb.z), pack_rest(p[1][2], p[1][3], pb.w));
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db], pl, oacc[db]);
        }
    };
    const bool late = w >= NW / 2;        // wave-uniform: this wave runs half a tile behind
    float cs_prev = 0.f;                  // chunk scale of the tile a late wave still owes its softmax
    auto tile_step = [&](int kt, int stage, float cscale) __attribute__((always_inline)) {
        const bool stamp = kt == kt_lo + 8;
        if (!late) {
            score_phase(kt, stage);
            FLY_PROF3(stamp, 2);
            soft_phase(kt, cscale);
        } else {
            if (kt > kt_lo) soft_phase(kt - 1, cs_prev);
            FLY_PROF3(stamp, 2);
            score_phase(kt, stage);
            cs_prev = cscale;
        }
        FLY_PROF3(stamp, 3);
    };

    FLY_PROF(2);
    // even steps: tile kt sits in stage 0 (from ra), rb holds kt + 1, ra is refilled with kt + 2;
    // odd steps the other way round
    // Fetches and stashes run on every pass, past the end with the last tile again: with loads under
    // conditions the compiler cannot tell which set is the newer one and drains both whenever it
    // waits for one.  After a stash only the other set is in flight, which the explicit counts record.
    drain_loads();                         // once, before the loop: from here on the counts below are exact
    for (int kt = kt_lo; kt < kt_hi; kt += 2) {
        const float cs0 = cs_lds[kt * TK / CH - c_lo];
        FLY_PROF3(kt == kt_lo + 8, 0);
        fetch(ra, min(kt + 2, kt_hi - 1));
        FLY_PROF3(kt == kt_lo + 8, 1);
        tile_step(kt, 0, cs0);
        stash(rb, 1);
        FLY_PROF3(kt == kt_lo + 8, 4);
        drain_loads_but<LOADS>();
        FLY_PROF3(kt == kt_lo + 8, 5);
        __syncthreads();
        FLY_PROF3(kt == kt_lo + 8, 6);
        // (no early exit between the halves: a path that leaves here with set A still in flight would
        // count, for the compiler, as a way back to the top of the loop)
        const bool second = kt + 1 < kt_hi;
        const float cs1 = cs_lds[min(kt + 1, kt_hi - 1) * TK / CH - c_lo];
        fetch(rb, min(kt + 3, kt_hi - 1));
        if (second) tile_step(kt + 1, 1, cs1);
        stash(ra, 0);
        drain_loads_but<LOADS>();
        __syncthreads();
    }
    if (late && kt_lo < kt_hi) soft_phase(kt_hi - 1, cs_prev);

    FLY_PROF(3);
    // global low-rank term: qkv^T[d][query] = sum_r KV[r][d] q'[query][r]; K'^T V comes as bf16, transposed,
    // features in the slot order of the overlap operand
    floatx4 lacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) lacc[db] = Frag<float>::zero();
    if (lowrank_here) {
        uint16_t* KVt = lds;
        // written by the combine kernel as bf16 [d][slot]: a plain copy in 16-byte pieces
        constexpr int KVC = D * M / 8;
#pragma unroll
        for (int piece = 1; piece >= 0; --piece) {       // the rest first, then the head (two bf16 pieces of K'^T V)
            const uint16_t* kvg = reinterpret_cast<const uint16_t*>(a.kvt) + ((long)bh * 2 + piece) * M * D;
            if (piece == 0) __syncthreads();             // the first piece has been read
#pragma unroll
            for (int j = 0; j < (KVC + NT - 1) / NT; ++j) {
                const int idx = tid + NT * j, d = idx / (M / 8), c8 = idx % (M / 8);
                if (KVC % NT == 0 || idx < KVC)
                    *reinterpret_cast<uint4*>(KVt + d * LDKV + 8 * c8) = *reinterpret_cast<const uint4*>(kvg + (long)d * M + 8 * c8);
            }
            __syncthreads();
#pragma unroll
            for (int ks = 0; ks < M / 32; ++ks)
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    lacc[db] = mma_bf16(*reinterpret_cast<const uint4*>(KVt + (16 * db + r16) * LDKV + 32 * ks + 8 * g), qfb[ks], lacc[db]);
        }
    }
    FLY_PROF(4);
    ze = group_sum(ze);
    zp = group_sum(zp);
    const float gamma = __builtin_amdgcn_exp2f(c0 - m_run);               // <= 1
    if (SPLIT) {
        // partials are kept per 64-query tile (the unit of sb_merge_kernel); this wave's tile:
        const int n_qt64 = (a.T + TQ64 - 1) / TQ64, t64 = (q0 + 16 * w) / TQ64;
        if (t64 < n_qt64) {                            // wave-uniform
            float* ws = a.part_ws + (((long)bh * n_qt64 + t64) * a.n_parts + part) * (TQ64 * (D + NSTAT));
            const int ql = (16 * w + r16) % TQ64;
#pragma unroll
            for (int db = 0; db < DB; ++db) *reinterpret_cast<floatx4*>(ws + ql * D + 16 * db + 4 * g) = oacc[db];
            if (g == 0) {
                float* st = ws + TQ64 * D;
                st[0 * TQ64 + ql] = m_run;
                st[1 * TQ64 + ql] = ze;
                st[2 * TQ64 + ql] = zp;
                st[3 * TQ64 + ql] = 0.f;
                st[4 * TQ64 + ql] = c0;
            }
        }
    } else {
        const float Z = ze + gamma * fmaxf(qk1 - zp, 1e-24f);
        const float inv = 1.0f / Z;
        if (qvalid) {
            T* optr = reinterpret_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq * a.o_ss;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                floatx4 o = (oacc[db] + gamma * lacc[db]) * inv;
                store4_f32(optr + 16 * db + 4 * g, o);
            }
            if (g == 0) a.log_norm[(long)bh * a.T + iq] = m_run * LN2 + __logf(Z);
        }
    }
    FLY_PROF(5);
}

// ---------------------------------------------------------------------------------------
// fused band kernel for bfloat16 inputs, 32 queries per wave
// ---------------------------------------------------------------------------------------
// The algorithm, tile formats and scratch layouts of sblocal_fwd_bf16_kernel on v_mfma_f32_32x32x16_bf16: a
// wave owns 32 queries, so every fragment it reads from LDS feeds twice the arithmetic (the 16-query kernel
// spends most of its time on those reads).  Lane (c = lane % 32, h = lane / 32) supplies eight consecutive
// k-slots 8h .. 8h+7 of row / column c per 16-slot step and receives D[8b + 4h + i][c], b = 0..3, i = 0..3, as
// element 4b + i: one query per lane, whose 32 keys of a tile are split between the lane pair (c, c + 32).
// The k-slot orders of the key pass's scratch fit without shuffles:
//   overlap K' q' : position 32ks + 8g + j holds feature 32ks + 16(j/4) + 4g + j%4; step s = 2ks + t takes
//                   positions 16s + 8h + j, i.e. (g = 2t + h) features 32ks + 8(2(j/4) + t) + 4h + j%4 -- elements
//                   4t + j%4 and 4(2 + t) + j%4 of the lane's own block of 32 projected features
//   P V           : position 8g + j of the V^T tile holds key 16(j/4) + 4g + j%4; step t takes positions
//                   16t + 8h + j, i.e. keys 8(2(j/4) + t) + 4h + j%4 -- the lane's own score elements again
// A workgroup is B32_WAVES waves of 32 queries.
typedef float floatx16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ floatx16 mma32_bf16(uint4 a, uint4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ float pair32_max(float v) { float x, y; rows_pair32(v, x, y); return fmaxf(x, y); }
__device__ __forceinline__ float pair32_sum(float v) { float x, y; rows_pair32(v, x, y); return x + y; }

// The tile loads of sblocal_fwd_b32_kernel: per-lane byte offsets from the tile bases, computed once (the K tile that
// runs past the last key row has its own), and the loads themselves -- wave w issues wave-loads w, w + NW, .. of every region.
template <int E, int D, int M, int NW>
struct B32Loads {
    static constexpr int K_ROW = 2 * E, F_ROW = 2 * M, V_ROW = 2 * TK;
    static constexpr int K_BYTES = TK * K_ROW, F_BYTES = TK * F_ROW, V_BYTES = D * V_ROW;
    static constexpr int NKL = (K_BYTES / 1024 + NW - 1) / NW, NFL = (F_BYTES / 1024 + NW - 1) / NW, NVL = (V_BYTES / 1024 + NW - 1) / NW;
    uint32_t kgo[NKL], kgo_last[NKL], fgo[NFL], vgo[NVL];
    __device__ __forceinline__ void plan(long k_ss, int rows_last, int w, int lane) {
#pragma unroll
        for (int x = 0; x < NKL; ++x) {
            const int o = 1024 * (NW * x + w) + 16 * lane, row = o / K_ROW, cp = (o % K_ROW) / 16;
            kgo[x] = (uint32_t)(row * k_ss * 2 + x3_swz(row, cp, K_ROW) * 16);
            kgo_last[x] = (uint32_t)(min(row, rows_last - 1) * k_ss * 2 + x3_swz(row, cp, K_ROW) * 16);
        }
#pragma unroll
        for (int x = 0; x < NFL; ++x) {
            const int o = 1024 * (NW * x + w) + 16 * lane, row = o / F_ROW, cp = (o % F_ROW) / 16;
            fgo[x] = (uint32_t)(row * F_ROW + x3_swz(row, cp, F_ROW) * 16);
        }
#pragma unroll
        for (int x = 0; x < NVL; ++x) {
            const int o = 1024 * (NW * x + w) + 16 * lane, row = o / V_ROW, cp = (o % V_ROW) / 16;
            vgo[x] = (uint32_t)(row * V_ROW + x3_swz(row, cp, V_ROW) * 16);
        }
    }
    __device__ __forceinline__ void issue(char* st, int w, bool last, const char* kg, const char* fg, const char* vg) const {
#pragma unroll
        for (int x = 0; x < NKL; ++x)
            if (K_BYTES / 1024 % NW == 0 || NW * x + w < K_BYTES / 1024)
                dma_to_lds(kg + (last ? kgo_last[x] : kgo[x]), st + 1024 * (NW * x + w));
#pragma unroll
        for (int x = 0; x < NFL; ++x)
            if (F_BYTES / 1024 % NW == 0 || NW * x + w < F_BYTES / 1024)
                dma_to_lds(fg + fgo[x], st + K_BYTES + 1024 * (NW * x + w));
#pragma unroll
        for (int x = 0; x < NVL; ++x)
            if (V_BYTES / 1024 % NW == 0 || NW * x + w < V_BYTES / 1024)
                dma_to_lds(vg + vgo[x], st + K_BYTES + F_BYTES + 1024 * (NW * x + w));
    }
};

template <int E, int M> constexpr size_t fwd_b32_smem() { return fwd_bf16_smem<E, M>(); }
// Four waves per workgroup (two workgroups per compute unit, which then overlap by themselves).  Eight with the skew
// below measured the same at 64 and 128 features and slower at 256, where the skewed form spills registers.
#ifndef B32_WAVES
#define B32_WAVES 4
#endif
#ifndef FLY_B32_FUSED_TILE
#define FLY_B32_FUSED_TILE 1
#endif

template <int E, int D, int M, bool SPLIT, int NW>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2, 2))) void sblocal_fwd_b32_kernel(FwdArgs a) {
    static_assert(TK == 32, "one 32-key tile is one row block of the 32x32 MFMA");
    constexpr int NT = 64 * NW, TQ = 32 * NW;          // shadow the constants of the fp32 kernels
    constexpr int TQ64 = 64;                           // queries per tile of the partial workspace / merge
    typedef bf16_t T;
    constexpr bool TWO_PIECE = M <= FLY_TWO_PIECE_MAX;
    constexpr int MH = M / 2, PB = MH / 32, KS = E / 16, FS = M / 16, DB = D / 32;
    static_assert(MH % 32 == 0 && D % 32 == 0, "whole 32-row blocks");
    constexpr int LDK = E + 8, LDKV = M + 8;           // LDS row strides in elements (projection rows, K'^T V)
    // a tile stage: K rows, feature rows and V^T rows without padding, the 16-byte chunks of every row XOR-swizzled
    // (x3_swz) -- the tiles come straight from global memory into LDS, a wave's 64 chunks to 1024 consecutive bytes
    constexpr int K_ROW = 2 * E, F_ROW = 2 * M, V_ROW = 2 * TK;           // row sizes in bytes
    constexpr int K_BYTES = TK * K_ROW, F_BYTES = TK * F_ROW, V_BYTES = D * V_ROW, STAGE_BYTES = K_BYTES + F_BYTES + V_BYTES;
    static_assert(K_BYTES % 1024 == 0 && F_BYTES % 1024 == 0 && V_BYTES % 1024 == 0, "whole wave loads");
    extern __shared__ __attribute__((aligned(128))) float smem[];
    uint16_t* lds = reinterpret_cast<uint16_t*>(smem);

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c = lane & 31, h = lane >> 5;
    // (the wave index as a scalar: the tests on the wave's range of queries -- does a tile touch its band, does it lie inside
    //  every query's band -- are then scalar branches, and the accumulators are not copied around exec-masked regions)
    if (SPLIT && (int)blockIdx.x >= a.band_wgs) {       // combine role, see sblocal_fwd_kernel
        const int ci = blockIdx.x - a.band_wgs;
        sb_combine_body(smem, a.kv_part, a.part_max, const_cast<float*>(a.kv), const_cast<float*>(a.ksum),
                        const_cast<float*>(a.kmax), nullptr, ci / a.cmb_wpb, ci % a.cmb_wpb, a.cmb_wpb, a.n_split, M, D);
        return;
    }
    const int n_qt = (a.T + TQ - 1) / TQ;
    const int n_items = a.B * a.H * n_qt * a.n_parts;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // see sblocal_fwd_kernel
    if (item >= n_items) return;                       // workgroup-uniform
    const int part = item % a.n_parts;
    const int qt = (item / a.n_parts) % n_qt;
    const int bh = item / (a.n_parts * n_qt), b = bh / a.H, hd = bh % a.H;
    const int q0 = qt * TQ;
    const int iq = q0 + 32 * w + c;
    const bool qvalid = iq < a.T;
    const uint16_t* qptr = reinterpret_cast<const uint16_t*>(a.q) + b * a.q_sb + hd * a.q_sh;
    const uint16_t* kptr = reinterpret_cast<const uint16_t*>(a.k) + b * a.k_sb + hd * a.k_sh;
    const uint16_t* vtp = reinterpret_cast<const uint16_t*>(a.vt) + (long)bh * a.n_chunks * CH * D;   // [tile][d][slot]
    const uint16_t* fptr = reinterpret_cast<const uint16_t*>(a.kfeat) + (long)bh * a.n_chunks * CH * M;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half = 0.5f * __logf(2.0f * a.mh_valid);
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi
    constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;

    // this workgroup's share of the band, in 32-key tiles (as in sblocal_fwd_kernel)
    const int q_last = min(q0 + TQ - 1, a.T - 1);
    const int lo = max(0, q0 - lc_lo);
    const int hi = min(len, q_last + lc_hi);
    int kt_lo = lo / TK;
    int kt_hi = (hi > lo) ? (hi + TK - 1) / TK : kt_lo;
    if (SPLIT) {
        const int nt = kt_hi - kt_lo, base = nt / a.n_parts, extra = nt % a.n_parts;
        const int first = kt_lo + part * base + min(part, extra);
        kt_lo = first;
        kt_hi = first + base + (part < extra ? 1 : 0);
    }

    // Key tiles travel global memory -> LDS directly, one step ahead of their use (two stages): wave-load j of a
    // region fills bytes 1024 j .. of it, lane l the chunk at 1024 j + 16 l, i.e. chunk position (1024 j + 16 l) % row
    // / 16 of row (1024 j + 16 l) / row -- which holds the row's chunk x3_swz(row, position).  The waves share the loads.
    const int last_tile = (a.S - 1) / TK;                 // the only K tile whose rows may not all exist
    B32Loads<E, D, M, NW> tl;
    tl.plan(a.k_ss, a.S - last_tile * TK, w, lane);
    const float* csp = a.chunk_scale + (long)bh * a.n_chunks;
    float cscale = (kt_lo < kt_hi) ? csp[kt_lo * TK / CH] : 0.f;
    const float kmax = SPLIT ? split_kmax(a.part_max, bh, a.n_split) : a.kmax[bh];

    // score operand: the query row as it is in memory, dims 16ks + 8h .. + 7
    const uint16_t* qrow = qptr + (long)min(iq, a.T - 1) * a.q_ss;
    uint4 qb[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qb[ks] = *reinterpret_cast<const uint4*>(qrow + 16 * ks + 8 * h);

    // overlap operand: step s = 2 kq + t holds features 32 kq + 8 (2 jj + t) + 4h + i of the [positive | negative] row
    uint4 qfb[FS];
    float lsq, qk1 = 0.f;
    if (SPLIT) {
        const long qr_ = (long)bh * a.T + min(iq, a.T - 1);
        const float* qfg = a.qfeat + qr_ * M;
#pragma unroll
        for (int s = 0; s < FS; ++s) {
            const floatx4 x0 = *reinterpret_cast<const floatx4*>(qfg + 32 * (s >> 1) + 8 * (s & 1) + 4 * h);
            const floatx4 x1 = *reinterpret_cast<const floatx4*>(qfg + 32 * (s >> 1) + 16 + 8 * (s & 1) + 4 * h);
            qfb[s] = make_uint4(pack_bf16x2(x0[0], x0[1]), pack_bf16x2(x0[2], x0[3]), pack_bf16x2(x1[0], x1[1]), pack_bf16x2(x1[2], x1[3]));
        }
        lsq = a.q_lsq[qr_];
    } else {
        // |q|^2 from the score operand (the lane pair holds the two halves of every 16 dims)
        float sq = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint32_t wds[4] = {qb[ks].x, qb[ks].y, qb[ks].z, qb[ks].w};
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const float lo_ = __uint_as_float(wds[x] << 16), hi_ = __uint_as_float(wds[x] & 0xffff0000u);
                sq += lo_ * lo_ + hi_ * hi_;
            }
        }
        const float diag_q = 0.5f * a.temp * pair32_sum(sq);
        // sqrt(t) P as bf16 head + bf16 remainder, rows of E + 8 elements
        uint16_t* Phi = lds;
        uint16_t* Plo = lds + MH * LDK;
        const float pscale = sqrtf(a.temp);
        for (int idx = tid; idx < MH * E / 4; idx += NT) {
            const int f = idx / (E / 4), c4 = idx % (E / 4);
            const floatx4 x = *reinterpret_cast<const floatx4*>(a.proj + (long)f * E + 4 * c4) * pscale;
            floatx4 rem;
            uint16_t hb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                hb[i] = f32_to_bf16(x[i]);
                rem[i] = x[i] - bf16_to_f32(hb[i]);
            }
            *reinterpret_cast<uint2*>(Phi + f * LDK + 4 * c4) = make_uint2(hb[0] | ((uint32_t)hb[1] << 16), hb[2] | ((uint32_t)hb[3] << 16));
            *reinterpret_cast<uint2*>(Plo + f * LDK + 4 * c4) = make_uint2(pack_bf16x2(rem[0], rem[1]), pack_bf16x2(rem[2], rem[3]));
        }
        __syncthreads();
        floatx16 dd[PB];                      // dd[pb][4b + i] = projection row 32 pb + 8b + 4h + i of this lane's query
        float qmax = 0.f;
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            floatx16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int off = (32 * pb + c) * LDK + 16 * ks + 8 * h;
                acc = mma32_bf16(*reinterpret_cast<const uint4*>(Phi + off), qb[ks], acc);
                acc = mma32_bf16(*reinterpret_cast<const uint4*>(Plo + off), qb[ks], acc);
            }
            dd[pb] = acc;
#pragma unroll
            for (int e = 0; e < 16; ++e)
                if (32 * pb + 8 * (e >> 2) + 4 * h + (e & 3) < a.mh_valid) qmax = fmaxf(qmax, fabsf(acc[e]));
        }
        qmax = pair32_max(qmax);
        lsq = -diag_q + qmax - lnm_half;
        // features, the normaliser q' . sum K' on the way, and the operand (positive blocks first, then negative)
        const float* ksg = a.ksum + (long)bh * M;
#pragma unroll
        for (int pb = 0; pb < PB; ++pb)
#pragma unroll
            for (int sg = 0; sg < 2; ++sg) {
                float f[16];
#pragma unroll
                for (int bq = 0; bq < 4; ++bq) {
                    const floatx4 ks4 = *reinterpret_cast<const floatx4*>(ksg + sg * MH + 32 * pb + 8 * bq + 4 * h);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float x = sg ? -dd[pb][4 * bq + i] : dd[pb][4 * bq + i];
                        const bool ok = 32 * pb + 8 * bq + 4 * h + i < a.mh_valid;
                        f[4 * bq + i] = ok ? bf16_round(__builtin_amdgcn_exp2f((x - qmax) * LOG2E)) : 0.f;     // (as the operand holds it)
                        qk1 += f[4 * bq + i] * ks4[i];
                    }
                }
                const int kq = sg * PB + pb;                  // 32-feature block of the [positive | negative] row
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    qfb[2 * kq + t] = make_uint4(pack_bf16x2(f[4 * t], f[4 * t + 1]), pack_bf16x2(f[4 * t + 2], f[4 * t + 3]),
                                                 pack_bf16x2(f[4 * (2 + t)], f[4 * (2 + t) + 1]), pack_bf16x2(f[4 * (2 + t) + 2], f[4 * (2 + t) + 3]));
            }
        qk1 = pair32_sum(qk1);
        __syncthreads();                 // the projection rows are dead; the tile buffers may overwrite them
    }

    const float sc = a.temp * LOG2E;             // scores leave the MFMA unscaled; exponents are base 2
    const float c0 = (lsq + kmax) * LOG2E;       // base-2 log-scale of the global low-rank term
    float m_run = c0;
    float ze = 0.f, zp = 0.f;
    floatx16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
    const int qw0 = q0 + 32 * w;
    const int smin = max(iq - lc_lo, 0);
    const unsigned span = qvalid ? (unsigned)max(min(iq + lc_hi, len) - smin, 0) : 0u;

    // fragment offsets inside a stage: step s of a row of 128 bytes or more reads chunk (2s + h) ^ (row & 7), i.e. one of
    // four lane-dependent offsets (by s % 4) plus 128 (s / 4) bytes
    static_assert(F_ROW >= 128, "feature rows of 64 features or more");
    int foff4[4], koff4[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        foff4[v] = c * F_ROW + (((2 * v + h) ^ (c & 7)) * 16);
        koff4[v] = K_ROW >= 128 ? c * K_ROW + (((2 * v + h) ^ (c & 7)) * 16) : c * K_ROW + x3_swz(c, (2 * v + h) & 3, K_ROW) * 16;
    }

    // One key tile takes two phases: scores (LDS fragment reads and the two score MFMA products) and softmax (the
    // arithmetic on the scores, and P V).  The first loads the LDS and matrix pipes, the second the vector ALU.  With
    // more than four waves per workgroup a SIMD holds two waves of it, and the upper half of the waves runs half a tile
    // behind the lower half (one reads fragments and multiplies while the other does its softmax arithmetic); a wave's
    // scores and V fragments of a tile stay in registers between the two phases.
    floatx16 s1, s2;
    uint4 vf[DB][2];
    auto touches = [&](int kt) __attribute__((always_inline)) {      // wave-uniform: does the tile touch the band of any of the wave's queries?
        const int s_base = kt * TK;
        return !(s_base + TK - 1 - qw0 < -lc_lo || s_base - (qw0 + 31) >= lc_hi || s_base >= len);
    };
    auto score_phase = [&](int kt, int stage) __attribute__((always_inline)) {
        if (!touches(kt)) return;
        const char* Ks = reinterpret_cast<const char*>(lds) + stage * STAGE_BYTES;
        const char* Fs = Ks + K_BYTES;
        const char* Vt = Fs + F_BYTES;
#pragma unroll
        for (int e = 0; e < 16; ++e) { s1[e] = 0.f; s2[e] = 0.f; }
        // fragments are requested from LDS in batches ahead of the MFMAs that use them
        uint4 kf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kf[ks] = *reinterpret_cast<const uint4*>(Ks + koff4[ks & 3] + 128 * (ks >> 2));
        // (feature fragments in small batches, the next batch requested before the MFMAs of the current one)
        constexpr int FBATCH = FS >= 16 ? 2 : (FS < 4 ? FS : 4), NBATCH = FS / FBATCH;    // (256 features leave room for pairs only)
        static_assert(FS % FBATCH == 0, "whole batches");
        uint4 ff[2][FBATCH];
#pragma unroll
        for (int s = 0; s < FBATCH; ++s) ff[0][s] = *reinterpret_cast<const uint4*>(Fs + foff4[s & 3] + 128 * (s >> 2));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s1 = mma32_bf16(kf[ks], qb[ks], s1);
#pragma unroll
        for (int bt = 0; bt < NBATCH; ++bt) {
            if (bt + 1 < NBATCH) {
#pragma unroll
                for (int s = 0; s < FBATCH; ++s) {
                    const int sn = (bt + 1) * FBATCH + s;
                    ff[(bt + 1) & 1][s] = *reinterpret_cast<const uint4*>(Fs + foff4[sn & 3] + 128 * (sn >> 2));
                }
            } else {
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int t = 0; t < 2; ++t)
                        vf[db][t] = *reinterpret_cast<const uint4*>(Vt + (32 * db + c) * V_ROW + x3_swz(32 * db + c, 2 * t + h, V_ROW) * 16);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < FBATCH; ++s) s2 = mma32_bf16(ff[bt & 1][s], qfb[bt * FBATCH + s], s2);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto soft_phase = [&](int kt, float cs) __attribute__((always_inline)) {
        if (!touches(kt)) return;
        const int s_base = kt * TK;
        const float wc = __builtin_amdgcn_exp2f((cs - kmax) * LOG2E);
        // the lane holds the raw scores q.k of its query against keys s_base + 8b + 4h + i (element 4b + i)
        const bool inside = s_base >= max(qw0 + 31 - lc_lo, 0) && s_base + TK <= min(qw0 + lc_hi, len) && qw0 + 31 < a.T;
        float p[16];
        float ovs = 0.f;
        auto soft = [&](auto masked_t) __attribute__((always_inline)) {
            constexpr bool MASKED = decltype(masked_t)::value;
            bool ok[16];
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int s = s_base + 8 * (e >> 2) + 4 * h + (e & 3);
                ok[e] = !MASKED || (unsigned)(s - smin) < span;
                mx = fmaxf(mx, ok[e] ? s1[e] : -INFINITY);
            }
            mx = pair32_max(mx) * sc;                               // sc > 0
            // The reference exponent is raised only when a tile exceeds it by more than 2^8 (wave-uniform vote), but the
            // rescale itself is unconditional (by 1 when nothing was raised): inside a branch the compiler gave the scaled
            // accumulators new registers and copied all 32 of them on the usual path and back at the end of every tile
            // (33 multiplies instead of 32 two-register moves and two waits for the matrix pipe).
            {
                const bool grow = __builtin_amdgcn_ballot_w64(mx > m_run + 8.f) != 0;
                const float m_new = grow ? fmaxf(m_run, mx) : m_run;
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                m_run = m_new;
                ze *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
            }
            const float beta = wc * __builtin_amdgcn_exp2f(c0 - m_run);      // scale of the overlap term
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float ex = ok[e] ? __builtin_amdgcn_exp2f(__builtin_fmaf(s1[e], sc, -m_run)) : 0.f;
                const float ov = ok[e] ? s2[e] : 0.f;
                ze += ex;
                ovs += ov;
                p[e] = ex - ov * beta;
            }
        };
        if (inside) soft(std::false_type{}); else soft(std::true_type{});
        // (see second_piece_wanted: where the band's low-rank part dwarfs the exact weights the probabilities go to
        //  the matrix pipe in two bf16 pieces)
        zp += ovs * wc;
        const bool two = TWO_PIECE && second_piece_wanted(zp * __builtin_amdgcn_exp2f(c0 - m_run), ze);
        // O^T[d][query] += sum_keys V[key][d] p[key][query]: step t takes the lane's elements 4t + i and 4(2 + t) + i
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint4 pb_ = make_uint4(pack_bf16x2(p[4 * t], p[4 * t + 1]), pack_bf16x2(p[4 * t + 2], p[4 * t + 3]),
                                         pack_bf16x2(p[4 * (2 + t)], p[4 * (2 + t) + 1]), pack_bf16x2(p[4 * (2 + t) + 2], p[4 * (2 + t) + 3]));
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma32_bf16(vf[db][t], pb_, oacc[db]);
            if (two) {                                           // wave-uniform
                const uint4 pl_ = make_uint4(pack_rest(p[4 * t], p[4 * t + 1], pb_.x), pack_rest(p[4 * t + 2], p[4 * t + 3], pb_.y),
                                             pack_rest(p[4 * (2 + t)], p[4 * (2 + t) + 1], pb_.z),
                                             pack_rest(p[4 * (2 + t) + 2], p[4 * (2 + t) + 3], pb_.w));
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] = mma32_bf16(vf[db][t], pl_, oacc[db]);
            }
        }
    };
    // Both phases of a tile in one piece, for waves that are not skewed.  The overlap products q'.k' of a tile are one chain of
    // FS MFMAs on one accumulator: each waits for the one before it, and a wave that has nothing else to issue waits with
    // it.  Everything of the softmax that needs only the scores -- maximum, reference exponent, rescale, the
    // exponentials and their sum -- is therefore placed between the links of that chain (sched_group_barrier: one MFMA,
    // then a share of the vector instructions), and only the subtraction of the overlap follows it.
    auto tile_phase = [&](int kt, int stage, float cs) __attribute__((always_inline)) {
        if (!touches(kt)) return;
        const char* Ks = reinterpret_cast<const char*>(lds) + stage * STAGE_BYTES;
        const char* Fs = Ks + K_BYTES;
        const char* Vt = Fs + F_BYTES;
#pragma unroll
        for (int e = 0; e < 16; ++e) { s1[e] = 0.f; s2[e] = 0.f; }
        uint4 kf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kf[ks] = *reinterpret_cast<const uint4*>(Ks + koff4[ks & 3] + 128 * (ks >> 2));
        constexpr int FBATCH = FS >= 16 ? 2 : (FS < 4 ? FS : 4), NBATCH = FS / FBATCH;
        static_assert(FS % FBATCH == 0, "whole batches");
        uint4 ff[2][FBATCH];
#pragma unroll
        for (int s = 0; s < FBATCH; ++s) ff[0][s] = *reinterpret_cast<const uint4*>(Fs + foff4[s & 3] + 128 * (s >> 2));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s1 = mma32_bf16(kf[ks], qb[ks], s1);
        __builtin_amdgcn_sched_barrier(0);
        const int s_base = kt * TK;
        const float wc = __builtin_amdgcn_exp2f((cs - kmax) * LOG2E);
        const bool inside = s_base >= max(qw0 + 31 - lc_lo, 0) && s_base + TK <= min(qw0 + lc_hi, len) && qw0 + 31 < a.T;
        float p[16];
        float ovs = 0.f;
        auto soft = [&](auto masked_t) __attribute__((always_inline)) {
            constexpr bool MASKED = decltype(masked_t)::value;
            // the chain, its fragments a batch ahead (V^T fragments with the last batch)
#pragma unroll
            for (int bt = 0; bt < NBATCH; ++bt) {
                if (bt + 1 < NBATCH) {
#pragma unroll
                    for (int s = 0; s < FBATCH; ++s) {
                        const int sn = (bt + 1) * FBATCH + s;
                        ff[(bt + 1) & 1][s] = *reinterpret_cast<const uint4*>(Fs + foff4[sn & 3] + 128 * (sn >> 2));
                    }
                } else {
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int t = 0; t < 2; ++t)
                            vf[db][t] = *reinterpret_cast<const uint4*>(Vt + (32 * db + c) * V_ROW + x3_swz(32 * db + c, 2 * t + h, V_ROW) * 16);
                }
#pragma unroll
                for (int s = 0; s < FBATCH; ++s) s2 = mma32_bf16(ff[bt & 1][s], qfb[bt * FBATCH + s], s2);
            }
            // in its shadow: what the scores alone decide
            bool ok[16];
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int s = s_base + 8 * (e >> 2) + 4 * h + (e & 3);
                ok[e] = !MASKED || (unsigned)(s - smin) < span;
                mx = fmaxf(mx, ok[e] ? s1[e] : -INFINITY);
            }
            mx = pair32_max(mx) * sc;                               // sc > 0
            {   // (see soft_phase: the vote is wave-uniform, the rescale unconditional)
                const bool grow = __builtin_amdgcn_ballot_w64(mx > m_run + 8.f) != 0;
                const float m_new = grow ? fmaxf(m_run, mx) : m_run;
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                m_run = m_new;
                ze *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                p[e] = ok[e] ? __builtin_amdgcn_exp2f(__builtin_fmaf(s1[e], sc, -m_run)) : 0.f;
                ze += p[e];
            }
            // the order asked of the scheduler: per batch its LDS reads, then link by link one MFMA and a share of the
            // vector work
            constexpr int VSHARE = (MASKED ? 176 : 144) / FS;
#pragma unroll
            for (int bt = 0; bt + 1 < NBATCH; ++bt) {
                __builtin_amdgcn_sched_group_barrier(0x100, FBATCH, 0);
#pragma unroll
                for (int s = 0; s < FBATCH; ++s) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, VSHARE, 0);
                }
            }
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * DB, 0);
#pragma unroll
            for (int s = 0; s < FBATCH; ++s) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, VSHARE, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            const float beta = wc * __builtin_amdgcn_exp2f(c0 - m_run);      // scale of the overlap term
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float ov = ok[e] ? s2[e] : 0.f;
                ovs += ov;
                p[e] = __builtin_fmaf(-ov, beta, p[e]);
            }
        };
        if (inside) soft(std::false_type{}); else soft(std::true_type{});
        zp += ovs * wc;
        const bool two = TWO_PIECE && second_piece_wanted(zp * __builtin_amdgcn_exp2f(c0 - m_run), ze);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint4 pb_ = make_uint4(pack_bf16x2(p[4 * t], p[4 * t + 1]), pack_bf16x2(p[4 * t + 2], p[4 * t + 3]),
                                         pack_bf16x2(p[4 * (2 + t)], p[4 * (2 + t) + 1]), pack_bf16x2(p[4 * (2 + t) + 2], p[4 * (2 + t) + 3]));
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma32_bf16(vf[db][t], pb_, oacc[db]);
            if (two) {                                           // wave-uniform
                const uint4 pl_ = make_uint4(pack_rest(p[4 * t], p[4 * t + 1], pb_.x), pack_rest(p[4 * t + 2], p[4 * t + 3], pb_.y),
                                             pack_rest(p[4 * (2 + t)], p[4 * (2 + t) + 1], pb_.z),
                                             pack_rest(p[4 * (2 + t) + 2], p[4 * (2 + t) + 3], pb_.w));
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] = mma32_bf16(vf[db][t], pl_, oacc[db]);
            }
        }
    };
    const bool late = NW > 4 && w >= NW / 2;      // wave-uniform: this wave runs half a tile behind
    float cs_prev = 0.f;                          // chunk scale of the tile a late wave still owes its softmax
    // (the first pass, kt = kt_lo - 1, only brings the first tile in)
    for (int kt = kt_lo - 1; kt < kt_hi; ++kt) {
        const int cur = (kt - kt_lo) & 1;
        const bool more = kt + 1 < kt_hi;
        float cscale_next = cscale;
        if (more) {                                      // next tile's loads fly during the MFMAs (every wave is past the barrier
            const int ktn = kt + 1, ktc = min(ktn, last_tile);      // that ended the last use of that stage; tiles past the keys
            tl.issue(reinterpret_cast<char*>(lds) + (cur ^ 1) * STAGE_BYTES, w, ktc == last_tile,      // are never used: stay in bounds)
                     reinterpret_cast<const char*>(kptr + (long)ktc * TK * a.k_ss),
                     reinterpret_cast<const char*>(fptr + (long)ktn * TK * M), reinterpret_cast<const char*>(vtp + (long)ktn * (D * TK)));
            cscale_next = csp[(kt + 1) * TK / CH];
        }
        if (kt >= kt_lo) {
            if (!late) {
#if FLY_B32_FUSED_TILE
                tile_phase(kt, cur, cscale);
#else
                score_phase(kt, cur);
                soft_phase(kt, cscale);
#endif
            } else {
                if (kt > kt_lo) soft_phase(kt - 1, cs_prev);
                score_phase(kt, cur);
                cs_prev = cscale;
            }
        }
        drain_loads();                                   // this wave's share of the next tile is in LDS
        cscale = cscale_next;
        __syncthreads();
    }
    if (late && kt_lo < kt_hi) soft_phase(kt_hi - 1, cs_prev);

    // global low-rank term: qkv^T[d][query] = sum_r KV[r][d] q'[query][r]; K'^T V comes as bf16, transposed,
    // features in the slot order of the overlap operand
    floatx16 lacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) lacc[db][e] = 0.f;
    if (!SPLIT) {
        uint16_t* KVt = lds;
        constexpr int KVC = D * M / 8;
#pragma nounroll                                 // (unrolled, the copies cost the key loop registers)
        for (int piece = 1; piece >= 0; --piece) {       // the rest first, then the head (two bf16 pieces of K'^T V)
            const uint16_t* kvg = reinterpret_cast<const uint16_t*>(a.kvt) + ((long)bh * 2 + piece) * M * D;
            if (piece == 0) __syncthreads();             // the first piece has been read
#pragma unroll
            for (int j = 0; j < (KVC + NT - 1) / NT; ++j) {
                const int idx = tid + NT * j, d = idx / (M / 8), c8 = idx % (M / 8);
                if (KVC % NT == 0 || idx < KVC)
                    *reinterpret_cast<uint4*>(KVt + d * LDKV + 8 * c8) = *reinterpret_cast<const uint4*>(kvg + (long)d * M + 8 * c8);
            }
            __syncthreads();
#pragma unroll
            for (int s = 0; s < FS; ++s)
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    lacc[db] = mma32_bf16(*reinterpret_cast<const uint4*>(KVt + (32 * db + c) * LDKV + 16 * s + 8 * h), qfb[s], lacc[db]);
        }
    }
    ze = pair32_sum(ze);
    zp = pair32_sum(zp);
    const float gamma = __builtin_amdgcn_exp2f(c0 - m_run);               // <= 1
    if (SPLIT) {
        // partials are kept per 64-query tile (the unit of sb_merge_kernel); this wave's tile:
        const int n_qt64 = (a.T + TQ64 - 1) / TQ64, t64 = (q0 + 32 * w) / TQ64;
        if (t64 < n_qt64) {                            // wave-uniform
            float* ws = a.part_ws + (((long)bh * n_qt64 + t64) * a.n_parts + part) * (TQ64 * (D + NSTAT));
            const int ql = (32 * w + c) % TQ64;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int bq = 0; bq < 4; ++bq) {
                    const floatx4 o4 = {oacc[db][4 * bq], oacc[db][4 * bq + 1], oacc[db][4 * bq + 2], oacc[db][4 * bq + 3]};
                    *reinterpret_cast<floatx4*>(ws + ql * D + 32 * db + 8 * bq + 4 * h) = o4;
                }
            if (h == 0) {
                float* st = ws + TQ64 * D;
                st[0 * TQ64 + ql] = m_run;
                st[1 * TQ64 + ql] = ze;
                st[2 * TQ64 + ql] = zp;
                st[3 * TQ64 + ql] = 0.f;
                st[4 * TQ64 + ql] = c0;
            }
        }
    } else {
        const float Z = ze + gamma * fmaxf(qk1 - zp, 1e-24f);
        const float inv = 1.0f / Z;
        if (qvalid) {
            T* optr = reinterpret_cast<T*>(a.out) + b * a.o_sb + hd * a.o_sh + (long)iq * a.o_ss;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int bq = 0; bq < 4; ++bq) {
                    floatx4 o4;
#pragma unroll
                    for (int i = 0; i < 4; ++i) o4[i] = (oacc[db][4 * bq + i] + gamma * lacc[db][4 * bq + i]) * inv;
                    store4_f32(optr + 32 * db + 8 * bq + 4 * h, o4);
                }
            if (h == 0) a.log_norm[(long)bh * a.T + iq] = m_run * LN2 + __logf(Z);
        }
    }
}

// (explicit instantiations: the launcher refers to these through a deduced return type)
#define FLY_B32_INST(EE, MM)                                                        \
    template __global__ void sblocal_fwd_b32_kernel<EE, EE, MM, false, B32_WAVES>(FwdArgs);   \
    template __global__ void sblocal_fwd_b32_kernel<EE, EE, MM, true, B32_WAVES>(FwdArgs);
FLY_B32_INST(32, 64) FLY_B32_INST(32, 128) FLY_B32_INST(32, 256)
FLY_B32_INST(64, 64) FLY_B32_INST(64, 128) FLY_B32_INST(64, 256)
#undef FLY_B32_INST

// ---------------------------------------------------------------------------------------
// key pass for bfloat16 inputs (key role only; used when no query features are asked for)
// ---------------------------------------------------------------------------------------
// The same outputs as the key role of sb_kfeat_kernel, with both contractions on the bf16 MFMA:
//   projection : S[key][feature] = K . (sqrt(t) log2e P)^T with K as it is in memory (bf16) and the
//                projection split into a bf16 head and remainder.  Rows = keys: a lane owns ONE
//                feature and receives keys 4g+i of every 16-key block -- which is the operand
//                layout (lane = feature, k-slots = keys) the second product needs, so the
//                features go from registers straight into it.
//   K'^T V     : KV[feature][d] = sum_keys F[key][feature] V[key][d] with V transposed through LDS
//                to [d][key slot]; the same LDS tile is what the band kernel wants in HBM (vt).
// Wave w owns the projection rows of blocks w, w+4, ... (both signs of each), for all 64 keys of
// the chunk.  The feature scratch for the band kernel ([key][k-slot order]) is assembled in LDS
// from 2-byte writes and leaves as 16-byte stores.
// (two workgroups per compute unit: the pass streams, and one workgroup's loads in flight do not fill the memory pipe;
//  the few registers this spills cost less than that)
template <int E, int D, int M>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, 2))) void sb_kfeat_bf16_kernel(KvArgs a) {
    constexpr int MH = M / 2, FB = MH / 16, DB = D / 16, KS = E / 32, KBN = CH / 16;
    constexpr int FPW = (FB + 3) / 4;                       // projection-row blocks per wave
    constexpr int LDK = E + 8, LDVT = CH + 8, LDFO = M + 8; // LDS row strides in 2-byte elements
    constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
    extern __shared__ __attribute__((aligned(128))) float smem[];
    uint16_t* Ks = reinterpret_cast<uint16_t*>(smem);      // [CH][LDK]   keys of the chunk
    uint16_t* Vt = Ks + CH * LDK;                           // [D][LDVT]   values, transposed, slot order
    uint16_t* Fo = Vt + D * LDVT;                           // [CH][LDFO]  features for the band kernel
    float* diag = reinterpret_cast<float*>(Fo + CH * LDFO); // [CH]        t log2e |k|^2 / 2
    float* red = diag + CH;                                 // [4]         wave maxima

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H, sp = blockIdx.x;
    const uint16_t* kptr = reinterpret_cast<const uint16_t*>(a.k) + b * a.k_sb + h * a.k_sh;
    const uint16_t* vptr = reinterpret_cast<const uint16_t*>(a.v) + b * a.v_sb + h * a.v_sh;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half2 = 0.5f * __log2f(2.0f * a.mh_valid);
    const int per = (a.n_chunks + a.n_split - 1) / a.n_split;
    const int c0 = sp * per, c1 = min(a.n_chunks, c0 + per);

    Tile16<CH, E, NT> rk;
    Tile16<CH, D, NT> rv;
    if (c0 < c1) {
        rk.fetch(kptr, a.k_ss, c0 * CH, a.S - 1, tid);
        rv.fetch(vptr, a.v_ss, c0 * CH, a.S - 1, tid);
    }
    // this wave's projection rows (feature c of block w + 4 fi), scaled by sqrt(t) log2e, as bf16 head
    // and remainder: lane (c = r16, g) holds columns 32ks + 8g .. + 7
    uint4 phi[FPW][KS], plo[FPW][KS];
    const float pscale = sqrtf(a.temp) * LOG2E;
#pragma unroll
    for (int fi = 0; fi < FPW; ++fi) {
        const int row = min(16 * (w + 4 * fi) + r16, MH - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const float* src = a.proj + (long)row * E + 32 * ks + 8 * g;
            const floatx4 x0 = *reinterpret_cast<const floatx4*>(src) * pscale;
            const floatx4 x1 = *reinterpret_cast<const floatx4*>(src + 4) * pscale;
            float xs[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
            uint32_t hw[4], lw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                hw[j] = pack_bf16x2(xs[2 * j], xs[2 * j + 1]);
                lw[j] = pack_bf16x2(xs[2 * j] - __uint_as_float(hw[j] << 16), xs[2 * j + 1] - __uint_as_float(hw[j] & 0xffff0000u));
            }
            phi[fi][ks] = make_uint4(hw[0], hw[1], hw[2], hw[3]);
            plo[fi][ks] = make_uint4(lw[0], lw[1], lw[2], lw[3]);
        }
    }
    // the tile in registers -> LDS: K rows as they are; V transposed into the slot order of the band
    // kernel's P V (column 32 t + 8g + 4h + i <- key 32 t + 16 h + 4 g + i); |k|^2 per key on the way
    auto stash = [&]() __attribute__((always_inline)) {
        rk.template stash<LDK>(Ks, tid);
#pragma unroll
        for (int j = 0; j < Tile16<CH, E, NT>::N; ++j) {
            constexpr int C8 = E / 8;
            const int idx = tid + NT * j, row = idx / C8;
            const uint32_t wds[4] = {rk.r[j][0], rk.r[j][1], rk.r[j][2], rk.r[j][3]};
            float sq = 0.f;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const float lo = __uint_as_float(wds[x] << 16), hi = __uint_as_float(wds[x] & 0xffff0000u);
                sq += lo * lo + hi * hi;
            }
#pragma unroll
            for (int off = 1; off < C8; off <<= 1) sq += __shfl_xor(sq, off);      // the C8 lanes of one key row
            if (idx % C8 == 0 && idx < CH * C8) diag[row] = 0.5f * a.temp * LOG2E * sq;
        }
#pragma unroll
        for (int j = 0; j < Tile16<CH, D, NT>::N; ++j) {
            constexpr int C8 = D / 8;
            const int idx = tid + NT * j, key = idx / C8, c8 = idx % C8;
            if (idx < CH * C8) {
                const int col = 32 * (key >> 5) + 8 * ((key >> 2) & 3) + 4 * ((key >> 4) & 1) + (key & 3);
                const uint32_t wds[4] = {rv.r[j][0], rv.r[j][1], rv.r[j][2], rv.r[j][3]};
#pragma unroll
                for (int x = 0; x < 8; ++x) Vt[(8 * c8 + x) * LDVT + col] = (uint16_t)(wds[x >> 1] >> (16 * (x & 1)));
            }
        }
    };
    if (c0 < c1) stash();
    __syncthreads();

    floatx4 kvacc[FPW][2][DB];                   // [block][sign][value block]
    float ksum_p[FPW], ksum_n[FPW];              // this lane's feature, summed over its keys
#pragma unroll
    for (int fi = 0; fi < FPW; ++fi) {
        ksum_p[fi] = ksum_n[fi] = 0.f;
#pragma unroll
        for (int sg = 0; sg < 2; ++sg)
#pragma unroll
            for (int db = 0; db < DB; ++db) kvacc[fi][sg][db] = Frag<float>::zero();
    }
    float run_max = -INFINITY;

    for (int c = c0; c < c1; ++c) {
        const int s_base = c * CH;
        if (c + 1 < c1) {
            rk.fetch(kptr, a.k_ss, s_base + CH, a.S - 1, tid);
            rv.fetch(vptr, a.v_ss, s_base + CH, a.S - 1, tid);
        }
        // projections: dd[fi][kb][i] = log2e sqrt(t) P[feature] . k[key 16kb + 4g + i]
        uint4 kf[KBN][KS];
#pragma unroll
        for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                kf[kb][ks] = *reinterpret_cast<const uint4*>(Ks + (16 * kb + r16) * LDK + 32 * ks + 8 * g);
        floatx4 dg[KBN];
#pragma unroll
        for (int kb = 0; kb < KBN; ++kb) dg[kb] = *reinterpret_cast<const floatx4*>(diag + 16 * kb + 4 * g);
        floatx4 dd[FPW][KBN];
#pragma unroll
        for (int fi = 0; fi < FPW; ++fi)
#pragma unroll
            for (int kb = 0; kb < KBN; ++kb) {
                dd[fi][kb] = Frag<float>::zero();
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    dd[fi][kb] = mma_bf16(kf[kb][ks], phi[fi][ks], dd[fi][kb]);
                    dd[fi][kb] = mma_bf16(kf[kb][ks], plo[fi][ks], dd[fi][kb]);
                }
            }
        // chunk stabiliser: max over valid keys and features of |dd| - diag
        float cs = -INFINITY;
#pragma unroll
        for (int fi = 0; fi < FPW; ++fi) {
            const bool fvalid = (w + 4 * fi) < FB && 16 * (w + 4 * fi) + r16 < a.mh_valid;
#pragma unroll
            for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool ok = fvalid && (s_base + 16 * kb + 4 * g + i) < len;
                    cs = fmaxf(cs, ok ? fabsf(dd[fi][kb][i]) - dg[kb][i] : -INFINITY);
                }
        }
        // a valid key whose features are all masked (mh_valid rows only in other waves) still bounds the max
#pragma unroll
        for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if ((s_base + 16 * kb + 4 * g + i) < len) cs = fmaxf(cs, -dg[kb][i]);
        cs = wave_max(cs) - lnm_half2;
        if (lane == 0) red[w] = cs;
        __syncthreads();
        const float lmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float new_max = fmaxf(run_max, lmax);
        const bool live = new_max != -INFINITY;              // workgroup-uniform: some valid key so far
        const float rescale = (run_max == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(run_max - new_max);
        if (live) run_max = new_max;
        // per (block, sign): features of the lane's feature for all 64 keys -> column sums, the feature
        // scratch in LDS (band kernel's order: block bm of the [positive | negative] row, feature c of it
        // -> position 32 (bm/2) + 8 (c/4) + 4 (bm%2) + c%4 of the key's row) and K'^T V
#pragma unroll
        for (int fi = 0; fi < FPW; ++fi) {
            const bool fvalid = (w + 4 * fi) < FB && 16 * (w + 4 * fi) + r16 < a.mh_valid;
            ksum_p[fi] *= rescale;
            ksum_n[fi] *= rescale;
#pragma unroll
            for (int sg = 0; sg < 2; ++sg) {
#pragma unroll
                for (int db = 0; db < DB; ++db) kvacc[fi][sg][db] *= rescale;
                // the features as the bf16 pairs every later product reads; their sum is taken from
                // the same rounded values, so that numerator and normaliser see one set of features
                uint32_t fp[KBN][2];
                float tot = 0.f;
#pragma unroll
                for (int kb = 0; kb < KBN; ++kb) {
                    float f[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const bool ok = live && fvalid && (s_base + 16 * kb + 4 * g + i) < len;
                        const float x = sg ? -dd[fi][kb][i] : dd[fi][kb][i];
                        f[i] = ok ? __builtin_amdgcn_exp2f(x - dg[kb][i] - lnm_half2 - new_max) : 0.f;
                    }
                    fp[kb][0] = pack_bf16x2(f[0], f[1]);
                    fp[kb][1] = pack_bf16x2(f[2], f[3]);
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        tot += __uint_as_float(fp[kb][h] << 16) + __uint_as_float(fp[kb][h] & 0xffff0000u);
                }
                if (sg) ksum_n[fi] += tot; else ksum_p[fi] += tot;
                if ((w + 4 * fi) < FB) {
                    const int bm = sg * FB + w + 4 * fi;
                    const int pos = 32 * (bm >> 1) + 8 * (r16 >> 2) + 4 * (bm & 1) + (r16 & 3);
#pragma unroll
                    for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            Fo[(16 * kb + 4 * g + i) * LDFO + pos] = (uint16_t)(fp[kb][i >> 1] >> (16 * (i & 1)));
                }
                // KV[feature][d] += sum_keys F[key][feature] V[key][d], 32 keys per MFMA step
#pragma unroll
                for (int t = 0; t < CH / 32; ++t) {
                    const uint4 fa = make_uint4(fp[2 * t][0], fp[2 * t][1], fp[2 * t + 1][0], fp[2 * t + 1][1]);
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        kvacc[fi][sg][db] = mma_bf16(fa, *reinterpret_cast<const uint4*>(Vt + (16 * db + r16) * LDVT + 32 * t + 8 * g),
                                                     kvacc[fi][sg][db]);
                }
            }
        }
        if (tid == 0) a.chunk_scale[(long)bh * a.n_chunks + c] = live ? new_max * LN2 : 0.f;
        __syncthreads();                         // Fo complete
        // LDS -> HBM in 16-byte pieces: the chunk's features, and its V as two transposed 32-key tiles
        {
            uint16_t* fdst = reinterpret_cast<uint16_t*>(a.kfeat) + ((long)bh * a.n_chunks * CH + s_base) * M;
#pragma unroll
            for (int j = 0; j < CH * M / 8 / NT; ++j) {
                const int idx = tid + NT * j, row = idx / (M / 8), c8 = idx % (M / 8);
                *reinterpret_cast<uint4*>(fdst + (long)row * M + 8 * c8) = *reinterpret_cast<const uint4*>(Fo + row * LDFO + 8 * c8);
            }
            uint16_t* vdst = reinterpret_cast<uint16_t*>(a.vt) + ((long)bh * a.n_chunks + c) * (CH * D);
#pragma unroll
            for (int j = 0; j < (CH * D / 8 + NT - 1) / NT; ++j) {
                const int idx = tid + NT * j, tile = idx / (D * 4), rem = idx % (D * 4), d = rem / 4, c8 = rem % 4;
                if (idx < CH * D / 8)
                    *reinterpret_cast<uint4*>(vdst + tile * (D * 32) + d * 32 + 8 * c8) =
                        *reinterpret_cast<const uint4*>(Vt + d * LDVT + 32 * tile + 8 * c8);
            }
        }
        __syncthreads();                         // everyone is done with this chunk's tiles
        if (c + 1 < c1) stash();
        __syncthreads();
    }

    // partial K'^T V in accumulator order: tile (rb, db) -> 64 lanes x 4 floats (see sb_combine_kernel)
    float* part = a.kv_part + ((long)bh * a.n_split + sp) * (M * (D + 1));
#pragma unroll
    for (int fi = 0; fi < FPW; ++fi) {
        if ((w + 4 * fi) < FB) {
#pragma unroll
            for (int sg = 0; sg < 2; ++sg) {
                const int rb = sg * FB + w + 4 * fi;
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    *reinterpret_cast<floatx4*>(part + ((rb * DB + db) * 64 + lane) * 4) = kvacc[fi][sg][db];
                const float tot = group_sum(sg ? ksum_n[fi] : ksum_p[fi]);       // over the four key groups g
                if (g == 0) part[M * D + sg * MH + 16 * (w + 4 * fi) + r16] = tot;
            }
        }
    }
    if (tid == 0) a.part_max[(long)bh * a.n_split + sp] = run_max * LN2;
}

// ---------------------------------------------------------------------------------------
// plain local attention (no random features): softmax over the band, P V
// ---------------------------------------------------------------------------------------
// The band kernel without its low-rank half: per (batch, head, 64-query tile) scores^T = (t log2e) K q
// on fp32 MFMA, band / length masks, online softmax, P V; key tiles double-buffered through LDS.
// A query without any valid key gets a zero output row.
struct LocalArgs {
    const void* q; const void* k; const void* v; const int64_t* lens; void* out;
    int B, H, T, S, lc;
    long q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss;
    float temp;
    float* lse;                     // optional (B, H, T): log of the softmax denominator, for the backward pass
    int n_xcd;                      // dies the dispatcher deals workgroup ids to (set at launch)
    // dropout of the probabilities (drop_thresh != 0): pair (query i, key s) of (b, h) is kept when the hash of
    // (seed, row = (b H + h) T + i, s) reaches the threshold, and scaled by 1 / (1 - p); the denominator sums all
    uint32_t drop_seed, drop_thresh; float drop_scale;
    // optional additive mask (T, S), float32, rows contiguous: added to q.k before the temperature.  Entries of -1e24
    // absorb the product (every masked score is the same float), so a query whose visible keys are all masked gets
    // equal weights 1 / local_context -- over the positions of its band that fall outside the keys as well, which
    // count in the denominator only; its lse entry is -inf, the marker the backward kernel reads.
    const float* add_mask;
};

template <typename T, int E, int D>
__global__ __launch_bounds__(NT) void local_fwd_kernel(LocalArgs a) {
    constexpr int LDK = E + 4, LDV = D + 4, EC = E / 16, DB = D / 16, KB = TK / 16;
    constexpr int STAGE = TK * (LDK + LDV);
    constexpr float LOG2E = 1.4426950408889634f;
    extern __shared__ __attribute__((aligned(128))) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int n_qt = (a.T + TQ - 1) / TQ;
    const int n_items = a.B * a.H * n_qt;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // see sblocal_fwd_kernel
    if (item >= n_items) return;                       // workgroup-uniform
    const int qt = item % n_qt, bh = item / n_qt, b = bh / a.H, h = bh % a.H;
    const int q0 = qt * TQ, iq = q0 + 16 * w + r16;
    const bool qvalid = iq < a.T;
    const T* qptr = reinterpret_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh;
    const T* kptr = reinterpret_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh;
    const T* vptr = reinterpret_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi

    const int q_last = min(q0 + TQ - 1, a.T - 1);
    const int lo = max(0, q0 - lc_lo), hi = min(len, q_last + lc_hi);
    const int kt_lo = lo / TK, kt_hi = (hi > lo) ? (hi + TK - 1) / TK : kt_lo;
    RowTile<TK, E> rk;
    RowTile<TK, D> rv;
    if (kt_lo < kt_hi) {
        rk.fetch(kptr, a.k_ss, kt_lo * TK, a.S - 1, tid);
        rv.fetch(vptr, a.v_ss, kt_lo * TK, a.S - 1, tid);
    }
    floatx4 qr[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        qr[c] = Frag<float>::zero();
        if (qvalid) qr[c] = load4_f32(qptr + (long)iq * a.q_ss + 16 * c + 4 * g) * (a.temp * LOG2E);
    }
    float m_run = -1e30f;           // finite, so that the first rescale is exp2(-huge) = 0 and not inf - inf
    float ze = 0.f;
    floatx4 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = Frag<float>::zero();
    const int qw0 = q0 + 16 * w;
    const int smin = max(iq - lc_lo, 0);
    const unsigned span = qvalid ? (unsigned)max(min(iq + lc_hi, len) - smin, 0) : 0u;
    const uint32_t drop_row = a.drop_thresh != 0u ? drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + iq)) : 0u;
    if (kt_lo < kt_hi) {
        rk.template stash<LDK>(smem, tid);
        rv.template stash<LDV>(smem + TK * LDK, tid);
    }
    __syncthreads();
    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        const int s_base = kt * TK, cur = (kt - kt_lo) & 1;
        const float* Ks = smem + cur * STAGE;
        const float* Vs = Ks + TK * LDK;
        const bool more = kt + 1 < kt_hi;
        if (more) {
            rk.fetch(kptr, a.k_ss, s_base + TK, a.S - 1, tid);
            rv.fetch(vptr, a.v_ss, s_base + TK, a.S - 1, tid);
        }
        const bool any = !(s_base + TK - 1 - qw0 < -lc_lo || s_base - (qw0 + 15) >= lc_hi || s_base >= len);
        if (any) {
            floatx4 s1[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) s1[kb] = Frag<float>::zero();
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                floatx4 ka[KB];
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
                    ka[kb] = *reinterpret_cast<const floatx4*>(Ks + (16 * kb + r16) * LDK + 4 * g + 16 * c);
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
                        s1[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[kb][j], qr[c][j], s1[kb], 0, 0, 0);
            }
            bool ok[KB][4];
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int s = s_base + 16 * kb + 4 * g + i;
                    ok[kb][i] = (unsigned)(s - smin) < span;
                }
            if (a.add_mask) {                                // (uniform)
                const float* am = a.add_mask + (long)min(iq, a.T - 1) * a.S;
                const float cs = a.temp * LOG2E;
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (ok[kb][i]) s1[kb][i] += am[s_base + 16 * kb + 4 * g + i] * cs;
            }
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) mx = fmaxf(mx, ok[kb][i] ? s1[kb][i] : -INFINITY);
            mx = group_max(mx);
            if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.f) != 0) {
                const float m_new = fmaxf(m_run, mx);
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                m_run = m_new;
                ze *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
            }
            floatx4 p[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    p[kb][i] = ok[kb][i] ? __builtin_amdgcn_exp2f(s1[kb][i] - m_run) : 0.f;
                    ze += p[kb][i];
                }
            if (a.drop_thresh != 0u) {                   // (uniform) dropped weights leave the product, not the denominator
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (!drop_keep(drop_row, (uint32_t)(s_base + 16 * kb + 4 * g + i), a.drop_thresh)) p[kb][i] = 0.f;
            }
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        oacc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                            Vs[(16 * kb + 4 * g + i) * LDV + 16 * db + r16], p[kb][i], oacc[db], 0, 0, 0);
        }
        if (more) {
            float* nxt = smem + (cur ^ 1) * STAGE;
            rk.template stash<LDK>(nxt, tid);
            rv.template stash<LDV>(nxt + TK * LDK, tid);
        }
        __syncthreads();
    }
    ze = group_sum(ze);
    // every visible key masked: the positions of the band outside the keys carry the same score in the reference's
    // softmax over the packed band (local_attention.py:68-81), so they count in the denominator
    const bool all_masked = a.add_mask != nullptr && span > 0u && m_run < -1e20f;
    if (all_masked) ze += (float)(a.lc - (int)span);
    if (qvalid) {
        const float inv = (ze > 0.f ? 1.0f / ze : 0.f) * (a.drop_thresh != 0u ? a.drop_scale : 1.0f);
        T* optr = reinterpret_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq * a.o_ss;
#pragma unroll
        for (int db = 0; db < DB; ++db) store4_f32(optr + 16 * db + 4 * g, oacc[db] * inv);
        if (a.lse && g == 0)        // a query without visible keys has no pair that would read its entry
            a.lse[((long)b * a.H + h) * a.T + iq] = all_masked ? -INFINITY
                                                    : ze > 0.f ? m_run * 0.6931471805599453f + __logf(ze) : 0.f;
    }
}

// ---------------------------------------------------------------------------------------
// plain local attention for 2-byte inputs: both products on the 16x16x32 MFMA of the input type
// ---------------------------------------------------------------------------------------
// The same work decomposition, masks, online softmax and outputs as local_fwd_kernel; key tiles of 64 keys, K and V
// row-major in LDS as they are in memory (rows padded by 16 bytes).
//   scores^T block (hf, b) = K rows {32 hf + 8 (r / 4) + 4 b + r % 4 : r = 0 .. 15} . q : lane (query r16, group g)
//       receives keys 32 hf + 8 g + 4 b + i, i = 0 .. 3 -- over b = 0, 1 the eight consecutive keys 32 hf + 8 g .. + 7,
//       which is the contraction slot order of the second product, so the weights go from registers into it;
//   out^T[d][query] += V^T[d][key] P[key][query], 32 keys per step: V^T fragments by transposing LDS reads
//       (ds_read_b64_tr_b16: column d of four consecutive key rows per read).
template <typename T> __device__ __forceinline__ uint32_t pack_pair(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack_pair<bf16_t>(float lo, float hi) { return pack_bf16x2(lo, hi); }
template <> __device__ __forceinline__ uint32_t pack_pair<f16_t>(float lo, float hi) {
    const _Float16 l = (_Float16)lo, h = (_Float16)hi;
    return (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, h) << 16);
}
constexpr int TKL = 64;                                // keys per tile of local_fwd_b16_kernel
template <int E> constexpr size_t local_b16_smem() { return (size_t)2 * TKL * 2 * (E + 8) * 2; }

// QB: 16-query blocks per wave.  With two, every K and V^T fragment read from LDS feeds two products (the LDS fragment
// traffic is what bounds the one-block form on long problems); a workgroup then covers 128 queries.
template <typename T, int E, int D, int QB>
__global__ __launch_bounds__(NT) void local_fwd_b16_kernel(LocalArgs a) {
    static_assert(sizeof(T) == 2 && E % 32 == 0 && D % 16 == 0, "2-byte inputs, whole MFMA steps");
    constexpr int LDK = E + 8, LDV = D + 8, KS = E / 32, DB = D / 16;
    constexpr int STAGE = TKL * (LDK + LDV);           // 2-byte elements of a stage
    constexpr int QW = 16 * QB, TQB = 4 * QW;          // queries per wave, per workgroup
    constexpr float LOG2E = 1.4426950408889634f;
    extern __shared__ __attribute__((aligned(128))) float smem[];
    uint16_t* lds = reinterpret_cast<uint16_t*>(smem);
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), r16 = lane & 15, g = lane >> 4;
    const int n_qt = (a.T + TQB - 1) / TQB;
    const int n_items = a.B * a.H * n_qt;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // see sblocal_fwd_kernel
    if (item >= n_items) return;                       // workgroup-uniform
    const int qt = item % n_qt, bh = item / n_qt, b = bh / a.H, h = bh % a.H;
    const int q0 = qt * TQB, qw0 = q0 + QW * w;
    const uint16_t* qptr = reinterpret_cast<const uint16_t*>(a.q) + b * a.q_sb + h * a.q_sh;
    const uint16_t* kptr = reinterpret_cast<const uint16_t*>(a.k) + b * a.k_sb + h * a.k_sh;
    const uint16_t* vptr = reinterpret_cast<const uint16_t*>(a.v) + b * a.v_sb + h * a.v_sh;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi

    const int q_last = min(q0 + TQB - 1, a.T - 1);
    const int lo = max(0, q0 - lc_lo), hi = min(len, q_last + lc_hi);
    const int kt_lo = lo / TKL, kt_hi = (hi > lo) ? (hi + TKL - 1) / TKL : kt_lo;
    Tile16<TKL, E, NT> rk;
    Tile16<TKL, D, NT> rv;
    if (kt_lo < kt_hi) {
        rk.fetch(kptr, a.k_ss, kt_lo * TKL, a.S - 1, tid);
        rv.fetch(vptr, a.v_ss, kt_lo * TKL, a.S - 1, tid);
    }
    // score operands: the query rows as they are in memory, dims 32 c + 8 g .. + 7 (the scale goes into the exponent)
    int iq[QB], smin[QB];
    unsigned span[QB];
    uint32_t drop_row[QB];
    uint4 qb[QB][KS];
    float m_run[QB], ze[QB];
    floatx4 oacc[QB][DB];
#pragma unroll
    for (int qq = 0; qq < QB; ++qq) {
        iq[qq] = qw0 + 16 * qq + r16;
        const uint16_t* qrow = qptr + (long)min(iq[qq], a.T - 1) * a.q_ss;
#pragma unroll
        for (int c = 0; c < KS; ++c) qb[qq][c] = *reinterpret_cast<const uint4*>(qrow + 32 * c + 8 * g);
        m_run[qq] = -1e30f;         // finite, so that the first rescale is exp2(-huge) = 0 and not inf - inf
        ze[qq] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) oacc[qq][db] = Frag<float>::zero();
        smin[qq] = max(iq[qq] - lc_lo, 0);
        span[qq] = iq[qq] < a.T ? (unsigned)max(min(iq[qq] + lc_hi, len) - smin[qq], 0) : 0u;
        drop_row[qq] = a.drop_thresh != 0u ? drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + iq[qq])) : 0u;
    }
    const float sc = a.temp * LOG2E;
    // fragment addresses inside a stage: the K row of this lane in block (hf, b), the two V rows of its transposing reads
    const int koff = (8 * (r16 >> 2) + (r16 & 3)) * LDK + 8 * g;        // + (32 hf + 4 b) LDK + 32 c
    const int voff = (8 * g + (r16 >> 2)) * LDV + 4 * (r16 & 3);        // + 32 hf LDV (+ 4 LDV) + 16 db
    if (kt_lo < kt_hi) {
        rk.template stash<LDK>(lds, tid);
        rv.template stash<LDV>(lds + TKL * LDK, tid);
    }
    __syncthreads();
    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        const int s_base = kt * TKL, cur = (kt - kt_lo) & 1;
        const uint16_t* Ks = lds + cur * STAGE;
        const uint16_t* Vs = Ks + TKL * LDK;
        const bool more = kt + 1 < kt_hi;
        if (more) {
            rk.fetch(kptr, a.k_ss, s_base + TKL, a.S - 1, tid);
            rv.fetch(vptr, a.v_ss, s_base + TKL, a.S - 1, tid);
        }
        // (wave-uniform, scalar: w is) does the tile touch the band of one of the wave's queries; does it lie inside all
        const bool any = !(s_base + TKL - 1 - qw0 < -lc_lo || s_base - (qw0 + QW - 1) >= lc_hi || s_base >= len);
        const bool inside = s_base - (qw0 + QW - 1) >= -lc_lo && s_base + TKL - 1 - qw0 < lc_hi && s_base + TKL <= len &&
                            qw0 + QW - 1 < a.T;
        if (any) {
            floatx4 s1[QB][4];                           // block 2 hf + b, unscaled
#pragma unroll
            for (int qq = 0; qq < QB; ++qq)
#pragma unroll
                for (int hb = 0; hb < 4; ++hb) s1[qq][hb] = Frag<float>::zero();
#pragma unroll
            for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                for (int c = 0; c < KS; ++c) {
                    const uint4 kf = *reinterpret_cast<const uint4*>(Ks + koff + (32 * (hb >> 1) + 4 * (hb & 1)) * LDK + 32 * c);
#pragma unroll
                    for (int qq = 0; qq < QB; ++qq) s1[qq][hb] = Frag32<T>::mma(kf, qb[qq][c], s1[qq][hb]);
                }
            if (a.add_mask) {                                // (uniform)
#pragma unroll
                for (int qq = 0; qq < QB; ++qq) {
                    const float* am = a.add_mask + (long)min(iq[qq], a.T - 1) * a.S;
#pragma unroll
                    for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int s = s_base + 32 * (hb >> 1) + 8 * g + 4 * (hb & 1) + i;
                            // (an absorbing entry becomes -2^80: its product with the scale is exact, so the multiply-add
                            //  of the exponent below gives exactly 0 for a row whose keys are all hidden)
                            if ((unsigned)(s - smin[qq]) < span[qq])
                                s1[qq][hb][i] = am[s] < -1e20f ? -0x1p80f : s1[qq][hb][i] + am[s];
                        }
                }
            }
            if (!inside) {
#pragma unroll
                for (int qq = 0; qq < QB; ++qq)
#pragma unroll
                    for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int s = s_base + 32 * (hb >> 1) + 8 * g + 4 * (hb & 1) + i;
                            if (!((unsigned)(s - smin[qq]) < span[qq])) s1[qq][hb][i] = -INFINITY;
                        }
            }
            float mx[QB];
            bool moved = false;
#pragma unroll
            for (int qq = 0; qq < QB; ++qq) {
                mx[qq] = -INFINITY;
#pragma unroll
                for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) mx[qq] = fmaxf(mx[qq], s1[qq][hb][i]);
                mx[qq] = group_max(mx[qq]) * sc;
                moved = moved || mx[qq] > m_run[qq] + 8.f;
            }
            if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
                for (int qq = 0; qq < QB; ++qq) {
                    const float m_new = fmaxf(m_run[qq], mx[qq]);
                    const float alpha = __builtin_amdgcn_exp2f(m_run[qq] - m_new);
                    m_run[qq] = m_new;
                    ze[qq] *= alpha;
#pragma unroll
                    for (int db = 0; db < DB; ++db) oacc[qq][db] *= alpha;
                }
            }
#pragma unroll
            for (int qq = 0; qq < QB; ++qq)
#pragma unroll
                for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s1[qq][hb][i] = __builtin_amdgcn_exp2f(fmaf(s1[qq][hb][i], sc, -m_run[qq]));   // (masked: -inf, weight 0)
                        ze[qq] += s1[qq][hb][i];
                    }
            if (a.drop_thresh != 0u) {                   // (uniform) dropped weights leave the product, not the denominator
#pragma unroll
                for (int qq = 0; qq < QB; ++qq)
#pragma unroll
                    for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (!drop_keep(drop_row[qq], (uint32_t)(s_base + 32 * (hb >> 1) + 8 * g + 4 * (hb & 1) + i), a.drop_thresh))
                                s1[qq][hb][i] = 0.f;
            }
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                uint4 pb[QB];
#pragma unroll
                for (int qq = 0; qq < QB; ++qq)
                    pb[qq] = make_uint4(pack_pair<T>(s1[qq][2 * hf][0], s1[qq][2 * hf][1]), pack_pair<T>(s1[qq][2 * hf][2], s1[qq][2 * hf][3]),
                                        pack_pair<T>(s1[qq][2 * hf + 1][0], s1[qq][2 * hf + 1][1]),
                                        pack_pair<T>(s1[qq][2 * hf + 1][2], s1[qq][2 * hf + 1][3]));
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const uint16_t* vp = Vs + voff + 32 * hf * LDV + 16 * db;
                    const uint4 va = __builtin_bit_cast(uint4, lds_read_tr8(reinterpret_cast<const char*>(vp),
                                                                             reinterpret_cast<const char*>(vp + 4 * LDV)));
#pragma unroll
                    for (int qq = 0; qq < QB; ++qq) oacc[qq][db] = Frag32<T>::mma(va, pb[qq], oacc[qq][db]);
                }
            }
        }
        if (more) {
            uint16_t* nxt = lds + (cur ^ 1) * STAGE;
            rk.template stash<LDK>(nxt, tid);
            rv.template stash<LDV>(nxt + TKL * LDK, tid);
        }
        __syncthreads();
    }
#pragma unroll
    for (int qq = 0; qq < QB; ++qq) {
        float z = group_sum(ze[qq]);
        // (every visible key masked: see local_fwd_kernel)
        const bool all_masked = a.add_mask != nullptr && span[qq] > 0u && m_run[qq] < -1e20f;
        if (all_masked) z += (float)(a.lc - (int)span[qq]);
        if (iq[qq] < a.T) {
            const float inv = (z > 0.f ? 1.0f / z : 0.f) * (a.drop_thresh != 0u ? a.drop_scale : 1.0f);
            T* optr = reinterpret_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq[qq] * a.o_ss;
#pragma unroll
            for (int db = 0; db < DB; ++db) store4_f32(optr + 16 * db + 4 * g, oacc[qq][db] * inv);
            if (a.lse && g == 0)
                a.lse[((long)b * a.H + h) * a.T + iq[qq]] = all_masked ? -INFINITY
                                                            : z > 0.f ? m_run[qq] * 0.6931471805599453f + __logf(z) : 0.f;
        }
    }
}

// ---------------------------------------------------------------------------------------
// gradients of plain local attention for 2-byte inputs
// ---------------------------------------------------------------------------------------
// With P_is = exp(t q_i.k_s - lse_i) on the band, g = d out and delta_i = g_i.out_i (local_attention.py:68-92 leaves
// these to autograd):  d v_s = sum_i P_is g_i,  dS_is = P_is (g_i.v_s - delta_i),  d q_i = t sum_s dS_is k_s,
// d k_s = t sum_i dS_is q_i.  One kernel in two orientations, built like local_fwd_b16_kernel: a wave owns QB blocks
// of 16 "outer" rows (queries, or keys when KEYMAJOR) whose two operands stay in registers, and walks 64-row tiles of
// the "inner" side (keys with values, or queries with their output gradients) through LDS.
//   S^T  = Y1 . x1  and  G^T = Y2 . x2   (inner rows of a 16-row block picked so that a lane's results over two
//                                         blocks are eight consecutive inner rows, the contraction slots below)
//   P = exp2(sc S - lse log2e) where the pair is in the band, dS = P (G - delta)   (lse, delta: of the query)
//   d x^T[e][outer] += Y^T[e][inner] . {P, dS}[inner][outer]   (Y^T fragments by transposing LDS reads)
// Query-major: d q from (K, dS).  Key-major: d v from (d out, P) and d k from (Q, dS).
struct LocalBwdArgs {
    const void* q; const void* k; const void* v; const void* go; const void* out;
    const float* lse; float* delta;                 // (B, H, T); delta is written by the query-major launch
    const int64_t* lens;
    void* dq; void* dk; void* dv;
    int B, H, T, S, lc;
    long q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, g_sb, g_sh, g_ss, o_sb, o_sh, o_ss;
    long dq_sb, dq_sh, dq_ss, dk_sb, dk_sh, dk_ss, dv_sb, dv_sh, dv_ss;
    float temp;
    int n_xcd;
};
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w);
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w);
template <> __device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t w) { return __uint_as_float(w << 16); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
template <> __device__ __forceinline__ float unpack_lo<f16_t>(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu)); }
template <> __device__ __forceinline__ float unpack_hi<f16_t>(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }
template <int E> constexpr size_t local_bwd_smem() { return (size_t)2 * (TKL * 2 * (E + 8) * 2 + 2 * TKL * sizeof(float)); }

template <typename T, int E, bool KEYMAJOR, int QB>
__global__ __launch_bounds__(NT) void local_bwd_b16_kernel(LocalBwdArgs a) {
    static_assert(sizeof(T) == 2 && E % 32 == 0, "2-byte inputs, whole MFMA steps");
    constexpr int LD = E + 8, KS = E / 32, EB = E / 16;
    constexpr int STAGE_BYTES = TKL * 2 * LD * 2 + 2 * TKL * (int)sizeof(float);
    constexpr int QW = 16 * QB, TQB = 4 * QW;          // outer rows per wave, per workgroup
    constexpr float LOG2E = 1.4426950408889634f;
    extern __shared__ __attribute__((aligned(128))) float smem[];
    char* lds = reinterpret_cast<char*>(smem);
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), r16 = lane & 15, g = lane >> 4;
    const int R_out = KEYMAJOR ? a.S : a.T, R_in = KEYMAJOR ? a.T : a.S;
    const int n_ot = (R_out + TQB - 1) / TQB;
    const int n_items = a.B * a.H * n_ot;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // see sblocal_fwd_kernel
    if (item >= n_items) return;                       // workgroup-uniform
    const int ot = item % n_ot, bh = item / n_ot, b = bh / a.H, h = bh % a.H;
    const int o0 = ot * TQB, ow0 = o0 + QW * w;
    const uint16_t* qptr = reinterpret_cast<const uint16_t*>(a.q) + b * a.q_sb + h * a.q_sh;
    const uint16_t* kptr = reinterpret_cast<const uint16_t*>(a.k) + b * a.k_sb + h * a.k_sh;
    const uint16_t* vptr = reinterpret_cast<const uint16_t*>(a.v) + b * a.v_sb + h * a.v_sh;
    const uint16_t* gptr = reinterpret_cast<const uint16_t*>(a.go) + b * a.g_sb + h * a.g_sh;
    const uint16_t* x1p = KEYMAJOR ? kptr : qptr;  const long x1s = KEYMAJOR ? a.k_ss : a.q_ss;     // outer operands
    const uint16_t* x2p = KEYMAJOR ? vptr : gptr;  const long x2s = KEYMAJOR ? a.v_ss : a.g_ss;
    const uint16_t* y1p = KEYMAJOR ? qptr : kptr;  const long y1s = KEYMAJOR ? a.q_ss : a.k_ss;     // inner tiles
    const uint16_t* y2p = KEYMAJOR ? gptr : vptr;  const long y2s = KEYMAJOR ? a.g_ss : a.v_ss;
    const float* lsep = a.lse + (long)bh * a.T;
    const float* delp = a.delta + (long)bh * a.T;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    // the pair (outer o, inner n) is in the band when n - o lies in [-A, Bq), o < Lo and n < Ln
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;
    const int A = KEYMAJOR ? lc_hi - 1 : lc_lo, Bq = KEYMAJOR ? lc_lo + 1 : lc_hi;
    const int Lo = KEYMAJOR ? len : a.T, Ln = KEYMAJOR ? a.T : len;

    const int o_last = min(min(o0 + TQB - 1, R_out - 1), Lo - 1);
    const int lo = max(0, o0 - A), hi = o_last >= o0 ? min(Ln, o_last + Bq) : 0;
    const int it_lo = lo / TKL, it_hi = (hi > lo) ? (hi + TKL - 1) / TKL : it_lo;
    Tile16<TKL, E, NT> r1, r2;
    float rl = 0.f, rd = 0.f;                          // key-major: lse log2e and delta of inner row tid (threads 0 .. 63)
    auto fetch = [&](int it) __attribute__((always_inline)) {
        r1.fetch(y1p, y1s, it * TKL, R_in - 1, tid);
        r2.fetch(y2p, y2s, it * TKL, R_in - 1, tid);
        if (KEYMAJOR && tid < TKL) {
            const int i = min(it * TKL + tid, a.T - 1);
            rl = lsep[i] * LOG2E;
            rd = delp[i];
        }
    };
    auto stash = [&](int stage) __attribute__((always_inline)) {
        uint16_t* t1 = reinterpret_cast<uint16_t*>(lds + stage * STAGE_BYTES);
        r1.template stash<LD>(t1, tid);
        r2.template stash<LD>(t1 + TKL * LD, tid);
        if (KEYMAJOR && tid < TKL) {
            float* sc_ = reinterpret_cast<float*>(lds + stage * STAGE_BYTES + TKL * 2 * LD * 2);
            sc_[tid] = rl;
            sc_[TKL + tid] = rd;
        }
    };
    if (it_lo < it_hi) fetch(it_lo);

    int io[QB], vmin[QB];
    unsigned vspan[QB];
    uint4 x1[QB][KS], x2[QB][KS];
    float l_own[QB], d_own[QB];
    floatx4 acc1[QB][EB], acc2[KEYMAJOR ? QB : 1][KEYMAJOR ? EB : 1];     // d q | d k, and d v
#pragma unroll
    for (int qq = 0; qq < QB; ++qq) {
        io[qq] = ow0 + 16 * qq + r16;
        const long row = min(io[qq], R_out - 1);
#pragma unroll
        for (int c = 0; c < KS; ++c) {
            x1[qq][c] = *reinterpret_cast<const uint4*>(x1p + row * x1s + 32 * c + 8 * g);
            x2[qq][c] = *reinterpret_cast<const uint4*>(x2p + row * x2s + 32 * c + 8 * g);
        }
        vmin[qq] = max(io[qq] - A, 0);
        vspan[qq] = io[qq] < Lo ? (unsigned)max(min(io[qq] + Bq, Ln) - vmin[qq], 0) : 0u;
        l_own[qq] = d_own[qq] = 0.f;
        if (!KEYMAJOR) {
            l_own[qq] = lsep[min(io[qq], a.T - 1)] * LOG2E;
            // delta of the query, g . out, from the output row in the layout of the gradient row; kept for the key-major launch
            const uint16_t* orow = reinterpret_cast<const uint16_t*>(a.out) + b * a.o_sb + h * a.o_sh + row * a.o_ss;
            float dsum = 0.f;
#pragma unroll
            for (int c = 0; c < KS; ++c) {
                const uint4 ov = *reinterpret_cast<const uint4*>(orow + 32 * c + 8 * g);
                const uint32_t ow[4] = {ov.x, ov.y, ov.z, ov.w}, gw[4] = {x2[qq][c].x, x2[qq][c].y, x2[qq][c].z, x2[qq][c].w};
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    dsum += unpack_lo<T>(ow[x]) * unpack_lo<T>(gw[x]) + unpack_hi<T>(ow[x]) * unpack_hi<T>(gw[x]);
            }
            d_own[qq] = group_sum(dsum);
            if (g == 0 && io[qq] < a.T) a.delta[(long)bh * a.T + io[qq]] = d_own[qq];
        }
#pragma unroll
        for (int eb = 0; eb < EB; ++eb) acc1[qq][eb] = Frag<float>::zero();
    }
    if (KEYMAJOR) {
#pragma unroll
        for (int qq = 0; qq < QB; ++qq)
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) acc2[qq][eb] = Frag<float>::zero();
    }
    const float sc = a.temp * LOG2E;
    const int foff = (8 * (r16 >> 2) + (r16 & 3)) * LD + 8 * g;         // + (32 hf + 4 b) LD + 32 c   (elements)
    const int toff = (8 * g + (r16 >> 2)) * LD + 4 * (r16 & 3);         // + 32 hf LD (+ 4 LD) + 16 eb
    if (it_lo < it_hi) stash(0);
    __syncthreads();
    for (int it = it_lo; it < it_hi; ++it) {
        const int i_base = it * TKL, cur = (it - it_lo) & 1;
        const uint16_t* Y1 = reinterpret_cast<const uint16_t*>(lds + cur * STAGE_BYTES);
        const uint16_t* Y2 = Y1 + TKL * LD;
        const float* Ls = reinterpret_cast<const float*>(lds + cur * STAGE_BYTES + TKL * 2 * LD * 2);
        const bool more = it + 1 < it_hi;
        if (more) fetch(it + 1);
        // (wave-uniform, scalar) does the tile touch the band of one of the wave's outer rows; does it lie inside all
        const bool any = !(i_base + TKL - 1 - ow0 < -A || i_base - (ow0 + QW - 1) >= Bq || i_base >= Ln || ow0 >= Lo);
        const bool inside = i_base - (ow0 + QW - 1) >= -A && i_base + TKL - 1 - ow0 < Bq && i_base + TKL <= Ln && ow0 + QW - 1 < Lo;
        if (any) {
            floatx4 s1[QB][4], gp[QB][4];                // block 2 hf + b: scores (unscaled) and g.v
#pragma unroll
            for (int qq = 0; qq < QB; ++qq)
#pragma unroll
                for (int hb = 0; hb < 4; ++hb) { s1[qq][hb] = Frag<float>::zero(); gp[qq][hb] = Frag<float>::zero(); }
#pragma unroll
            for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                for (int c = 0; c < KS; ++c) {
                    const int off = foff + (32 * (hb >> 1) + 4 * (hb & 1)) * LD + 32 * c;
                    const uint4 f1 = *reinterpret_cast<const uint4*>(Y1 + off);
                    const uint4 f2 = *reinterpret_cast<const uint4*>(Y2 + off);
#pragma unroll
                    for (int qq = 0; qq < QB; ++qq) {
                        s1[qq][hb] = Frag32<T>::mma(f1, x1[qq][c], s1[qq][hb]);
                        gp[qq][hb] = Frag32<T>::mma(f2, x2[qq][c], gp[qq][hb]);
                    }
                }
            floatx4 ln4[4], dl4[4];                      // key-major: the queries' lse log2e and delta, by block
            if (KEYMAJOR) {
#pragma unroll
                for (int hb = 0; hb < 4; ++hb) {
                    ln4[hb] = *reinterpret_cast<const floatx4*>(Ls + 32 * (hb >> 1) + 8 * g + 4 * (hb & 1));
                    dl4[hb] = *reinterpret_cast<const floatx4*>(Ls + TKL + 32 * (hb >> 1) + 8 * g + 4 * (hb & 1));
                }
            }
            // weights P into s1, dS into gp
#pragma unroll
            for (int qq = 0; qq < QB; ++qq)
#pragma unroll
                for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int n = i_base + 32 * (hb >> 1) + 8 * g + 4 * (hb & 1) + i;
                        const float lrow = KEYMAJOR ? ln4[hb][i] : l_own[qq], drow = KEYMAJOR ? dl4[hb][i] : d_own[qq];
                        float pr = __builtin_amdgcn_exp2f(fmaf(s1[qq][hb][i], sc, -lrow));
                        if (!inside && !((unsigned)(n - vmin[qq]) < vspan[qq])) pr = 0.f;
                        s1[qq][hb][i] = pr;
                        gp[qq][hb][i] = pr * (gp[qq][hb][i] - drow);
                    }
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                uint4 pb[KEYMAJOR ? QB : 1], sb[QB];
#pragma unroll
                for (int qq = 0; qq < QB; ++qq) {
                    sb[qq] = make_uint4(pack_pair<T>(gp[qq][2 * hf][0], gp[qq][2 * hf][1]), pack_pair<T>(gp[qq][2 * hf][2], gp[qq][2 * hf][3]),
                                        pack_pair<T>(gp[qq][2 * hf + 1][0], gp[qq][2 * hf + 1][1]),
                                        pack_pair<T>(gp[qq][2 * hf + 1][2], gp[qq][2 * hf + 1][3]));
                    if (KEYMAJOR)
                        pb[qq] = make_uint4(pack_pair<T>(s1[qq][2 * hf][0], s1[qq][2 * hf][1]), pack_pair<T>(s1[qq][2 * hf][2], s1[qq][2 * hf][3]),
                                            pack_pair<T>(s1[qq][2 * hf + 1][0], s1[qq][2 * hf + 1][1]),
                                            pack_pair<T>(s1[qq][2 * hf + 1][2], s1[qq][2 * hf + 1][3]));
                }
#pragma unroll
                for (int eb = 0; eb < EB; ++eb) {
                    const uint16_t* p1 = Y1 + toff + 32 * hf * LD + 16 * eb;
                    const uint4 t1 = __builtin_bit_cast(uint4, lds_read_tr8(reinterpret_cast<const char*>(p1),
                                                                             reinterpret_cast<const char*>(p1 + 4 * LD)));
#pragma unroll
                    for (int qq = 0; qq < QB; ++qq) acc1[qq][eb] = Frag32<T>::mma(t1, sb[qq], acc1[qq][eb]);
                    if (KEYMAJOR) {
                        const uint16_t* p2 = Y2 + toff + 32 * hf * LD + 16 * eb;
                        const uint4 t2 = __builtin_bit_cast(uint4, lds_read_tr8(reinterpret_cast<const char*>(p2),
                                                                                 reinterpret_cast<const char*>(p2 + 4 * LD)));
#pragma unroll
                        for (int qq = 0; qq < QB; ++qq) acc2[qq][eb] = Frag32<T>::mma(t2, pb[qq], acc2[qq][eb]);
                    }
                }
            }
        }
        if (more) stash(cur ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int qq = 0; qq < QB; ++qq) {
        if (io[qq] < R_out) {
            T* d1 = KEYMAJOR ? reinterpret_cast<T*>(a.dk) + b * a.dk_sb + h * a.dk_sh + (long)io[qq] * a.dk_ss
                             : reinterpret_cast<T*>(a.dq) + b * a.dq_sb + h * a.dq_sh + (long)io[qq] * a.dq_ss;
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) store4_f32(d1 + 16 * eb + 4 * g, acc1[qq][eb] * a.temp);
            if (KEYMAJOR) {
                T* d2 = reinterpret_cast<T*>(a.dv) + b * a.dv_sb + h * a.dv_sh + (long)io[qq] * a.dv_ss;
#pragma unroll
                for (int eb = 0; eb < EB; ++eb) store4_f32(d2 + 16 * eb + 4 * g, acc2[qq][eb]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// fused band kernel
// ---------------------------------------------------------------------------------------
template <typename T, int E, int D, int M, bool SPLIT, bool LIST = false>
__global__ __launch_bounds__(NT) void sblocal_fwd_kernel(FwdArgs a) {
    constexpr int MH = M / 2, LDK = E + 4, LDV = D + 4, LDF = M + 4;
    constexpr int FB = MH / 16, EC = E / 16, DB = D / 16, KB = TK / 16;
    constexpr int STAGE = TK * (LDK + LDV + LDF);     // floats per LDS stage
    extern __shared__ __attribute__((aligned(128))) float smem[];
    float* Ps = smem;                                  // only live before the key loop

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    if (SPLIT && !LIST && (int)blockIdx.x >= a.band_wgs) {
        // combine role: the partial K'^T V / sum K' of the key pass become kv / ksum / kmax for the merge
        // kernel (nothing in THIS launch reads them: the parts take kmax from the partial maxima)
        const int ci = blockIdx.x - a.band_wgs;
        sb_combine_body(smem, a.kv_part, a.part_max, const_cast<float*>(a.kv), const_cast<float*>(a.ksum),
                        const_cast<float*>(a.kmax), nullptr, ci / a.cmb_wpb, ci % a.cmb_wpb, a.cmb_wpb, a.n_split, M, D);
        return;
    }
    // Workgroups are handed to the 8 XCDs round-robin in launch order, and every XCD has its own
    // L2.  The linear id is therefore re-mapped so that one XCD works on a contiguous run of
    // (batch-head, query tile, part) items: neighbours in that order share key tiles.
    const int n_qt = (a.T + TQ - 1) / TQ;
    int part, qt, bh;
    // part_role: this workgroup writes an un-normalised partial for the merge kernel.  Always with SPLIT; on a
    // block-sparse support the first workgroups of the launch, which walk the long lists in parts
    bool part_role = SPLIT;
    long slot = 0;                  // long lists: index of the tile's partials and compact query features
    const int n_part_wgs = LIST ? (a.B * a.n_heavy * a.n_parts + a.n_xcd - 1) / a.n_xcd * a.n_xcd : 0;
    if (LIST && (int)blockIdx.x < n_part_wgs) {
        const int idx = blockIdx.x;
        if (idx >= a.B * a.n_heavy * a.n_parts) return;            // workgroup-uniform
        part_role = true;
        part = idx % a.n_parts;
        slot = idx / a.n_parts;
        const int hq = a.tl_heavy[slot % a.n_heavy];
        qt = hq % n_qt;
        bh = (int)(slot / a.n_heavy) * a.H + hq / n_qt;
    } else if (LIST) {
        // Lists differ in length by orders of magnitude (a block-row of global tokens against a window), so
        // the tiles start longest first: an XCD takes the (batch, head) pairs congruent to its number and
        // walks them rank by rank -- all their longest tiles, then all their second longest ...
        const int blk_id = blockIdx.x - n_part_wgs;
        const int nbh = a.B * a.H, x = blk_id % a.n_xcd, i = blk_id / a.n_xcd;
        const int mine = (nbh - x + a.n_xcd - 1) / a.n_xcd;            // pairs of this XCD
        if (mine <= 0 || i >= mine * n_qt) return;                 // workgroup-uniform
        const int rank = i / mine;
        bh = x + a.n_xcd * (i % mine);
        qt = a.tl_order ? a.tl_order[(bh % a.H) * n_qt + rank] : rank;
        if (qt < 0) return;                                        // a long list: walked in parts by the first workgroups
        part = 0;
    } else {
        const int n_items = a.B * a.H * n_qt * a.n_parts;
        const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
        const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;
        if (item >= n_items) return;                       // workgroup-uniform
        part = item % a.n_parts;
        qt = (item / a.n_parts) % n_qt;
        bh = item / (a.n_parts * n_qt);
    }
    const int b = bh / a.H, h = bh % a.H;
    const int q0 = qt * TQ;
    const int iq = q0 + 16 * w + r16;
    const bool qvalid = iq < a.T;
    const T* qptr = reinterpret_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh;
    const T* kptr = reinterpret_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh;
    const T* vptr = reinterpret_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh;
    const float* fptr = reinterpret_cast<const float*>(a.kfeat) + (long)bh * a.n_chunks * CH * M;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half = 0.5f * __logf(2.0f * a.mh_valid);
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi

    FLY_PROF(0);
    // this workgroup's share of the band, in 32-key tiles
    const int q_last = min(q0 + TQ - 1, a.T - 1);
    const int lo = max(0, q0 - lc_lo);
    const int hi = min(len, q_last + lc_hi);
    int kt_lo = lo / TK;
    int kt_hi = (hi > lo) ? (hi + TK - 1) / TK : kt_lo;
    if (SPLIT && !LIST) {
        // an even split: the first (tiles % parts) parts take one tile more
        const int nt = kt_hi - kt_lo, base = nt / a.n_parts, extra = nt % a.n_parts;
        const int first = kt_lo + part * base + min(part, extra);
        kt_lo = first;
        kt_hi = first + base + (part < extra ? 1 : 0);
    }
    // LIST: the loop counter walks the tile's list of 32-key tiles instead of a range of them; the tile index and
    // this wave's presence mask of an entry (bit h: the wave's 16 queries see keys 16 h .. 16 h + 15 of the tile --
    // a block-row of 16 x 16 blocks is one wave, two waves share a block-row of 32 x 32 blocks and see whole tiles)
    // are read one iteration ahead of their use
    const int32_t* tl_inner = nullptr;
    const int32_t* tl_blk = nullptr;
    int tile_cur = 0, tile_next = 0;
    int pres_cur = 0, pres_next = 0;
    bool seen_block = false;
    if (LIST) {
        int lp0 = a.tl_ptr[h * n_qt + qt];
        kt_lo = 0;
        kt_hi = a.tl_ptr[h * n_qt + qt + 1] - lp0;
        if (part_role) {
            // this part's share of the list: the first (entries % parts) parts take one entry more
            const int base = kt_hi / a.n_parts, extra = kt_hi % a.n_parts;
            lp0 += part * base + min(part, extra);
            kt_hi = base + (part < extra ? 1 : 0);
        }
        tl_inner = a.tl_inner + lp0;
        tl_blk = a.tl_blk + 4 * (long)lp0 + w;              // four masks per entry, one per wave
        if (kt_hi > 0) { tile_cur = tl_inner[0]; pres_cur = tl_blk[0] & 3; }
        if (kt_hi > 1) { tile_next = tl_inner[1]; pres_next = tl_blk[4] & 3; }
    }
    const int first_tile = LIST ? tile_cur : kt_lo;

    // start the first tile's loads before anything else
    RowTile<TK, E> rk;
    RowTile<TK, D> rv;
    RowTile<TK, M> rf;
    const int f_last = a.n_chunks * CH - 1;
    if (kt_lo < kt_hi) {
        rk.fetch(kptr, a.k_ss, first_tile * TK, a.S - 1, tid);
        rv.fetch(vptr, a.v_ss, first_tile * TK, a.S - 1, tid);
        rf.fetch(fptr, M, first_tile * TK, f_last, tid);
    }
    // tiles after the first: per-thread offsets once, then one load per piece from the tile's base
    // (tiles that run past the last key row keep the clamping fetch)
    uint32_t offk[RowTile<TK, E>::N], offv[RowTile<TK, D>::N], offf[RowTile<TK, M>::N];
    rk.template offsets<T>(offk, a.k_ss, tid);
    rv.template offsets<T>(offv, a.v_ss, tid);
    rf.template offsets<float>(offf, M, tid);
    const float* csp = a.chunk_scale + (long)bh * a.n_chunks;
    float cscale = (kt_lo < kt_hi) ? csp[first_tile * TK / CH] : 0.f;
    constexpr bool OWN_Q = !SPLIT || LIST;       // query features formed here (not by the key pass), kmax combined
    const float kmax = OWN_Q ? a.kmax[bh] : split_kmax(a.part_max, bh, a.n_split);

    // query operand (B side: column = query, k = 16c+4g+j) and its squared norm
    floatx4 qr[EC];
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        qr[c] = Frag<float>::zero();
        if (qvalid) qr[c] = load4_f32(qptr + (long)iq * a.q_ss + 16 * c + 4 * g);
        sq += qr[c][0] * qr[c][0] + qr[c][1] * qr[c][1] + qr[c][2] * qr[c][2] + qr[c][3] * qr[c][3];
    }
    const float diag_q = 0.5f * a.temp * group_sum(sq);

    // query features, kept in registers: qf[c] is the B operand for feature slice c of K'
    floatx4 qf[2 * FB];
    float lsq;
    if (!OWN_Q) {
        // several parts share a query tile: the key pass has computed the features once
        const long qrow = (long)bh * a.T + min(iq, a.T - 1);
#pragma unroll
        for (int c = 0; c < 2 * FB; ++c) qf[c] = *reinterpret_cast<const floatx4*>(a.qfeat + qrow * M + 16 * c + 4 * g);
        lsq = a.q_lsq[qrow];
    } else {
        load_proj<E, MH>(Ps, a.proj, sqrtf(a.temp), tid);
        __syncthreads();
        float qmax = 0.f;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) qf[fb] = Frag<float>::zero();
#pragma unroll
        for (int c = 0; c < EC; ++c) {                      // the FB accumulation chains advance together
            floatx4 pa[FB];
#pragma unroll
            for (int fb = 0; fb < FB; ++fb)
                pa[fb] = *reinterpret_cast<const floatx4*>(Ps + (16 * fb + r16) * LDK + 16 * c + 4 * g);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int fb = 0; fb < FB; ++fb)
                    qf[fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[fb][j], qr[c][j], qf[fb], 0, 0, 0);
        }
#pragma unroll
        for (int fb = 0; fb < FB; ++fb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (16 * fb + 4 * g + i < a.mh_valid) qmax = fmaxf(qmax, fabsf(qf[fb][i]));
        qmax = group_max(qmax);
        lsq = -diag_q + qmax - lnm_half;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
            floatx4 dd = qf[fb];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = 16 * fb + 4 * g + i < a.mh_valid;
                qf[fb][i] = ok ? __expf(dd[i] - qmax) : 0.f;
                qf[FB + fb][i] = ok ? __expf(-dd[i] - qmax) : 0.f;
            }
        }
    }
    if (OWN_Q) __syncthreads();      // Ps is dead; the tile buffers may overwrite it
    if (LIST && part_role && part == 0) {
        // the merge kernel's operand for the global low-rank term
        float* dst = const_cast<float*>(a.qfeat) + (slot * TQ + 16 * w + r16) * M;
#pragma unroll
        for (int c = 0; c < 2 * FB; ++c) *reinterpret_cast<floatx4*>(dst + 16 * c + 4 * g) = qf[c];
    }
    FLY_PROF(1);

    // From here on all exponents are base 2 (one v_exp_f32 each): scores carry t*log2(e) through
    // the query operand, the log-scales are converted once.
    constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
    const float c0 = (lsq + kmax) * LOG2E;       // base-2 log-scale of the global low-rank term
#pragma unroll
    for (int c = 0; c < EC; ++c) qr[c] *= a.temp * LOG2E;
    float m_run = c0;               // reference exponent: max(running row max, log-scale of the low-rank part)
    float ze = 0.f, zp = 0.f;       // per-lane partial sums (reduced over g at the end)
    floatx4 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = Frag<float>::zero();
    const int qw0 = q0 + 16 * w;    // first query of this wave
    // keys this lane's query may see: smin <= s < smin + span
    const int smin = max(iq - lc_lo, 0);
    const unsigned span = qvalid ? (unsigned)max(min(iq + lc_hi, len) - smin, 0) : 0u;
    const bool drop_on = a.drop_thresh != 0u;          // (kernel-uniform) dropout of the exact weights
    const uint32_t drop_row = drop_on ? drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + iq)) : 0u;

    if (kt_lo < kt_hi) {
        rk.template stash<LDK>(smem, tid);
        rv.template stash<LDV>(smem + TK * LDK, tid);
        rf.template stash<LDF>(smem + TK * (LDK + LDV), tid);
    }
    __syncthreads();

    FLY_PROF(2);
    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        const int s_base = (LIST ? tile_cur : kt) * TK;
        const int s_next = LIST ? tile_next * TK : s_base + TK;      // first key of the next tile
        const int cur = (kt - kt_lo) & 1;
        const float* Ks = smem + cur * STAGE;
        const float* Vs = Ks + TK * LDK;
        const float* Fs = Vs + TK * LDV;
        const bool more = kt + 1 < kt_hi;
        float cscale_next = cscale;
        // LIST: the entry after the next one (block column, presence) is requested now
        int tile_n2 = 0;
        int pres_n2 = 0;
        if (LIST && kt + 2 < kt_hi) { tile_n2 = tl_inner[kt + 2]; pres_n2 = tl_blk[4 * (kt + 2)] & 3; }
        if (more) {                                      // next tile's loads fly during the MFMAs
            if (s_next + TK <= a.S) {
                rk.fetch_fast(kptr + (long)s_next * a.k_ss, offk, tid);
                rv.fetch_fast(vptr + (long)s_next * a.v_ss, offv, tid);
                rf.fetch_fast(fptr + (long)s_next * M, offf, tid);
            } else {
                rk.fetch(kptr, a.k_ss, s_next, a.S - 1, tid);
                rv.fetch(vptr, a.v_ss, s_next, a.S - 1, tid);
                rf.fetch(fptr, M, s_next, f_last, tid);
            }
            cscale_next = csp[s_next / CH];
        }
        // weight of this chunk's features relative to the global key stabiliser (<= 1); the same
        // expression weights the chunk in the combine role
        const float wc = __builtin_amdgcn_exp2f((cscale - kmax) * LOG2E);

        // wave-uniform: does this tile touch the band of any of the wave's 16 queries?  (Blocks of a
        // touched tile that lie outside the band are computed and masked: no branches among the MFMAs.)
        const bool any = LIST ? pres_cur != 0
                              : !(s_base + TK - 1 - qw0 < -lc_lo || s_base - (qw0 + 15) >= lc_hi || s_base >= len);
        if (any) {
            // scores^T: s1 = (t log2e) K q, s2 = K' q'.  The accumulation chains of the two key
            // blocks and of the two products are interleaved so that no MFMA waits on its predecessor.
            floatx4 s1[KB], s2[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) { s1[kb] = Frag<float>::zero(); s2[kb] = Frag<float>::zero(); }
            constexpr int CMAX = EC > 2 * FB ? EC : 2 * FB;
#pragma unroll
            for (int c = 0; c < CMAX; ++c) {
                floatx4 ka[KB], fa[KB];
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    if (c < EC) ka[kb] = *reinterpret_cast<const floatx4*>(Ks + (16 * kb + r16) * LDK + 4 * g + 16 * c);
                    if (c < 2 * FB) fa[kb] = *reinterpret_cast<const floatx4*>(Fs + (16 * kb + r16) * LDF + 4 * g + 16 * c);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb) {
                        if (c < EC) s1[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[kb][j], qr[c][j], s1[kb], 0, 0, 0);
                        if (c < 2 * FB) s2[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[kb][j], qf[c][j], s2[kb], 0, 0, 0);
                    }
                }
            }

            // lane holds the scores of query iq against keys s_base + 16kb + 4g + i.  A tile that lies
            // inside the band of all 16 queries of the wave and below the key length (wave-uniform) needs
            // no masks.
            // (LIST: a present half tile is wholly visible; the caller guarantees whole blocks of keys and queries)
            const bool interior = LIST ? pres_cur == 3
                                       : (s_base - (qw0 + 15) >= -lc_lo && s_base + TK - 1 - qw0 < lc_hi &&
                                          s_base + TK <= len && qw0 + 15 < a.T);
            floatx4 p[KB];
            float ovs = 0.f;
            auto soft = [&](auto masked_tag) __attribute__((always_inline)) {
                constexpr bool MASKED = decltype(masked_tag)::value;
                bool ok[KB][4];
                float mx = -INFINITY;
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int s = s_base + 16 * kb + 4 * g + i;
                        ok[kb][i] = !MASKED || (LIST ? ((pres_cur >> kb) & 1) != 0 : (unsigned)(s - smin) < span);
                        mx = fmaxf(mx, ok[kb][i] ? s1[kb][i] : -INFINITY);
                    }
                mx = group_max(mx);
                // the reference exponent is raised only when a tile exceeds it by more than 2^8: until
                // then the exponentials may exceed 1, which fp32 holds without loss
                if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.f) != 0) {      // wave-uniform
                    const float m_new = fmaxf(m_run, mx);
                    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                    m_run = m_new;
                    ze *= alpha;
#pragma unroll
                    for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
                }
                const float beta = wc * __builtin_amdgcn_exp2f(c0 - m_run);      // scale of the overlap term
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float e = ok[kb][i] ? __builtin_amdgcn_exp2f(s1[kb][i] - m_run) : 0.f;
                        const float ov = ok[kb][i] ? s2[kb][i] : 0.f;
                        ze += e;                                   // the normaliser sees no dropout
                        ovs += ov;
                        float ek = e;
                        if (drop_on) ek = drop_keep(drop_row, (uint32_t)(s_base + 16 * kb + 4 * g + i), a.drop_thresh) ? e * a.drop_scale : 0.f;
                        p[kb][i] = ek - ov * beta;
                    }
            };
            if (interior) soft(std::false_type{}); else soft(std::true_type{});
            zp += ovs * wc;
            // O^T[d][query] += sum_keys V[key][d] p[key][query]
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        oacc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                            Vs[(16 * kb + 4 * g + i) * LDV + 16 * db + r16], p[kb][i], oacc[db], 0, 0, 0);
            }
        }
        if (more) {
            float* nxt = smem + (cur ^ 1) * STAGE;
            rk.template stash<LDK>(nxt, tid);
            rv.template stash<LDV>(nxt + TK * LDK, tid);
            rf.template stash<LDF>(nxt + TK * (LDK + LDV), tid);
        }
        cscale = cscale_next;
        if (LIST) { seen_block |= pres_cur != 0; tile_cur = tile_next; tile_next = tile_n2; pres_cur = pres_next; pres_next = pres_n2; }
        __syncthreads();
    }
    if (LIST && !part_role && !seen_block) {
        // A block-row without any block: the reference's row logsumexp returns 0 there, not -inf
        // (blocksparse_logsumexp.py:132), so its normaliser carries an extra exp(0); reproduced.
        m_run = fmaxf(m_run, 0.f);
        ze = g == 0 ? __builtin_amdgcn_exp2f(-m_run) : 0.f;
    }

    FLY_PROF(3);
    // global low-rank term: qkv^T[d][query] = sum_r KV[r][d] q'[query][r],  qk1 = q' . Ksum
    // (with several parts the merge kernel adds it)
    floatx4 lacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) lacc[db] = Frag<float>::zero();
    float qk1 = 0.f;
    if (!part_role) {
        // K'^T V (M x D) and sum K' (M) staged in LDS: coalesced loads, all in flight together
        float* KVs = smem;
        float* KSs = smem + M * LDV;
        {
            RowTile<M, D> kvt;
            kvt.fetch(a.kv + (long)bh * M * D, D, 0, M - 1, tid);
            if (tid < M) KSs[tid] = a.ksum[(long)bh * M + tid];
            kvt.template stash<LDV>(KVs, tid);
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 2 * FB; ++c) {
            const floatx4 ks = *reinterpret_cast<const floatx4*>(KSs + 16 * c + 4 * g);
            qk1 += qf[c][0] * ks[0] + qf[c][1] * ks[1] + qf[c][2] * ks[2] + qf[c][3] * ks[3];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    lacc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                        KVs[(16 * c + 4 * g + j) * LDV + 16 * db + r16], qf[c][j], lacc[db], 0, 0, 0);
        }
        qk1 = group_sum(qk1);
    }
    ze = group_sum(ze);
    zp = group_sum(zp);
    FLY_PROF(4);
    const float gamma = __builtin_amdgcn_exp2f(c0 - m_run);               // <= 1
    if (part_role) {
        // un-normalised partial in this part's own (base-2) exponent m_run
        float* ws = a.part_ws + ((LIST ? slot : (long)bh * n_qt + qt) * a.n_parts + part) * (TQ * (D + NSTAT));
        const int ql = 16 * w + r16;
#pragma unroll
        for (int db = 0; db < DB; ++db) *reinterpret_cast<floatx4*>(ws + ql * D + 16 * db + 4 * g) = oacc[db];
        if (g == 0) {
            float* st = ws + TQ * D;
            st[0 * TQ + ql] = m_run;
            st[1 * TQ + ql] = ze;
            st[2 * TQ + ql] = zp;
            st[3 * TQ + ql] = 0.f;
            st[4 * TQ + ql] = c0;
        }
    } else {
        const float Z = ze + gamma * fmaxf(qk1 - zp, 1e-24f);
        const float inv = 1.0f / Z;
        if (qvalid) {
            T* optr = reinterpret_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq * a.o_ss;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                floatx4 o = (oacc[db] + gamma * lacc[db]) * inv;
                store4_f32(optr + 16 * db + 4 * g, o);
            }
            if (g == 0) a.log_norm[(long)bh * a.T + iq] = m_run * LN2 + __logf(Z);
        }
    }
    FLY_PROF(5);
}

// ---------------------------------------------------------------------------------------
// fused band kernel for float inputs on the bf16 matrix pipe (operands in bf16 pieces)
// ---------------------------------------------------------------------------------------
// Same work decomposition, masks, online softmax and outputs as sblocal_fwd_kernel; the three products
// of the key loop run on v_mfma_f32_16x16x32_bf16 from the tile images the key pass has left (see
// X3Tile): per 32-key tile and wave 12 MFMAs for the scores (three piece products), 4 M / 16 for the
// overlap (four), 5 D / 16 for P V (five; six with three V pieces) instead of (E + M + D) / 2 fp32 MFMAs of twice the duration.
// A tile image is copied global -> registers -> LDS as it is (16-byte pieces in thread order), two LDS
// stages.
// LIST: the exact part lives on a block-sparse support instead of a band (see sblocal_fwd_kernel: the same lists of 32-key
// tiles with a two-bit mask per wave and entry, the same start order, long lists walked in parts by the first workgroups
// of the launch, which write un-normalised partials for sb_merge_kernel).  One part per ordinary tile: SPLIT is false.
// TIO: the element type of q and out in memory (float, or a 2-byte type widened as it is loaded / rounded as it is stored).
template <int E, int D, int M, bool SPLIT, bool DROPOUT = false, bool LIST = false, typename TIO = float>
__global__ __launch_bounds__(NT) void sblocal_fwd_x3_kernel(FwdArgs a) {
    static_assert(!(LIST && SPLIT), "a block-sparse support is walked with one part per tile (long lists: a runtime role)");
    typedef X3Tile<E, D, M> TL;
    constexpr int MH = M / 2, LDK = E + 4, LDV = D + 4;
    constexpr int FB = MH / 16, EC = E / 16, DB = D / 16, KB = TK / 16, KS = E / 32, FS = M / 32;
    static_assert(KB == 2 && TK == 32, "one P V step per tile: eight k-slots per lane are the lane's two score quads");
    extern __shared__ __attribute__((aligned(128))) float smem[];
    char* lds = reinterpret_cast<char*>(smem);
    float* Ps = smem;                                  // only live before the key loop

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int n_qt = (a.T + TQ - 1) / TQ;
    // (LIST: every workgroup has an item of the lists below; n_items = 0 keeps the band's mapping out of the way)
    const int n_items = LIST ? 0 : a.B * a.H * n_qt * a.n_parts;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const bool tail = (int)blockIdx.x >= a.band_wgs;
    const int item = tail ? n_items : (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // see sblocal_fwd_kernel
    if (!LIST && item >= n_items) {                    // workgroup-uniform
        // Combine role, see sblocal_fwd_kernel: the workgroups behind the band workgroups, and the band range's own
        // padding (its size is a whole number of rounds over the XCDs), which would otherwise hold a slot for nothing
        if (!SPLIT) return;
        const int n_pad = a.band_wgs - n_items;
        const int ci = tail ? n_pad + (int)blockIdx.x - a.band_wgs : item - n_items;
        if (ci >= a.B * a.H * a.cmb_wpb) return;
        FLY_PROF(0);
        sb_combine_body(smem, a.kv_part, a.part_max, const_cast<float*>(a.kv), const_cast<float*>(a.ksum),
                        const_cast<float*>(a.kmax), nullptr, ci / a.cmb_wpb, ci % a.cmb_wpb, a.cmb_wpb, a.n_split, M, D);
        FLY_PROF(7);
        return;
    }
    int part = LIST ? 0 : item % a.n_parts;
    int qt = LIST ? 0 : (item / a.n_parts) % n_qt;
    int bh = LIST ? 0 : item / (a.n_parts * n_qt);
    // part_role: this workgroup writes an un-normalised partial instead of the result (always with SPLIT; with LIST the
    // first workgroups of the launch, which walk the long lists in parts)
    bool part_role = SPLIT;
    long slot = 0;                  // long lists: index of the tile's partials and compact query features
    if (LIST) {                     // (as in sblocal_fwd_kernel)
        const int n_part_wgs = (a.B * a.n_heavy * a.n_parts + a.n_xcd - 1) / a.n_xcd * a.n_xcd;
        if ((int)blockIdx.x < n_part_wgs) {
            const int idx = blockIdx.x;
            if (idx >= a.B * a.n_heavy * a.n_parts) return;            // workgroup-uniform
            part_role = true;
            part = idx % a.n_parts;
            slot = idx / a.n_parts;
            const int hq = a.tl_heavy[slot % a.n_heavy];
            qt = hq % n_qt;
            bh = (int)(slot / a.n_heavy) * a.H + hq / n_qt;
        } else {
            const int blk_id = blockIdx.x - n_part_wgs;
            const int nbh = a.B * a.H, x = blk_id % a.n_xcd, i = blk_id / a.n_xcd;
            const int mine = (nbh - x + a.n_xcd - 1) / a.n_xcd;            // (batch, head) pairs of this XCD
            if (mine <= 0 || i >= mine * n_qt) return;                 // workgroup-uniform
            const int rank = i / mine;
            bh = x + a.n_xcd * (i % mine);
            qt = a.tl_order ? a.tl_order[(bh % a.H) * n_qt + rank] : rank;
            if (qt < 0) return;                                        // a long list: walked in parts by the first workgroups
        }
    }
    const int b = bh / a.H, h = bh % a.H;
    const int q0 = qt * TQ;
    const int iq = q0 + 16 * w + r16;
    const bool qvalid = iq < a.T;
    const TIO* qptr = reinterpret_cast<const TIO*>(a.q) + b * a.q_sb + h * a.q_sh;
    const char* kv_img = reinterpret_cast<const char*>(a.vt) + (long)bh * a.n_chunks * (2 * (long)TL::KV_BYTES);
    const char* f_img = reinterpret_cast<const char*>(a.kfeat) + (long)bh * a.n_chunks * (2 * (long)TL::F_BYTES);
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half = 0.5f * __logf(2.0f * a.mh_valid);
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi

    FLY_PROF(0);
    const int q_last = min(q0 + TQ - 1, a.T - 1);
    const int lo = max(0, q0 - lc_lo);
    const int hi = min(len, q_last + lc_hi);
    int kt_lo = lo / TK;
    int kt_hi = (hi > lo) ? (hi + TK - 1) / TK : kt_lo;
    if (SPLIT) {
        const int nt = kt_hi - kt_lo, base = nt / a.n_parts, extra = nt % a.n_parts;
        const int first = kt_lo + part * base + min(part, extra);
        kt_lo = first;
        kt_hi = first + base + (part < extra ? 1 : 0);
    }
    // LIST: the loop counter walks the tile's list; tile index and this wave's presence mask of an entry (bit h: the wave's
    // 16 queries see keys 16 h .. 16 h + 15 of the tile) are read one iteration ahead of their use
    const int32_t* tl_inner = nullptr;
    const int32_t* tl_blk = nullptr;
    int tile_cur = 0, tile_next = 0;
    int pres_cur = 0, pres_next = 0;
    bool seen_block = false;
    if (LIST) {
        int lp0 = a.tl_ptr[h * n_qt + qt];
        kt_lo = 0;
        kt_hi = a.tl_ptr[h * n_qt + qt + 1] - lp0;
        if (part_role) {
            const int base = kt_hi / a.n_parts, extra = kt_hi % a.n_parts;
            lp0 += part * base + min(part, extra);
            kt_hi = base + (part < extra ? 1 : 0);
        }
        tl_inner = a.tl_inner + lp0;
        tl_blk = a.tl_blk + 4 * (long)lp0 + w;              // four masks per entry, one per wave
        if (kt_hi > 0) { tile_cur = tl_inner[0]; pres_cur = tl_blk[0] & 3; }
        if (kt_hi > 1) { tile_next = tl_inner[1]; pres_next = tl_blk[4] & 3; }
    }
    const int first_tile = LIST ? tile_cur : kt_lo;

    // tile images: flat copies, 16-byte pieces in thread order
    constexpr int NKV = (TL::KV_BYTES / 16 + NT - 1) / NT, NF = (TL::F_BYTES / 16 + NT - 1) / NT;
    constexpr bool KV_EXACT = TL::KV_BYTES / 16 % NT == 0, F_EXACT = TL::F_BYTES / 16 % NT == 0;
    uintx4 rkv[NKV], rf[NF];
    auto fetch = [&](int kt) __attribute__((always_inline)) {
        const uintx4* gk = reinterpret_cast<const uintx4*>(kv_img + (long)kt * TL::KV_BYTES);
        const uintx4* gf = reinterpret_cast<const uintx4*>(f_img + (long)kt * TL::F_BYTES);
#pragma unroll
        for (int j = 0; j < NKV; ++j)
            if (KV_EXACT || tid + NT * j < TL::KV_BYTES / 16) rkv[j] = gk[tid + NT * j];
#pragma unroll
        for (int j = 0; j < NF; ++j)
            if (F_EXACT || tid + NT * j < TL::F_BYTES / 16) rf[j] = gf[tid + NT * j];
    };
    auto stash = [&](int stage) __attribute__((always_inline)) {
        uintx4* dk = reinterpret_cast<uintx4*>(lds + stage * TL::BYTES);
        uintx4* df = reinterpret_cast<uintx4*>(lds + stage * TL::BYTES + TL::KV_BYTES);
#pragma unroll
        for (int j = 0; j < NKV; ++j)
            if (KV_EXACT || tid + NT * j < TL::KV_BYTES / 16) dk[tid + NT * j] = rkv[j];
#pragma unroll
        for (int j = 0; j < NF; ++j)
            if (F_EXACT || tid + NT * j < TL::F_BYTES / 16) df[tid + NT * j] = rf[j];
    };
    // the tiles after the first go straight from global memory into the stage (the first is asked for here, through
    // registers, because the stages hold the projection until the query features are done)
    auto transfer = [&](int kt, int stage) __attribute__((always_inline)) {
        const char* gk = kv_img + (long)kt * TL::KV_BYTES;
        const char* gf = f_img + (long)kt * TL::F_BYTES;
        const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
#pragma unroll
        for (int j = 0; j < NKV; ++j)
            if (KV_EXACT || tid + NT * j < TL::KV_BYTES / 16)
                dma_to_lds(gk + 16 * (tid + NT * j), lds + stage * TL::BYTES + 16 * (NT * j + 64 * wv));
#pragma unroll
        for (int j = 0; j < NF; ++j)
            if (F_EXACT || tid + NT * j < TL::F_BYTES / 16)
                dma_to_lds(gf + 16 * (tid + NT * j), lds + stage * TL::BYTES + TL::KV_BYTES + 16 * (NT * j + 64 * wv));
    };
    if (kt_lo < kt_hi) fetch(first_tile);
    const float* csp = a.chunk_scale + (long)bh * a.n_chunks;
    float cscale = (kt_lo < kt_hi) ? csp[first_tile * TK / CH] : 0.f;
    const float kmax = SPLIT ? split_kmax(a.part_max, bh, a.n_split) : a.kmax[bh];

    // query operand: lane (r16, g) holds elements 16c + 4g + i of its query row
    floatx4 qr[EC];
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        qr[c] = Frag<float>::zero();
        if (qvalid) qr[c] = load4_f32(qptr + (long)iq * a.q_ss + 16 * c + 4 * g);
        sq += qr[c][0] * qr[c][0] + qr[c][1] * qr[c][1] + qr[c][2] * qr[c][2] + qr[c][3] * qr[c][3];
    }
    const float diag_q = 0.5f * a.temp * group_sum(sq);

    // query features rounded to 17 bits, as two bf16 pieces in B-operand order (k-slot 8g + 4h + i of step ks
    // = feature 32 ks + 16 h + 4 g + i, i.e. blocks 2 ks and 2 ks + 1 of the lane's features)
    uintx4 qfh[FS], qfl[FS];
    float lsq;
    {
        floatx4 qf[2 * FB];
        if (SPLIT) {
            const long qrow = (long)bh * a.T + min(iq, a.T - 1);
#pragma unroll
            for (int c = 0; c < 2 * FB; ++c) qf[c] = *reinterpret_cast<const floatx4*>(a.qfeat + qrow * M + 16 * c + 4 * g);
            lsq = a.q_lsq[qrow];
        } else {
            // sqrt(t) P q on the bf16 matrix pipe: P in three pieces (exact), q in two, five piece products
            char* Pp = reinterpret_cast<char*>(smem);
            constexpr int P_ROW = 2 * E, P_PIECE = MH * P_ROW;
            static_assert(3 * P_PIECE <= 2 * TL::BYTES, "the projection pieces must fit the tile stages");
            load_proj_pieces<E, MH>(Pp, a.proj, sqrtf(a.temp), tid);
            __syncthreads();
            float qmax = 0.f;
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) qf[fb] = Frag<float>::zero();
#pragma unroll
            for (int ks = 0; ks < E / 32; ++ks) {
                uintx4 uh, ul;
                split2(qr[2 * ks], qr[2 * ks + 1], uh, ul);
#pragma unroll
                for (int fb = 0; fb < FB; ++fb) {
                    const int row = 16 * fb + r16;
                    const char* pp_ = Pp + row * P_ROW + x3_swz(row, 4 * ks + g, P_ROW) * 16;
                    const uintx4 ph = *reinterpret_cast<const uintx4*>(pp_), pm = *reinterpret_cast<const uintx4*>(pp_ + P_PIECE);
                    const uintx4 pl = *reinterpret_cast<const uintx4*>(pp_ + 2 * P_PIECE);
                    qf[fb] = mma_bf16(pl, uh, qf[fb]);
                    qf[fb] = mma_bf16(pm, ul, qf[fb]);
                    qf[fb] = mma_bf16(ph, ul, qf[fb]);
                    qf[fb] = mma_bf16(pm, uh, qf[fb]);
                    qf[fb] = mma_bf16(ph, uh, qf[fb]);
                }
            }
#pragma unroll
            for (int fb = 0; fb < FB; ++fb)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (16 * fb + 4 * g + i < a.mh_valid) qmax = fmaxf(qmax, fabsf(qf[fb][i]));
            qmax = group_max(qmax);
            lsq = -diag_q + qmax - lnm_half;
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                floatx4 dd = qf[fb];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool ok = 16 * fb + 4 * g + i < a.mh_valid;
                    qf[fb][i] = ok ? quant16(__expf(dd[i] - qmax)) : 0.f;
                    qf[FB + fb][i] = ok ? quant16(__expf(-dd[i] - qmax)) : 0.f;
                }
            }
            __syncthreads();      // Ps is dead; the tile buffers may overwrite it
        }
        if (LIST && part_role && part == 0) {
            // the merge kernel's operand for the global low-rank term
            float* dst = const_cast<float*>(a.qfeat) + (slot * TQ + 16 * w + r16) * M;
#pragma unroll
            for (int c = 0; c < 2 * FB; ++c) *reinterpret_cast<floatx4*>(dst + 16 * c + 4 * g) = qf[c];
        }
#pragma unroll
        for (int ks = 0; ks < FS; ++ks) split2(qf[2 * ks], qf[2 * ks + 1], qfh[ks], qfl[ks]);   // exact: 17-bit values
    }
    FLY_PROF(1);

    // From here on all exponents are base 2: the score operand carries t log2(e)
    constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
    const float c0 = (lsq + kmax) * LOG2E;       // base-2 log-scale of the global low-rank term
    uintx4 qh[KS], ql[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) split2(qr[2 * ks] * (a.temp * LOG2E), qr[2 * ks + 1] * (a.temp * LOG2E), qh[ks], ql[ks]);
    float m_run = c0;
    float ze = 0.f, zp = 0.f;
    floatx4 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = Frag<float>::zero();
    const int qw0 = q0 + 16 * w;
    const int smin = max(iq - lc_lo, 0);
    const unsigned span = qvalid ? (unsigned)max(min(iq + lc_hi, len) - smin, 0) : 0u;
    const uint32_t drop_row = DROPOUT ? drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + iq)) : 0u;

    // fragment addresses inside a stage (bytes): rows 16 kb + r16 share the swizzle of r16
    int koff[KS], foff[FS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) koff[ks] = r16 * TL::K_ROW + x3_swz(r16, 4 * ks + g, TL::K_ROW) * 16;
#pragma unroll
    for (int ks = 0; ks < FS; ++ks) foff[ks] = TL::KV_BYTES + r16 * TL::F_ROW + x3_swz(r16, 4 * ks + g, TL::F_ROW) * 16;
    const int voff = 2 * TL::K_PIECE + r16 * TL::V_ROW + x3_swz(r16, g, TL::V_ROW) * 16;

    if (kt_lo < kt_hi) stash(0);
    __syncthreads();

    FLY_PROF(2);
    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        const int s_base = (LIST ? tile_cur : kt) * TK;
        const int cur = (kt - kt_lo) & 1;
        const char* st = lds + cur * TL::BYTES;
        const bool more = kt + 1 < kt_hi;
        float cscale_next = cscale;
        // LIST: the entry after the next one (tile, presence) is requested now
        int tile_n2 = 0, pres_n2 = 0;
        if (LIST && kt + 2 < kt_hi) { tile_n2 = tl_inner[kt + 2]; pres_n2 = tl_blk[4 * (kt + 2)] & 3; }
        if (more) {                                      // next tile's transfer flies during the MFMAs (every wave is past
            const int nxt = LIST ? tile_next : kt + 1;   // the barrier that ended the last use of that stage)
            transfer(nxt, cur ^ 1);
            cscale_next = csp[nxt * TK / CH];
        }
        const float wc = __builtin_amdgcn_exp2f((cscale - kmax) * LOG2E);
        const bool any = LIST ? pres_cur != 0
                              : !(s_base + TK - 1 - qw0 < -lc_lo || s_base - (qw0 + 15) >= lc_hi || s_base >= len);
        const bool stamp = kt == kt_lo + 1;
        FLY_PROF2(stamp, 0);
        if (any) {
            floatx4 s1[KB], s2[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) { s1[kb] = Frag<float>::zero(); s2[kb] = Frag<float>::zero(); }
            // LDS fragments are requested a phase ahead of the MFMAs that use them (the scheduling barriers keep the
            // requests where they are written): K and the first half of K' before the scores, the second half
            // of K' before the first half of the overlap, V^T before the second half and the softmax arithmetic
            // (small problems, where a workgroup's few tiles are a chain of latencies; with one part per tile the registers
            // this takes would cost the second workgroup of a compute unit, and fragments are requested where they are used)
            constexpr bool AHEAD = SPLIT;
            constexpr int FA = (FS + 1) / 2, DA = (DB + 1) / 2;
            uintx4 kf[KS][KB][2], ff[FS][KB][2], vf[DB][X3_VP];
            auto load_f = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    ff[ks][kb][0] = *reinterpret_cast<const uintx4*>(st + foff[ks] + 16 * kb * TL::F_ROW);
                    ff[ks][kb][1] = *reinterpret_cast<const uintx4*>(st + foff[ks] + 16 * kb * TL::F_ROW + TL::F_PIECE);
                }
            };
            auto load_v = [&](int db) __attribute__((always_inline)) {
                vf[db][0] = *reinterpret_cast<const uintx4*>(st + voff + 16 * db * TL::V_ROW);
                vf[db][1] = *reinterpret_cast<const uintx4*>(st + voff + 16 * db * TL::V_ROW + TL::V_PIECE);
                if (X3_VP == 3) vf[db][X3_VP - 1] = *reinterpret_cast<const uintx4*>(st + voff + 16 * db * TL::V_ROW + 2 * TL::V_PIECE);
            };
            // overlap of one feature step: all four piece products (exact product of the rounded features)
            // (consecutive MFMAs go to different accumulators: one that adds to the result of the one before it waits
            //  for that result)
            auto overlap = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s2[kb] = mma_bf16(ff[ks][kb][1], qfl[ks], s2[kb]);
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s2[kb] = mma_bf16(ff[ks][kb][1], qfh[ks], s2[kb]);
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s2[kb] = mma_bf16(ff[ks][kb][0], qfl[ks], s2[kb]);
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s2[kb] = mma_bf16(ff[ks][kb][0], qfh[ks], s2[kb]);
            };
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    kf[ks][kb][0] = *reinterpret_cast<const uintx4*>(st + koff[ks] + 16 * kb * TL::K_ROW);
                    kf[ks][kb][1] = *reinterpret_cast<const uintx4*>(st + koff[ks] + 16 * kb * TL::K_ROW + TL::K_PIECE);
                }
            if (AHEAD) {
#pragma unroll
                for (int ks = 0; ks < FA; ++ks) load_f(ks);
                __builtin_amdgcn_sched_barrier(0);
            }
            FLY_PROF2(stamp, 1);
            // scores: three piece products, smallest first
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s1[kb] = mma_bf16(kf[ks][kb][1], qh[ks], s1[kb]);
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s1[kb] = mma_bf16(kf[ks][kb][0], ql[ks], s1[kb]);
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s1[kb] = mma_bf16(kf[ks][kb][0], qh[ks], s1[kb]);
            }
            if (AHEAD) {
                __builtin_amdgcn_sched_barrier(0);
                FLY_PROF2(stamp, 2);
#pragma unroll
                for (int ks = FA; ks < FS; ++ks) load_f(ks);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < FA; ++ks) overlap(ks);
                __builtin_amdgcn_sched_barrier(0);
                FLY_PROF2(stamp, 3);
#pragma unroll
                for (int db = 0; db < DA; ++db) load_v(db);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = FA; ks < FS; ++ks) overlap(ks);
                __builtin_amdgcn_sched_barrier(0);
                FLY_PROF2(stamp, 4);
#pragma unroll
                for (int db = DA; db < DB; ++db) load_v(db);
                __builtin_amdgcn_sched_barrier(0);
            } else {
#pragma unroll
                for (int ks = 0; ks < FS; ++ks) { load_f(ks); overlap(ks); }
            }
            // (LIST: a present half tile is wholly visible; the caller guarantees whole blocks of keys and queries)
            const bool interior = LIST ? pres_cur == 3
                                       : (s_base - (qw0 + 15) >= -lc_lo && s_base + TK - 1 - qw0 < lc_hi &&
                                          s_base + TK <= len && qw0 + 15 < a.T);
            floatx4 p[KB];
            float ovs = 0.f;
            auto soft = [&](auto masked_tag, auto drop_tag) __attribute__((always_inline)) {
                constexpr bool MASKED = decltype(masked_tag)::value, DROP = decltype(drop_tag)::value;
                bool ok[KB][4];
                float mx = -INFINITY;
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int s = s_base + 16 * kb + 4 * g + i;
                        ok[kb][i] = !MASKED || (LIST ? ((pres_cur >> kb) & 1) != 0 : (unsigned)(s - smin) < span);
                        mx = fmaxf(mx, ok[kb][i] ? s1[kb][i] : -INFINITY);
                    }
                mx = group_max(mx);
                if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.f) != 0) {      // wave-uniform
                    const float m_new = fmaxf(m_run, mx);
                    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                    m_run = m_new;
                    ze *= alpha;
#pragma unroll
                    for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
                }
                const float beta = wc * __builtin_amdgcn_exp2f(c0 - m_run);      // scale of the overlap term
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float e = ok[kb][i] ? __builtin_amdgcn_exp2f(s1[kb][i] - m_run) : 0.f;
                        const float ov = ok[kb][i] ? s2[kb][i] : 0.f;
                        ze += e;                                   // the normaliser sees no dropout
                        ovs += ov;
                        float ek = e;
                        if (DROP) ek = drop_keep(drop_row, (uint32_t)(s_base + 16 * kb + 4 * g + i), a.drop_thresh) ? e * a.drop_scale : 0.f;
                        p[kb][i] = ek - ov * beta;
                    }
            };
            if (interior) soft(std::false_type{}, std::integral_constant<bool, DROPOUT>{});
            else soft(std::true_type{}, std::integral_constant<bool, DROPOUT>{});
            FLY_PROF2(stamp, 5);
            zp += ovs * wc;
            // O^T[d][query] += sum_keys V[key][d] p[key][query]: P exactly in three pieces, five or six products
            // (P always in three exact pieces: its in-band low-rank part cancels against the global term, which is formed
            //  in fp32.  V may be two: the key pass multiplies the same rounded V, so that cancellation is not touched.)
            uintx4 ph, pm, pl;
            split3(p[0], p[1], ph, pm, pl);
            if (!AHEAD) {
#pragma unroll
                for (int db = 0; db < DB; ++db) load_v(db);
            }
            if (X3_VP == 3) {
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db][X3_VP - 1], ph, oacc[db]);
            }
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db][0], pl, oacc[db]);
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db][1], pm, oacc[db]);
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db][1], ph, oacc[db]);
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db][0], pm, oacc[db]);
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[db] = mma_bf16(vf[db][0], ph, oacc[db]);
        }
        FLY_PROF2(stamp, 6);
        drain_loads();                                   // this wave's share of the next tile is in LDS
        cscale = cscale_next;
        if (LIST) { seen_block |= pres_cur != 0; tile_cur = tile_next; tile_next = tile_n2; pres_cur = pres_next; pres_next = pres_n2; }
        FLY_PROF2(stamp, 7);
        __syncthreads();
        FLY_PROF2(stamp, 8);
    }
    if (LIST && !part_role && !seen_block) {
        // A block-row without any block: the reference's row logsumexp returns 0 there, not -inf
        // (blocksparse_logsumexp.py:132), so its normaliser carries an extra exp(0); reproduced.
        m_run = fmaxf(m_run, 0.f);
        ze = g == 0 ? __builtin_amdgcn_exp2f(-m_run) : 0.f;
    }

    FLY_PROF(3);
    floatx4 lacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) lacc[db] = Frag<float>::zero();
    float qk1 = 0.f;
    if (!part_role) {
        // global low-rank term on the bf16 matrix pipe: K'^T V in three pieces, the rounded query features in their two;
        // as many of the D columns at a time as the three pieces fit into the tile stages
        constexpr int ROOM = 2 * X3Tile<E, D, M>::BYTES - (int)sizeof(float) * M;
        constexpr int CW = 3 * M * 2 * D <= ROOM ? D : (3 * M * D <= ROOM ? D / 2 : D / 4);
        static_assert(3 * M * 2 * CW <= ROOM && CW % 16 == 0, "K'^T V pieces must fit the tile stages");
        char* KVp = reinterpret_cast<char*>(smem);
        float* KSs = reinterpret_cast<float*>(KVp + 3 * M * 2 * CW);
        if (tid < M) KSs[tid] = a.ksum[(long)bh * M + tid];
#pragma unroll
        for (int sl = 0; sl < D / CW; ++sl) {
            RowTile<M, CW> kvt;
            kvt.fetch(a.kv + (long)bh * M * D + sl * CW, D, 0, M - 1, tid);
            if (sl) __syncthreads();                 // the last slice's pieces have been read
            stash_pieces3<M, CW>(kvt, KVp, tid);
            __syncthreads();
            lowrank_pieces<M, CW, CW / 16>(KVp, qfh, qfl, *reinterpret_cast<floatx4(*)[CW / 16]>(&lacc[sl * (CW / 16)]), r16, g);
        }
#pragma unroll
        for (int c = 0; c < 2 * FB; ++c) {
            const uintx4 hw = qfh[c >> 1], lw = qfl[c >> 1];
            floatx4 qf;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t wh = hw[2 * (c & 1) + (i >> 1)], wl = lw[2 * (c & 1) + (i >> 1)];
                qf[i] = ((i & 1) ? __uint_as_float(wh & 0xffff0000u) : __uint_as_float(wh << 16)) +
                        ((i & 1) ? __uint_as_float(wl & 0xffff0000u) : __uint_as_float(wl << 16));
            }
            const floatx4 ks = *reinterpret_cast<const floatx4*>(KSs + 16 * c + 4 * g);
            qk1 += qf[0] * ks[0] + qf[1] * ks[1] + qf[2] * ks[2] + qf[3] * ks[3];
        }
        qk1 = group_sum(qk1);
    }
    ze = group_sum(ze);
    zp = group_sum(zp);
    FLY_PROF(4);
    const float gamma = __builtin_amdgcn_exp2f(c0 - m_run);               // <= 1
    if (part_role) {
        float* ws = a.part_ws + ((LIST ? slot : (long)bh * n_qt + qt) * a.n_parts + part) * (TQ * (D + NSTAT));
        const int ql_ = 16 * w + r16;
        float* stp = ws + TQ * D;
#pragma unroll
        for (int db = 0; db < DB; ++db) FLY_STORE(oacc[db], reinterpret_cast<floatx4*>(ws + ql_ * D + 16 * db + 4 * g));
        if (g == 0) {
            stp[0 * TQ + ql_] = m_run;
            stp[1 * TQ + ql_] = ze;
            stp[2 * TQ + ql_] = zp;
            stp[3 * TQ + ql_] = 0.f;
            stp[4 * TQ + ql_] = c0;
        }
    } else {
        const float Z = ze + gamma * fmaxf(qk1 - zp, 1e-24f);
        const float inv = 1.0f / Z;
        if (qvalid) {
            TIO* optr = reinterpret_cast<TIO*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq * a.o_ss;
#pragma unroll
            for (int db = 0; db < DB; ++db) store4_f32(optr + 16 * db + 4 * g, (oacc[db] + gamma * lacc[db]) * inv);
            if (g == 0) a.log_norm[(long)bh * a.T + iq] = m_run * LN2 + __logf(Z);
        }
    }
    FLY_PROF(5);
}

// Finish of a query tile that was computed in parts: one workgroup per (64-query tile, batch-head),
// in the register layout of the band kernel (wave w, lane (r16, g): query 16w + r16, output columns
// 16db + 4g + i).  It merges the parts' un-normalised partials -- taken in batches whose loads are all
// issued before the first is used (slots past n_parts re-read the last part and are ignored), with an
// online rescale to the running maximum between batches -- and adds the global low-rank term
// q' (K'^T V), q' . sum K' on fp32 MFMA from the query features of the key pass and the combined
// reductions, then normalises.
template <typename T, int D, int M>
__global__ __launch_bounds__(NT) void sb_merge_kernel(FwdArgs a) {
    constexpr float LN2 = 0.6931471805599453f;
    constexpr int FC = M / 16, LDV = 16 + 4;
    constexpr int PB = 8;                            // parts per batch
    __shared__ __attribute__((aligned(16))) float KVs[M * LDV];      // 16 columns of K'^T V
    __shared__ __attribute__((aligned(16))) float KSs[M];            // sum K'
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    // one workgroup per (64-query tile, 16 output columns, batch-head): the tile's finish is spread over
    // D/16 workgroups because it is all latency (a short chain of loads, 2 M/16 MFMAs, a store)
    // (long lists of a block-sparse support: blockIdx.x = batch * n_heavy + entry of tl_heavy, see FwdArgs)
    const bool heavy = a.tl_heavy != nullptr;
    const int n_qt = heavy ? (a.T + TQ - 1) / TQ : gridDim.x;
    const int hq = heavy ? a.tl_heavy[blockIdx.x % a.n_heavy] : 0;
    const int qt = heavy ? hq % n_qt : blockIdx.x;
    const int db = blockIdx.y, bh = heavy ? (blockIdx.x / a.n_heavy) * a.H + hq / n_qt : blockIdx.z;
    const int b = bh / a.H, h = bh % a.H;
    const long slot = heavy ? blockIdx.x : (long)bh * n_qt + qt;
    const int ql = 16 * w + r16, iq = qt * TQ + ql;
    {
        RowTile<M, 16> kvt;
        kvt.fetch(a.kv + (long)bh * M * D + 16 * db, D, 0, M - 1, tid);
        if (tid < M) KSs[tid] = a.ksum[(long)bh * M + tid];
        kvt.template stash<LDV>(KVs, tid);
    }
    const long qrow = heavy ? slot * TQ + ql : (long)bh * a.T + min(iq, a.T - 1);
    floatx4 qf[FC];
#pragma unroll
    for (int c = 0; c < FC; ++c) qf[c] = *reinterpret_cast<const floatx4*>(a.qfeat + qrow * M + 16 * c + 4 * g);

    const long stride = (long)TQ * (D + NSTAT);
    const float* ws = a.part_ws + slot * a.n_parts * stride;
    const float* st = ws + TQ * D + ql;
    const float c0 = st[4 * TQ];                     // base-2 log-scale of the low-rank term (same in every part)
    float m_star = -INFINITY, ze = 0.f, zp = 0.f;
    floatx4 acc = Frag<float>::zero();
    for (int p0 = 0; p0 < a.n_parts; p0 += PB) {
        float mv[PB], zev[PB], zpv[PB];
        floatx4 ov[PB];
#pragma unroll
        for (int j = 0; j < PB; ++j) {
            const long off = (long)min(p0 + j, a.n_parts - 1) * stride;
            mv[j] = st[off];
            zev[j] = st[off + TQ];
            zpv[j] = st[off + 2 * TQ];
            ov[j] = *reinterpret_cast<const floatx4*>(ws + off + ql * D + 16 * db + 4 * g);
        }
        float m_new = m_star;
#pragma unroll
        for (int j = 0; j < PB; ++j) m_new = fmaxf(m_new, mv[j]);      // repeated slots repeat a valid value
        const float keep = (m_star == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_star - m_new);
        m_star = m_new;
        ze *= keep;
        acc *= keep;
#pragma unroll
        for (int j = 0; j < PB; ++j) {
            if (p0 + j < a.n_parts) {
                const float wgt = __builtin_amdgcn_exp2f(mv[j] - m_star);
                ze += wgt * zev[j];
                zp += zpv[j];
                acc += wgt * ov[j];
            }
        }
    }
    __syncthreads();                                 // K'^T V and sum K' are in LDS
    floatx4 lacc0 = Frag<float>::zero(), lacc1 = Frag<float>::zero();    // two chains
    float qk1 = 0.f;
#pragma unroll
    for (int c = 0; c < FC; ++c) {
        const floatx4 ks = *reinterpret_cast<const floatx4*>(KSs + 16 * c + 4 * g);
        qk1 += qf[c][0] * ks[0] + qf[c][1] * ks[1] + qf[c][2] * ks[2] + qf[c][3] * ks[3];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float kvv = KVs[(16 * c + 4 * g + j) * LDV + r16];
            if (j & 1) lacc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kvv, qf[c][j], lacc1, 0, 0, 0);
            else lacc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kvv, qf[c][j], lacc0, 0, 0, 0);
        }
    }
    qk1 = group_sum(qk1);
    if (iq >= a.T) return;
    const float gamma = __builtin_amdgcn_exp2f(c0 - m_star);              // <= 1: every part starts its maximum at c0
    const float Z = ze + gamma * fmaxf(qk1 - zp, 1e-24f);
    const float inv = 1.0f / Z;
    T* optr = reinterpret_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq * a.o_ss;
    store4_f32(optr + 16 * db + 4 * g, (acc + gamma * (lacc0 + lacc1)) * inv);
    if (g == 0 && db == 0) a.log_norm[(long)bh * a.T + iq] = m_star * LN2 + __logf(Z);
}

// The same finish for the band kernel on bf16 pieces, arranged for locality: a workgroup takes 16 NDB output
// columns of a tile (NDB = D / 16: the whole tile, so that the query features and the parts' statistics are
// read once), and the one-dimensional grid is laid out so that a tile is finished on the XCD whose
// workgroups wrote its parts (the dispatcher deals consecutive workgroup ids to the XCDs in turn): the
// partials are then still in that XCD's L2.  xcd_items = band items (tile, part) per XCD of the band launch.
// (the finish of tile tl, columns 16 NDB slice .. of it, by one workgroup; KVp: 3 M rows of 32 NDB bytes, KSs: M floats of LDS)
template <int D, int M, int NDB, typename TOUT = float>
__device__ __forceinline__ void sb_merge_tile(const FwdArgs& a, int tl, int slice, char* KVp, float* KSs) {
    constexpr float LN2 = 0.6931471805599453f;
    constexpr int FC = M / 16, COLS = 16 * NDB, LDV = COLS + 4;
    constexpr int PB = NDB >= 4 ? 5 : 8;              // parts per batch (their loads are all in flight together)
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int n_qt = (a.T + TQ - 1) / TQ;
    const int qt = tl % n_qt, bh = tl / n_qt, b = bh / a.H, h = bh % a.H;
    const int col0 = slice * COLS;
    const int ql = 16 * w + r16, iq = qt * TQ + ql;
    // every operand comes from memory (another launch, or another workgroup, wrote it): all loads are issued
    // before the first is used, so that the finish costs one round trip, not one per operand
    RowTile<M, COLS> kvt;
    kvt.fetch(a.kv + (long)bh * M * D + col0, D, 0, M - 1, tid);
    const float ksv = a.ksum[(long)bh * M + min(tid, M - 1)];
    const long qrow = (long)bh * a.T + min(iq, a.T - 1);
    floatx4 qf[FC];
#pragma unroll
    for (int c = 0; c < FC; ++c) qf[c] = *reinterpret_cast<const floatx4*>(a.qfeat + qrow * M + 16 * c + 4 * g);

    const long stride = (long)TQ * (D + NSTAT);
    const float* ws = a.part_ws + (long)tl * a.n_parts * stride;
    const float* st = ws + TQ * D + ql;
    const float c0 = st[4 * TQ];
    float m_star = -INFINITY, ze = 0.f, zp = 0.f;
    floatx4 acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) acc[db] = Frag<float>::zero();
    for (int p0 = 0; p0 < a.n_parts; p0 += PB) {
        float mv[PB], zev[PB], zpv[PB];
        floatx4 ov[PB][NDB];
#pragma unroll
        for (int jj = 0; jj < PB; ++jj) {
            const long off = (long)min(p0 + jj, a.n_parts - 1) * stride;
            mv[jj] = st[off];
            zev[jj] = st[off + TQ];
            zpv[jj] = st[off + 2 * TQ];
#pragma unroll
            for (int db = 0; db < NDB; ++db)
                ov[jj][db] = *reinterpret_cast<const floatx4*>(ws + off + ql * D + col0 + 16 * db + 4 * g);
        }
        if (p0 == 0) {
            stash_pieces3<M, COLS>(kvt, KVp, tid);
            if (tid < M) KSs[tid] = ksv;
        }
        float m_new = m_star;
#pragma unroll
        for (int jj = 0; jj < PB; ++jj) m_new = fmaxf(m_new, mv[jj]);
        const float keep = (m_star == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_star - m_new);
        m_star = m_new;
        ze *= keep;
#pragma unroll
        for (int db = 0; db < NDB; ++db) acc[db] *= keep;
#pragma unroll
        for (int jj = 0; jj < PB; ++jj) {
            if (p0 + jj < a.n_parts) {
                const float wgt = __builtin_amdgcn_exp2f(mv[jj] - m_star);
                ze += wgt * zev[jj];
                zp += zpv[jj];
#pragma unroll
                for (int db = 0; db < NDB; ++db) acc[db] += wgt * ov[jj][db];
            }
        }
    }
    __syncthreads();                                 // K'^T V and sum K' are in LDS
    floatx4 lacc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) lacc[db] = Frag<float>::zero();
    float qk1 = 0.f;
    uintx4 qph[M / 32], qpl[M / 32];
#pragma unroll
    for (int c = 0; c < FC; ++c) {
        const floatx4 ks = *reinterpret_cast<const floatx4*>(KSs + 16 * c + 4 * g);
        qk1 += qf[c][0] * ks[0] + qf[c][1] * ks[1] + qf[c][2] * ks[2] + qf[c][3] * ks[3];
        if (c & 1) split2(qf[c - 1], qf[c], qph[c >> 1], qpl[c >> 1]);      // (exact: the features carry 17 bits)
    }
    lowrank_pieces<M, COLS, NDB>(KVp, qph, qpl, lacc, r16, g);
    qk1 = group_sum(qk1);
    if (iq >= a.T) return;
    const float gamma = __builtin_amdgcn_exp2f(c0 - m_star);
    const float Z = ze + gamma * fmaxf(qk1 - zp, 1e-24f);
    const float inv = 1.0f / Z;
    TOUT* optr = reinterpret_cast<TOUT*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq * a.o_ss + col0;
#pragma unroll
    for (int db = 0; db < NDB; ++db) store4_f32(optr + 16 * db + 4 * g, (acc[db] + gamma * lacc[db]) * inv);
    if (g == 0 && slice == 0) a.log_norm[(long)bh * a.T + iq] = m_star * LN2 + __logf(Z);
}

template <int D, int M, int NDB, typename TOUT = float>
__global__ __launch_bounds__(NT) void sb_merge_x_kernel(FwdArgs a, int xcd_items, int tiles_per_xcd) {
    constexpr int COLS = 16 * NDB, NSL = D / COLS;
    __shared__ __attribute__((aligned(16))) char KVp[3 * M * 2 * COLS];
    __shared__ __attribute__((aligned(16))) float KSs[M];
    const int n_qt = (a.T + TQ - 1) / TQ, n_tiles = a.B * a.H * n_qt;
    const int x = blockIdx.x % a.n_xcd, i = blockIdx.x / a.n_xcd, slice = i % NSL, j = i / NSL;
    // tiles whose first part is one of XCD x's band items
    const int t_lo = (x * xcd_items + a.n_parts - 1) / a.n_parts;
    const int t_hi = min(((x + 1) * xcd_items + a.n_parts - 1) / a.n_parts, n_tiles);
    const int tl = t_lo + j;
    if (j >= tiles_per_xcd || tl >= t_hi) return;     // workgroup-uniform
    sb_merge_tile<D, M, NDB, TOUT>(a, tl, slice, KVp, KSs);
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
template <int E, int M> constexpr size_t kfeat_smem() {
    // one K and one V tile, one feature tile, reduction scratch
    return sizeof(float) * (2 * CH * (E + 4) + CH * (M + 4) + 8);
}
template <int E, int M> constexpr size_t fwd_smem() {
    constexpr size_t stage = (size_t)TK * ((E + 4) + (E + 4) + (M + 4));
    constexpr size_t proj = (size_t)(M / 2) * (E + 4);
    constexpr size_t lowrank = (size_t)M * (E + 4) + M;
    constexpr size_t need = 2 * stage > proj ? (2 * stage > lowrank ? 2 * stage : lowrank)
                                             : (proj > lowrank ? proj : lowrank);
    return sizeof(float) * need;
}

template <int E, int M> constexpr size_t kfeat_bf16_smem() {
    return 2 * ((size_t)CH * (E + 8) + (size_t)E * (CH + 8) + (size_t)CH * (M + 8)) + sizeof(float) * (CH + 8);
}
template <int E, int M> constexpr size_t kfeat_x3_smem() {
    return 2 * (size_t)X3Tile<E, E, M>::BYTES + sizeof(float) * CH * (E + 4) + 3 * (size_t)(M / 2) * 2 * E +
           sizeof(float) * (CH + 4 + 4 * M);
}
template <int E, int M>
static int launch_kfeat_x3(const KvArgs& a, hipStream_t st) {
    if constexpr (E <= 64 && M <= 128) {
        // both products on the bf16 matrix pipe, images assembled in LDS
        constexpr size_t smem = kfeat_x3_smem<E, M>();
        static_assert(smem <= 160 * 1024, "two tile images, the V chunk and the projection image must fit the LDS");
        static std::atomic<unsigned long long> lds_set[3] = {{0}, {0}, {0}};     // (devices on which a kernel has its LDS limit)
        const void* kern = a.in_code == 1   ? reinterpret_cast<const void*>(sb_kfeat_x3_kernel<E, E, M, bf16_t>)
                           : a.in_code == 2 ? reinterpret_cast<const void*>(sb_kfeat_x3_kernel<E, E, M, f16_t>)
                                            : reinterpret_cast<const void*>(sb_kfeat_x3_kernel<E, E, M, float>);
        if (int rc = ensure_dynamic_lds(kern, smem, lds_set[a.in_code], "sb_kfeat_x3")) return rc;
        const dim3 grid(a.n_split + a.q_tiles, a.B * a.H);
        if (a.in_code == 1) hipLaunchKernelGGL((sb_kfeat_x3_kernel<E, E, M, bf16_t>), grid, dim3(NT), smem, st, a);
        else if (a.in_code == 2) hipLaunchKernelGGL((sb_kfeat_x3_kernel<E, E, M, f16_t>), grid, dim3(NT), smem, st, a);
        else hipLaunchKernelGGL((sb_kfeat_x3_kernel<E, E, M, float>), grid, dim3(NT), smem, st, a);
        return check_launch("sb_kfeat_x3_kernel");
    }
    if (a.in_code != 0) return fail(ERR_UNSUPPORTED, "sb_kv_reduce: 2-byte inputs on the image path need head dims up to 64 and up to 128 features");
    auto kern = sb_kfeat_kernel<float, E, E, M, true>;
    constexpr size_t smem = kfeat_smem<E, M>();
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "sb_kfeat (piece images)")) return rc;
    hipLaunchKernelGGL(kern, dim3(a.n_split + a.q_tiles, a.B * a.H), dim3(NT), smem, st, a);
    return check_launch("sb_kfeat_kernel (piece images)");
}

template <typename T, int E, int M>
static int launch_kfeat(const KvArgs& a, hipStream_t st) {
    if (sizeof(T) == 2 && !a.q) {            // bfloat16 keys, no query role: both products on the bf16 MFMA
        auto kern16 = sb_kfeat_bf16_kernel<E, E, M>;
        constexpr size_t smem16 = kfeat_bf16_smem<E, M>();
        static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern16), smem16, lds_set, "sb_kfeat_bf16")) return rc;
        hipLaunchKernelGGL(kern16, dim3(a.n_split, a.B * a.H), dim3(NT), smem16, st, a);
        return check_launch("sb_kfeat_bf16_kernel");
    }
    if (sizeof(T) == 4 && a.vt) return launch_kfeat_x3<E, M>(a, st);      // float inputs, piece images asked for
    auto kern = sb_kfeat_kernel<T, E, E, M>;
    constexpr size_t smem = kfeat_smem<E, M>();
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "sb_kfeat")) return rc;
    // per (batch, head): key-role workgroups, then query-role ones
    hipLaunchKernelGGL(kern, dim3(a.n_split + a.q_tiles, a.B * a.H), dim3(NT), smem, st, a);
    return check_launch("sb_kfeat_kernel");
}

// Optional timing hooks: two caller-owned events recorded immediately before and after the fused
// band kernel of the next flyhip_sblocal_fwd call made by this thread (then cleared).
static thread_local hipEvent_t g_ev_before = nullptr, g_ev_after = nullptr;

// float inputs: fp32 MFMA kernel; bfloat16 inputs: bf16 MFMA kernel
template <typename T, int E, int M, bool SPLIT> struct FwdKernel {
    static constexpr size_t smem = fwd_smem<E, M>();
    static constexpr int threads = NT, tq = TQ;       // threads and queries per workgroup
    static auto get() { return sblocal_fwd_kernel<T, E, E, M, SPLIT>; }
};
#ifndef FLY_BF16_WIDE
#define FLY_BF16_WIDE 1
#endif
// bfloat16 inputs: 32 queries per wave where the registers hold the wider operands (head dim up to 64) and the
// projection rows fill 32-row blocks (64 features or more); 16 queries per wave otherwise.  Both: 128 queries per workgroup.
template <int E, int M> constexpr bool bf16_wide() { return FLY_BF16_WIDE && M >= 64 && E <= 64; }
template <int E, int M, bool SPLIT> struct FwdKernel<bf16_t, E, M, SPLIT> {
    static constexpr size_t smem = fwd_bf16_smem<E, M>();
    static constexpr int threads = bf16_wide<E, M>() ? 64 * B32_WAVES : 64 * BF16_WAVES;
    static constexpr int tq = bf16_wide<E, M>() ? 32 * B32_WAVES : 16 * BF16_WAVES;
    static auto get() {
        if constexpr (bf16_wide<E, M>()) return sblocal_fwd_b32_kernel<E, E, M, SPLIT, B32_WAVES>;
        else return sblocal_fwd_bf16_kernel<E, E, M, SPLIT, BF16_WAVES>;
    }
};

template <typename T, int E, int M, bool SPLIT>
static int launch_fwd_impl(const FwdArgs& a, hipStream_t st) {
    auto kern = FwdKernel<T, E, M, SPLIT>::get();
    typedef FwdKernel<T, E, M, SPLIT> K;
    // the bf16 kernel keeps the chunk log-scales of a workgroup's share of the band behind its tile stages
    const long band_keys = (long)a.lc + K::tq + 2 * CH;
    const size_t smem = K::smem + (sizeof(T) == 2 ? (size_t)(band_keys / CH + 2) * sizeof(float) : 0);
    constexpr size_t LDS_MAX = 160 * 1024;
    if (smem > LDS_MAX) return fail(ERR_ARG, "sblocal_fwd: local_context %d needs %zu bytes of LDS (limit %zu)", a.lc, smem, LDS_MAX);
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_MAX, lds_set, "sblocal_fwd")) return rc;
    const Machine& mach = machine();
    const int qt = (a.T + TQ - 1) / TQ;                           // 64-query tiles (partials, merge)
    const long items = (long)a.B * a.H * ((a.T + K::tq - 1) / K::tq) * a.n_parts;
    long grid = (items + mach.xcds - 1) / mach.xcds * mach.xcds;             // whole rounds over the XCDs
    FwdArgs args = a;
    args.n_xcd = mach.xcds;
    args.band_wgs = (int)grid;
    if (SPLIT) {
        // combine role: as many workgroups per (batch, head) as fit beside the band workgroups in one
        // residency round (two workgroups of this kernel per CU), at least one, at most one thread per output
        const long bhn = (long)a.B * a.H, free_slots = mach.slots - grid;
        long wpb = free_slots / bhn;
        const long most = (M * (E + 1) / 4 + K::threads - 1) / K::threads;   // one 16-byte piece of the result per thread
        if (wpb > most) wpb = most;
        if (wpb < 1) wpb = 1;
        args.cmb_wpb = (int)wpb;
        grid += bhn * wpb;
    }
    if (grid > 2147483647L) return fail(ERR_ARG, "sblocal_fwd: too many workgroups");
    // (measurement hook: the two events take the launch's own begin and end time stamps)
    if (g_ev_before && g_ev_after)
        hipExtLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(K::threads), (uint32_t)smem, st, g_ev_before, g_ev_after, 0, args);
    else
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(K::threads), smem, st, args);
    g_ev_before = g_ev_after = nullptr;
    int rc = check_launch("sblocal_fwd_kernel");
    if (rc || !SPLIT) return rc;
    hipLaunchKernelGGL((sb_merge_kernel<T, E, M>), dim3(qt, E / 16, a.B * a.H), dim3(NT), 0, st, args);
    return check_launch("sb_merge_kernel");
}
#ifndef MERGE_NDB
#define MERGE_NDB 2
#endif
// float inputs with the piece images of the key pass: the band kernel on the bf16 matrix pipe
template <int E, int M> constexpr size_t fwd_x3_smem() {
    constexpr size_t tiles = 2 * (size_t)X3Tile<E, E, M>::BYTES;
    constexpr size_t proj = sizeof(float) * (size_t)(M / 2) * (E + 4);
    constexpr size_t lowrank = sizeof(float) * ((size_t)M * (E + 4) + M);
    return tiles > proj ? (tiles > lowrank ? tiles : lowrank) : (proj > lowrank ? proj : lowrank);
}
template <int E, int M, bool SPLIT, bool DROPOUT = false, typename TIO = float>
static int launch_fwd_x3(const FwdArgs& a, hipStream_t st) {
    auto kern = sblocal_fwd_x3_kernel<E, E, M, SPLIT, DROPOUT, false, TIO>;
#ifdef FLY_X3_PAD
    constexpr size_t smem = fwd_x3_smem<E, M>() + FLY_X3_PAD;
#else
    constexpr size_t smem = fwd_x3_smem<E, M>();
#endif
    static_assert(smem <= 160 * 1024, "two tile stages must fit the LDS");
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "sblocal_fwd (bf16 pieces)")) return rc;
    const Machine& mach = machine();
    const int qt = (a.T + TQ - 1) / TQ;
    const long items = (long)a.B * a.H * qt * a.n_parts;
    long grid = (items + mach.xcds - 1) / mach.xcds * mach.xcds;
    FwdArgs args = a;
    args.n_xcd = mach.xcds;
    args.band_wgs = (int)grid;
    if (SPLIT) {
        // combine role: as many workgroups per (batch, head) as fit beside the band workgroups in one residency round,
        // at least one, at most one thread per 16-byte piece of the result; the padding of the band range serves first
        const long bhn = (long)a.B * a.H, free_slots = mach.slots - items;
        long wpb = free_slots / bhn;
        const long most = (M * (E + 1) / 4 + NT - 1) / NT;
        if (wpb > most) wpb = most;
        if (wpb < 1) wpb = 1;
        args.cmb_wpb = (int)wpb;
        const long pad = grid - items;
        if (bhn * wpb > pad) grid += bhn * wpb - pad;
    }
    if (grid > 2147483647L) return fail(ERR_ARG, "sblocal_fwd: too many workgroups");
    // (measurement hook: the two events take the launch's own begin and end time stamps)
    if (g_ev_before && g_ev_after)
        hipExtLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), (uint32_t)smem, st, g_ev_before, g_ev_after, 0, args);
    else
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), smem, st, args);
    g_ev_before = g_ev_after = nullptr;
    int rc = check_launch("sblocal_fwd_x3_kernel");
    if (rc || !SPLIT) return rc;
    constexpr int NDB = MERGE_NDB < E / 16 ? MERGE_NDB : E / 16;
    const int xcd_items = (int)((items + mach.xcds - 1) / mach.xcds);
    const int tiles_per_xcd = (xcd_items + a.n_parts - 1) / a.n_parts + 1;
    hipLaunchKernelGGL((sb_merge_x_kernel<E, M, NDB, TIO>), dim3((unsigned)(mach.xcds * tiles_per_xcd * (E / 16 / NDB))), dim3(NT), 0, st,
                       args, xcd_items, tiles_per_xcd);
    return check_launch("sb_merge_x_kernel");
}
template <typename T, int E, int M>
static int launch_fwd(const FwdArgs& a, hipStream_t st) {
    if (a.io_code != 0) {
        // float16 q and out on the kernels on operand images (bfloat16 tensors have kernels of their own)
        if constexpr (sizeof(T) == 4 && E <= 64 && M <= 128) {
            if (a.vt && a.io_code == 2) {
                if (a.drop_thresh)
                    return a.n_parts > 1 ? launch_fwd_x3<E, M, true, true, f16_t>(a, st) : launch_fwd_x3<E, M, false, true, f16_t>(a, st);
                return a.n_parts > 1 ? launch_fwd_x3<E, M, true, false, f16_t>(a, st) : launch_fwd_x3<E, M, false, false, f16_t>(a, st);
            }
        }
        return fail(ERR_UNSUPPORTED, "sblocal_fwd: 2-byte q and out (code %d) are read and written by the kernels on operand images "
                                     "only: float16, head dims up to 64, up to 128 features", a.io_code);
    }
    if (sizeof(T) == 4 && a.vt) {
        // (dropout of the exact weights: a variant of its own, so that the kernel without it carries nothing of it)
        if (a.drop_thresh) {
            if constexpr (E <= 64 && M <= 128)
                return a.n_parts > 1 ? launch_fwd_x3<E, M, true, true>(a, st) : launch_fwd_x3<E, M, false, true>(a, st);
            return fail(ERR_UNSUPPORTED, "sblocal_fwd: no dropout variant for head dim %d with %d features", E, M);
        }
        return a.n_parts > 1 ? launch_fwd_x3<E, M, true>(a, st) : launch_fwd_x3<E, M, false>(a, st);
    }
    return a.n_parts > 1 ? launch_fwd_impl<T, E, M, true>(a, st) : launch_fwd_impl<T, E, M, false>(a, st);
}

// band kernel on a block-sparse support (lists of key tiles per query tile), one part per tile: on bf16 pieces when the
// key pass has left tile images (a.vt; head dims up to 64, up to 128 features, no dropout), else the fp32 kernel
template <typename T, int E, int M>
static int launch_fwd_list(const FwdArgs& a, hipStream_t st) {
    constexpr bool X3 = E <= 64 && M <= 128;
    const bool pieces = X3 && a.vt != nullptr;
    if (a.vt && !X3)
        return fail(ERR_UNSUPPORTED, "sbblocksparse_fwd: tile images are for head dims up to 64 and up to 128 features "
                                     "(got %d, %d)", E, M);
    const bool dropping = a.drop_thresh != 0u;
    const void* kern_fp32 = reinterpret_cast<const void*>(sblocal_fwd_kernel<float, E, E, M, false, true>);
    const void* kern = kern_fp32;
    size_t smem = fwd_smem<E, M>();
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which the kernels have their LDS limit)
    if (a.io_code != 0 && !pieces)
        return fail(ERR_UNSUPPORTED, "sbblocksparse_fwd: 2-byte q and out are read and written by the kernel on operand images only");
    static std::atomic<unsigned long long> lds_set_x3v[6] = {{0}, {0}, {0}, {0}, {0}, {0}};
    if constexpr (X3) {
        if (pieces) {
#define FLY_X3_LIST(DROP_, TIO_) reinterpret_cast<const void*>(sblocal_fwd_x3_kernel<E, E, M, false, DROP_, true, TIO_>)
            kern = a.io_code == 1   ? (dropping ? FLY_X3_LIST(true, bf16_t) : FLY_X3_LIST(false, bf16_t))
                   : a.io_code == 2 ? (dropping ? FLY_X3_LIST(true, f16_t) : FLY_X3_LIST(false, f16_t))
                                    : (dropping ? FLY_X3_LIST(true, float) : FLY_X3_LIST(false, float));
#undef FLY_X3_LIST
            smem = fwd_x3_smem<E, M>();
        }
    }
    if (int rc = ensure_dynamic_lds(kern, smem, pieces ? lds_set_x3v[2 * a.io_code + (dropping ? 1 : 0)] : lds_set, "sbblocksparse_fwd")) return rc;
    // every XCD gets room for ceil(B H / dies) (batch, head) pairs
    const Machine& mach = machine();
    const long grid = (((long)a.B * a.H + mach.xcds - 1) / mach.xcds) * ((a.T + TQ - 1) / TQ) * mach.xcds;
    if (grid > 2147483647L) return fail(ERR_ARG, "sbblocksparse_fwd: too many workgroups");
    // long lists: the first workgroups of the launch walk them in parts (they are the longest pieces of work)
    const long tiles = (long)a.B * a.n_heavy;
    const long part_wgs = (tiles * a.n_parts + mach.xcds - 1) / mach.xcds * mach.xcds;
    if (grid + part_wgs > 2147483647L) return fail(ERR_ARG, "sbblocksparse_fwd: too many workgroups");
    FwdArgs args = a;
    args.n_xcd = mach.xcds;
    args.band_wgs = (int)(grid + part_wgs);
    if constexpr (X3) {
        if (pieces) {
            const dim3 grd((unsigned)(grid + part_wgs));
#define FLY_X3_LIST_GO(DROP_, TIO_) hipLaunchKernelGGL((sblocal_fwd_x3_kernel<E, E, M, false, DROP_, true, TIO_>), grd, dim3(NT), smem, st, args)
            if (a.io_code == 1) { if (dropping) FLY_X3_LIST_GO(true, bf16_t); else FLY_X3_LIST_GO(false, bf16_t); }
            else if (a.io_code == 2) { if (dropping) FLY_X3_LIST_GO(true, f16_t); else FLY_X3_LIST_GO(false, f16_t); }
            else { if (dropping) FLY_X3_LIST_GO(true, float); else FLY_X3_LIST_GO(false, float); }
#undef FLY_X3_LIST_GO
        }
    }
    if (!pieces)
        hipLaunchKernelGGL((sblocal_fwd_kernel<float, E, E, M, false, true>), dim3((unsigned)(grid + part_wgs)), dim3(NT), smem, st, args);
    int rc = check_launch("sblocal_fwd_kernel (block-sparse support)");
    if (rc || a.n_heavy <= 0) return rc;
    const dim3 mgrid((unsigned)tiles, E / 16, 1);
    if (a.io_code == 1) hipLaunchKernelGGL((sb_merge_kernel<bf16_t, E, M>), mgrid, dim3(NT), 0, st, args);
    else if (a.io_code == 2) hipLaunchKernelGGL((sb_merge_kernel<f16_t, E, M>), mgrid, dim3(NT), 0, st, args);
    else hipLaunchKernelGGL((sb_merge_kernel<float, E, M>), mgrid, dim3(NT), 0, st, args);
    return check_launch("sb_merge_kernel (long lists)");
}

#ifndef FLY_LOCAL_B16
#define FLY_LOCAL_B16 1
#endif
// 2-byte inputs whose rows allow 16-byte loads: the kernel on the 16x16x32 MFMA of the input type
template <typename T, int E, int QB>
static int launch_local_b16_as(const LocalArgs& a, hipStream_t st) {
    auto kern = local_fwd_b16_kernel<T, E, E, QB>;
    constexpr size_t smem = local_b16_smem<E>();
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "local_fwd_b16")) return rc;
    const Machine& mach = machine();
    const long items = (long)a.B * a.H * ((a.T + 64 * QB - 1) / (64 * QB));
    const long grid = (items + mach.xcds - 1) / mach.xcds * mach.xcds;
    if (grid > 2147483647L) return fail(ERR_ARG, "local_fwd: too many workgroups");
    LocalArgs args = a;
    args.n_xcd = mach.xcds;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), smem, st, args);
    return check_launch("local_fwd_b16_kernel");
}
#ifndef FLY_LOCAL_B16_WIDE
#define FLY_LOCAL_B16_WIDE 1
#endif
#ifndef FLY_LOCAL_B16_WIDE_ROUNDS
#define FLY_LOCAL_B16_WIDE_ROUNDS 2
#endif
// 32 queries per wave once workgroups of 128 queries still fill the device twice over (three of them share a compute
// unit; measured at 2.7 rounds: 0.152 -> 0.129 ms at 16 heads of 16384 tokens; head dims up to 64: the wide form's
// accumulators and score sets need the registers)
template <typename T, int E>
static int launch_local_b16(const LocalArgs& a, hipStream_t st) {
    if constexpr (E <= 64) {
        const long wide_items = (long)a.B * a.H * ((a.T + 127) / 128);
        if (FLY_LOCAL_B16_WIDE && wide_items >= (long)FLY_LOCAL_B16_WIDE_ROUNDS * 3 * machine().cus) return launch_local_b16_as<T, E, 2>(a, st);
    }
    return launch_local_b16_as<T, E, 1>(a, st);
}
static bool local_b16_ready(const LocalArgs& a) {
    const long strides = a.q_sb | a.q_sh | a.q_ss | a.k_sb | a.k_sh | a.k_ss | a.v_sb | a.v_sh | a.v_ss;
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(a.q) | reinterpret_cast<uintptr_t>(a.k) | reinterpret_cast<uintptr_t>(a.v);
    return FLY_LOCAL_B16 && strides % 8 == 0 && ptrs % 16 == 0;
}

#ifndef FLY_LOCAL_BWD_QB
#define FLY_LOCAL_BWD_QB 1
#endif
template <typename T, int E, bool KEYMAJOR, int QB>
static int launch_local_bwd_as(const LocalBwdArgs& a, hipStream_t st) {
    auto kern = local_bwd_b16_kernel<T, E, KEYMAJOR, QB>;
    constexpr size_t smem = local_bwd_smem<E>();
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "local_bwd_b16")) return rc;
    const Machine& mach = machine();
    const int rows = KEYMAJOR ? a.S : a.T;
    const long items = (long)a.B * a.H * ((rows + 64 * QB - 1) / (64 * QB));
    const long grid = (items + mach.xcds - 1) / mach.xcds * mach.xcds;
    if (grid > 2147483647L) return fail(ERR_ARG, "local_bwd: too many workgroups");
    LocalBwdArgs args = a;
    args.n_xcd = mach.xcds;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), smem, st, args);
    return check_launch("local_bwd_b16_kernel");
}
template <typename T, int E>
static int launch_local_bwd(const LocalBwdArgs& a, hipStream_t st) {
    // (query-major first: it leaves delta for the key-major launch)
    if (int rc = launch_local_bwd_as<T, E, false, FLY_LOCAL_BWD_QB>(a, st)) return rc;
    return launch_local_bwd_as<T, E, true, FLY_LOCAL_BWD_QB>(a, st);
}

template <typename T, int E>
static int launch_local(const LocalArgs& a, hipStream_t st) {
    auto kern = local_fwd_kernel<T, E, E>;
    constexpr size_t smem = sizeof(float) * 2 * TK * 2 * (E + 4);
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "local_fwd")) return rc;
    const Machine& mach = machine();
    const long items = (long)a.B * a.H * ((a.T + TQ - 1) / TQ);
    const long grid = (items + mach.xcds - 1) / mach.xcds * mach.xcds;
    if (grid > 2147483647L) return fail(ERR_ARG, "local_fwd: too many workgroups");
    LocalArgs args = a;
    args.n_xcd = mach.xcds;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), smem, st, args);
    return check_launch("local_fwd_kernel");
}

// ---------------------------------------------------------------------------------------
// band terms of the backward pass
// ---------------------------------------------------------------------------------------
// Inside the band a (query i, key s) pair carries  a = exp(t q_i.k_s - log Z_i),  kb = psi_i.phik_s
// (the low-rank weight, psi = Phi(q) scaled by 1/Z),  df = g_i.v_s - c_i  and  dm = a df.  The
// gradients need five band-limited sums of them:
//   over keys    : sum_s dm k_s (-> d q),  sum_s df phik_s                     (query-major pass)
//   over queries : sum_i dm q_i (-> d k),  sum_i df psi_i,  sum_i (a - kb) g_i (key-major pass)
// Both passes are one kernel: an "outer" side whose rows are owned by lanes (64 per workgroup, 16 per
// wave, operands in registers) meets 32-row tiles of the "inner" side staged through LDS, with the
// products formed transposed (rows = inner, columns = outer) exactly as in the forward kernel, so the
// pair weights leave the score MFMAs in the operand layout of the output MFMAs.
//   query-major: outer = (q, -, g), inner = (k, phik, v): s1 = K q, s3 = V g;
//                out1 = t K^T dm, out2 = phik^T df
//   key-major  : outer = (k, phik, v), inner = (q, psi, g): s1 = Q k, s2 = psi phik, s3 = G v;
//                out1 = t Q^T dm, out2 = psi^T df, out3 = G^T (a - kb)
// log Z and c belong to the query: lane-owned in the query-major pass, staged with the tile (two
// extra LDS rows) in the key-major pass.  All tensors are fp32, contiguous (batch*head, rows, width).
struct BwdArgs {
    const float* x1; const float* x2; const float* x3;      // outer rows (x2 only key-major)
    const float* y1; const float* y2; const float* y3;      // inner rows
    const float* ln; const float* c;                        // per query: log Z, g.out
    const int64_t* lens;
    float* o1; float* o2; float* o3;                        // outer rows (o3 only key-major)
    int BH, H, T, S, lc;
    float temp;
    // finishing pass: global low-rank terms and the chain rule through the feature map in the epilogue
    const float* gmat; const float* gvec; const float* proj;
    int n_xcd;                      // dies the dispatcher deals workgroup ids to (set at launch)
    // dropout of the exact weights in the forward (drop_thresh != 0): with m = 0 on dropped pairs (the hash of
    // (seed, (b H + h) T + query, key), see drop_keep) and 1 / (1 - p) on kept ones, dm = a (m g.v - c) and the
    // weight of g in d v is m a - kb
    uint32_t drop_seed, drop_thresh; float drop_scale;
    // optional additive mask (T, S) of plain local attention, added to q.k before the temperature (see LocalArgs); a
    // query whose log Z entry is -inf had all its visible keys masked and weighs each of them 1 / local_context
    const float* add_mask;
};

//
// With FINISH the epilogue turns the sums into the gradients themselves.  The low-rank weight outside
// the band is "all keys minus the band", and the sums over all keys are products with small per-head
// matrices computed beforehand: gmat | gvec = K'^T V | sum K' for the query-major pass (K' = phik),
// Q'^T g | Q'^T c for the key-major pass (Q' = psi).  With x2 = the outer row's own features (psi
// resp. phik), u_f = x2_f (gmat_f . x3 - c gvec_f - out2_f) is the gradient with respect to the log of
// feature f (c = the query's g.out, resp. 1 for a key), and
//   d x1 = out1 + sqrt(t) P^T (u+ - u-) - t x1 sum_f u_f,    d v = out3 + gmat^T phik   (key-major)
// where features f < M/2 are the exp(+.) half and f + M/2 their exp(-.) partners.  o1 (and o3)
// receive the gradients; o2 is not written.
template <int E, int M, bool KEYMAJOR, bool FINISH>
__global__ __launch_bounds__(NT) void sblocal_bwd_band_kernel(BwdArgs a) {
    constexpr int D = E, LDK = E + 4, LDV = D + 4, LDF = M + 4;
    constexpr int EC = E / 16, FC = M / 16, DB = D / 16, KB = TK / 16;
    constexpr int STAGE = TK * (LDK + LDV + LDF) + 2 * TK;      // floats per LDS stage (+ log Z and c of the tile)
    constexpr float LOG2E = 1.4426950408889634f;
    extern __shared__ __attribute__((aligned(128))) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int Lo = KEYMAJOR ? a.S : a.T, Li = KEYMAJOR ? a.T : a.S;
    const int n_ot = (Lo + TQ - 1) / TQ;
    const int n_items = a.BH * n_ot;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // see sblocal_fwd_kernel
    if (item >= n_items) return;                       // workgroup-uniform
    const int ot = item % n_ot, bh = item / n_ot, b = bh / a.H;
    const int o0 = ot * TQ, ow0 = o0 + 16 * w, o = ow0 + r16;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi
    // the same band seen from the outer row: lo <= n - o < hi
    const int lo = KEYMAJOR ? -(lc_hi - 1) : -lc_lo, hi = KEYMAJOR ? lc_lo + 1 : lc_hi;
    const int o_limit = KEYMAJOR ? len : a.T, n_limit = KEYMAJOR ? a.T : len;
    const bool ovalid = o < o_limit;

    const float* y1 = a.y1 + (long)bh * Li * E;
    const float* y2 = a.y2 + (long)bh * Li * M;
    const float* y3 = a.y3 + (long)bh * Li * D;
    const float* lnp = a.ln + (long)bh * a.T;
    const float* cp = a.c + (long)bh * a.T;

    // inner tiles this workgroup meets
    const int o_last = min(o0 + TQ - 1, o_limit - 1);
    const int n_lo = max(0, o0 + lo), n_hi = min(n_limit, o_last + hi);
    const int kt_lo = n_lo / TK;
    const int kt_hi = (o_last >= o0 && n_hi > n_lo) ? (n_hi + TK - 1) / TK : kt_lo;

    RowTile<TK, E> r1;
    RowTile<TK, M> r2;
    RowTile<TK, D> r3;
    float rs = 0.f;                                   // key-major: log Z (threads 0..31) / c (32..63) of the tile
    auto fetch = [&](int kt) __attribute__((always_inline)) {
        r1.fetch(y1, E, kt * TK, Li - 1, tid);
        r2.fetch(y2, M, kt * TK, Li - 1, tid);
        r3.fetch(y3, D, kt * TK, Li - 1, tid);
        if (KEYMAJOR && tid < 2 * TK) {
            const int row = min(kt * TK + (tid & (TK - 1)), Li - 1);
            rs = tid < TK ? lnp[row] * LOG2E : cp[row];
        }
    };
    auto stash = [&](int buf) __attribute__((always_inline)) {
        float* st = smem + buf * STAGE;
        r1.template stash<LDK>(st, tid);
        r3.template stash<LDV>(st + TK * LDK, tid);
        r2.template stash<LDF>(st + TK * (LDK + LDV), tid);
        if (KEYMAJOR && tid < 2 * TK) st[TK * (LDK + LDV + LDF) + tid] = rs;
    };
    if (kt_lo < kt_hi) fetch(kt_lo);

    // outer operands (B side: column = outer row, k = 16c + 4g + j); exponents are base 2
    const int orow = min(o, Lo - 1);
    floatx4 x1[EC], x3[DB], x2[(KEYMAJOR || FINISH) ? FC : 1];
#pragma unroll
    for (int c = 0; c < EC; ++c)
        x1[c] = load4_f32(a.x1 + ((long)bh * Lo + orow) * E + 16 * c + 4 * g) * (a.temp * LOG2E);
#pragma unroll
    for (int c = 0; c < DB; ++c) x3[c] = load4_f32(a.x3 + ((long)bh * Lo + orow) * D + 16 * c + 4 * g);
    if (KEYMAJOR || FINISH) {
#pragma unroll
        for (int c = 0; c < FC; ++c) x2[c] = load4_f32(a.x2 + ((long)bh * Lo + orow) * M + 16 * c + 4 * g);
    }
    const float ln_o = KEYMAJOR ? 0.f : lnp[orow] * LOG2E, c_o = KEYMAJOR ? 0.f : cp[orow];
    // inner rows this lane's outer row may meet: nmin <= n < nmin + span
    const int nmin = max(o + lo, 0);
    const unsigned span = ovalid ? (unsigned)max(min(o + hi, n_limit) - nmin, 0) : 0u;
    const uint32_t drop_row = (!KEYMAJOR && a.drop_thresh != 0u) ? drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + o)) : 0u;

    floatx4 acc1[EC], acc2[FC], acc3[KEYMAJOR ? DB : 1];
#pragma unroll
    for (int c = 0; c < EC; ++c) acc1[c] = Frag<float>::zero();
#pragma unroll
    for (int c = 0; c < FC; ++c) acc2[c] = Frag<float>::zero();
#pragma unroll
    for (int c = 0; c < (KEYMAJOR ? DB : 1); ++c) acc3[c] = Frag<float>::zero();

    if (kt_lo < kt_hi) stash(0);
    __syncthreads();

    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        const int n_base = kt * TK;
        const int cur = (kt - kt_lo) & 1;
        const float* Y1s = smem + cur * STAGE;
        const float* Y3s = Y1s + TK * LDK;
        const float* Y2s = Y3s + TK * LDV;
        const float* Ss = Y2s + TK * LDF;
        const bool more = kt + 1 < kt_hi;
        if (more) fetch(kt + 1);                       // next tile's loads fly during the MFMAs

        // wave-uniform: does this tile meet the band of any of the wave's 16 outer rows?
        const bool any = !(n_base + TK - 1 - ow0 < lo || n_base - (ow0 + 15) >= hi || n_base >= n_limit || ow0 >= o_limit);
        if (any) {
            floatx4 s1[KB], s2[KB], s3[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) { s1[kb] = Frag<float>::zero(); s2[kb] = Frag<float>::zero(); s3[kb] = Frag<float>::zero(); }
#pragma unroll
            for (int c = 0; c < EC; ++c) {               // E == D: the two chains advance together
                floatx4 ya[KB], yc[KB];
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    ya[kb] = *reinterpret_cast<const floatx4*>(Y1s + (16 * kb + r16) * LDK + 4 * g + 16 * c);
                    yc[kb] = *reinterpret_cast<const floatx4*>(Y3s + (16 * kb + r16) * LDV + 4 * g + 16 * c);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb) {
                        s1[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ya[kb][j], x1[c][j], s1[kb], 0, 0, 0);
                        s3[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(yc[kb][j], x3[c][j], s3[kb], 0, 0, 0);
                    }
            }
            if (KEYMAJOR) {
#pragma unroll
                for (int c = 0; c < FC; ++c) {
                    floatx4 yb[KB];
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
                        yb[kb] = *reinterpret_cast<const floatx4*>(Y2s + (16 * kb + r16) * LDF + 4 * g + 16 * c);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int kb = 0; kb < KB; ++kb)
                            s2[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(yb[kb][j], x2[c][j], s2[kb], 0, 0, 0);
                }
            }
            // lane holds the pair (outer row o, inner row n_base + 16kb + 4g + i)
            floatx4 wdm[KB], wdf[KB], wak[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                floatx4 lnq, cq;
                if (KEYMAJOR) {
                    lnq = *reinterpret_cast<const floatx4*>(Ss + 16 * kb + 4 * g);
                    cq = *reinterpret_cast<const floatx4*>(Ss + TK + 16 * kb + 4 * g);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n_base + 16 * kb + 4 * g + i;
                    const bool ok = (unsigned)(n - nmin) < span;
                    float av = ok ? __builtin_amdgcn_exp2f(s1[kb][i] - (KEYMAJOR ? lnq[i] : ln_o)) : 0.f;
                    if (a.add_mask) {                        // (uniform)
                        const float lq = KEYMAJOR ? lnq[i] : ln_o;
                        const long at = KEYMAJOR ? (long)n * a.S + o : (long)o * a.S + n;
                        const float sm = ok ? s1[kb][i] + a.add_mask[at] * (a.temp * LOG2E) : 0.f;
                        av = !ok ? 0.f : lq == -INFINITY ? 1.0f / (float)a.lc : __builtin_amdgcn_exp2f(sm - lq);
                    }
                    const float df = ok ? s3[kb][i] - (KEYMAJOR ? cq[i] : c_o) : 0.f;
                    wdf[kb][i] = df;
                    if (a.drop_thresh != 0u) {               // (uniform)
                        const uint32_t rh = KEYMAJOR ? drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + n)) : drop_row;
                        const float m = drop_keep(rh, (uint32_t)(KEYMAJOR ? o : n), a.drop_thresh) ? a.drop_scale : 0.f;
                        wdm[kb][i] = ok ? av * (m * s3[kb][i] - (KEYMAJOR ? cq[i] : c_o)) : 0.f;
                        wak[kb][i] = av * m - (ok ? s2[kb][i] : 0.f);
                    } else {
                        wdm[kb][i] = av * df;
                        wak[kb][i] = av - (ok ? s2[kb][i] : 0.f);
                    }
                }
            }
            // out^T[col][outer] += sum_inner Y[inner][col] w[inner][outer]
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int row = 16 * kb + 4 * g + i;
#pragma unroll
                    for (int c = 0; c < EC; ++c)
                        acc1[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(Y1s[row * LDK + 16 * c + r16], wdm[kb][i], acc1[c], 0, 0, 0);
#pragma unroll
                    for (int c = 0; c < FC; ++c)
                        acc2[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(Y2s[row * LDF + 16 * c + r16], wdf[kb][i], acc2[c], 0, 0, 0);
                    if (KEYMAJOR) {
#pragma unroll
                        for (int c = 0; c < DB; ++c)
                            acc3[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(Y3s[row * LDV + 16 * c + r16], wak[kb][i], acc3[c], 0, 0, 0);
                    }
                }
        }
        if (more) stash(cur ^ 1);
        __syncthreads();
    }

    if (FINISH) {
        // per-head matrices into the tile stages (dead now; the loop ended on a barrier)
        constexpr int MH = M / 2;
        float* GMs = smem;                          // gmat (M, D), rows of LDV
        float* GVs = GMs + M * LDV;                 // gvec (M)
        float* Ps = GVs + M;                        // projection (M/2, E), rows of LDK
        static_assert(M * LDV + M + MH * LDK <= 2 * STAGE, "epilogue operands must fit the tile stages");
        {
            RowTile<M, D> gm;
            gm.fetch(a.gmat + (long)bh * M * D, D, 0, M - 1, tid);
            RowTile<MH, E> pt;
            pt.fetch(a.proj, E, 0, MH - 1, tid);
            if (tid < M) GVs[tid] = a.gvec[(long)bh * M + tid];
            gm.template stash<LDV>(GMs, tid);
            pt.template stash<LDK>(Ps, tid);
        }
        __syncthreads();
        // u^T[f][outer] = sum_d gmat[f][d] x3[d][outer]
        floatx4 u[FC];
#pragma unroll
        for (int c = 0; c < FC; ++c) u[c] = Frag<float>::zero();
#pragma unroll
        for (int cd = 0; cd < DB; ++cd) {
            floatx4 ga[FC];
#pragma unroll
            for (int c = 0; c < FC; ++c) ga[c] = *reinterpret_cast<const floatx4*>(GMs + (16 * c + r16) * LDV + 16 * cd + 4 * g);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int c = 0; c < FC; ++c) u[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(ga[c][j], x3[cd][j], u[c], 0, 0, 0);
        }
        const float cmul = KEYMAJOR ? 1.0f : c_o;
        float usum = 0.f;
#pragma unroll
        for (int c = 0; c < FC; ++c) {
            const floatx4 gv = *reinterpret_cast<const floatx4*>(GVs + 16 * c + 4 * g);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                u[c][i] = x2[c][i] * (u[c][i] - cmul * gv[i] - acc2[c][i]);
                usum += u[c][i];
            }
        }
        usum = group_sum(usum);
        // chain rule through the projection: dp^T[e][outer] = sum_r P[r][e] (u_r - u_{r + M/2})
        floatx4 dp[EC];
#pragma unroll
        for (int c = 0; c < EC; ++c) dp[c] = Frag<float>::zero();
#pragma unroll
        for (int c = 0; c < FC / 2; ++c) {
            const floatx4 du = u[c] - u[c + FC / 2];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int eb = 0; eb < EC; ++eb)
                    dp[eb] = __builtin_amdgcn_mfma_f32_16x16x4f32(Ps[(16 * c + 4 * g + j) * LDK + 16 * eb + r16], du[j], dp[eb], 0, 0, 0);
        }
        if (KEYMAJOR) {
            // d v^T[d][key] += sum_f gmat[f][d] phik[f][key]
#pragma unroll
            for (int c = 0; c < FC; ++c)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        acc3[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(GMs[(16 * c + 4 * g + j) * LDV + 16 * db + r16], x2[c][j], acc3[db], 0, 0, 0);
        }
        if (o < Lo) {
            const float st = sqrtf(a.temp), back = 1.0f / LOG2E;     // x1 carries t log2(e)
            float* p1 = a.o1 + ((long)bh * Lo + o) * E;
#pragma unroll
            for (int c = 0; c < EC; ++c) store4_f32(p1 + 16 * c + 4 * g, acc1[c] * a.temp + dp[c] * st - x1[c] * (back * usum));
            if (KEYMAJOR) {
                float* p3 = a.o3 + ((long)bh * Lo + o) * D;
#pragma unroll
                for (int c = 0; c < DB; ++c) store4_f32(p3 + 16 * c + 4 * g, acc3[c]);
            }
        }
        return;
    }
    if (o < Lo) {
        float* p1 = a.o1 + ((long)bh * Lo + o) * E;
        float* p2 = a.o2 + ((long)bh * Lo + o) * M;
#pragma unroll
        for (int c = 0; c < EC; ++c) store4_f32(p1 + 16 * c + 4 * g, acc1[c] * a.temp);
#pragma unroll
        for (int c = 0; c < FC; ++c) store4_f32(p2 + 16 * c + 4 * g, acc2[c]);
        if (KEYMAJOR) {
            float* p3 = a.o3 + ((long)bh * Lo + o) * D;
#pragma unroll
            for (int c = 0; c < DB; ++c) store4_f32(p3 + 16 * c + 4 * g, acc3[c]);
        }
    }
}

template <int E, int M, bool KEYMAJOR, bool FINISH>
static int launch_bwd_band(const BwdArgs& a, hipStream_t st) {
    auto kern = sblocal_bwd_band_kernel<E, M, KEYMAJOR, FINISH>;
    constexpr size_t smem = sizeof(float) * 2 * (TK * (3 * 4 + 2 * E + M) + 2 * TK);
    static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "sblocal_bwd_band")) return rc;
    const Machine& mach = machine();
    const long items = (long)a.BH * (((KEYMAJOR ? a.S : a.T) + TQ - 1) / TQ);
    const long grid = (items + mach.xcds - 1) / mach.xcds * mach.xcds;
    if (grid > 2147483647L) return fail(ERR_ARG, "sblocal_bwd_band: too many workgroups");
    BwdArgs args = a;
    args.n_xcd = mach.xcds;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), smem, st, args);
    return check_launch("sblocal_bwd_band_kernel");
}

template <int E, int M>
static int launch_bwd_band_both(const BwdArgs& a, bool key_major, hipStream_t st) {
    if (a.gmat)
        return key_major ? launch_bwd_band<E, M, true, true>(a, st) : launch_bwd_band<E, M, false, true>(a, st);
    return key_major ? launch_bwd_band<E, M, true, false>(a, st) : launch_bwd_band<E, M, false, false>(a, st);
}

#define SB_DISPATCH_M(FN, T, EE, ARGS)                                       \
    switch (m) {                                                              \
        case 32: return FN<T, EE, 32>(ARGS, st);                              \
        case 64: return FN<T, EE, 64>(ARGS, st);                              \
        case 128: return FN<T, EE, 128>(ARGS, st);                            \
        case 256: return FN<T, EE, 256>(ARGS, st);                            \
        default: return fail(ERR_UNSUPPORTED, "feature count m=%d not in {32,64,128,256}", m); \
    }
#define SB_DISPATCH_E(FN, T, ARGS)                                            \
    switch (E) {                                                              \
        case 32: SB_DISPATCH_M(FN, T, 32, ARGS)                               \
        case 64: SB_DISPATCH_M(FN, T, 64, ARGS)                               \
        case 128: SB_DISPATCH_M(FN, T, 128, ARGS)                             \
        default: return fail(ERR_UNSUPPORTED, "head dim E=%d not in {32,64,128}", E); \
    }

static int dispatch_kfeat(int dtype, int E, int m, const KvArgs& a, hipStream_t st) {
    if (dtype == F32) { SB_DISPATCH_E(launch_kfeat, float, a) }
    if (dtype == BF16) { SB_DISPATCH_E(launch_kfeat, bf16_t, a) }
    return fail(ERR_UNSUPPORTED, "sblocal supports float32 and bfloat16, got dtype code %d", dtype);
}
static int dispatch_fwd(int dtype, int E, int m, const FwdArgs& a, hipStream_t st) {
    if (dtype == F32) { SB_DISPATCH_E(launch_fwd, float, a) }
    if (dtype == BF16) { SB_DISPATCH_E(launch_fwd, bf16_t, a) }
    return fail(ERR_UNSUPPORTED, "sblocal supports float32 and bfloat16, got dtype code %d", dtype);
}

// number of parts the band of every query tile is split into: enough workgroups for two per CU
// on small problems, one part (no partials, no merge) once the grid fills the chip by itself
static int plan_parts(int B, int H, int T, int S, int lc) {
    const long tiles = (long)B * H * ((T + TQ - 1) / TQ);
    long band = (long)lc + TQ;
    if (band > S) band = S;
    const int key_tiles = (int)((band + TK - 1) / TK);
    long want = machine().slots / tiles;                 // never more than two workgroups per CU
    if (want > 8) want = 8;
    if (want > key_tiles / 2) want = key_tiles / 2;      // at least two key tiles per part
    return want < 1 ? 1 : (int)want;
}

// workgroups of the key pass that a compute unit holds together: the fp32 pass that writes the bf16 operand images
// (sb_kfeat_x3_kernel: more than 256 registers a lane and 108 KB of LDS) runs one, the others two
static int key_pass_wgs_per_cu(int dtype, int E, int mh) { return (dtype == F32 && E <= 64 && 2 * mh <= 128) ? 1 : 2; }

static int plan(int B, int H, int S, int wgs_per_cu, int* n_chunks, int* n_split) {
    const int nc = (S + CH - 1) / CH;
    // aim for about four workgroups per CU over the chip, at least one chunk each
    const long slots = machine().slots;
    long want = (2 * slots + (long)B * H - 1) / ((long)B * H);
    if (want < 1) want = 1;
    if (want > nc) want = nc;
    int per = (nc + (int)want - 1) / (int)want;
    const long resident = (long)machine().cus * wgs_per_cu;
    if ((long)B * H * nc > resident) {
        // more work than one residency round: the pass takes about rounds x chunks per workgroup, and a round that
        // is full costs no more than one that is not; among equals the larger share wins (fewer partial reductions
        // to combine)
        long best = -1;
        for (int p = 1; p <= nc; ++p) {
            const long wgs = (long)B * H * ((nc + p - 1) / p);
            const long cost = ((wgs + resident - 1) / resident) * p;
            if (best < 0 || cost <= best) { best = cost; per = p; }
        }
    }
    *n_chunks = nc;
    *n_split = (nc + per - 1) / per;
    return OK;
}

}  // namespace flyhip

using namespace flyhip;

#ifdef FLY_PROFILE
extern "C" int flyhip_prof_reset(void) {
    hipDeviceSynchronize();
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_prof)) != hipSuccess) return -1;
    if (hipMemset(p, 0, sizeof(long long) * 16384 * 8) != hipSuccess) return -1;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_prof_k)) != hipSuccess) return -1;
    if (hipMemset(p, 0, sizeof(long long) * 4096 * 8) != hipSuccess) return -1;
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}
extern "C" int flyhip_prof_read_k(long long* dst, int n_workgroups) {
    hipDeviceSynchronize();
    hipError_t e = hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_prof_k), sizeof(long long) * 8 * n_workgroups);
    return e == hipSuccess ? 0 : -1;
}
extern "C" int flyhip_prof_read2(long long* dst, int n_workgroups) {
    hipDeviceSynchronize();
    hipError_t e = hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_prof2), sizeof(long long) * 16 * n_workgroups);
    return e == hipSuccess ? 0 : -1;
}
extern "C" int flyhip_prof_read(long long* dst, int n_workgroups) {
    hipDeviceSynchronize();
    hipError_t e = hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_prof), sizeof(long long) * 8 * n_workgroups);
    return e == hipSuccess ? 0 : -1;
}
#endif

extern "C" int flyhip_sb_time_next_fwd(void* event_before, void* event_after) {
    g_ev_before = reinterpret_cast<hipEvent_t>(event_before);
    g_ev_after = reinterpret_cast<hipEvent_t>(event_after);
    return OK;
}

extern "C" int flyhip_sb_plan(int B, int H, int T, int S, int local_context,
                              int* n_chunks, int* n_split, int* n_parts) {
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0 && local_context > 0 && n_chunks && n_split && n_parts,
                "sb_plan: bad arguments");
    *n_parts = plan_parts(B, H, T, S, local_context);
    return plan(B, H, S, 2, n_chunks, n_split);
}

extern "C" int flyhip_sb_plan_for(int B, int H, int T, int S, int local_context, int E, int mh, int dtype,
                                  int* n_chunks, int* n_split, int* n_parts) {
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0 && local_context > 0 && E > 0 && mh > 0 && n_chunks && n_split && n_parts,
                "sb_plan_for: bad arguments");
    *n_parts = plan_parts(B, H, T, S, local_context);
    return plan(B, H, S, key_pass_wgs_per_cu(dtype, E, mh), n_chunks, n_split);
}

static int check_sb_dims(const char* who, int E, int D, int mh, int mh_valid, int dtype,
                         int64_t s0, int64_t s1, int64_t s2) {
    FLY_REQUIRE(E == D, "%s: padded head dims must be equal (E=%d, D=%d)", who, E, D);
    FLY_REQUIRE(mh_valid >= 1 && mh_valid <= mh, "%s: mh_valid=%d outside [1, mh=%d]", who, mh_valid, mh);
    const int64_t gran = dtype == BF16 ? 8 : 4;
    FLY_REQUIRE((s0 % gran) == 0 && (s1 % gran) == 0 && (s2 % gran) == 0,
                "%s: strides must be multiples of %d elements (16-byte vector access)", who, (int)gran);
    return OK;
}

extern "C" int flyhip_sb_kv_reduce(const void* k, const void* v, const float* proj, const int64_t* key_lengths,
                                   void* kfeat, float* chunk_scale, float* kv_part, float* part_max,
                                   float* kv, float* ksum, float* kmax,
                                   const void* q, float* qfeat, float* q_lsq, int T,
                                   int64_t q_sb, int64_t q_sh, int64_t q_ss, void* vt, void* kvt,
                                   int B, int H, int S, int E, int D, int mh, int mh_valid, int n_split,
                                   int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                   int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                   float softmax_temp, int dtype, void* stream) {
    FLY_REQUIRE(k && v && proj && kfeat && chunk_scale && kv_part && part_max && kv && ksum && kmax,
                "sb_kv_reduce: null pointer");
    FLY_REQUIRE(B > 0 && H > 0 && S > 0, "sb_kv_reduce: empty problem B=%d H=%d S=%d", B, H, S);
    FLY_REQUIRE(softmax_temp > 0.f, "sb_kv_reduce: softmax_temp must be positive");
    // (float32 with operand images: bits 8..15 of dtype name the element type of q, k, v in memory, see flyhip_sbblocksparse_fwd)
    const int in_code = (dtype >> 8) & 0xff;
    dtype &= 0xff;
    FLY_REQUIRE(in_code >= 0 && in_code <= 2 && (in_code == 0 || (dtype == F32 && vt)), "sb_kv_reduce: 2-byte tensors (code %d) go with float32 arithmetic on operand images", in_code);
    int rc = check_sb_dims("sb_kv_reduce", E, D, mh, mh_valid, dtype, k_sb | k_sh, k_ss, v_sb | v_sh | v_ss);
    if (rc) return rc;
    int nc, ns;
    plan(B, H, S, 2, &nc, &ns);
    FLY_REQUIRE(n_split >= 1 && n_split <= nc && n_split <= MAX_SPLIT,
                "sb_kv_reduce: n_split=%d outside [1, min(%d, %d)]", n_split, nc, MAX_SPLIT);
    FLY_REQUIRE((long)B * H <= 65535, "sb_kv_reduce: B*H=%ld exceeds the grid limit 65535", (long)B * H);
    FLY_REQUIRE(dtype != BF16 || (vt && kvt), "sb_kv_reduce: bfloat16 inputs need the vt and kvt scratch");
    if (dtype != BF16) kvt = nullptr;           // (float inputs: vt, when given, receives the operand images)
    if (q) {
        FLY_REQUIRE(qfeat && q_lsq && T > 0, "sb_kv_reduce: query features asked for without qfeat / q_lsq / T");
        FLY_REQUIRE(((q_sb | q_sh | q_ss) % 4) == 0, "sb_kv_reduce: q strides must be multiples of 4 elements");
    }
    KvArgs a{k, v, proj, key_lengths, kfeat, chunk_scale, kv_part, part_max,
             B, H, S, mh_valid, nc, n_split, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, softmax_temp,
             q, qfeat, q_lsq, q ? T : 0, q_sb, q_sh, q_ss,
             q ? (T + TQ - 1) / TQ : 0, vt};
    a.in_code = in_code;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    const int m = 2 * mh;
    rc = dispatch_kfeat(dtype, E, m, a, st);
    if (rc || q) return rc;          // with query features asked for (several parts per query tile) the
                                     // partial reductions are combined inside flyhip_sblocal_fwd's launch
    const int per = m * (D + 1);
    hipLaunchKernelGGL(sb_combine_kernel, dim3((per / 4 + NT - 1) / NT, B * H), dim3(NT), 0, st,
                       kv_part, part_max, kv, ksum, kmax, reinterpret_cast<uint16_t*>(kvt), n_split, m, D);
    return check_launch("sb_combine_kernel");
}

static int sblocal_fwd_checked(const void* q, const void* k, const void* v, const float* proj,
                                  const void* kfeat, const float* chunk_scale,
                                  float* kv, float* ksum, float* kmax,
                                  const float* qfeat, const float* q_lsq, const void* vt, const void* kvt,
                                  const float* kv_part, const float* part_max, int n_split,
                                  const int64_t* key_lengths, void* out, float* log_norm,
                                  float* part_ws, int n_parts,
                                  int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                                  int local_context,
                                  int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                  int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                  int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                  int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                  float softmax_temp, int dtype, void* stream, DropArgs drop = DropArgs{0, 0, 1.f}) {
    FLY_REQUIRE(q && k && v && proj && kfeat && chunk_scale && kv && ksum && kmax && out && log_norm,
                "sblocal_fwd: null pointer");
    // (float32 with operand images: bits 8..15 of dtype name the element type of q and out in memory, see flyhip_sbblocksparse_fwd)
    const int io_code = (dtype >> 8) & 0xff;
    dtype &= 0xff;
    FLY_REQUIRE(io_code == 0 || (io_code == 2 && dtype == F32 && vt), "sblocal_fwd: 2-byte tensors (code %d) are float16 with float32 arithmetic on operand images", io_code);
    // dropout lives in the band kernel on bf16 pieces (float inputs with the key pass's tile images)
    FLY_REQUIRE(drop.thresh == 0 || (dtype == F32 && vt && E <= 64 && 2 * mh <= 128),
                "sblocal_fwd: dropout is implemented for float32 inputs with head dims up to 64 and up to 128 features "
                "(the kernels on bf16 pieces)");
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0, "sblocal_fwd: empty problem");
    FLY_REQUIRE(local_context >= 1, "sblocal_fwd: local_context must be >= 1");
    FLY_REQUIRE(softmax_temp > 0.f, "sblocal_fwd: softmax_temp must be positive");
    int rc = check_sb_dims("sblocal_fwd", E, D, mh, mh_valid, dtype, q_sb | q_sh | q_ss | k_sb | k_sh | k_ss,
                           v_sb | v_sh | v_ss, o_sb | o_sh | o_ss);
    if (rc) return rc;
    FLY_REQUIRE((long)B * H <= 65535, "sblocal_fwd: B*H=%ld exceeds the grid limit 65535", (long)B * H);
    FLY_REQUIRE(n_parts >= 1 && n_parts <= 64, "sblocal_fwd: n_parts=%d outside [1, 64]", n_parts);
    FLY_REQUIRE(dtype != BF16 || (vt && kvt), "sblocal_fwd: bfloat16 inputs need the vt and kvt scratch of the key pass");
    FLY_REQUIRE(n_parts == 1 || (part_ws && qfeat && q_lsq && kv_part && part_max && n_split >= 1 && n_split <= MAX_SPLIT),
                "sblocal_fwd: n_parts > 1 needs the partial workspace, the query features and the partial "
                "reductions (kv_part, part_max, n_split) of the key pass");
    int nc, ns;
    plan(B, H, S, 2, &nc, &ns);
    FwdArgs a{q, k, v, proj, kfeat, chunk_scale, kv, ksum, kmax, qfeat, q_lsq, vt, kvt, kv_part, part_max, n_split, 0, 1, key_lengths, out, log_norm, part_ws,
              B, H, T, S, mh_valid, local_context, nc, n_parts,
              q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss, softmax_temp,
              nullptr, nullptr, nullptr};
    a.drop_seed = drop.seed; a.drop_thresh = drop.thresh; a.drop_scale = drop.scale;
    a.io_code = io_code;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    return dispatch_fwd(dtype, E, 2 * mh, a, st);
}

extern "C" int flyhip_sblocal_fwd(const void* q, const void* k, const void* v, const float* proj,
                                  const void* kfeat, const float* chunk_scale,
                                  float* kv, float* ksum, float* kmax,
                                  const float* qfeat, const float* q_lsq, const void* vt, const void* kvt,
                                  const float* kv_part, const float* part_max, int n_split,
                                  const int64_t* key_lengths, void* out, float* log_norm,
                                  float* part_ws, int n_parts,
                                  int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                                  int local_context,
                                  int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                  int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                  int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                  int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                  float softmax_temp, int dtype, void* stream) {
    return sblocal_fwd_checked(q, k, v, proj, kfeat, chunk_scale, kv, ksum, kmax, qfeat, q_lsq, vt, kvt, kv_part, part_max,
                               n_split, key_lengths, out, log_norm, part_ws, n_parts, B, H, T, S, E, D, mh, mh_valid,
                               local_context, q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss,
                               softmax_temp, dtype, stream);
}

// ---------------------------------------------------------------------------------------
// the whole forward on one caller-provided workspace
// ---------------------------------------------------------------------------------------
namespace {
struct SbWorkspace {
    size_t kfeat, chunk_scale, kv_part, part_max, kv, ksum, kmax, vt, kvt, part_ws, qfeat, q_lsq, total;
    int n_chunks, n_split, n_parts;
};
// Every piece starts at a multiple of 256 bytes.  E: padded head dim (= D), mh: padded projection rows.
SbWorkspace sb_workspace(int B, int H, int T, int S, int E, int mh, int local_context, int dtype, bool exact_fp32) {
    SbWorkspace w{};
    // (the fp32-pipe key pass, like the bf16 one, keeps two workgroups per compute unit resident)
    plan(B, H, S, exact_fp32 ? 2 : key_pass_wgs_per_cu(dtype, E, mh), &w.n_chunks, &w.n_split);
    w.n_parts = plan_parts(B, H, T, S, local_context);
    const size_t bh = (size_t)B * H, nc = w.n_chunks, ns = w.n_split, m = 2 * (size_t)mh, n_qt = (T + TQ - 1) / TQ;
    const size_t esize = dtype == F32 ? 4 : 2;
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t at = off; off += (bytes + 255) / 256 * 256; return at; };
    w.kfeat = take(bh * nc * CH * m * esize);
    w.chunk_scale = take(bh * nc * 4);
    w.kv_part = take(bh * ns * m * (E + 1) * 4);
    w.part_max = take(bh * ns * 4);
    w.kv = take(bh * m * E * 4);
    w.ksum = take(bh * m * 4);
    w.kmax = take(bh * 4);
    w.vt = take(dtype == F32 ? bh * nc * 2 * (128 * (size_t)E + 64 * (size_t)X3_VP * (size_t)E) : bh * nc * CH * E * 2);
    w.kvt = take(dtype == F32 ? 0 : bh * E * m * 2 * 2);      // two bf16 pieces
    w.part_ws = take(w.n_parts > 1 ? bh * n_qt * w.n_parts * TQ * (E + NSTAT) * 4 : 0);
    w.qfeat = take(w.n_parts > 1 ? bh * T * m * 4 : 0);
    w.q_lsq = take(w.n_parts > 1 ? bh * T * 4 : 0);
    w.total = off;
    return w;
}
}  // namespace

// flags of flyhip_sblocal_forward / flyhip_sb_workspace_bytes
constexpr int SB_EXACT_FP32 = 1;

extern "C" int64_t flyhip_sb_workspace_bytes(int B, int H, int T, int S, int E, int mh, int local_context, int dtype, int flags) {
    if (B <= 0 || H <= 0 || T <= 0 || S <= 0 || E <= 0 || mh <= 0 || local_context <= 0 || (dtype != F32 && dtype != BF16)) return -1;
    if (flags & ~SB_EXACT_FP32) return -1;
    return (int64_t)sb_workspace(B, H, T, S, E, mh, local_context, dtype, dtype == F32 && (flags & SB_EXACT_FP32)).total;
}

extern "C" int flyhip_sblocal_forward(const void* q, const void* k, const void* v, const float* proj,
                                      const int64_t* key_lengths, void* out, float* log_norm,
                                      void* workspace, int64_t workspace_bytes,
                                      int B, int H, int T, int S, int E, int D, int mh, int mh_valid, int local_context,
                                      int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                      int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                      int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                      int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                      float softmax_temp, int dtype, int flags,
                                      float dropout_p, uint64_t dropout_seed, void* stream) {
    FLY_REQUIRE(q && k && v && proj && out && log_norm && workspace, "sblocal_forward: null pointer");
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "sblocal_forward: dropout probability %g outside [0, 1)", (double)dropout_p);
    FLY_REQUIRE(dropout_p == 0.f || !(flags & SB_EXACT_FP32), "sblocal_forward: dropout is not implemented on the fp32-pipe kernels");
    FLY_REQUIRE((flags & ~SB_EXACT_FP32) == 0, "sblocal_forward: unknown flags 0x%x", flags);
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0 && local_context >= 1, "sblocal_forward: empty problem");
    // (float32 on operand images: bits 8..15 of dtype = 2 for float16 q, k, v and out, widened as they are loaded, rounded as stored)
    const int io_bits = dtype & 0xff00;
    dtype &= 0xff;
    FLY_REQUIRE(io_bits == 0 || (io_bits == (2 << 8) && dtype == F32 && !(flags & SB_EXACT_FP32)),
                "sblocal_forward: 2-byte tensors are float16 with float32 arithmetic on operand images (dtype 0x%x)", dtype | io_bits);
    FLY_REQUIRE(dtype == F32 || dtype == BF16, "sblocal_forward supports float32 and bfloat16, got dtype code %d", dtype);
    FLY_REQUIRE(E == D && E > 0 && mh > 0, "sblocal_forward: padded head dims must be equal (E=%d, D=%d)", E, D);
    FLY_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "sblocal_forward: the workspace must be aligned to 256 bytes");
    // float inputs: products on the bf16 matrix pipe from operands in bf16 pieces (the key pass leaves tile images in
    // `vt`), unless the caller asks for the fp32 matrix pipe throughout (no images: vt stays unused)
    const bool exact_fp32 = dtype == F32 && (flags & SB_EXACT_FP32);
    const SbWorkspace w = sb_workspace(B, H, T, S, E, mh, local_context, dtype, exact_fp32);
    FLY_REQUIRE(workspace_bytes >= (int64_t)w.total, "sblocal_forward: the workspace holds %lld bytes, this problem needs %lld "
                "(flyhip_sb_workspace_bytes)", (long long)workspace_bytes, (long long)w.total);
    char* ws = reinterpret_cast<char*>(workspace);
    auto f = [&](size_t at) { return reinterpret_cast<float*>(ws + at); };
    const bool split = w.n_parts > 1;
    void* vt = exact_fp32 ? nullptr : ws + w.vt;
    void* kvt = dtype == BF16 ? ws + w.kvt : nullptr;
    int rc = flyhip_sb_kv_reduce(k, v, proj, key_lengths, ws + w.kfeat, f(w.chunk_scale), f(w.kv_part), f(w.part_max),
                                 f(w.kv), f(w.ksum), f(w.kmax),
                                 split ? q : nullptr, split ? f(w.qfeat) : nullptr, split ? f(w.q_lsq) : nullptr, T,
                                 q_sb, q_sh, q_ss, vt, kvt, B, H, S, E, D, mh, mh_valid, w.n_split,
                                 k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, softmax_temp, dtype | io_bits, stream);
    if (rc) return rc;
    return sblocal_fwd_checked(q, k, v, proj, ws + w.kfeat, f(w.chunk_scale), f(w.kv), f(w.ksum), f(w.kmax),
                               split ? f(w.qfeat) : nullptr, split ? f(w.q_lsq) : nullptr, vt, kvt,
                               f(w.kv_part), f(w.part_max), w.n_split, key_lengths, out, log_norm,
                               split ? f(w.part_ws) : nullptr, w.n_parts, B, H, T, S, E, D, mh, mh_valid, local_context,
                               q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss,
                               softmax_temp, dtype | io_bits, stream, drop_args(dropout_p, dropout_seed));
}

// ---------------------------------------------------------------------------------------
// flyhip_sblocal_fwd for callers that cannot allocate
// ---------------------------------------------------------------------------------------
// The un-normalised partial outputs of the band kernel (one per part of a query tile) live in a
// fixed array inside the library's code object instead of a caller-provided workspace.  Every GPU
// the library runs on holds its own copy of the array for the life of the process.
constexpr size_t STATIC_SCRATCH_FLOATS = (size_t)4 << 20;                  // 16 MiB
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

// The array's address on each device, resolved once per device on first use.  In host code the
// array's name is only a handle for hipGetSymbolAddress, never an address a kernel may receive.
constexpr int MAX_DEVICES = 64;
static std::atomic<float*> g_scratch_ptr[MAX_DEVICES];

static int static_scratch(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(ERR_LAUNCH, "sblocal_fwd_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(ERR_UNSUPPORTED, "sblocal_fwd_static: device index %d outside [0, %d)", dev, MAX_DEVICES);
    float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        // (two threads racing here resolve the same address; the second store is harmless)
        void* sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !sym)
            return fail(ERR_LAUNCH, "sblocal_fwd_static: hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        p = reinterpret_cast<float*>(sym);
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return OK;
}

extern "C" int flyhip_sblocal_fwd_static(const void* q, const void* k, const void* v, const float* proj,
                                         const void* kfeat, const float* chunk_scale,
                                         float* kv, float* ksum, float* kmax,
                                         const float* qfeat, const float* q_lsq, const void* vt, const void* kvt,
                                         const float* kv_part, const float* part_max, int n_split,
                                         const int64_t* key_lengths, void* out, float* log_norm,
                                         int n_parts,
                                         int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                                         int local_context,
                                         int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                         int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                         int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                         int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                         float softmax_temp, int dtype, void* stream) {
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && D > 0, "sblocal_fwd_static: empty problem");
    FLY_REQUIRE(n_parts >= 1 && n_parts <= 64, "sblocal_fwd_static: n_parts=%d outside [1, 64]", n_parts);
    float* ws = nullptr;
    if (n_parts > 1) {
        // the partials of flyhip_sblocal_fwd's part_ws: every part writes all 64 rows of its tile and its
        // five statistics before the merge kernel reads them, so nothing has to start at zero
        const size_t need = (size_t)B * H * ((T + TQ - 1) / TQ) * n_parts * TQ * (size_t)(D + NSTAT);
        FLY_REQUIRE(need <= STATIC_SCRATCH_FLOATS,
                    "sblocal_fwd_static: the partial outputs of this problem need %zu floats, the built-in scratch "
                    "holds %zu (B*H*ceil(T/64)*n_parts*64*(D+5) must not exceed it); use flyhip_sblocal_fwd with a "
                    "caller-allocated part_ws", need, STATIC_SCRATCH_FLOATS);
        int rc = static_scratch(&ws);
        if (rc) return rc;
    }
    return flyhip_sblocal_fwd(q, k, v, proj, kfeat, chunk_scale, kv, ksum, kmax, qfeat, q_lsq, vt, kvt, kv_part, part_max,
                              n_split, key_lengths, out, log_norm, ws, n_parts, B, H, T, S, E, D, mh, mh_valid,
                              local_context, q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss,
                              softmax_temp, dtype, stream);
}

extern "C" int flyhip_sbblocksparse_fwd(const void* q, const void* k, const void* v, const float* proj,
                                        const void* kfeat, const void* vt, const float* chunk_scale,
                                        const float* kv, const float* ksum, const float* kmax,
                                        const int32_t* tl_ptr, const int32_t* tl_inner, const int32_t* tl_blk,
                                        const int32_t* tl_order, const int32_t* tl_heavy, int n_heavy, int heavy_parts,
                                        float* part_ws, float* qfeat, void* out, float* log_norm,
                                        int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                                        int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                        int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                        int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                        int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                        float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed, void* stream) {
    FLY_REQUIRE(q && k && v && proj && kfeat && chunk_scale && kv && ksum && kmax && tl_ptr && tl_inner && tl_blk &&
                out && log_norm, "sbblocksparse_fwd: null pointer");
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "sbblocksparse_fwd: dropout_p %g not in [0, 1)", (double)dropout_p);
    FLY_REQUIRE((long)B * H * T <= 4294967295L, "sbblocksparse_fwd: more than 2^32 query rows");
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0, "sbblocksparse_fwd: empty problem");
    FLY_REQUIRE(T % 16 == 0 && S % 16 == 0, "sbblocksparse_fwd: sequence lengths %d, %d must be multiples of 16", T, S);
    FLY_REQUIRE(softmax_temp > 0.f, "sbblocksparse_fwd: softmax_temp must be positive");
    // dtype: float32, optionally with the element type of q, k, v and out in memory in bits 8..15 (FLYHIP_IO_BF16 /
    // FLYHIP_IO_F16: the kernels on operand images widen what they load and round what they store)
    const int io_code = (dtype >> 8) & 0xff;
    dtype &= 0xff;
    FLY_REQUIRE(dtype == F32, "sbblocksparse_fwd: float32 arithmetic only (got dtype code %d)", dtype);
    FLY_REQUIRE(io_code >= 0 && io_code <= 2 && (io_code == 0 || vt), "sbblocksparse_fwd: 2-byte tensors (code %d) need the operand images", io_code);
    int rc = check_sb_dims("sbblocksparse_fwd", E, D, mh, mh_valid, dtype, q_sb | q_sh | q_ss | k_sb | k_sh | k_ss,
                           v_sb | v_sh | v_ss, o_sb | o_sh | o_ss);
    if (rc) return rc;
    int nc, ns;
    plan(B, H, S, 2, &nc, &ns);
    FLY_REQUIRE(n_heavy >= 0 && (n_heavy == 0 || (tl_heavy && tl_order && part_ws && qfeat && heavy_parts >= 2 && heavy_parts <= 64)),
                "sbblocksparse_fwd: long lists need tl_heavy, tl_order (with the long tiles marked), part_ws, qfeat and "
                "2 <= heavy_parts <= 64");
    FwdArgs a{q, k, v, proj, kfeat, chunk_scale, kv, ksum, kmax, qfeat, nullptr, vt, nullptr, nullptr, nullptr, 0, 0, 1,
              nullptr, out, log_norm, part_ws,
              B, H, T, S, mh_valid, 1, nc, n_heavy > 0 ? heavy_parts : 1,
              q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss, softmax_temp,
              tl_ptr, tl_inner, tl_blk, tl_order, tl_heavy, n_heavy};
    const DropArgs drop = drop_args(dropout_p, dropout_seed);
    a.drop_seed = drop.seed; a.drop_thresh = drop.thresh; a.drop_scale = drop.scale;
    a.io_code = io_code;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    const int m = 2 * mh;
    SB_DISPATCH_E(launch_fwd_list, float, a)
}

extern "C" int flyhip_local_fwd_dropout(const void* q, const void* k, const void* v, const int64_t* key_lengths, void* out,
                                    float* lse,
                                int B, int H, int T, int S, int E, int D, int local_context,
                                int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed, void* stream);
extern "C" int flyhip_sblocal_bwd_band_dropout(const float* x1, const float* x2, const float* x3,
                                       const float* y1, const float* y2, const float* y3,
                                       const float* log_norm, const float* c, const int64_t* key_lengths,
                                       float* o1, float* o2, float* o3,
                                       int BH, int H, int T, int S, int E, int M, int local_context,
                                       float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                       void* stream);

extern "C" int flyhip_local_fwd_lse(const void* q, const void* k, const void* v, const int64_t* key_lengths, void* out,
                                    float* lse,
                                int B, int H, int T, int S, int E, int D, int local_context,
                                int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                float softmax_temp, int dtype, void* stream) {
    return flyhip_local_fwd_dropout(q, k, v, key_lengths, out, lse, B, H, T, S, E, D, local_context,
                                    q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss,
                                    softmax_temp, dtype, 0.f, 0, stream);
}

extern "C" int flyhip_local_fwd_masked(const void* q, const void* k, const void* v, const int64_t* key_lengths,
                                       const float* attn_mask, void* out, float* lse,
                                       int B, int H, int T, int S, int E, int D, int local_context,
                                       int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                       int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                       int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                       int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                       float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed,
                                       void* stream);

extern "C" int flyhip_local_fwd_dropout(const void* q, const void* k, const void* v, const int64_t* key_lengths, void* out,
                                    float* lse,
                                int B, int H, int T, int S, int E, int D, int local_context,
                                int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed, void* stream) {
    return flyhip_local_fwd_masked(q, k, v, key_lengths, nullptr, out, lse, B, H, T, S, E, D, local_context,
                                   q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss,
                                   softmax_temp, dtype, dropout_p, dropout_seed, stream);
}

extern "C" int flyhip_local_fwd_masked(const void* q, const void* k, const void* v, const int64_t* key_lengths,
                                       const float* attn_mask, void* out, float* lse,
                                       int B, int H, int T, int S, int E, int D, int local_context,
                                       int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                       int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                       int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                       int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                       float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed,
                                       void* stream) {
    FLY_REQUIRE(q && k && v && out, "local_fwd: null pointer");
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "local_fwd: dropout_p %g not in [0, 1)", (double)dropout_p);
    FLY_REQUIRE((long)B * H * T <= 4294967295L, "local_fwd: more than 2^32 query rows");
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0, "local_fwd: empty problem");
    FLY_REQUIRE(local_context >= 1, "local_fwd: local_context must be >= 1");
    FLY_REQUIRE(softmax_temp > 0.f, "local_fwd: softmax_temp must be positive");
    FLY_REQUIRE(E == D, "local_fwd: padded head dims must be equal (E=%d, D=%d)", E, D);
    FLY_REQUIRE(((q_sb | q_sh | q_ss | k_sb | k_sh | k_ss | v_sb | v_sh | v_ss | o_sb | o_sh | o_ss) % 4) == 0,
                "local_fwd: strides must be multiples of 4 elements (16-byte vector access)");
    LocalArgs a{q, k, v, key_lengths, out, B, H, T, S, local_context,
                q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss, softmax_temp, lse};
    const DropArgs drop = drop_args(dropout_p, dropout_seed);
    a.drop_seed = drop.seed; a.drop_thresh = drop.thresh; a.drop_scale = drop.scale;
    a.add_mask = attn_mask;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
#define LOCAL_DISPATCH(TT)                                                                          \
    switch (E) {                                                                                    \
        case 32: return launch_local<TT, 32>(a, st);                                                \
        case 64: return launch_local<TT, 64>(a, st);                                                \
        case 128: return launch_local<TT, 128>(a, st);                                              \
        default: return fail(ERR_UNSUPPORTED, "local_fwd: head dim E=%d not in {32,64,128}", E);     \
    }
    if (dtype == F32) { LOCAL_DISPATCH(float) }
#define LOCAL_DISPATCH_B16(TT)                                                                      \
    switch (E) {                                                                                    \
        case 32: return launch_local_b16<TT, 32>(a, st);                                            \
        case 64: return launch_local_b16<TT, 64>(a, st);                                            \
        case 128: return launch_local_b16<TT, 128>(a, st);                                          \
        default: return fail(ERR_UNSUPPORTED, "local_fwd: head dim E=%d not in {32,64,128}", E);     \
    }
    if (dtype == BF16 && local_b16_ready(a)) { LOCAL_DISPATCH_B16(bf16_t) }
    if (dtype == BF16) { LOCAL_DISPATCH(bf16_t) }
    if (dtype == F16) {
        FLY_REQUIRE(local_b16_ready(a), "local_fwd: float16 rows must allow 16-byte loads (strides in multiples of 8 elements, aligned pointers)");
        LOCAL_DISPATCH_B16(f16_t)
    }
#undef LOCAL_DISPATCH
#undef LOCAL_DISPATCH_B16
    return fail(ERR_UNSUPPORTED, "local_fwd supports float32, bfloat16 and float16, got dtype code %d", dtype);
}

extern "C" int flyhip_local_bwd(const void* q, const void* k, const void* v, const void* out, const void* grad_out,
                               const float* lse, const int64_t* key_lengths, float* delta,
                               void* dq, void* dk, void* dv,
                               int B, int H, int T, int S, int E, int local_context,
                               int64_t q_sb, int64_t q_sh, int64_t q_ss,
                               int64_t k_sb, int64_t k_sh, int64_t k_ss,
                               int64_t v_sb, int64_t v_sh, int64_t v_ss,
                               int64_t o_sb, int64_t o_sh, int64_t o_ss,
                               int64_t g_sb, int64_t g_sh, int64_t g_ss,
                               int64_t dq_sb, int64_t dq_sh, int64_t dq_ss,
                               int64_t dk_sb, int64_t dk_sh, int64_t dk_ss,
                               int64_t dv_sb, int64_t dv_sh, int64_t dv_ss,
                               float softmax_temp, int dtype, void* stream) {
    FLY_REQUIRE(q && k && v && out && grad_out && lse && delta && dq && dk && dv, "local_bwd: null pointer");
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0, "local_bwd: empty problem");
    FLY_REQUIRE(local_context >= 1, "local_bwd: local_context must be >= 1");
    FLY_REQUIRE(softmax_temp > 0.f, "local_bwd: softmax_temp must be positive");
    FLY_REQUIRE(((q_sb | q_sh | q_ss | k_sb | k_sh | k_ss | v_sb | v_sh | v_ss | g_sb | g_sh | g_ss | o_sb | o_sh | o_ss) % 8) == 0,
                "local_bwd: input strides must be multiples of 8 elements (16-byte loads)");
    FLY_REQUIRE(((dq_sb | dq_sh | dq_ss | dk_sb | dk_sh | dk_ss | dv_sb | dv_sh | dv_ss) % 4) == 0,
                "local_bwd: output strides must be multiples of 4 elements (8-byte stores)");
    FLY_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                  reinterpret_cast<uintptr_t>(grad_out) | reinterpret_cast<uintptr_t>(out)) % 16) == 0 &&
                ((reinterpret_cast<uintptr_t>(dq) | reinterpret_cast<uintptr_t>(dk) | reinterpret_cast<uintptr_t>(dv)) % 8) == 0,
                "local_bwd: pointers must be 16-byte (inputs) and 8-byte (outputs) aligned");
    LocalBwdArgs a{q, k, v, grad_out, out, lse, delta, key_lengths, dq, dk, dv, B, H, T, S, local_context,
                   q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, g_sb, g_sh, g_ss, o_sb, o_sh, o_ss,
                   dq_sb, dq_sh, dq_ss, dk_sb, dk_sh, dk_ss, dv_sb, dv_sh, dv_ss, softmax_temp, 0};
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
#define LOCAL_BWD_DISPATCH(TT)                                                                      \
    switch (E) {                                                                                    \
        case 32: return launch_local_bwd<TT, 32>(a, st);                                            \
        case 64: return launch_local_bwd<TT, 64>(a, st);                                            \
        case 128: return launch_local_bwd<TT, 128>(a, st);                                          \
        default: return fail(ERR_UNSUPPORTED, "local_bwd: head dim E=%d not in {32,64,128}", E);     \
    }
    if (dtype == BF16) { LOCAL_BWD_DISPATCH(bf16_t) }
    if (dtype == F16) { LOCAL_BWD_DISPATCH(f16_t) }
#undef LOCAL_BWD_DISPATCH
    return fail(ERR_UNSUPPORTED, "local_bwd supports bfloat16 and float16, got dtype code %d", dtype);
}

extern "C" int flyhip_local_fwd(const void* q, const void* k, const void* v, const int64_t* key_lengths, void* out,
                                int B, int H, int T, int S, int E, int D, int local_context,
                                int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                float softmax_temp, int dtype, void* stream) {
    return flyhip_local_fwd_lse(q, k, v, key_lengths, out, nullptr, B, H, T, S, E, D, local_context,
                                q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss,
                                softmax_temp, dtype, stream);
}

static int dispatch_bwd_band(const BwdArgs& a, int E, int M, int key_major, void* stream);

extern "C" int flyhip_sblocal_bwd_band(const float* x1, const float* x2, const float* x3,
                                       const float* y1, const float* y2, const float* y3,
                                       const float* log_norm, const float* c, const int64_t* key_lengths,
                                       float* o1, float* o2, float* o3,
                                       int BH, int H, int T, int S, int E, int M, int local_context,
                                       float softmax_temp, int key_major, void* stream) {
    return flyhip_sblocal_bwd_band_dropout(x1, x2, x3, y1, y2, y3, log_norm, c, key_lengths, o1, o2, o3, BH, H, T, S, E, M,
                                           local_context, softmax_temp, key_major, 0.f, 0, stream);
}

extern "C" int flyhip_sblocal_bwd_band_masked(const float* x1, const float* x2, const float* x3,
                                       const float* y1, const float* y2, const float* y3,
                                       const float* log_norm, const float* c, const int64_t* key_lengths,
                                       const float* attn_mask,
                                       float* o1, float* o2, float* o3,
                                       int BH, int H, int T, int S, int E, int M, int local_context,
                                       float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                       void* stream);

extern "C" int flyhip_sblocal_bwd_band_dropout(const float* x1, const float* x2, const float* x3,
                                       const float* y1, const float* y2, const float* y3,
                                       const float* log_norm, const float* c, const int64_t* key_lengths,
                                       float* o1, float* o2, float* o3,
                                       int BH, int H, int T, int S, int E, int M, int local_context,
                                       float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                       void* stream) {
    return flyhip_sblocal_bwd_band_masked(x1, x2, x3, y1, y2, y3, log_norm, c, key_lengths, nullptr, o1, o2, o3,
                                          BH, H, T, S, E, M, local_context, softmax_temp, key_major, dropout_p,
                                          dropout_seed, stream);
}

extern "C" int flyhip_sblocal_bwd_band_masked(const float* x1, const float* x2, const float* x3,
                                       const float* y1, const float* y2, const float* y3,
                                       const float* log_norm, const float* c, const int64_t* key_lengths,
                                       const float* attn_mask,
                                       float* o1, float* o2, float* o3,
                                       int BH, int H, int T, int S, int E, int M, int local_context,
                                       float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                       void* stream) {
    FLY_REQUIRE(x1 && x3 && y1 && y2 && y3 && log_norm && c && o1 && o2, "sblocal_bwd_band: null pointer");
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "sblocal_bwd_band: dropout_p %g not in [0, 1)", (double)dropout_p);
    FLY_REQUIRE((long)BH * T <= 4294967295L, "sblocal_bwd_band: more than 2^32 query rows");
    FLY_REQUIRE(!key_major || (x2 && o3), "sblocal_bwd_band: the key-major pass needs x2 and o3");
    FLY_REQUIRE(BH > 0 && H > 0 && BH % H == 0 && T > 0 && S > 0, "sblocal_bwd_band: empty or inconsistent problem");
    FLY_REQUIRE(local_context >= 1, "sblocal_bwd_band: local_context must be >= 1");
    FLY_REQUIRE(softmax_temp > 0.f, "sblocal_bwd_band: softmax_temp must be positive");
    BwdArgs a{x1, x2, x3, y1, y2, y3, log_norm, c, key_lengths, o1, o2, o3, BH, H, T, S, local_context, softmax_temp,
              nullptr, nullptr, nullptr};
    const DropArgs drop = drop_args(dropout_p, dropout_seed);
    a.drop_seed = drop.seed; a.drop_thresh = drop.thresh; a.drop_scale = drop.scale;
    a.add_mask = attn_mask;
    return dispatch_bwd_band(a, E, M, key_major, stream);
}

extern "C" int flyhip_sblocal_bwd(const float* x1, const float* x2, const float* x3,
                                  const float* y1, const float* y2, const float* y3,
                                  const float* log_norm, const float* c, const int64_t* key_lengths,
                                  const float* gmat, const float* gvec, const float* proj,
                                  float* d1, float* d3,
                                  int BH, int H, int T, int S, int E, int M, int local_context,
                                  float softmax_temp, int key_major, void* stream) {
    FLY_REQUIRE(x1 && x2 && x3 && y1 && y2 && y3 && log_norm && c && gmat && gvec && proj && d1,
                "sblocal_bwd: null pointer");
    FLY_REQUIRE(!key_major || d3, "sblocal_bwd: the key-major pass needs d3");
    FLY_REQUIRE(BH > 0 && H > 0 && BH % H == 0 && T > 0 && S > 0, "sblocal_bwd: empty or inconsistent problem");
    FLY_REQUIRE(local_context >= 1, "sblocal_bwd: local_context must be >= 1");
    FLY_REQUIRE(softmax_temp > 0.f, "sblocal_bwd: softmax_temp must be positive");
    BwdArgs a{x1, x2, x3, y1, y2, y3, log_norm, c, key_lengths, d1, nullptr, d3, BH, H, T, S, local_context, softmax_temp,
              gmat, gvec, proj};
    return dispatch_bwd_band(a, E, M, key_major, stream);
}

static int dispatch_bwd_band(const BwdArgs& a, int E, int M, int key_major, void* stream) {
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    if (E == 32 && M == 32) return launch_bwd_band_both<32, 32>(a, key_major != 0, st);
    if (E == 32 && M == 64) return launch_bwd_band_both<32, 64>(a, key_major != 0, st);
    if (E == 64 && M == 32) return launch_bwd_band_both<64, 32>(a, key_major != 0, st);
    if (E == 64 && M == 64) return launch_bwd_band_both<64, 64>(a, key_major != 0, st);
    if (E == 64 && M == 128) return launch_bwd_band_both<64, 128>(a, key_major != 0, st);
    return fail(ERR_UNSUPPORTED, "sblocal_bwd_band: (head dim, features) = (%d, %d) not in "
                                 "{(32,32), (32,64), (64,32), (64,64), (64,128)}", E, M);
}
