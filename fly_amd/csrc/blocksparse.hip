// Block-sparse matmuls (SDD / DSD / DDS) and block-sparse row operations for gfx950.
//
// Sparse tensors are (Z, nnz, blk, blk) with block n the n-th nonzero of the (H, rows, cols)
// layout in row-major order.  Every matmul wave owns one register tile of the output (up to
// 32x32, built from 16x16 MFMA results) and walks its reduction list, reading operand fragments
// straight from global memory (16-byte / 8-byte vector loads when the contraction index is
// contiguous, strided gathers otherwise).  Products are formed with the operand that supplies
// the output columns on the MFMA "A" side, so a lane ends up with four consecutive output
// columns of one row and writes them with a single vector store.
#include "common.h"
#include <math.h>

namespace flyhip {

template <typename T>
__device__ __forceinline__ typename Frag<T>::type frag_at(const T* p, long k_stride) {
    // four contraction elements starting at p, spaced by k_stride
    if (k_stride == 1) return Frag<T>::load(p);
    return Frag<T>::gather(p, k_stride);
}

template <typename T>
__device__ __forceinline__ void store_tile_row(T* p, long col_stride, floatx4 v, int ncols_left) {
    // v holds four consecutive output columns starting at p
    if (col_stride == 1 && ncols_left >= 4) { store4_f32(p, v); return; }
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (i < ncols_left) p[i * col_stride] = Elem<T>::from_f32(v[i]);
}

// ---------------------------------------------------------------------------------------
// SDD: sparse = dense x dense^T
// ---------------------------------------------------------------------------------------
struct SddArgs {
    const void* a; const void* b; void* c; const int32_t* lut;
    int nnz, K;
    long a_sz, a_sh, a_sm, a_sk, b_sz, b_sh, b_sn, b_sk;
};

template <typename T, int BLK>
__global__ __launch_bounds__(256) void bs_sdd_kernel(SddArgs a) {
    constexpr int TILE = BLK >= 32 ? 32 : 16, NTL = TILE / 16, SUB = BLK / TILE;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    const long wid = (long)blockIdx.x * 4 + w;
    const int n = (int)(wid / (SUB * SUB)), sub = (int)(wid % (SUB * SUB));
    if (n >= a.nnz) return;
    const int z = blockIdx.y;
    const int head = a.lut[4 * n], bi = a.lut[4 * n + 1], bj = a.lut[4 * n + 2], id = a.lut[4 * n + 3];
    const int ml = (sub / SUB) * TILE, nl = (sub % SUB) * TILE;      // tile origin inside the block
    const T* ap = reinterpret_cast<const T*>(a.a) + z * a.a_sz + head * a.a_sh + (long)(bi * BLK + ml) * a.a_sm;
    const T* bp = reinterpret_cast<const T*>(a.b) + z * a.b_sz + head * a.b_sh + (long)(bj * BLK + nl) * a.b_sn;

    floatx4 acc[NTL][NTL];
#pragma unroll
    for (int tm = 0; tm < NTL; ++tm)
#pragma unroll
        for (int tn = 0; tn < NTL; ++tn) acc[tm][tn] = Frag<float>::zero();

    for (int kk = 0; kk < a.K; kk += 16) {
        typename Frag<T>::type fa[NTL], fb[NTL];
#pragma unroll
        for (int t = 0; t < NTL; ++t) {
            fa[t] = frag_at<T>(ap + (long)(16 * t + r16) * a.a_sm + (long)(kk + 4 * g) * a.a_sk, a.a_sk);
            fb[t] = frag_at<T>(bp + (long)(16 * t + r16) * a.b_sn + (long)(kk + 4 * g) * a.b_sk, a.b_sk);
        }
#pragma unroll
        for (int tm = 0; tm < NTL; ++tm)
#pragma unroll
            for (int tn = 0; tn < NTL; ++tn) acc[tm][tn] = Frag<T>::mma(fb[tn], fa[tm], acc[tm][tn]);
    }
    // lane holds C[m = 16tm + r16][n = 16tn + 4g + i]
    T* cp = reinterpret_cast<T*>(a.c) + ((long)z * a.nnz + id) * (BLK * BLK);
#pragma unroll
    for (int tm = 0; tm < NTL; ++tm)
#pragma unroll
        for (int tn = 0; tn < NTL; ++tn)
            store4_f32(cp + (ml + 16 * tm + r16) * BLK + nl + 16 * tn + 4 * g, acc[tm][tn]);
}

// Fast SDD for 32x32 blocks of a 2-byte type with contiguous contraction (K a multiple of 32, at
// most 128): one wave per (head, block-row).  The wave loads the A fragments of its block-row once
// (16-byte loads, kept in registers) and then produces the row's blocks one after the other: B fragments with 16-byte loads, 16x16x32 MFMAs, 8-byte stores of a 2 KiB block.
// The hardware hands consecutive workgroup ids to the XCDs in turn (n_xcd of them), and every XCD has an L2
// of its own.  unit_of() turns a 1-D workgroup id into (unit, position inside the unit) such
// that all `per_unit` workgroups of a unit -- one (batch, head) matrix, whose dense operand they
// all re-read -- run on one XCD, so that operand comes from HBM once instead of once per XCD.
__device__ __forceinline__ bool unit_of(unsigned id, int n_xcd, int per_unit, int n_units, int& unit, int& pos) {
    const unsigned xcd = id % (unsigned)n_xcd, slot = id / (unsigned)n_xcd;
    unit = (int)(slot / per_unit) * n_xcd + (int)xcd;
    pos = (int)(slot % per_unit);
    return unit < n_units;
}
static long unit_grid(long n_units, long per_unit) {
    const long x = machine().xcds;
    return (n_units + x - 1) / x * x * per_unit;
}

template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float lo, float hi) { return pack_bf16x2(lo, hi); }
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float lo, float hi) {
    const _Float16 l = (_Float16)lo, h = (_Float16)hi;
    return (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, h) << 16);
}
template <typename T> __device__ __forceinline__ floatx4 mma32(uintx4 a, uintx4 b, floatx4 c);
template <> __device__ __forceinline__ floatx4 mma32<bf16_t>(uintx4 a, uintx4 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ floatx4 mma32<f16_t>(uintx4 a, uintx4 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8_t, a), __builtin_bit_cast(halfx8_t, b), c, 0, 0, 0);
}

struct SddRowArgs {
    const void* a; const void* b; void* c;
    const int32_t* row_ptr; const int32_t* row_blk; const int32_t* row_col;
    int nnz, K, brows_per_head, n_heads, Z;
    long a_sz, a_sh, a_sm, b_sz, b_sh, b_sn;
    int n_xcd;          // dies the dispatcher deals workgroup ids to (set where the kernel is launched)
};

constexpr int SDD_RING = 3;

template <typename T, int KS>     // KS = K / 32
__global__ __launch_bounds__(256) void bs_sdd32_kernel(const SddRowArgs a) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    // one block-row per wave: the four waves of a workgroup walk neighbouring block-rows, whose
    // column lists mostly coincide, so their B-tile loads meet in the L1 cache
    int unit, grp;
    if (!unit_of(blockIdx.x, a.n_xcd, (a.brows_per_head + 3) / 4, a.n_heads * a.Z, unit, grp)) return;
    const int z = unit / a.n_heads, head = unit % a.n_heads, bi = grp * 4 + w;
    if (bi >= a.brows_per_head) return;
    const int brow = head * a.brows_per_head + bi;
    const int p0 = a.row_ptr[brow], nb = a.row_ptr[brow + 1] - p0;
    const T* ap = reinterpret_cast<const T*>(a.a) + z * a.a_sz + head * a.a_sh + (long)(bi * 32 + r16) * a.a_sm + 8 * g;
    // MFMA row i of B-tile tn is block column 8*(i/4) + 4*tn + i%4: the four results a lane gets from
    // tile 0 and the four from tile 1 are then eight consecutive columns -> one 16-byte store
    const T* bp = reinterpret_cast<const T*>(a.b) + z * a.b_sz + head * a.b_sh +
                  (long)(8 * (r16 >> 2) + (r16 & 3)) * a.b_sn + 8 * g;
    T* cz = reinterpret_cast<T*>(a.c) + (long)z * a.nnz * 1024;
    if (nb == 0) return;
    uint4 fa[2][KS];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fa[tm][ks] = *reinterpret_cast<const uint4*>(ap + 16 * tm * a.a_sm + 32 * ks);
    // B tiles travel through a ring of SDD_RING register sets: the loads of block j + SDD_RING - 1
    // are issued before block j is multiplied and stored, so a wave keeps several tiles in flight
    uint4 fb[SDD_RING][2][KS];
    auto fetch = [&](uint4 (&dst)[2][KS], int j) {
        const long brow_b = (long)a.row_col[p0 + min(j, nb - 1)] * 32;
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                dst[tn][ks] = *reinterpret_cast<const uint4*>(bp + (brow_b + 4 * tn) * a.b_sn + 32 * ks);
    };
#pragma unroll
    for (int u = 0; u < SDD_RING - 1; ++u) fetch(fb[u], u);
    for (int j0 = 0; j0 < nb; j0 += SDD_RING) {
#pragma unroll
        for (int u = 0; u < SDD_RING; ++u) {
            const int j = j0 + u;
            if (j >= nb) break;
            fetch(fb[(u + SDD_RING - 1) % SDD_RING], j + SDD_RING - 1);
            floatx4 acc[2][2];
#pragma unroll
            for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                for (int tn = 0; tn < 2; ++tn) {
                    acc[tm][tn] = Frag<float>::zero();
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) acc[tm][tn] = Frag32<T>::mma(fb[u][tn][ks], fa[tm][ks], acc[tm][tn]);
                }
            // lane holds C[m = 16tm + r16][n = 8g + 4tn + i]: rows of 64 bytes, 16 consecutive rows per store
            T* cp = cz + (long)a.row_blk[p0 + j] * 1024;
#pragma unroll
            for (int tm = 0; tm < 2; ++tm) store8_f32(cp + (16 * tm + r16) * 32 + 8 * g, acc[tm][0], acc[tm][1]);
        }
    }
}

// Operand of a 16x16x32 MFMA whose contraction index runs down the rows of a row-major LDS tile
// ([k][feature]): lane (r16, g) needs feature f0 + r16 at k = 8g .. 8g + 7.  ds_read_b64_tr_b16 hands a lane
// the element column of a 16-lane group's 16 x 4 block of 2-byte values: with lane j of the group
// pointing at some row (its choice) for k-slot j / 4, columns 4 (j % 4) .. + 3, lane j receives column j of the
// four rows.  Two such reads (k-slots 8g .. 8g + 3 and 8g + 4 .. 8g + 7) make the eight k-slots; row_lo /
// row_hi are the LDS rows that hold k = 8g + r16 / 4 and k = 8g + 4 + r16 / 4 (tiles may keep their rows
// in any order).
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uintx4 frag_down_rows_at(const uint16_t* tile, int ld, int f0, int r16, int row_lo, int row_hi) {
    typedef __attribute__((address_space(3))) shortx4 lds_shortx4;
    const uint16_t* p = tile + f0 + 4 * (r16 & 3);
    const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(p + row_lo * ld));
    const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(p + row_hi * ld));
    const uintx2 l = __builtin_bit_cast(uintx2, lo), h = __builtin_bit_cast(uintx2, hi);
    return uintx4{l[0], l[1], h[0], h[1]};
}
__device__ __forceinline__ uintx4 frag_down_rows(const uint16_t* tile, int ld, int f0, int r16, int g) {
    return frag_down_rows_at(tile, ld, f0, r16, 8 * g + (r16 >> 2), 8 * g + 4 + (r16 >> 2));
}

// SDD for layouts whose neighbouring block-rows share most of their columns (band and butterfly
// patterns do): one workgroup per (batch, head, four consecutive block-rows), wave w owning row
// 4*group + w with its A fragments in registers.  The workgroup walks the union of the four
// column lists (uni_inner), stages each 32 x K tile of B once in LDS -- a quarter of the cache
// traffic of the one-wave-per-row kernel -- and every wave whose row holds that column
// (uni_blk[step][w] >= 0) multiplies and stores its 2 KiB block.  Tiles are double-buffered:
// the global loads of step s+1 are in flight while step s is multiplied.
struct SddUniArgs {
    const void* a; const void* b; void* c;
    const int32_t* uni_ptr; const int32_t* uni_inner; const int32_t* uni_blk;
    int nnz, brows_per_head, grps_per_head, n_heads, Z;
    long a_sz, a_sh, a_sm, b_sz, b_sh, b_sn;
    // EPI 1: c = scale * p * (a b^T - delta[row]) on the nonzero blocks, the gradient of the scores of a
    // softmax(scale * s) -> p -> p v chain from a = d out, b = v, delta = rowsum(d out * out)
    // EPI 2: c = 2^(scale * a b^T - delta[row]): the probabilities again from a = q, b = k, scale =
    // softmax scale * log2(e) and delta = the rows' base-2 log-denominators of the one-kernel attention
    const void* p; const float* delta; float scale;
    // EPI 3: both at once from a = d out, b = v and a2 = q, b2 = k (strides as a, b): p2 = 2^(scale2 * a2 b2^T -
    // lse2[row]) is written to p2 and c = scale * p2 * (a b^T - delta[row])
    const void* a2; const void* b2; const float* lse2; void* p2; float scale2;
    long a2_sz, a2_sh, a2_sm, b2_sz, b2_sh, b2_sn;
    // ... and the gradient of a2 on the way: dq = c b2 (rows of a2), accumulated over the row's blocks
    void* dq; long dq_sz, dq_sh, dq_sm;
    // ... with delta formed here when `out` is given (delta may then be null): rowsum(a * out), out laid out like a
    const void* out; long o_sz, o_sh, o_sm;
    int n_xcd;          // dies the dispatcher deals workgroup ids to (set where the kernel is launched)
    // EPI 3 with DROP: the forward dropped probabilities by the hash of (seed, row = (z H + head) L + query, key)
    // (drop_keep): p2 is then written with the dropped ones zeroed and the kept ones scaled by 1 / (1 - p) -- the
    // operand of dV -- and c = scale * p * (m * (a b^T) - delta[row]) with m that 0 or 1 / (1 - p)
    uint32_t drop_seed, drop_thresh; float drop_scale;
};

template <typename T, int KS, int EPI = 0, bool DROP = false>     // KS = K / 32; EPI: 0 product, 1 softmax gradient, 2 probabilities
__global__ __launch_bounds__(256) void bs_sdd32u_kernel(const SddUniArgs a) {
    static_assert(!DROP || EPI == 3, "dropout belongs to the epilogue that forms the probabilities again");
    constexpr bool DSOFT = EPI == 1, PROB = EPI == 2, BOTH = EPI == 3;
    constexpr int K = 32 * KS, LD = K + 8;              // LDS row stride: 16 rows of a tile hit all banks once
    constexpr int CPR = K / 8;                          // 16-byte chunks per tile row
    constexpr int NCH = (32 * CPR + 255) / 256;         // chunks per thread
    __shared__ __attribute__((aligned(16))) uint16_t tile[2][32 * LD];
    __shared__ __attribute__((aligned(16))) uint16_t tile2[BOTH ? 2 : 1][BOTH ? 32 * LD : 8];
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    int unit, grp;
    if (!unit_of(blockIdx.x, a.n_xcd, a.grps_per_head, a.n_heads * a.Z, unit, grp)) return;
    const int z = unit / a.n_heads, head = unit % a.n_heads;
    const int ug = head * a.grps_per_head + grp;
    const int p0 = a.uni_ptr[ug], n = a.uni_ptr[ug + 1] - p0;
    const int bi = grp * 4 + w;
    const bool have_row = bi < a.brows_per_head;
    if (n == 0) {
        if (EPI == 3 && have_row) {                     // rows without blocks: zero gradient
            T* dqp = reinterpret_cast<T*>(a.dq) + z * a.dq_sz + head * a.dq_sh;
            for (int e = lane; e < 32 * K / 4; e += 64)
                store4_f32(dqp + (long)(bi * 32 + e / (K / 4)) * a.dq_sm + 4 * (e % (K / 4)), Frag<float>::zero());
        }
        return;
    }
    const T* ap = reinterpret_cast<const T*>(a.a) + z * a.a_sz + head * a.a_sh +
                  (long)(min(bi, a.brows_per_head - 1) * 32 + r16) * a.a_sm + 8 * g;
    const T* bz = reinterpret_cast<const T*>(a.b) + z * a.b_sz + head * a.b_sh;
    T* cz = reinterpret_cast<T*>(a.c) + (long)z * a.nnz * 1024;
    // DSOFT: this lane's rows are 16 tm + r16 of block-row bi
    const long rowvec_off = ((long)z * a.n_heads + head) * a.brows_per_head * 32 + (long)min(bi, a.brows_per_head - 1) * 32 + r16;
    const float* dlt = (DSOFT || PROB || (BOTH && a.delta)) ? a.delta + rowvec_off : nullptr;
    uintx4 fa[2][KS];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fa[tm][ks] = *reinterpret_cast<const uintx4*>(ap + 16 * tm * a.a_sm + 32 * ks);
    // EPI 3: the second product's row operand, column tiles and row vector
    uintx4 fa2[BOTH ? 2 : 1][BOTH ? KS : 1];
    const T* bz2 = nullptr;
    float lse_row[2] = {0.f, 0.f}, dl_row[2] = {0.f, 0.f};
    if (BOTH) {
        const T* ap2 = reinterpret_cast<const T*>(a.a2) + z * a.a2_sz + head * a.a2_sh +
                       (long)(min(bi, a.brows_per_head - 1) * 32 + r16) * a.a2_sm + 8 * g;
#pragma unroll
        for (int tm = 0; tm < 2; ++tm) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) fa2[BOTH ? tm : 0][BOTH ? ks : 0] = *reinterpret_cast<const uintx4*>(ap2 + 16 * tm * a.a2_sm + 32 * ks);
            lse_row[tm] = a.lse2[rowvec_off + 16 * tm];
            if (a.out) {
                // delta = sum over the head dim of d out * out for this lane's row: the lane holds 8 KS of the
                // row's values, the four lanes r16 + 16g the rest
                const T* op = reinterpret_cast<const T*>(a.out) + z * a.o_sz + head * a.o_sh +
                              (long)(min(bi, a.brows_per_head - 1) * 32 + 16 * tm + r16) * a.o_sm + 8 * g;
                float part = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const uintx4 ov = *reinterpret_cast<const uintx4*>(op + 32 * ks);
                    const uintx4 gv = fa[tm][ks];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        T x, y;
                        *reinterpret_cast<uint16_t*>(&x) = (uint16_t)(gv[e >> 1] >> (16 * (e & 1)));
                        *reinterpret_cast<uint16_t*>(&y) = (uint16_t)(ov[e >> 1] >> (16 * (e & 1)));
                        part += Elem<T>::to_f32(x) * Elem<T>::to_f32(y);
                    }
                }
                dl_row[tm] = group_sum(part);
            } else {
                dl_row[tm] = dlt[16 * tm];
            }
        }
        bz2 = reinterpret_cast<const T*>(a.b2) + z * a.b2_sz + head * a.b2_sh;
    }
    uint32_t drop_row[2] = {0u, 0u};
    if (DROP) {
        const uint32_t row0 = (uint32_t)rowvec_off;     // (z H + head) L + 32 bi + r16
        drop_row[0] = drop_row_hash(a.drop_seed, row0);
        drop_row[1] = drop_row_hash(a.drop_seed, row0 + 16u);
    }

    // staging: chunk c = tid + 256 i is 16 bytes of tile row c / CPR.  Block column n lands in LDS row
    // 16*((n>>2)&1) + 4*(n>>3) + (n&3), so that MFMA tile tn reads the 16 consecutive LDS rows
    // 16 tn .. 16 tn + 15 and its row i is block column 8*(i/4) + 4*tn + i%4: the four results a lane
    // gets from tile 0 and the four from tile 1 are eight consecutive columns -> one 16-byte store
    uintx4 reg[NCH], reg2[BOTH ? NCH : 1];
    auto fetch = [&](int inner) __attribute__((always_inline)) {
        const long brow_b = (long)inner * 32;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            if (c < 32 * CPR) reg[i] = *reinterpret_cast<const uintx4*>(bz + (brow_b + c / CPR) * a.b_sn + 8 * (c % CPR));
            if (BOTH && c < 32 * CPR)
                reg2[BOTH ? i : 0] = *reinterpret_cast<const uintx4*>(bz2 + (brow_b + c / CPR) * a.b2_sn + 8 * (c % CPR));
        }
    };
    auto stash = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i, nrow = c / CPR;
            const int lrow = 16 * ((nrow >> 2) & 1) + 4 * (nrow >> 3) + (nrow & 3);
            if (c < 32 * CPR) *reinterpret_cast<uintx4*>(&tile[buf][lrow * LD + 8 * (c % CPR)]) = reg[i];
            if (BOTH && c < 32 * CPR) *reinterpret_cast<uintx4*>(&tile2[BOTH ? buf : 0][lrow * LD + 8 * (c % CPR)]) = reg2[BOTH ? i : 0];
        }
    };
    floatx4 dqa[BOTH ? 2 * KS : 1][2];                  // dq^T[feature 16dt + 4g + i][row 16tm + r16]
    if (BOTH) {
#pragma unroll
        for (int dt = 0; dt < 2 * KS; ++dt) { dqa[BOTH ? dt : 0][0] = Frag<float>::zero(); dqa[BOTH ? dt : 0][1] = Frag<float>::zero(); }
    }
    // the index lists are read two steps (block-column) and one step (block id) ahead of their use
    int inner_n1 = n > 1 ? a.uni_inner[p0 + 1] : 0;
    int blk = a.uni_blk[(long)p0 * 4 + w];
    int inner_cur = a.uni_inner[p0];
    fetch(inner_cur);
    stash(0);
    drain_loads();
    __syncthreads();
    for (int s = 0; s < n; ++s) {
        const int inner_n2 = s + 2 < n ? a.uni_inner[p0 + s + 2] : 0;
        const int blk_n1 = s + 1 < n ? a.uni_blk[(long)(p0 + s + 1) * 4 + w] : -1;
        if (s + 1 < n) fetch(inner_n1);
        const bool mine = blk >= 0 && have_row;
        floatx4 acc[2][2], acc2[2][2];
        uintx4 pv[2];
        if (DSOFT && mine) {                              // requested before the products, used after them
            const T* pp = reinterpret_cast<const T*>(a.p) + ((long)z * a.nnz + blk) * 1024;
#pragma unroll
            for (int tm = 0; tm < 2; ++tm)
                pv[tm] = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(pp + (16 * tm + r16) * 32 + 8 * g));
        }
        if (mine) {
            const uint16_t* tp = tile[s & 1];
            uintx4 fb[2][KS];
#pragma unroll
            for (int tn = 0; tn < 2; ++tn)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    fb[tn][ks] = *reinterpret_cast<const uintx4*>(tp + (16 * tn + r16) * LD + 32 * ks + 8 * g);
#pragma unroll
            for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                for (int tn = 0; tn < 2; ++tn) {
                    acc[tm][tn] = Frag<float>::zero();
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) acc[tm][tn] = mma32<T>(fb[tn][ks], fa[tm][ks], acc[tm][tn]);
                }
            if (BOTH) {
                const uint16_t* tp2 = tile2[BOTH ? (s & 1) : 0];
#pragma unroll
                for (int tn = 0; tn < 2; ++tn)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        fb[tn][ks] = *reinterpret_cast<const uintx4*>(tp2 + (16 * tn + r16) * LD + 32 * ks + 8 * g);
#pragma unroll
                for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                    for (int tn = 0; tn < 2; ++tn) {
                        acc2[tm][tn] = Frag<float>::zero();
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks)
                            acc2[tm][tn] = mma32<T>(fb[tn][ks], fa2[BOTH ? tm : 0][BOTH ? ks : 0], acc2[tm][tn]);
                    }
            }
        }
        // the next tile goes to LDS before this step's stores are issued: the wait for its loads would
        // otherwise wait for the stores too (one counter covers both)
        if (s + 1 < n) stash((s + 1) & 1);
        if (mine) {
            // lane holds C[m = 16tm + r16][n = 8g + 4tn + i]
            T* cp = cz + (long)blk * 1024;
#pragma unroll
            for (int tm = 0; tm < 2; ++tm) {
                if (DSOFT) {
                    const float dl = dlt[16 * tm];
#pragma unroll
                    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint32_t word = pv[tm][2 * tn + (i >> 1)];
                            T e;
                            *reinterpret_cast<uint16_t*>(&e) = (i & 1) ? (uint16_t)(word >> 16) : (uint16_t)(word & 0xffffu);
                            acc[tm][tn][i] = a.scale * Elem<T>::to_f32(e) * (acc[tm][tn][i] - dl);
                        }
                }
                if (BOTH) {
#pragma unroll
                    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(acc2[tm][tn][i], a.scale2, -lse_row[tm]));
                            if (DROP) {
                                const uint32_t col = (uint32_t)inner_cur * 32u + 8u * g + 4u * tn + i;
                                const float m = drop_keep(drop_row[tm], col, a.drop_thresh) ? a.drop_scale : 0.f;
                                acc2[tm][tn][i] = m * pr;
                                acc[tm][tn][i] = a.scale * pr * (m * acc[tm][tn][i] - dl_row[tm]);
                            } else {
                                acc2[tm][tn][i] = pr;
                                acc[tm][tn][i] = a.scale * pr * (acc[tm][tn][i] - dl_row[tm]);
                            }
                        }
                    T* pp2 = reinterpret_cast<T*>(a.p2) + ((long)z * a.nnz + blk) * 1024;
                    store8_f32(pp2 + (16 * tm + r16) * 32 + 8 * g, acc2[tm][0], acc2[tm][1]);
                    // the lane's eight ds values are columns 8g .. 8g+7 of row 16tm + r16: an MFMA operand as they are
                    const uintx4 dsb = {pack2<T>(acc[tm][0][0], acc[tm][0][1]), pack2<T>(acc[tm][0][2], acc[tm][0][3]),
                                        pack2<T>(acc[tm][1][0], acc[tm][1][1]), pack2<T>(acc[tm][1][2], acc[tm][1][3])};
                    // ... against the b2 tile read down its rows (block column n sits in LDS row
                    // 16 ((n >> 2) & 1) + 4 (n >> 3) + (n & 3), see the staging)
                    const uint16_t* tt = tile2[BOTH ? (s & 1) : 0];
                    const int n_lo = 8 * g + (r16 >> 2), n_hi = n_lo + 4;
                    const int row_lo = 16 * ((n_lo >> 2) & 1) + 4 * (n_lo >> 3) + (n_lo & 3);
                    const int row_hi = 16 * ((n_hi >> 2) & 1) + 4 * (n_hi >> 3) + (n_hi & 3);
#pragma unroll
                    for (int dt = 0; dt < 2 * KS; ++dt) {
                        const uintx4 fk = frag_down_rows_at(tt, LD, 16 * dt, r16, row_lo, row_hi);
                        dqa[BOTH ? dt : 0][tm] = mma32<T>(fk, dsb, dqa[BOTH ? dt : 0][tm]);
                    }
                }
                if (PROB) {
                    const float dl = dlt[16 * tm];
#pragma unroll
                    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            acc[tm][tn][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[tm][tn][i], a.scale, -dl));
                }
                store8_f32(cp + (16 * tm + r16) * 32 + 8 * g, acc[tm][0], acc[tm][1]);
            }
        }
        inner_cur = inner_n1;
        inner_n1 = inner_n2;
        blk = blk_n1;
        __syncthreads();
    }
    if (BOTH && have_row) {
        T* dqp = reinterpret_cast<T*>(a.dq) + z * a.dq_sz + head * a.dq_sh;
#pragma unroll
        for (int tm = 0; tm < 2; ++tm)
#pragma unroll
            for (int dt = 0; dt < 2 * KS; ++dt)
                store4_f32(dqp + (long)(bi * 32 + 16 * tm + r16) * a.dq_sm + 16 * dt + 4 * g, dqa[BOTH ? dt : 0][tm]);
    }
}

// ---------------------------------------------------------------------------------------
// SDD with the contraction index slowest in both operands: sparse = A^T B, A (K x M), B (K x N)
// ---------------------------------------------------------------------------------------
// The weight gradient of a block-sparse linear layer: K = tokens (tens of thousands), M / N = output /
// input features, 32x32 blocks of a 2-byte type.  One workgroup per (group of <= 4 consecutive
// block-rows with identical column lists, chunk of <= 4 of their block-columns, slice of K): a
// 128 x 128 output tile, the 2 x 2 waves owning 64 x 64 each.  Per step of 32 tokens the 32 x 128
// tiles of A and B are loaded with 16-byte pieces along the features and kept row-major in LDS; the
// MFMA fragments, whose contraction index runs down the rows, are two transposing 8-byte LDS reads
// each (ds_read_b64_tr_b16), so nothing is transposed with 2-byte stores; the
// slices' partial blocks meet in an fp32 buffer through hardware float atomics (the caller zeroes
// it and rounds it to the output type afterwards).
struct SddKArgs {
    const void* a; const void* b; float* c32;
    const int32_t* seg_ptr; const int32_t* seg_blk; const int32_t* seg_inner;
    const int32_t* grp_row0; const int32_t* grp_n;
    int per_head, K, k_slice, chunks, nnz;
    long a_sz, a_sh, a_sk, b_sz, b_sh, b_sk;
};
constexpr int SDDK_LD = 144;    // LDS row stride in elements ([token][128 features + 16]: the four token rows a
                                // 16-lane group reads together start 32 bytes apart modulo 256)

template <typename T>
__global__ __launch_bounds__(256) void bs_sdd32k_kernel(const SddKArgs a) {
    constexpr int LD = SDDK_LD;
    __shared__ __attribute__((aligned(16))) uint16_t at[2][32 * LD];
    __shared__ __attribute__((aligned(16))) uint16_t bt[2][32 * LD];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int wm = w >> 1, wn = w & 1;
    const int grp = blockIdx.x / a.chunks, chunk = blockIdx.x % a.chunks, z = blockIdx.z;
    const int row0 = a.grp_row0[grp], gn = a.grp_n[grp];
    const int head = row0 / a.per_head, brow0 = row0 % a.per_head;
    const int p0 = a.seg_ptr[row0], nin = a.seg_ptr[row0 + 1] - p0;
    const int j0 = chunk * 4, jn = min(4, nin - j0);       // this chunk's block-columns: list entries j0 .. j0 + jn - 1
    if (jn <= 0) return;                                    // workgroup-uniform
    const int k0 = blockIdx.y * a.k_slice, k1 = min(a.K, k0 + a.k_slice);
    if (k0 >= k1) return;
    const uint16_t* ap = reinterpret_cast<const uint16_t*>(a.a) + z * a.a_sz + head * a.a_sh + (long)brow0 * 32;
    const uint16_t* bp = reinterpret_cast<const uint16_t*>(a.b) + z * a.b_sz + head * a.b_sh;

    // staging: piece c = tid + 256 i (i < 2) of each 32-token x 128-feature tile is token c / 16, features
    // 8 (c % 16) .. + 7: the tiles stay row-major ([token][feature]) in LDS, one 16-byte store per piece; the
    // MFMA fragments -- tokens are the contraction index -- come out of them through the transposing read.
    // Feature block (c % 16) / 4 is output block-row ob (A) or list entry j0 + jb (B); absent blocks read
    // block 0 of the tile and are zeroed when parked
    int fcol_a[2], fcol_b[2];                               // feature offset of the piece in its operand
    bool live_a[2], live_b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int c = tid + 256 * i, fb = (c & 15) >> 2, f8 = 8 * (c & 3);
        live_a[i] = fb < gn;
        live_b[i] = fb < jn;
        fcol_a[i] = 32 * (live_a[i] ? fb : 0) + f8;
        fcol_b[i] = a.seg_inner[p0 + j0 + (live_b[i] ? fb : 0)] * 32 + f8;
    }
    // two register sets: the loads of step s+2 are issued while step s is multiplied and are parked in LDS
    // one step later, so every global load has two steps to arrive (every fetch issues the same four
    // loads per thread on every path, so the wait for the older set can leave the newer one in flight)
    uintx4 ra0[2], rb0[2], ra1[2], rb1[2];
    auto fetch = [&](int kt, uintx4 (&ra)[2], uintx4 (&rb)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int tok = min(kt + ((tid + 256 * i) >> 4), a.K - 1);     // clamped; tokens past k1 are zeroed below
            ra[i] = *reinterpret_cast<const uintx4*>(ap + (long)tok * a.a_sk + fcol_a[i]);
            rb[i] = *reinterpret_cast<const uintx4*>(bp + (long)tok * a.b_sk + fcol_b[i]);
        }
    };
    auto stash = [&](int buf, int kt, const uintx4 (&ra)[2], const uintx4 (&rb)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + 256 * i, tok = c >> 4, f0 = 8 * (c & 15);
            const bool in = kt + tok < k1;
            *reinterpret_cast<uintx4*>(&at[buf][tok * LD + f0]) = (live_a[i] && in) ? ra[i] : uintx4{0, 0, 0, 0};
            *reinterpret_cast<uintx4*>(&bt[buf][tok * LD + f0]) = (live_b[i] && in) ? rb[i] : uintx4{0, 0, 0, 0};
        }
    };

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = Frag<float>::zero();
    const bool wave_active = 2 * wm < gn && 2 * wn < jn;    // its output blocks exist

    auto compute = [&](int buf) __attribute__((always_inline)) {
        if (wave_active) {
            uintx4 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                fa[i] = frag_down_rows(at[buf], LD, 64 * wm + 16 * i, r16, g);
                fb[i] = frag_down_rows(bt[buf], LD, 64 * wn + 16 * i, r16, g);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mma32<T>(fa[i], fb[j], acc[i][j]);
        }
    };
    fetch(k0, ra0, rb0);
    stash(0, k0, ra0, rb0);
    fetch(k0 + 32, ra1, rb1);                               // set 1 holds odd steps, set 0 even steps
    drain_loads_but<4>();                                   // only set 1 (four loads a thread) is in flight
    __syncthreads();
    for (int kt = k0; kt < k1; kt += 64) {
        fetch(kt + 64, ra0, rb0);                           // (past the slice: loaded, zeroed, never used)
        compute(0);
        stash(1, kt + 32, ra1, rb1);
        drain_loads_but<4>();                               // set 1 is parked: only set 0 is in flight
        __syncthreads();
        fetch(kt + 96, ra1, rb1);
        if (kt + 32 < k1) compute(1);
        stash(0, kt + 64, ra0, rb0);
        drain_loads_but<4>();
        __syncthreads();
    }
    if (!wave_active) return;
    // lane holds C[out = 64 wm + 16 i + 4 g + x][in = 64 wn + 16 j + r16]
    float* cz = a.c32 + (long)z * a.nnz * 1024;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ob = 2 * wm + (i >> 1);
        if (ob >= gn) continue;
        const int* blks = a.seg_blk + a.seg_ptr[row0 + ob] + j0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int jb = 2 * wn + (j >> 1);
            if (jb >= jn) continue;
            float* cb = cz + (long)blks[jb] * 1024 + (16 * (i & 1) + 4 * g) * 32 + 16 * (j & 1) + r16;
#pragma unroll
            for (int x = 0; x < 4; ++x) unsafeAtomicAdd(cb + 32 * x, acc[i][j][x]);
        }
    }
}

// ---------------------------------------------------------------------------------------
// DSD: dense = sparse x dense
// ---------------------------------------------------------------------------------------
struct DxdArgs {
    const void* sp; const void* dn; void* c;
    const int32_t* seg_ptr; const int32_t* seg_blk; const int32_t* seg_inner;
    int n_seg, per_head, X, trans;      // X = N (DSD: dense columns) or M (DDS: dense rows)
    long sp_sz;
    long dn_sz, dn_sh, dn_s0, dn_s1;    // DSD: (k, n) strides; DDS: (m, k) strides
    long c_sz, c_sh, c_sm, c_sn;
    int Z;
    int n_xcd;          // dies the dispatcher deals workgroup ids to (set where the kernel is launched)
};

template <typename T, int BLK>
__global__ __launch_bounds__(256) void bs_dsd_kernel(DxdArgs a) {
    constexpr int TILE = BLK >= 32 ? 32 : 16, NTL = TILE / 16, SUBM = BLK / TILE;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    const int ntn = (a.X + 31) / 32;
    const long wid = (long)blockIdx.x * 4 + w;
    const long per_seg = (long)SUBM * ntn;
    const int seg = (int)(wid / per_seg);
    if (seg >= a.n_seg) return;
    const int rem = (int)(wid % per_seg), subm = rem / ntn, nt = rem % ntn;
    const int z = blockIdx.y;
    const int head = seg / a.per_head, brow = seg % a.per_head;
    const int n0 = nt * 32;
    const T* spz = reinterpret_cast<const T*>(a.sp) + z * a.sp_sz;
    const T* dnp = reinterpret_cast<const T*>(a.dn) + z * a.dn_sz + head * a.dn_sh;

    floatx4 acc[NTL][2];
#pragma unroll
    for (int tm = 0; tm < NTL; ++tm) { acc[tm][0] = Frag<float>::zero(); acc[tm][1] = Frag<float>::zero(); }
    bool nok[2];
    nok[0] = n0 + r16 < a.X;
    nok[1] = n0 + 16 + r16 < a.X;

    const int p1 = a.seg_ptr[seg + 1];
    for (int p = a.seg_ptr[seg]; p < p1; ++p) {
        const T* blkp = spz + (long)a.seg_blk[p] * (BLK * BLK);
        const long krow0 = (long)a.seg_inner[p] * BLK;
#pragma unroll
        for (int kk = 0; kk < BLK; kk += 16) {
            typename Frag<T>::type fs[NTL], fd[2];
#pragma unroll
            for (int tm = 0; tm < NTL; ++tm) {
                const int m = subm * TILE + 16 * tm + r16;
                fs[tm] = a.trans ? Frag<T>::gather(blkp + (kk + 4 * g) * BLK + m, BLK)
                                 : Frag<T>::load(blkp + m * BLK + kk + 4 * g);
            }
#pragma unroll
            for (int tn = 0; tn < 2; ++tn) {
                fd[tn] = Frag<T>::zero();
                if (nok[tn])
                    fd[tn] = frag_at<T>(dnp + (krow0 + kk + 4 * g) * a.dn_s0 + (long)(n0 + 16 * tn + r16) * a.dn_s1, a.dn_s0);
            }
#pragma unroll
            for (int tm = 0; tm < NTL; ++tm) {
                acc[tm][0] = Frag<T>::mma(fd[0], fs[tm], acc[tm][0]);
                acc[tm][1] = Frag<T>::mma(fd[1], fs[tm], acc[tm][1]);
            }
        }
    }
    T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh;
#pragma unroll
    for (int tm = 0; tm < NTL; ++tm) {
        const long m = (long)brow * BLK + subm * TILE + 16 * tm + r16;
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) {
            const int n = n0 + 16 * tn + 4 * g;
            if (n < a.X) store_tile_row<T>(cp + m * a.c_sm + n * a.c_sn, a.c_sn, acc[tm][tn], a.X - n);
        }
    }
}

// Fast DSD for 32x32 blocks of a 2-byte type, dense operand with contiguous columns (the V of
// attention): one workgroup per (head, block-row, 64-column tile).  Wave w reduces the row's blocks
// w, w+4, ...: the sparse block supplies k-contiguous fragments straight from global memory; the
// 32 x 64 tile of the dense operand is staged in a wave-private LDS buffer (16-byte global loads)
// and read back column-wise, which is the transposition a [k][n] operand needs.  The four partial
// sums meet in LDS and leave as 16-byte stores.
constexpr int DSD_LD = 68;      // LDS row stride in elements: the four k-groups of a read hit distinct banks

template <typename T>
__global__ __launch_bounds__(256) void bs_dsd32_kernel(DxdArgs a) {
    __shared__ __attribute__((aligned(16))) uint16_t vt[4][32 * DSD_LD];
    __shared__ float part[4][32][64 + 1];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int ntn = (a.X + 63) / 64, n_heads = a.n_seg / a.per_head;
    int unit, pos;
    if (!unit_of(blockIdx.x, a.n_xcd, a.per_head * ntn, n_heads * a.Z, unit, pos)) return;
    const int z = unit / n_heads, head = unit % n_heads, brow = pos / ntn, n0 = (pos % ntn) * 64;
    const int seg = head * a.per_head + brow;
    const T* spz = reinterpret_cast<const T*>(a.sp) + z * a.sp_sz;
    const T* dnp = reinterpret_cast<const T*>(a.dn) + z * a.dn_sz + head * a.dn_sh;
    const int ncols = min(64, a.X - n0);            // valid columns of this tile (a multiple of 8)

    floatx4 acc[2][4];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) acc[tm][tn] = Frag<float>::zero();
    uint16_t* my = vt[w];
    const int p1 = a.seg_ptr[seg + 1];
    for (int p = a.seg_ptr[seg] + w; p < p1; p += 4) {
        const T* blkp = spz + (long)a.seg_blk[p] * 1024;
        const long krow0 = (long)a.seg_inner[p] * 32;
        // dense tile rows krow0..+31, columns n0..n0+63 -> LDS (lane: row 8*it + lane/8, 8 columns)
        uint4 stage[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int k = 8 * it + (lane >> 3), c8 = 8 * (lane & 7);
            stage[it] = make_uint4(0, 0, 0, 0);
            if (c8 < ncols) stage[it] = *reinterpret_cast<const uint4*>(dnp + (krow0 + k) * a.dn_s0 + n0 + c8);
        }
        uint4 fs[2];
#pragma unroll
        for (int tm = 0; tm < 2; ++tm) fs[tm] = *reinterpret_cast<const uint4*>(blkp + (16 * tm + r16) * 32 + 8 * g);
        __builtin_amdgcn_wave_barrier();            // previous iteration's LDS reads are done (in-order DS)
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int k = 8 * it + (lane >> 3), c8 = 8 * (lane & 7);
            uint2* dst = reinterpret_cast<uint2*>(my + k * DSD_LD + c8);
            dst[0] = make_uint2(stage[it].x, stage[it].y);
            dst[1] = make_uint2(stage[it].z, stage[it].w);
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) {
            // column n = 16tn + r16 of the tile, rows k = 8g..8g+7
            const uint16_t* src = my + (8 * g) * DSD_LD + 16 * tn + r16;
            uint4 fd;
            fd.x = (uint32_t)src[0] | ((uint32_t)src[DSD_LD] << 16);
            fd.y = (uint32_t)src[2 * DSD_LD] | ((uint32_t)src[3 * DSD_LD] << 16);
            fd.z = (uint32_t)src[4 * DSD_LD] | ((uint32_t)src[5 * DSD_LD] << 16);
            fd.w = (uint32_t)src[6 * DSD_LD] | ((uint32_t)src[7 * DSD_LD] << 16);
            acc[0][tn] = Frag32<T>::mma(fd, fs[0], acc[0][tn]);
            acc[1][tn] = Frag32<T>::mma(fd, fs[1], acc[1][tn]);
        }
    }
    // lane holds C[m = 16tm + r16][n = 16tn + 4g + i]; sum the four waves
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int tn = 0; tn < 4; ++tn)
#pragma unroll
            for (int i = 0; i < 4; ++i) part[w][16 * tm + r16][16 * tn + 4 * g + i] = acc[tm][tn][i];
    __syncthreads();
    const int m = tid >> 3, c8 = 8 * (tid & 7);
    if (c8 < ncols) {
        floatx4 lo, hi;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lo[i] = (part[0][m][c8 + i] + part[1][m][c8 + i]) + (part[2][m][c8 + i] + part[3][m][c8 + i]);
            hi[i] = (part[0][m][c8 + 4 + i] + part[1][m][c8 + 4 + i]) + (part[2][m][c8 + 4 + i] + part[3][m][c8 + 4 + i]);
        }
        T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh + ((long)brow * 32 + m) * a.c_sm + n0 + c8;
        store4_f32(cp, lo);
        store4_f32(cp + 4, hi);
    }
}

// DSD for layouts whose neighbouring block-rows share most of their columns: one workgroup per
// (batch, head, four consecutive block-rows, 64-column tile of the dense operand), wave w owning
// output rows of block-row 4*group + w -- no split of the reduction, so no partial sums to merge.
// The workgroup walks the union of the four column lists; each 32 x 64 tile of the dense operand
// is loaded once (16-byte global loads) and written to LDS transposed, [column][k], which turns the
// MFMA fragment of a [k][n] operand into one 16-byte LDS read.  Sparse blocks come straight from
// global memory, each read by exactly one wave.  Tiles and sparse fragments of step s+1 are in
// flight while step s is multiplied.
struct DsdUniArgs {
    const void* sp; const void* dn; void* c;
    const int32_t* uni_ptr; const int32_t* uni_inner; const int32_t* uni_blk;
    int per_head, grps_per_head, n_heads, Z, N;
    long sp_sz, dn_sz, dn_sh, dn_sk, c_sz, c_sh, c_sm;
    int n_xcd;          // dies the dispatcher deals workgroup ids to (set where the kernel is launched)
};
constexpr int DSDU_LD = 40;     // LDS row stride in elements ([column][k], 32 k + 8): 16 columns hit all banks once

template <typename T, bool TA>     // TA: every sparse block is used transposed (segments are block-columns of the layout)
__global__ __launch_bounds__(256) void bs_dsd32u_kernel(const DsdUniArgs a) {
    __shared__ __attribute__((aligned(16))) uint16_t vt[2][64 * DSDU_LD];
    // TA: a wave turns its 32x32 block through a private LDS tile, [column][row]
    __shared__ __attribute__((aligned(16))) uint16_t bt[TA ? 4 : 1][TA ? 32 * DSDU_LD : 8];
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ntn = (a.N + 63) / 64;
    int unit, pos;
    if (!unit_of(blockIdx.x, a.n_xcd, a.grps_per_head * ntn, a.n_heads * a.Z, unit, pos)) return;
    const int z = unit / a.n_heads, head = unit % a.n_heads, grp = pos / ntn, n0 = (pos % ntn) * 64;
    const int ug = head * a.grps_per_head + grp;
    const int p0 = a.uni_ptr[ug], n = a.uni_ptr[ug + 1] - p0;
    const int bi = grp * 4 + w;
    const bool have_row = bi < a.per_head;
    const int ncols = min(64, a.N - n0);            // valid columns of this tile (a multiple of 8)
    const T* spz = reinterpret_cast<const T*>(a.sp) + z * a.sp_sz;
    const T* dnp = reinterpret_cast<const T*>(a.dn) + z * a.dn_sz + head * a.dn_sh + n0;

    floatx4 acc[2][4];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) acc[tm][tn] = Frag<float>::zero();

    // staging: thread holds dense row k = tid / 8, columns c8 .. c8 + 7.  Column n lands in LDS row
    // 32*(n>>5) + 16*((n>>2)&1) + 4*((n>>3)&3) + (n&3): MFMA tile tn reads LDS rows 16 tn .. 16 tn + 15
    // and its row i is column 32*(tn/2) + 8*(i/4) + 4*(tn%2) + i%4, so tiles 2q and 2q+1 give a lane
    // eight consecutive output columns.
    const int sk = tid >> 3, c8 = 8 * (tid & 7);
    uint4 stage, fs[2], fs_next[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
    int blk_next = -1;
    auto fetch = [&](int inner, int blk_id) {
        const long krow0 = (long)inner * 32;
        stage = make_uint4(0, 0, 0, 0);
        if (c8 < ncols) stage = *reinterpret_cast<const uint4*>(dnp + (krow0 + sk) * a.dn_sk + c8);
        blk_next = have_row ? blk_id : -1;
        if (blk_next >= 0) {
            const T* blkp = spz + (long)blk_next * 1024;
#pragma unroll
            for (int tm = 0; tm < 2; ++tm) {
                // every sparse block is read by exactly one wave: nontemporal
                const uintx4 t_ = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(blkp + (16 * tm + r16) * 32 + 8 * g));
                fs_next[tm] = make_uint4(t_[0], t_[1], t_[2], t_[3]);
            }
        }
    };
    auto stash = [&](int buf) {
        const uint32_t v[4] = {stage.x, stage.y, stage.z, stage.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int nn = c8 + i;
            const int lrow = 32 * (nn >> 5) + 16 * ((nn >> 2) & 1) + 4 * ((nn >> 3) & 3) + (nn & 3);
            vt[buf][lrow * DSDU_LD + sk] = (uint16_t)(v[i >> 1] >> (16 * (i & 1)));
        }
    };
    // the index lists are read one step ahead of the fetch that uses them
    int inner_n1 = n > 1 ? a.uni_inner[p0 + 1] : 0, id_n1 = n > 1 ? a.uni_blk[(long)(p0 + 1) * 4 + w] : -1;
    if (n > 0) {
        fetch(a.uni_inner[p0], a.uni_blk[(long)p0 * 4 + w]);
        stash(0);
    }
    drain_loads();
    __syncthreads();
    for (int s = 0; s < n; ++s) {
        const int blk = blk_next;
        fs[0] = fs_next[0];
        fs[1] = fs_next[1];
        const int inner_n2 = s + 2 < n ? a.uni_inner[p0 + s + 2] : 0;
        const int id_n2 = s + 2 < n ? a.uni_blk[(long)(p0 + s + 2) * 4 + w] : -1;
        if (s + 1 < n) fetch(inner_n1, id_n1);
        inner_n1 = inner_n2;
        id_n1 = id_n2;
        if (blk >= 0) {
            if (TA) {
                // the lane holds rows 16 tm + r16 of the block, columns 8g .. 8g + 7: they go to LDS as
                // [column][row] and come back as fragments of the transposed block (a wave-private tile;
                // LDS operations of a wave complete in order)
                uint16_t* my = bt[w];
#pragma unroll
                for (int tm = 0; tm < 2; ++tm) {
                    const uint32_t v[4] = {fs[tm].x, fs[tm].y, fs[tm].z, fs[tm].w};
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        my[(8 * g + e) * DSDU_LD + 16 * tm + r16] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
                }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int tm = 0; tm < 2; ++tm) fs[tm] = *reinterpret_cast<const uint4*>(my + (16 * tm + r16) * DSDU_LD + 8 * g);
                __builtin_amdgcn_wave_barrier();
            }
            const uint16_t* tp = vt[s & 1];
#pragma unroll
            for (int tn = 0; tn < 4; ++tn) {
                const uint4 fd = *reinterpret_cast<const uint4*>(tp + (16 * tn + r16) * DSDU_LD + 8 * g);
                acc[0][tn] = Frag32<T>::mma(fd, fs[0], acc[0][tn]);
                acc[1][tn] = Frag32<T>::mma(fd, fs[1], acc[1][tn]);
            }
        }
        if (s + 1 < n) stash((s + 1) & 1);
        __syncthreads();
    }
    if (!have_row) return;
    // lane holds C[m = 16tm + r16][n = 32q + 8g + 4(tn%2) + i], tn = 2q, 2q+1
    T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh + n0;
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int nn = 32 * q + 8 * g;
            if (nn < ncols) store8_f32(cp + ((long)bi * 32 + 16 * tm + r16) * a.c_sm + nn, acc[tm][2 * q], acc[tm][2 * q + 1]);
        }
}

// ---------------------------------------------------------------------------------------
// DDS: dense = dense x sparse
// ---------------------------------------------------------------------------------------
template <typename T, int BLK>
__global__ __launch_bounds__(256) void bs_dds_kernel(DxdArgs a) {
    constexpr int TILE = BLK >= 32 ? 32 : 16, NTL = TILE / 16, SUBN = BLK / TILE;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    const long wid = (long)blockIdx.x * 4 + w;
    const long per_mt = (long)a.n_seg * SUBN;
    const long mt = wid / per_mt;
    if (mt * 32 >= a.X) return;
    const int rem = (int)(wid % per_mt), seg = rem / SUBN, subn = rem % SUBN;
    const int z = blockIdx.y;
    const int head = seg / a.per_head, bcol = seg % a.per_head;
    const long m0 = mt * 32;
    const T* spz = reinterpret_cast<const T*>(a.sp) + z * a.sp_sz;
    const T* dnp = reinterpret_cast<const T*>(a.dn) + z * a.dn_sz + head * a.dn_sh;

    floatx4 acc[2][NTL];
#pragma unroll
    for (int tn = 0; tn < NTL; ++tn) { acc[0][tn] = Frag<float>::zero(); acc[1][tn] = Frag<float>::zero(); }
    bool mok[2];
    mok[0] = m0 + r16 < a.X;
    mok[1] = m0 + 16 + r16 < a.X;

    const int p1 = a.seg_ptr[seg + 1];
    for (int p = a.seg_ptr[seg]; p < p1; ++p) {
        const T* blkp = spz + (long)a.seg_blk[p] * (BLK * BLK);
        const long kcol0 = (long)a.seg_inner[p] * BLK;
#pragma unroll
        for (int kk = 0; kk < BLK; kk += 16) {
            typename Frag<T>::type fs[NTL], fd[2];
#pragma unroll
            for (int tn = 0; tn < NTL; ++tn) {
                const int n = subn * TILE + 16 * tn + r16;
                fs[tn] = a.trans ? Frag<T>::load(blkp + n * BLK + kk + 4 * g)
                                 : Frag<T>::gather(blkp + (kk + 4 * g) * BLK + n, BLK);
            }
#pragma unroll
            for (int tm = 0; tm < 2; ++tm) {
                fd[tm] = Frag<T>::zero();
                if (mok[tm])
                    fd[tm] = frag_at<T>(dnp + (m0 + 16 * tm + r16) * a.dn_s0 + (kcol0 + kk + 4 * g) * a.dn_s1, a.dn_s1);
            }
#pragma unroll
            for (int tn = 0; tn < NTL; ++tn) {
                acc[0][tn] = Frag<T>::mma(fs[tn], fd[0], acc[0][tn]);
                acc[1][tn] = Frag<T>::mma(fs[tn], fd[1], acc[1][tn]);
            }
        }
    }
    // lane holds C[m = m0 + 16tm + r16][n = 16tn + 4g + i]
    T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh;
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
        if (!mok[tm]) continue;
        const long m = m0 + 16 * tm + r16;
#pragma unroll
        for (int tn = 0; tn < NTL; ++tn) {
            const long n = (long)bcol * BLK + subn * TILE + 16 * tn + 4 * g;
            store_tile_row<T>(cp + m * a.c_sm + n * a.c_sn, a.c_sn, acc[tm][tn], 4);
        }
    }
}

// Fast DDS (y = x W^T, W block-sparse, blocks read transposed) for 32x32 blocks of a 2-byte type,
// the Pixelfly linear.  Consecutive output block-rows that reduce over the same input blocks are
// grouped (at most four per group, table built on the host): a group is a small dense GEMM
// y[M x 32g] = x[:, listed input blocks] . W_group^T.  A workgroup owns one group and walks a stream
// of 128-token tiles with one continuous pipeline: per input block the 128 x 32 activation tile and
// the group's 32g x 32 weight tile are staged in LDS (registers hold the next-but-one step's tiles
// while the MFMAs of the current one run, across tile boundaries), the 2 x 2 waves own 64 x 64
// outputs each, form them with 16x16x32 MFMAs and store them after the tile's last input block.
struct DdsGroupArgs {
    const void* sp; const void* dn; void* c;
    const int32_t* seg_ptr; const int32_t* seg_blk; const int32_t* seg_inner;
    const int32_t* grp_row0; const int32_t* grp_n;
    int per_head, M;
    long sp_sz, dn_sz, dn_sh, dn_sm, c_sz, c_sh, c_sm;
    int n_xcd;          // dies the dispatcher deals workgroup ids to (set where the kernel is launched)
    int n_grp;          // groups (the weight-stationary kernel deals (token stream, group) pairs itself)
};
constexpr int DDS_MAX_STEPS = 128;   // longest reduction list the tiled kernel accepts
#ifndef FLY_DDS_STATIONARY
#define FLY_DDS_STATIONARY 2         // weight-stationary kernels where the group's weights fit the LDS: 1 = activation
#endif                               // fragments straight from memory, 2 = staged through LDS when there are enough tokens
#ifndef FLY_DDS_DEPTH
#define FLY_DDS_DEPTH 2              // steps (of two input blocks) its activation loads run ahead
#endif
#ifndef FLY_DDS_DIST
#define FLY_DDS_DIST 2               // steps the loads of the 128-token kernel run ahead of its MFMAs
#endif

template <typename T, bool WT, int DIST = FLY_DDS_DIST>     // WT: blocks are [k][n] (y = x W) and are transposed on their way into LDS
__global__ __launch_bounds__(256) void bs_dds32_kernel(DdsGroupArgs a) {
    // A pipeline step takes TWO entries of the reduction list.  The LDS tiles are [row][64 k] with 128-byte rows, the
    // first entry's 32 inputs in front; the eight 16-byte chunks of a row are stored at chunk ^ ((row >> 1) & 7).  Then
    // both the 16-byte fragment reads (16 consecutive rows, one chunk) and the staging writes (2 rows x 8 chunks per 16
    // lanes) cover all 64 banks.  Neighbouring entries of a list are mostly neighbouring input blocks: a staging wave
    // then reads whole 128-byte lines of eight token rows (a compute unit's vector memory path takes one line about
    // every four cycles whether half of it is used or all of it).
    constexpr int LD = 64;
    extern __shared__ __attribute__((aligned(16))) uint16_t dds_smem[];
    uint16_t (*xs)[128 * LD] = reinterpret_cast<uint16_t (*)[128 * LD]>(dds_smem);
    uint16_t (*ws)[128 * LD] = reinterpret_cast<uint16_t (*)[128 * LD]>(dds_smem + 2 * 128 * LD);
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int wm = w >> 1, wn = w & 1;                      // this wave: tokens 64wm.., outputs 64wn..
    const int z = blockIdx.z;
    // Workgroups go to the XCDs (each with its own L2) round-robin in launch order.  The launch
    // index is re-mapped so that the groups working on one stream of token tiles -- they read the same
    // activations -- run on one XCD, one after the other: stream = n_xcd * (slot / groups) + XCD.
    const int lin = blockIdx.x + gridDim.x * blockIdx.y, slot = lin / a.n_xcd;
    const int grp = slot % (int)gridDim.x, ty = a.n_xcd * (slot / (int)gridDim.x) + lin % a.n_xcd, gy = gridDim.y;   // gridDim.y is a multiple of n_xcd
    // token tiles ty, ty + gy, ... : the group's tables are read once and the load -> LDS -> MFMA
    // pipeline runs on across tile boundaries
    const int tiles_all = (a.M + 127) / 128;
    if (ty >= tiles_all) return;                            // workgroup-uniform
    const int my_tiles = (tiles_all - ty + gy - 1) / gy;
    const int row0 = a.grp_row0[grp], gn = a.grp_n[grp];    // first output block-row (segment) and count
    const int head = row0 / a.per_head, bcol0 = row0 % a.per_head;
    const int p0 = a.seg_ptr[row0], nin = a.seg_ptr[row0 + 1] - p0;
    const uint16_t* spz = reinterpret_cast<const uint16_t*>(a.sp) + z * a.sp_sz;
    const uint16_t* xp = reinterpret_cast<const uint16_t*>(a.dn) + z * a.dn_sz + head * a.dn_sh;

    // the group's reduction list (inner block per entry, block id per entry and output block-row) is
    // read once into LDS: the per-step loads then depend on no other global load
    __shared__ int s_inner[DDS_MAX_STEPS];
    __shared__ int s_blk[4][DDS_MAX_STEPS];
    for (int i = tid; i < nin; i += 256) s_inner[i] = a.seg_inner[p0 + i];
    for (int i = tid; i < 4 * nin; i += 256) {
        const int ob = i / nin, t = i % nin;
        s_blk[ob][t] = ob < gn ? a.seg_blk[a.seg_ptr[row0 + ob] + t] : -1;
    }
    __syncthreads();

    // staging roles: thread -> (row = tid/8 + 32 hh, 16-byte chunk = tid%8) of the x and W tiles; chunks 0..3 belong
    // to the step's first entry, 4..7 to its second
    const int srow = tid >> 3, sc = tid & 7, sel = sc >> 2, schunk = (sc & 3) * 8;
    const int npair = (nin + 1) / 2;
    const int n_steps = my_tiles * npair;
    // DIST register sets: the loads of step s+DIST are issued while step s computes and are parked in LDS
    // one iteration before they are used
    // (native vectors: arrays of the uint4 struct passed by reference do not stay in registers)
    // Every fetch issues the same number of loads on every path (a step past the end re-reads the last
    // one, an absent weight block reads block 0 and is zeroed when it is parked): only then can the
    // compiler count how many newer loads may stay in flight when it waits for the older set.
    uintx4 rx[DIST][4], rw[DIST][4];                        // set j holds the steps congruent to j modulo DIST
    bool wl[DIST][4];                                       // weight block present?
    int f_tile = 0, f_t = 0;                                // fetch cursor: (token tile, step inside it)
    // A load is "base + per-thread byte offset": the two input blocks of a step and the weight blocks of its eight
    // (output block, entry) pairs come out of LDS once through the first lane; a thread picks the entry its chunk
    // belongs to; the per-thread offsets change only with the token tile.
    const uint32_t woff = (uint32_t)((srow * 32 + schunk) * 2);
    uint32_t xoff[4] = {0, 0, 0, 0};
    auto fetch = [&](uintx4 (&rx)[4], uintx4 (&rw)[4], bool (&wl)[4]) __attribute__((always_inline)) {
        const bool live = f_tile < my_tiles;                 // past the end: re-read the last step, zero weights
        const int tc = live ? f_t : npair - 1;
        if (f_t == 0) {
            const long m0 = ((long)ty + (long)min(f_tile, my_tiles - 1) * gy) * 128;
#pragma unroll
            for (int hh = 0; hh < 4; ++hh) {
                const long m = min(m0 + srow + 32 * hh, (long)a.M - 1);          // clamped: masked at the store
                xoff[hh] = (uint32_t)((m * a.dn_sm + schunk) * 2);
            }
        }
        const int t0 = 2 * tc, t1 = min(2 * tc + 1, nin - 1);
        const bool second = 2 * tc + 1 < nin;                // an odd list's last step: its second entry is absent
        const int in0 = __builtin_amdgcn_readfirstlane(s_inner[t0]), in1 = __builtin_amdgcn_readfirstlane(s_inner[t1]);
        const char* xb = reinterpret_cast<const char*>(xp + (long)(sel ? in1 : in0) * 32);
#pragma unroll
        for (int hh = 0; hh < 4; ++hh) {
            rx[hh] = *reinterpret_cast<const uintx4*>(xb + xoff[hh]);
            const int b0 = __builtin_amdgcn_readfirstlane(s_blk[hh][t0]), b1 = __builtin_amdgcn_readfirstlane(s_blk[hh][t1]);
            const int blk_id = sel ? (second ? b1 : -1) : b0;
            wl[hh] = live && blk_id >= 0;                    // a missing block contributes zero weights
            rw[hh] = *reinterpret_cast<const uintx4*>(reinterpret_cast<const char*>(spz + (long)max(blk_id, 0) * 1024) + woff);
        }
        if (++f_t == npair) { f_t = 0; ++f_tile; }
    };
    // The weight tile sits in LDS in the order the MFMAs read it: row 64*(n/64) + 16*i + r holds output
    // n = 64*(n/64) + 32*(i/2) + 8*(r/4) + 4*(i%2) + r%4, so that a wave's fragment read walks 16
    // consecutive LDS rows.
    auto wrow = [](int n) { const int b = n & 31; return (n & 64) + 16 * (2 * ((n >> 5) & 1) + ((b >> 2) & 1)) + 4 * (b >> 3) + (b & 3); };
    auto slot_of = [](int row, int chunk) { return row * LD + 8 * (chunk ^ ((row >> 1) & 7)); };
    auto stash = [&](int buf, const uintx4 (&rx)[4], const uintx4 (&rw)[4], const bool (&wl)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int hh = 0; hh < 4; ++hh) {
            *reinterpret_cast<uintx4*>(&xs[buf][slot_of(srow + 32 * hh, sc)]) = rx[hh];
            const uintx4 wv = wl[hh] ? rw[hh] : uintx4{0, 0, 0, 0};
            if (!WT) {
                // block row srow of output block hh, inputs schunk .. of entry `sel`
                *reinterpret_cast<uintx4*>(&ws[buf][slot_of(wrow(32 * hh + srow), sc)]) = wv;
            } else {
                // the thread holds row k = srow of the block [k][n], columns n = schunk .. schunk + 7: the
                // LDS tile is [n][k] either way, so these eight go out one by one
                const int kk = 32 * sel + srow;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int n = wrow(32 * hh + schunk + e);
                    ws[buf][slot_of(n, kk >> 3) + (kk & 7)] = (uint16_t)(wv[e >> 1] >> (16 * (e & 1)));
                }
            }
        }
    };

    floatx4 acc[4][4];
#pragma unroll
    for (int tm = 0; tm < 4; ++tm)
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) acc[tm][tn] = Frag<float>::zero();
    const bool wave_active = 2 * wn < gn;                   // its output blocks exist in this group

    T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh;
    // lane holds y[m = 64wm + 16tm + r16][n = 32*(output block) + 8g + 4*(tn%2) + i]: 16-byte stores
    auto store_tile = [&](int tile) __attribute__((always_inline)) {
        const long m0 = ((long)ty + (long)tile * gy) * 128;
#pragma unroll
        for (int tm = 0; tm < 4; ++tm) {
            const long m = m0 + 64 * wm + 16 * tm + r16;
#pragma unroll
            for (int o2 = 0; o2 < 2; ++o2) {
                const int ob = 2 * wn + o2;
                if (m < a.M && ob < gn)
                    store8_f32(cp + m * a.c_sm + (long)(bcol0 + ob) * 32 + 8 * g, acc[tm][2 * o2], acc[tm][2 * o2 + 1]);
            }
#pragma unroll
            for (int tn = 0; tn < 4; ++tn) acc[tm][tn] = Frag<float>::zero();
        }
    };
    int c_tile = 0, c_t = 0;                                // compute cursor
    // this lane's 16 bytes inside a 16-row fragment, per entry of the step (fragments start at multiples of 16 rows)
    const int frag_off[2] = {r16 * LD + 8 * (g ^ (r16 >> 1)), r16 * LD + 8 * ((4 + g) ^ (r16 >> 1))};
    auto compute = [&](int cur) __attribute__((always_inline)) {
        if (wave_active) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                uint4 fx[4], fw[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    fx[i] = *reinterpret_cast<const uint4*>(&xs[cur][(64 * wm + 16 * i) * LD + frag_off[kb]]);
                    // W-tile i covers output block i/2; its MFMA row r is block row 8*(r/4) + 4*(i%2) + r%4
                    fw[i] = *reinterpret_cast<const uint4*>(&ws[cur][(64 * wn + 16 * i) * LD + frag_off[kb]]);
                }
#pragma unroll
                for (int tm = 0; tm < 4; ++tm)
#pragma unroll
                    for (int tn = 0; tn < 4; ++tn) acc[tm][tn] = Frag32<T>::mma(fw[tn], fx[tm], acc[tm][tn]);
            }
            if (++c_t == npair) { store_tile(c_tile); c_t = 0; ++c_tile; }   // the tile's last entries
        }
    };
    if (nin == 0) {                                         // no input block: zero rows
        if (wave_active)
            for (int tile = 0; tile < my_tiles; ++tile) store_tile(tile);
        return;
    }
    // Loads run DIST steps ahead of the MFMAs in DIST register sets: a step's tiles are asked for, parked in LDS
    // DIST - 1 iterations later (one iteration before they are used), and every global load has that long to arrive.
    // The loop is unrolled over the least common multiple of the two LDS stages and the DIST sets, so that every
    // register set and stage index is a constant.
#pragma unroll
    for (int j = 0; j < DIST; ++j) fetch(rx[j], rw[j], wl[j]);
    drain_loads_but<8 * (DIST - 1)>();                       // set 0 has arrived
    stash(0, rx[0], rw[0], wl[0]);
    __syncthreads();
    constexpr int U = (DIST % 2 == 0) ? DIST : 2 * DIST;
    for (int step = 0; step < n_steps; step += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // (no early exit inside: every path through the body issues the same loads, so the compiler can count how
            //  many newer ones may stay in flight when it waits for a set)
            fetch(rx[u % DIST], rw[u % DIST], wl[u % DIST]);                    // step + u + DIST; its set was parked an iteration ago
            if (step + u < n_steps) compute(u & 1);
            stash((u + 1) & 1, rx[(u + 1) % DIST], rw[(u + 1) % DIST], wl[(u + 1) % DIST]);
            drain_loads_but<8 * (DIST - 1)>();              // the set parked next iteration has arrived
            __syncthreads();
        }
    }
}

// Weight-stationary DDS for groups whose weights fit the LDS (reduction lists of up to 9 input blocks: layers that
// widen, such as the first linear of a channel MLP).  The group's weight tiles -- the same for every token tile -- are
// brought into LDS once; after that a wave needs nothing from its neighbours: it owns 64 tokens against all outputs of
// the group, takes its activation fragments STRAIGHT from global memory in MFMA operand order (lane (r, g): token r,
// inputs 8 g .. 8 g + 7 of the step's block, 16 contiguous bytes), DEPTH steps ahead in DEPTH register sets, and reads
// the step's weight fragments from LDS.  No barrier in the loop, no activation staging, no weight traffic per token
// tile; every weight fragment read feeds four MFMAs.  Tokens are the rows of the products and the weight tiles are
// dealt so that tile n holds outputs 8 r + n (r = 0..15): a lane then ends up with eight CONSECUTIVE outputs of four
// tokens, and one store instruction writes four whole 256-byte rows of the result (with 64-byte pieces per row the
// stores of the 308 MB result were 40 % of the kernel's time).  Two workgroups of four waves per compute unit; the
// (token stream, group) pairs are dealt to the XCDs in contiguous runs, so that the groups reading one stream's
// activations share an L2.
constexpr int DDS_STAT_STEPS = 9;         // longest reduction list: 8 KB of weight tiles per step, 72 KB, two workgroups per CU

template <typename T, bool WT, int DEPTH>
__global__ __launch_bounds__(256) void bs_dds32s_kernel(DdsGroupArgs a, int n_streams) {
    constexpr int STEP = 8 * 16 * 32;                       // elements of a step's eight weight tiles
    extern __shared__ __attribute__((aligned(16))) uint16_t wres[];     // [step][tile n][row r][32 k]: output 8 r + n of the group
    __shared__ int s_inner[DDS_STAT_STEPS];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int z = blockIdx.y;
    // pair index: the dispatcher deals workgroup ids to the XCDs in turn; XCD x takes the pairs x * per_xcd ...
    const int per_xcd = (int)gridDim.x / a.n_xcd;
    const int pair = ((int)blockIdx.x % a.n_xcd) * per_xcd + (int)blockIdx.x / a.n_xcd;
    const int n_grp = a.n_grp;
    if (pair >= n_streams * n_grp) return;                  // workgroup-uniform
    const int ty = pair / n_grp, grp = pair % n_grp, gy = n_streams;
    const int tiles_all = (a.M + 255) / 256;
    if (ty >= tiles_all) return;
    const int my_tiles = (tiles_all - ty + gy - 1) / gy;
    const int row0 = a.grp_row0[grp], gn = a.grp_n[grp];
    const int head = row0 / a.per_head, bcol0 = row0 % a.per_head;
    const int p0 = a.seg_ptr[row0], nin = a.seg_ptr[row0 + 1] - p0;
    const uint16_t* spz = reinterpret_cast<const uint16_t*>(a.sp) + z * a.sp_sz;
    const uint16_t* xp = reinterpret_cast<const uint16_t*>(a.dn) + z * a.dn_sz + head * a.dn_sh;
    T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh;

    for (int i = tid; i < nin; i += 256) s_inner[i] = a.seg_inner[p0 + i];
    // the group's weights, once (output blocks the group lacks: zeros)
    for (int idx = tid; idx < nin * 512; idx += 256) {
        const int chunk = idx & 3, row = (idx >> 2) & 31, ob = (idx >> 7) & 3, t = idx >> 9;
        const int blk_id = ob < gn ? a.seg_blk[a.seg_ptr[row0 + ob] + t] : -1;
        uintx4 v = {0, 0, 0, 0};
        if (blk_id >= 0) v = *reinterpret_cast<const uintx4*>(spz + (long)blk_id * 1024 + row * 32 + chunk * 8);
        uint16_t* dst = wres + (size_t)t * STEP;
        if (!WT) {
            // block row `row` is output 32 ob + row: tile row % 8, row 4 ob + row / 8; the thread's 8 inputs stay together
            *reinterpret_cast<uintx4*>(dst + (row & 7) * 512 + (4 * ob + (row >> 3)) * 32 + 8 * chunk) = v;
        } else {
            // the block is [input][output]: the thread holds input `row`, outputs 32 ob + 8 chunk + e -> tile e, row 4 ob + chunk
#pragma unroll
            for (int e = 0; e < 8; ++e)
                dst[e * 512 + (4 * ob + chunk) * 32 + row] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
        }
    }
    __syncthreads();

    floatx4 acc[4][8];
#pragma unroll
    for (int tm = 0; tm < 4; ++tm)
#pragma unroll
        for (int n = 0; n < 8; ++n) acc[tm][n] = Frag<float>::zero();
    const bool col_live = 8 * r16 < 32 * gn;                // this lane's eight outputs exist in the group
    // lane holds y[m = 64 w + 16 tm + 4 g + i][n0 + 8 r16 .. + 7]: one 16-byte store per (tm, i), 256 bytes per row and
    // instruction
    auto store_tile = [&](int tile) __attribute__((always_inline)) {
        const long m0 = ((long)ty + (long)tile * gy) * 256 + 64 * w + 4 * g;
        T* base = cp + (long)bcol0 * 32 + 8 * r16;
#pragma unroll
        for (int tm = 0; tm < 4; ++tm) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const long m = m0 + 16 * tm + i;
                if (m < a.M && col_live) {
                    const floatx4 lo = {acc[tm][0][i], acc[tm][1][i], acc[tm][2][i], acc[tm][3][i]};
                    const floatx4 hi = {acc[tm][4][i], acc[tm][5][i], acc[tm][6][i], acc[tm][7][i]};
                    store8_f32(base + m * a.c_sm, lo, hi);
                }
            }
#pragma unroll
            for (int n = 0; n < 8; ++n) acc[tm][n] = Frag<float>::zero();
        }
    };
    if (nin == 0) {                                         // no input block: zero rows
        for (int tile = 0; tile < my_tiles; ++tile) store_tile(tile);
        return;
    }

    // a step takes two entries of the reduction list: neighbouring input blocks share their 128-byte lines, and asked for
    // together the second block's loads find them on their way (a step apart they had left the L1 again)
    const int npair = (nin + 1) / 2;
    const int n_steps = my_tiles * npair;
    uintx4 fx[DEPTH][2][4];
    int f_tile = 0, f_t = 0;                                // fetch cursor: (token tile, pair of entries inside it)
    uint32_t xoff[4] = {0, 0, 0, 0};
    auto fetch = [&](uintx4 (&rx)[2][4]) __attribute__((always_inline)) {
        const int tp = f_tile < my_tiles ? f_t : npair - 1; // past the end: re-read the last step (never used)
        if (f_t == 0) {
            const long m0 = ((long)ty + (long)min(f_tile, my_tiles - 1) * gy) * 256 + 64 * w;
#pragma unroll
            for (int tm = 0; tm < 4; ++tm) {
                const long m = min(m0 + 16 * tm + r16, (long)a.M - 1);           // clamped: masked at the store
                xoff[tm] = (uint32_t)((m * a.dn_sm + 8 * g) * 2);
            }
        }
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {                    // (an odd list's last step reads its last entry twice and uses it once)
            const int inner = __builtin_amdgcn_readfirstlane(s_inner[min(2 * tp + hf, nin - 1)]);
            const char* xb = reinterpret_cast<const char*>(xp + (long)inner * 32);
#pragma unroll
            for (int tm = 0; tm < 4; ++tm) rx[hf][tm] = *reinterpret_cast<const uintx4*>(xb + xoff[tm]);
        }
        if (++f_t == npair) { f_t = 0; ++f_tile; }
    };
    int c_tile = 0, c_t = 0;                                // compute cursor
    const int frag_off = r16 * 32 + 8 * g;                  // this lane's 16 bytes of a weight tile: a wave reads its 1 KB in lane order
    auto compute = [&](const uintx4 (&rx)[2][4]) __attribute__((always_inline)) {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            if (2 * c_t + hf < nin) {                       // workgroup-uniform
                const uint16_t* wt = wres + (size_t)(2 * c_t + hf) * STEP + frag_off;
#pragma unroll
                for (int n = 0; n < 8; ++n) {
                    const uint4 fw = *reinterpret_cast<const uint4*>(wt + n * 512);
#pragma unroll
                    for (int tm = 0; tm < 4; ++tm)
                        acc[tm][n] = Frag32<T>::mma(__builtin_bit_cast(uint4, rx[hf][tm]), fw, acc[tm][n]);
                }
            }
        }
        if (++c_t == npair) { store_tile(c_tile); c_t = 0; ++c_tile; }   // the tile's last entries: results out
    };
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) fetch(fx[j]);
    for (int step = 0; step < n_steps; step += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            if (step + u < n_steps) compute(fx[u]);
            fetch(fx[u]);                                   // step + u + DEPTH
        }
    }
}

// The weight-stationary DDS with the activations staged through LDS by direct-to-LDS transfers.  A compute unit's
// vector memory path takes about one 128-byte line every four cycles whether half of the line is asked for or all of
// it, and bs_dds32s_kernel's fragment loads (64-byte pieces of 16 token rows per instruction) are what bounds it.  Here
// a wave fetches a step's two input blocks of its 64 tokens as whole 128-byte pieces of token rows (eight rows per
// instruction, the two blocks side by side when they are neighbours) into a stage of its own, 8 KB, and reads the MFMA
// fragments from there.  One workgroup of eight waves per compute unit shares the group's weights (72 KB) and leaves
// room for the eight stages; a wave touches no other wave's stage, so the loop has no barrier: it waits for its
// transfer, reads the step's fragments into registers, starts the next step's transfer into the same stage and then
// multiplies.  16-byte chunk c of token t sits at chunk c ^ ((t >> 1) & 7) of the token's 128 bytes: the transfer
// writes lane by lane, so the lane asks for the chunk that belongs in its slot, and the 16 lanes of a fragment read
// cover all 64 banks.
template <typename T, bool WT>
__global__ __launch_bounds__(512) void bs_dds32d_kernel(DdsGroupArgs a, int n_streams) {
    constexpr int STEP = 8 * 16 * 32;                       // elements of a step's eight weight tiles
    constexpr int WBYTES = DDS_STAT_STEPS * 8192;           // the weights' share of the LDS
    extern __shared__ __attribute__((aligned(1024))) uint16_t wres[];   // [step][tile n][row r][32 k], then 8 stages of 8 KB
    __shared__ int s_inner[DDS_STAT_STEPS];
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int z = blockIdx.y;
    const int per_xcd = (int)gridDim.x / a.n_xcd;
    const int pair = ((int)blockIdx.x % a.n_xcd) * per_xcd + (int)blockIdx.x / a.n_xcd;
    const int n_grp = a.n_grp;
    if (pair >= n_streams * n_grp) return;                  // workgroup-uniform
    const int ty = pair / n_grp, grp = pair % n_grp, gy = n_streams;
    const int tiles_all = (a.M + 511) / 512;
    if (ty >= tiles_all) return;
    const int my_tiles = (tiles_all - ty + gy - 1) / gy;
    const int row0 = a.grp_row0[grp], gn = a.grp_n[grp];
    const int head = row0 / a.per_head, bcol0 = row0 % a.per_head;
    const int p0 = a.seg_ptr[row0], nin = a.seg_ptr[row0 + 1] - p0;
    const uint16_t* spz = reinterpret_cast<const uint16_t*>(a.sp) + z * a.sp_sz;
    const uint16_t* xp = reinterpret_cast<const uint16_t*>(a.dn) + z * a.dn_sz + head * a.dn_sh;
    T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh;

    for (int i = tid; i < nin; i += 512) s_inner[i] = a.seg_inner[p0 + i];
    for (int idx = tid; idx < nin * 512; idx += 512) {      // the group's weights, once (see bs_dds32s_kernel)
        const int chunk = idx & 3, row = (idx >> 2) & 31, ob = (idx >> 7) & 3, t = idx >> 9;
        const int blk_id = ob < gn ? a.seg_blk[a.seg_ptr[row0 + ob] + t] : -1;
        uintx4 v = {0, 0, 0, 0};
        if (blk_id >= 0) v = *reinterpret_cast<const uintx4*>(spz + (long)blk_id * 1024 + row * 32 + chunk * 8);
        uint16_t* dst = wres + (size_t)t * STEP;
        if (!WT) {
            *reinterpret_cast<uintx4*>(dst + (row & 7) * 512 + (4 * ob + (row >> 3)) * 32 + 8 * chunk) = v;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                dst[e * 512 + (4 * ob + chunk) * 32 + row] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
        }
    }
    __syncthreads();

    floatx4 acc[4][8];
#pragma unroll
    for (int tm = 0; tm < 4; ++tm)
#pragma unroll
        for (int n = 0; n < 8; ++n) acc[tm][n] = Frag<float>::zero();
    const bool col_live = 8 * r16 < 32 * gn;
    auto store_tile = [&](int tile) __attribute__((always_inline)) {
        const long m0 = ((long)ty + (long)tile * gy) * 512 + 64 * w + 4 * g;
        T* base = cp + (long)bcol0 * 32 + 8 * r16;
#pragma unroll
        for (int tm = 0; tm < 4; ++tm) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const long m = m0 + 16 * tm + i;
                if (m < a.M && col_live) {
                    const floatx4 lo = {acc[tm][0][i], acc[tm][1][i], acc[tm][2][i], acc[tm][3][i]};
                    const floatx4 hi = {acc[tm][4][i], acc[tm][5][i], acc[tm][6][i], acc[tm][7][i]};
                    store8_f32(base + m * a.c_sm, lo, hi);
                }
            }
#pragma unroll
            for (int n = 0; n < 8; ++n) acc[tm][n] = Frag<float>::zero();
        }
    };
    if (nin == 0) {                                         // no input block: zero rows
        for (int tile = 0; tile < my_tiles; ++tile) store_tile(tile);
        return;
    }

    const int npair = (nin + 1) / 2;
    const int n_steps = my_tiles * npair;
    char* stage = reinterpret_cast<char*>(wres) + WBYTES + 8192 * w;
    // transfer j of a step brings tokens 8 j .. 8 j + 7 of the wave: this lane's slot is chunk slot lane % 8 of token
    // 8 j + lane / 8, i.e. chunk (lane % 8) ^ ((token >> 1) & 7) of that token's two blocks
    const int tl = lane >> 3;
    uint32_t xoff[8];
    int sel[8];                                             // which of the step's two blocks the lane's chunk belongs to
#pragma unroll
    for (int j = 0; j < 8; ++j) { xoff[j] = 0; sel[j] = 0; }
    int f_tile = 0, f_t = 0;                                // transfer cursor: (token tile, pair of entries inside it)
    auto transfer = [&]() __attribute__((always_inline)) {
        if (f_t == 0) {
            const long m0 = ((long)ty + (long)f_tile * gy) * 512 + 64 * w;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int t = 8 * j + tl, c = (lane & 7) ^ ((t >> 1) & 7);
                const long m = min(m0 + t, (long)a.M - 1);                       // clamped: masked at the store
                xoff[j] = (uint32_t)((m * a.dn_sm + 8 * (c & 3)) * 2);
                sel[j] = c >> 2;
            }
        }
        const int in0 = __builtin_amdgcn_readfirstlane(s_inner[2 * f_t]);
        const int in1 = __builtin_amdgcn_readfirstlane(s_inner[min(2 * f_t + 1, nin - 1)]);   // (an odd list's last step: twice the same)
        const char* xb = reinterpret_cast<const char*>(xp);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            dma_to_lds(xb + xoff[j] + (uint32_t)((sel[j] ? in1 : in0) * 64), stage + 1024 * j);
        if (++f_t == npair) { f_t = 0; ++f_tile; }
    };
    int c_tile = 0, c_t = 0;                                // compute cursor
    const int wfrag = r16 * 32 + 8 * g;                     // this lane's 16 bytes of a weight tile
    // fragment of (token 16 tm + r16, block hf): chunk 4 hf + g, stored at chunk ^ ((token >> 1) & 7)
    int xfrag[2][4];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int tm = 0; tm < 4; ++tm) {
            const int t = 16 * tm + r16;
            xfrag[hf][tm] = t * 128 + 16 * ((4 * hf + g) ^ ((t >> 1) & 7));
        }
    transfer();
    for (int step = 0; step < n_steps; ++step) {
        drain_loads();                                      // this step's activations are in the stage
        uintx4 fx[2][4];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int tm = 0; tm < 4; ++tm) fx[hf][tm] = *reinterpret_cast<const uintx4*>(stage + xfrag[hf][tm]);
        __builtin_amdgcn_s_waitcnt(0xC07F);                 // lgkmcnt(0): the fragments are in registers, the stage is free
        if (step + 1 < n_steps) transfer();                 // (workgroup-uniform) flies under the products below
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            if (2 * c_t + hf < nin) {                       // workgroup-uniform
                const uint16_t* wt = wres + (size_t)(2 * c_t + hf) * STEP + wfrag;
#pragma unroll
                for (int n = 0; n < 8; ++n) {
                    const uint4 fw = *reinterpret_cast<const uint4*>(wt + n * 512);
#pragma unroll
                    for (int tm = 0; tm < 4; ++tm)
                        acc[tm][n] = Frag32<T>::mma(__builtin_bit_cast(uint4, fx[hf][tm]), fw, acc[tm][n]);
                }
            }
        }
        if (++c_t == npair) { store_tile(c_tile); c_t = 0; ++c_tile; }
    }
}

// The same per-wave scheme for reduction lists that do not fit the LDS (layers that narrow: 36 input blocks per output
// block in the second linear of a channel MLP).  The group's weights pass through LDS in chunks of DDS_CK list entries
// (32 KB), double-buffered and shared by the eight waves: a thread asks for its 64 bytes of the next chunk at the head
// of a chunk, parks them in the other buffer at its end, and one barrier per chunk (two steps of 64 MFMAs per wave)
// publishes them -- the tiled kernel pays a barrier, eight LDS writes and the wait for its loads per 32 MFMAs.  The
// activations go through a stage per wave exactly as in bs_dds32d_kernel.  The weights are fetched again for every tile
// of 512 tokens (from L2: a quarter of what the tiled kernel's 128-token tiles fetch).
constexpr int DDS_CK = 4;
typedef unsigned int uintx2 __attribute__((ext_vector_type(2)));

template <typename T, bool WT>
__global__ __launch_bounds__(512) void bs_dds32c_kernel(DdsGroupArgs a, int n_streams) {
    constexpr int STEP = 8 * 16 * 32;                       // elements of an entry's eight weight tiles
    constexpr int CHUNK = DDS_CK * STEP;                    // elements of a chunk buffer
    extern __shared__ __attribute__((aligned(1024))) uint16_t wres[];   // 2 x [entry][tile n][row r][32 k], then 8 stages of 8 KB
    __shared__ int s_inner[DDS_MAX_STEPS];
    __shared__ int s_blk[4][DDS_MAX_STEPS];
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int z = blockIdx.y;
    const int per_xcd = (int)gridDim.x / a.n_xcd;
    const int pair = ((int)blockIdx.x % a.n_xcd) * per_xcd + (int)blockIdx.x / a.n_xcd;
    const int n_grp = a.n_grp;
    if (pair >= n_streams * n_grp) return;                  // workgroup-uniform
    const int ty = pair / n_grp, grp = pair % n_grp, gy = n_streams;
    const int tiles_all = (a.M + 511) / 512;
    if (ty >= tiles_all) return;
    const int my_tiles = (tiles_all - ty + gy - 1) / gy;
    const int row0 = a.grp_row0[grp], gn = a.grp_n[grp];
    const int head = row0 / a.per_head, bcol0 = row0 % a.per_head;
    const int p0 = a.seg_ptr[row0], nin = a.seg_ptr[row0 + 1] - p0;
    const uint16_t* spz = reinterpret_cast<const uint16_t*>(a.sp) + z * a.sp_sz;
    const uint16_t* xp = reinterpret_cast<const uint16_t*>(a.dn) + z * a.dn_sz + head * a.dn_sh;
    T* cp = reinterpret_cast<T*>(a.c) + z * a.c_sz + head * a.c_sh;

    for (int i = tid; i < nin; i += 512) s_inner[i] = a.seg_inner[p0 + i];
    for (int i = tid; i < 4 * nin; i += 512) {
        const int ob = i / nin, t = i % nin;
        s_blk[ob][t] = ob < gn ? a.seg_blk[a.seg_ptr[row0 + ob] + t] : -1;
    }
    __syncthreads();

    floatx4 acc[4][8];
#pragma unroll
    for (int tm = 0; tm < 4; ++tm)
#pragma unroll
        for (int n = 0; n < 8; ++n) acc[tm][n] = Frag<float>::zero();
    // The group's 32 gn outputs are dealt to NT = 2 gn tiles of 16: tile n holds outputs NT r + n (r = 0..15), so no MFMA
    // column is padding whatever the group's size, and a lane ends up with NT consecutive outputs of four tokens.
    const int NT = 2 * gn;
    auto store_tile = [&](int tile) __attribute__((always_inline)) {
        const long m0 = ((long)ty + (long)tile * gy) * 512 + 64 * w + 4 * g;
        T* base = cp + (long)bcol0 * 32 + NT * r16;
#pragma unroll
        for (int tm = 0; tm < 4; ++tm) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const long m = m0 + 16 * tm + i;
                if (m < a.M) {
                    uint32_t* dst = reinterpret_cast<uint32_t*>(base + m * a.c_sm);
                    const uint32_t p0_ = pack2<T>(acc[tm][0][i], acc[tm][1][i]), p1_ = pack2<T>(acc[tm][2][i], acc[tm][3][i]);
                    const uint32_t p2_ = pack2<T>(acc[tm][4][i], acc[tm][5][i]), p3_ = pack2<T>(acc[tm][6][i], acc[tm][7][i]);
                    if (NT == 8) __builtin_nontemporal_store(uintx4{p0_, p1_, p2_, p3_}, reinterpret_cast<uintx4*>(dst));
                    else if (NT == 6) { __builtin_nontemporal_store(uintx2{p0_, p1_}, reinterpret_cast<uintx2*>(dst)); __builtin_nontemporal_store(p2_, dst + 2); }
                    else if (NT == 4) __builtin_nontemporal_store(uintx2{p0_, p1_}, reinterpret_cast<uintx2*>(dst));
                    else __builtin_nontemporal_store(p0_, dst);
                }
            }
#pragma unroll
            for (int n = 0; n < 8; ++n) acc[tm][n] = Frag<float>::zero();
        }
    };
    if (nin == 0) {                                         // no input block: zero rows
        for (int tile = 0; tile < my_tiles; ++tile) store_tile(tile);
        return;
    }

    const int npair = (nin + 1) / 2, nchunk = (npair + DDS_CK / 2 - 1) / (DDS_CK / 2);      // steps and chunks per tile
    const int n_steps = my_tiles * npair, n_chunks = my_tiles * nchunk;
    // the weights of a chunk: this thread's 16 bytes of each of its DDS_CK entries -- row `wrow` (its 8 inputs `wch`..) of
    // output block `wob`, parked at the place the MFMAs read (see bs_dds32s_kernel)
    const int wch = tid & 3, wrow = (tid >> 2) & 31, wob = (tid >> 7) & 3;
    const uint32_t wsrc = (uint32_t)((wrow * 32 + wch * 8) * 2);
    // where they go: output o of the group sits in tile o % NT, row o / NT
    int wdst[WT ? 8 : 1];
    if (!WT) {
        const int o = 32 * wob + wrow;
        wdst[0] = (o % NT) * 512 + (o / NT) * 32 + 8 * wch;
    } else {
#pragma unroll
        for (int e = 0; e < (WT ? 8 : 1); ++e) {
            const int o = 32 * wob + 8 * wch + e;
            wdst[e] = (o % NT) * 512 + (o / NT) * 32 + wrow;
        }
    }
    uintx4 rwq[DDS_CK];
    bool wlive[DDS_CK];
    auto fetch_w = [&](int q) __attribute__((always_inline)) {
        const int e0 = DDS_CK * (q % nchunk);
#pragma unroll
        for (int j = 0; j < DDS_CK; ++j) {
            const int blk_id = e0 + j < nin ? s_blk[wob][e0 + j] : -1;
            wlive[j] = blk_id >= 0;
            rwq[j] = *reinterpret_cast<const uintx4*>(reinterpret_cast<const char*>(spz + (long)max(blk_id, 0) * 1024) + wsrc);
        }
    };
    auto stash_w = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < DDS_CK; ++j) {
            const uintx4 v = wlive[j] ? rwq[j] : uintx4{0, 0, 0, 0};
            uint16_t* dst = wres + (size_t)buf * CHUNK + (size_t)j * STEP;
            if (wob < gn) {                                 // (an output block the group lacks has no place in the tiles)
                if (!WT) {
                    *reinterpret_cast<uintx4*>(dst + wdst[0]) = v;
                } else {
#pragma unroll
                    for (int e = 0; e < (WT ? 8 : 1); ++e) dst[wdst[e]] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
                }
            }
        }
    };

    char* stage = reinterpret_cast<char*>(wres) + 2 * CHUNK * 2 + 8192 * w;
    const int tl = lane >> 3;
    uint32_t xoff[8];
    int sel[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) { xoff[j] = 0; sel[j] = 0; }
    int f_tile = 0, f_t = 0;                                // transfer cursor: (token tile, pair of entries inside it)
    auto transfer = [&]() __attribute__((always_inline)) {  // (see bs_dds32d_kernel)
        if (f_t == 0) {
            const long m0 = ((long)ty + (long)f_tile * gy) * 512 + 64 * w;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int t = 8 * j + tl, c = (lane & 7) ^ ((t >> 1) & 7);
                const long m = min(m0 + t, (long)a.M - 1);
                xoff[j] = (uint32_t)((m * a.dn_sm + 8 * (c & 3)) * 2);
                sel[j] = c >> 2;
            }
        }
        const int in0 = __builtin_amdgcn_readfirstlane(s_inner[2 * f_t]);
        const int in1 = __builtin_amdgcn_readfirstlane(s_inner[min(2 * f_t + 1, nin - 1)]);
        const char* xb = reinterpret_cast<const char*>(xp);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            dma_to_lds(xb + xoff[j] + (uint32_t)((sel[j] ? in1 : in0) * 64), stage + 1024 * j);
        if (++f_t == npair) { f_t = 0; ++f_tile; }
    };
    const int wfrag = r16 * 32 + 8 * g;
    int xfrag[2][4];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int tm = 0; tm < 4; ++tm) {
            const int t = 16 * tm + r16;
            xfrag[hf][tm] = t * 128 + 16 * ((4 * hf + g) ^ ((t >> 1) & 7));
        }

    fetch_w(0);
    stash_w(0);
    __syncthreads();
    transfer();
    int c_tile = 0, c_t = 0, q = 0;                         // compute cursor: tile, step inside it; chunks done so far
    for (int step = 0; step < n_steps; ++step) {
        drain_loads();                                      // this step's activations are in the stage
        const bool chunk_head = (c_t & (DDS_CK / 2 - 1)) == 0;
        if (chunk_head && q + 1 < n_chunks) fetch_w(q + 1); // (workgroup-uniform) parked at the chunk's end
        uintx4 fx[2][4];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int tm = 0; tm < 4; ++tm) fx[hf][tm] = *reinterpret_cast<const uintx4*>(stage + xfrag[hf][tm]);
        __builtin_amdgcn_s_waitcnt(0xC07F);                 // lgkmcnt(0): the fragments are in registers, the stage is free
        if (step + 1 < n_steps) transfer();
        const uint16_t* wbuf = wres + (size_t)(q & 1) * CHUNK + (size_t)(2 * (c_t & (DDS_CK / 2 - 1))) * STEP + wfrag;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            if (2 * c_t + hf < nin) {                       // workgroup-uniform
                const uint16_t* wt = wbuf + (size_t)hf * STEP;
#pragma unroll
                for (int n = 0; n < 8; ++n) {
                    if (n < NT) {                           // workgroup-uniform
                        const uint4 fw = *reinterpret_cast<const uint4*>(wt + n * 512);
#pragma unroll
                        for (int tm = 0; tm < 4; ++tm)
                            acc[tm][n] = Frag32<T>::mma(__builtin_bit_cast(uint4, fx[hf][tm]), fw, acc[tm][n]);
                    }
                }
            }
        }
        bool chunk_end = false;
        if (++c_t == npair) { store_tile(c_tile); c_t = 0; ++c_tile; chunk_end = true; }
        else chunk_end = (c_t & (DDS_CK / 2 - 1)) == 0;
        if (chunk_end) {                                    // (workgroup-uniform)
            if (q + 1 < n_chunks) stash_w((q + 1) & 1);
            __syncthreads();
            ++q;
        }
    }
}

// ---------------------------------------------------------------------------------------
// fused block-sparse attention: out = softmax(scale * Q K^T + key mask) V over the nonzero blocks
// ---------------------------------------------------------------------------------------
// One pass for 32x32 blocks of a 2-byte type: the (Z, nnz, 32, 32) score and probability tensors of
// the SDD -> softmax -> DSD sequence never exist.  One workgroup per (batch, head, NW consecutive
// block-rows); wave w owns the 32 queries of block-row NW*group + w with their Q fragments in
// registers.  The workgroup walks the union of the rows' column lists; each step stages one 32 x D
// tile of K (row-major) and of V (transposed, [d][key slot]) in LDS, double-buffered, and every
// wave whose row holds that column forms S^T = K Q^T (rows = keys, columns = queries: a lane then
// owns one query per 16-column tile and its row statistics are lane scalars plus a 4-group
// butterfly), runs the online softmax in base 2, and accumulates O^T += V^T P with the
// probabilities going straight from the score registers into the MFMA operand: key 16kt + 4g + i
// sits in contraction slot 8g + 4kt + i, which is the order the V tile is transposed into.
struct AttnArgs {
    const void* q; const void* k; const void* v; void* out;
    const int32_t* uni_ptr; const int32_t* uni_inner; const int32_t* uni_blk;
    const float* kpm; long kpm_stride;
    int brows_per_head, grps_per_head, n_heads, Z;
    long q_sz, q_sh, q_sm, k_sz, k_sh, k_sn, v_sz, v_sh, v_sn, o_sz, o_sh, o_sm;
    float scale;
    float* lse2;        // optional (Z, H, 32 * brows_per_head): base-2 log of every row's softmax denominator
    int n_xcd;          // dies the dispatcher deals workgroup ids to (set where the kernel is launched)
    const float* am; long am_stride;     // optional (rows, cols) additive term per (query, key), shared by batch and heads
    // dropout of the probabilities (DROP kernels): element (z, head, query, key) is kept when the hash of
    // (seed, row = (z H + head) L + query, key) reaches the threshold; kept ones are scaled by 1 / (1 - p)
    uint32_t drop_seed, drop_thresh; float drop_scale;
};

// Maxima of scores.  A two-operand fmaxf costs three instructions here (each operand is first quieted
// by a self-maximum); three-operand maxima are emitted as they are, so pairs get -inf as a third.
__device__ __forceinline__ float max2_finite(float a, float b) { return fmaxf(fmaxf(a, b), -INFINITY); }
__device__ __forceinline__ float max8_finite(floatx4 a, floatx4 b) {
    const float m0 = fmaxf(fmaxf(a[0], a[1]), a[2]);
    const float m1 = fmaxf(fmaxf(m0, a[3]), b[0]);
    const float m2 = fmaxf(fmaxf(m1, b[1]), b[2]);
    return max2_finite(m2, b[3]);
}
__device__ __forceinline__ float group_max_finite(float v) {
    float a, b;
    rows_pair16(v, a, b); v = max2_finite(a, b);
    rows_pair32(v, a, b); return max2_finite(a, b);
}

// LDS image of a block-column's K and V tiles: rows of 2 D bytes without padding (a wave's direct-to-LDS load
// fills 1024 consecutive bytes), 16-byte chunks permuted within a row so that the fragment reads spread over the
// banks: the eight lanes of a 16-byte K read (eight consecutive keys, one chunk) and the sixteen lanes of a
// transposing V read (four consecutive keys, 32 bytes each) then cover a 128-byte line exactly.  Both maps are
// their own inverses.  CPR = chunks per row.
template <int CPR> __device__ __forceinline__ int attn_kslot(int row, int c) {
    constexpr int RPL = CPR >= 8 ? 1 : 8 / CPR;           // rows per 128-byte line
    return c ^ ((row / RPL) & (CPR - 1));
}
template <int CPR> __device__ __forceinline__ int attn_vslot(int row, int c) {
    constexpr int RPL = CPR >= 8 ? 1 : 8 / CPR;
    return c ^ ((((row / RPL) & 3) & (CPR / 2 - 1)) << 1);
}
template <typename T, int KS, int NW, bool MASKED, bool DROP = false>     // head dim 32*KS, NW block-rows (waves) per workgroup
__global__ __launch_bounds__(64 * NW) void bs_attn32_kernel(const AttnArgs a) {
    constexpr int D = 32 * KS, DT = D / 16, RB = 2 * D;   // RB: bytes of a tile row
    // block-columns per step: what 64 KB of LDS hold twice over -- half of that for workgroups of four waves at 64 dims,
    // of which a compute unit then holds four (the registers allow it) instead of two
    constexpr int CP = KS == 1 ? 4 : (KS == 2 && NW >= 8 ? 4 : 2);
    constexpr int CPR = D / 8;                            // 16-byte chunks per tile row
    constexpr int COLB = 64 * RB;                         // one column's image: rows 0..31 keys of K, 32..63 the same keys of V
    constexpr int U = COLB / 1024, NCH = (U + NW - 1) / NW;      // wave loads per column, and per wave
    constexpr float LOG2E = 1.4426950408889634f;
    // The running reference exponent of a query is only raised (and its accumulators rescaled) when
    // a block's maximum exceeds it by more than LAZY binary orders of magnitude; until then the
    // probabilities may exceed 1 (by at most 2^LAZY), which fp32 sums and 2-byte operands hold
    // without loss, and the result is the same quotient.
    constexpr float LAZY = 8.f;
    __shared__ __attribute__((aligned(1024))) char tiles[2][CP][COLB];
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    int unit, grp;
    if (!unit_of(blockIdx.x, a.n_xcd, a.grps_per_head, a.n_heads * a.Z, unit, grp)) return;
    const int z = unit / a.n_heads, head = unit % a.n_heads;
    const int ug = head * a.grps_per_head + grp;
    const int p0 = a.uni_ptr[ug], n = a.uni_ptr[ug + 1] - p0;
    const int bi = grp * NW + w;
    const bool have_row = bi < a.brows_per_head;
    const T* qp = reinterpret_cast<const T*>(a.q) + z * a.q_sz + head * a.q_sh +
                  (long)(min(bi, a.brows_per_head - 1) * 32 + r16) * a.q_sm + 8 * g;
    const T* kz = reinterpret_cast<const T*>(a.k) + z * a.k_sz + head * a.k_sh;
    const T* vz = reinterpret_cast<const T*>(a.v) + z * a.v_sz + head * a.v_sh;
    const float* kpm = a.kpm ? a.kpm + z * a.kpm_stride : nullptr;

    uintx4 fq[2][KS];                                     // B operand: query 16qt + r16, dims 32ks + 8g ..
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fq[qt][ks] = *reinterpret_cast<const uintx4*>(qp + 16 * qt * a.q_sm + 32 * ks);

    // staging: wave load x = w + NW i of a column fills bytes 1024 x .. of its image; this lane's 16 of them are
    // chunk slot `p` of image row `row`
    const T* src[NCH];           // the lane's chunk in block-column 0
    long src_step[NCH];          // elements from one block-column to the next (wave-uniform)
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int pos = 1024 * (w + NW * i) + 16 * lane, row = (pos / RB) & 63, p = (pos % RB) / 16;
        const bool is_k = 1024 * (w + NW * i) < 32 * RB;    // whole wave loads are K or V
        src[i] = is_k ? kz + (long)row * a.k_sn + 8 * attn_kslot<CPR>(row, p)
                      : vz + (long)(row - 32) * a.v_sn + 8 * attn_vslot<CPR>(row - 32, p);
        src_step[i] = is_k ? 32 * a.k_sn : 32 * a.v_sn;
    }
    auto fetch = [&](int j, int stage, int inner) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NCH; ++i)
            if (U % NW == 0 || w + NW * i < U) dma_to_lds(src[i] + inner * src_step[i], tiles[stage][j] + 1024 * (w + NW * i));
    };

    floatx4 o[DT][2];                                     // O^T[d = 16dt + 4g + i][query 16qt + r16]
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) { o[dt][0] = Frag<float>::zero(); o[dt][1] = Frag<float>::zero(); }
    float m_run[2] = {-INFINITY, -INFINITY};
    floatx4 lsum[2] = {Frag<float>::zero(), Frag<float>::zero()};      // every element: sum of the query's probabilities
    const uint32_t one2 = pack2<T>(1.f, 1.f);
    const uintx4 ones = {one2, one2, one2, one2};
    const float scale2 = a.scale * LOG2E;

    // S^T[key 16kt + 4g + i][query 16qt + r16] of the K tile at `tile`
    floatx4 sc[2][2];
    floatx4 amk[2][2];                                    // the attention-mask entries of sc (asked for with the scores)
    const float* amrow = (MASKED && a.am) ? a.am + (long)(min(bi, a.brows_per_head - 1) * 32 + r16) * a.am_stride + 4 * g : nullptr;
    uint32_t drop_row[2] = {0u, 0u};                      // DROP: hash of (seed, global row) of the lane's two queries
    if (DROP) {
        const uint32_t row0 = (uint32_t)(z * a.n_heads + head) * (uint32_t)(a.brows_per_head * 32) +
                              (uint32_t)(min(bi, a.brows_per_head - 1) * 32 + r16);
        drop_row[0] = drop_row_hash(a.drop_seed, row0);
        drop_row[1] = drop_row_hash(a.drop_seed, row0 + 16u);
    }
    auto score = [&](const char* tile, int inner) __attribute__((always_inline)) {
        if (MASKED && amrow) {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int qt = 0; qt < 2; ++qt)
                    amk[kt][qt] = *reinterpret_cast<const floatx4*>(amrow + 16 * qt * a.am_stride + (long)inner * 32 + 16 * kt);
        }
        uintx4 fk[2][KS];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                fk[kt][ks] = *reinterpret_cast<const uintx4*>(tile + (16 * kt + r16) * RB + 16 * attn_kslot<CPR>(16 * kt + r16, 4 * ks + g));
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                sc[kt][qt] = Frag<float>::zero();
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) sc[kt][qt] = mma32<T>(fk[kt][ks], fq[qt][ks], sc[kt][qt]);
            }
    };
    // DROP: the probabilities that go to the product with V, the dropped ones zeroed (the denominator sums all of them)
    auto dropped = [&](float (&e0)[4], float (&e1)[4], uint32_t row_hash, int inner) __attribute__((always_inline)) {
        const uint32_t col0 = (uint32_t)inner * 32u + 4u * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (!drop_keep(row_hash, col0 + i, a.drop_thresh)) e0[i] = 0.f;
            if (!drop_keep(row_hash, col0 + 16u + i, a.drop_thresh)) e1[i] = 0.f;
        }
        return uintx4{pack2<T>(e0[0], e0[1]), pack2<T>(e0[2], e0[3]), pack2<T>(e1[0], e1[1]), pack2<T>(e1[2], e1[3])};
    };
    // online softmax of sc and O^T += V^T P with the V tile that follows the K tile at `tile`; `inner` = its block-column
    auto soft_pv = [&](const char* tile, int inner) __attribute__((always_inline)) {
        // A operand: column d = 16dt + r16 of V, keys 4g .. 4g+3 and 16+4g .. 16+4g+3
        const int vrow = 4 * g + (r16 >> 2);
        const char* vp = tile + (32 + vrow) * RB + 8 * (r16 & 1);
        uintx4 fv[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const char* p0 = vp + 16 * attn_vslot<CPR>(vrow, 2 * dt + ((r16 & 3) >> 1));
            fv[dt] = lds_read_tr8(p0, p0 + 16 * RB);
        }
        uintx4 pb[2], pd[2];                              // probabilities, and (DROP) the kept ones
        if (!MASKED) {
            // scale > 0 and no mask: the maximum is taken on the raw scores and the scale rides in
            // the exponent's fma
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                const floatx4 s0 = sc[0][qt], s1 = sc[1][qt];
                const float mx = group_max_finite(max8_finite(s0, s1)) * scale2;
                if (__builtin_amdgcn_ballot_w64(mx > m_run[qt] + LAZY) != 0) {      // wave-uniform: some row maximum grew a lot
                    const float m_new = fmaxf(m_run[qt], mx);
                    const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_new);
                    m_run[qt] = m_new;
                    lsum[qt] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) o[dt][qt] *= alpha;
                }
                const float nm = -m_run[qt];
                float e0[4], e1[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    e0[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s0[i], scale2, nm));
                    e1[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s1[i], scale2, nm));
                }
                pb[qt] = uintx4{pack2<T>(e0[0], e0[1]), pack2<T>(e0[2], e0[3]), pack2<T>(e1[0], e1[1]), pack2<T>(e1[2], e1[3])};
                if (DROP) pd[qt] = dropped(e0, e1, drop_row[qt], inner);
            }
        } else {
            floatx4 mk[2] = {Frag<float>::zero(), Frag<float>::zero()};
            if (kpm) {
                const float* mp = kpm + (long)inner * 32 + 4 * g;
                mk[0] = *reinterpret_cast<const floatx4*>(mp) * LOG2E;
                mk[1] = *reinterpret_cast<const floatx4*>(mp + 16) * LOG2E;
            }
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                floatx4 t0 = sc[0][qt] * scale2 + mk[0], t1 = sc[1][qt] * scale2 + mk[1];
                if (amrow) { t0 += amk[0][qt] * LOG2E; t1 += amk[1][qt] * LOG2E; }
                float mx = fmaxf(fmaxf(fmaxf(t0[0], t0[1]), t0[2]), fmaxf(fmaxf(t0[3], t1[0]), t1[1]));
                mx = fmaxf(fmaxf(mx, t1[2]), t1[3]);
                mx = group_max(mx);
                if (__builtin_amdgcn_ballot_w64(mx > m_run[qt] + LAZY) != 0) {
                    const float m_new = fmaxf(m_run[qt], mx);
                    const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run[qt] - m_new);
                    m_run[qt] = m_new;
                    lsum[qt] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) o[dt][qt] *= alpha;
                }
                const float mref = (m_run[qt] == -INFINITY) ? 0.f : m_run[qt];     // all keys masked so far: p = 0
                float e0[4], e1[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    e0[i] = __builtin_amdgcn_exp2f(t0[i] - mref);
                    e1[i] = __builtin_amdgcn_exp2f(t1[i] - mref);
                }
                pb[qt] = uintx4{pack2<T>(e0[0], e0[1]), pack2<T>(e0[2], e0[3]), pack2<T>(e1[0], e1[1]), pack2<T>(e1[2], e1[3])};
                if (DROP) pd[qt] = dropped(e0, e1, drop_row[qt], inner);
            }
        }
        // the row sums come from the matrix pipe as well: a row of ones times the rounded probabilities
        lsum[0] = mma32<T>(ones, pb[0], lsum[0]);
        lsum[1] = mma32<T>(ones, pb[1], lsum[1]);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            o[dt][0] = mma32<T>(fv[dt], DROP ? pd[0] : pb[0], o[dt][0]);
            o[dt][1] = mma32<T>(fv[dt], DROP ? pd[1] : pb[1], o[dt][1]);
        }
    };

    // The index lists are read two steps (block-column) and one step (presence) ahead of their use,
    // so that no step waits for a table load.  A step: ask for the next step's tiles (they go into the
    // other stage, which every wave has finished reading before the last barrier), work through this
    // step's columns, wait for the own loads, barrier.
    const int n_steps = (n + CP - 1) / CP;
    int inner_cur[CP], inner_n1[CP], blk_cur[CP];
#pragma unroll
    for (int j = 0; j < CP; ++j) {
        inner_cur[j] = j < n ? a.uni_inner[p0 + j] : 0;
        inner_n1[j] = CP + j < n ? a.uni_inner[p0 + CP + j] : 0;
        blk_cur[j] = j < n ? a.uni_blk[(long)(p0 + j) * NW + w] : -1;
    }
    if (n > 0) {
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < n) fetch(j, 0, inner_cur[j]);
    }
    drain_loads();
    __syncthreads();
    for (int st = 0; st < n_steps; ++st) {
        const int s1 = CP * (st + 1), s2 = CP * (st + 2);
        int inner_n2[CP], blk_n1[CP];
#pragma unroll
        for (int j = 0; j < CP; ++j) {
            inner_n2[j] = s2 + j < n ? a.uni_inner[p0 + s2 + j] : 0;
            blk_n1[j] = s1 + j < n ? a.uni_blk[(long)(p0 + s1 + j) * NW + w] : -1;
        }
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (s1 + j < n) fetch(j, (st + 1) & 1, inner_n1[j]);
#pragma unroll
        for (int j = 0; j < CP; ++j) {
            if (have_row && blk_cur[j] >= 0) {
                score(tiles[st & 1][j], inner_cur[j]);
                soft_pv(tiles[st & 1][j], inner_cur[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < CP; ++j) {
            inner_cur[j] = inner_n1[j];
            inner_n1[j] = inner_n2[j];
            blk_cur[j] = blk_n1[j];
        }
        drain_loads();                                    // this wave's part of the next step's tiles has landed
        __syncthreads();
    }
    if (!have_row) return;
    T* op = reinterpret_cast<T*>(a.out) + z * a.o_sz + head * a.o_sh;
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        const float l = lsum[qt][0];
        float inv = l > 0.f ? 1.0f / l : 0.f;             // rows without a finite score come out as zeros
        if (DROP) inv *= a.drop_scale;
        T* row = op + ((long)bi * 32 + 16 * qt + r16) * a.o_sm + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) store4_f32(row + 16 * dt, o[dt][qt] * inv);
        if (a.lse2 && g == 0)       // a row without a finite score: +inf, so that 2^(score - lse2) is 0
            a.lse2[(((long)z * a.n_heads + head) * a.brows_per_head + bi) * 32 + 16 * qt + r16] =
                l > 0.f ? m_run[qt] + __log2f(l) : INFINITY;
    }
}

// ---------------------------------------------------------------------------------------
// row operations: one wave per row of a block-row
// ---------------------------------------------------------------------------------------
struct RowArgs {
    void* x; void* out;
    const int32_t* row_ptr; const int32_t* row_blk; const int32_t* row_col;
    int n_brow, brows_per_head, blk_shift;
    long x_sz;
    float scale;
    const float* kpm; long kpm_stride; int kpm_mul;
    const float* am; long am_stride; int am_mul;
    int op;
};

__device__ __forceinline__ float mask_term(float v, int mul) {
    if (!mul) return v;
    return v == 0.f ? -INFINITY : 0.f;
}

// value of element e (0 <= e < nb*blk) of the row, with scale and masks applied
template <typename T>
__device__ __forceinline__ float row_value(const RowArgs& a, const T* xz, int p0, int rl, int e, int z, int grow,
                                           long* addr) {
    const int BLK = 1 << a.blk_shift;
    const int bidx = e >> a.blk_shift, cl = e & (BLK - 1);
    const long off = (long)a.row_blk[p0 + bidx] * (BLK * BLK) + rl * BLK + cl;
    *addr = off;
    float v = Elem<T>::to_f32(xz[off]) * a.scale;
    if (a.kpm || a.am) {
        const long col = (long)a.row_col[p0 + bidx] * BLK + cl;
        if (a.kpm) v += mask_term(a.kpm[z * a.kpm_stride + col], a.kpm_mul);
        if (a.am) v += mask_term(a.am[grow * a.am_stride + col], a.am_mul);
    }
    return v;
}

template <typename T, int NREG>
__global__ __launch_bounds__(256) void bs_softmax_kernel(RowArgs a) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int BLK = 1 << a.blk_shift;
    const long R = (long)blockIdx.x * 4 + w;
    if (R >= (long)a.n_brow * BLK) return;
    const int brow = (int)(R >> a.blk_shift), rl = (int)(R & (BLK - 1));
    const int z = blockIdx.y;
    const int p0 = a.row_ptr[brow], nb = a.row_ptr[brow + 1] - p0;
    const int n = nb << a.blk_shift;
    const int grow = (brow % a.brows_per_head) * BLK + rl;
    T* xz = reinterpret_cast<T*>(a.x) + z * a.x_sz;

    float vals[NREG];
    long addr[NREG];
    float mx = -INFINITY;
#pragma unroll
    for (int it = 0; it < NREG; ++it) {
        const int e = lane + 64 * it;
        vals[it] = -INFINITY;
        addr[it] = 0;
        if (e < n) vals[it] = row_value<T>(a, xz, p0, rl, e, z, grow, &addr[it]);
        mx = fmaxf(mx, vals[it]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < NREG; ++it) {
        const int e = lane + 64 * it;
        if (e < n) { vals[it] = expf(vals[it] - mx); sum += vals[it]; }   // -inf - -inf = NaN, kept on purpose
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int it = 0; it < NREG; ++it) {
        const int e = lane + 64 * it;
        if (e < n) xz[addr[it]] = Elem<T>::from_f32(vals[it] * inv);
    }
}

// Fast path for 32x32 blocks of a 2-byte type: one workgroup per (block-row, 16-row half).  The
// 16 x 32 half of a block is 1 KiB of contiguous memory, which one wave moves with a single 16-byte
// load per lane (lane = 4*row + chunk of 8 columns); wave w owns blocks w, w+4, ... of the row and
// keeps them in registers (raw 2-byte form) across the max / sum / write passes, so HBM sees each
// element once in and once out.  Row statistics go quad -> wave (DPP) -> workgroup (LDS).
template <typename T, int MAXB, int NW>     // NW waves share a (block-row, 16-row half); wave w takes blocks w, w + NW, ...
__global__ __launch_bounds__(64 * NW) void bs_softmax32_kernel(RowArgs a) {
    constexpr float LOG2E = 1.4426950408889634f;
    __shared__ float red[2][NW][16];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, rl = lane >> 2, chunk = lane & 3;
    const int brow = blockIdx.x >> 1, row = (blockIdx.x & 1) * 16 + rl;       // row inside the block
    const int z = blockIdx.y;
    const int p0 = a.row_ptr[brow], nb = a.row_ptr[brow + 1] - p0;
    const int grow = (brow % a.brows_per_head) * 32 + row;
    T* xz = reinterpret_cast<T*>(a.x) + z * a.x_sz + row * 32 + chunk * 8;
    const bool masked = a.kpm || a.am;

    uint4 raw[MAXB];
    long off[MAXB];
#pragma unroll
    for (int it = 0; it < MAXB; ++it) {
        const int j = w + NW * it;
        off[it] = -1;
        if (j < nb) {
            off[it] = (long)a.row_blk[p0 + j] * 1024;
            // streamed once in, once out: nontemporal both ways
            const uintx4 t_ = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(xz + off[it]));
            raw[it] = make_uint4(t_[0], t_[1], t_[2], t_[3]);
        }
    }
    // element u (0..7) of block slot `it` as float, unscaled
    auto elem = [&](int it, int u) -> float {
        const uint32_t word = (&raw[it].x)[u >> 1];
        T e;
        *reinterpret_cast<uint16_t*>(&e) = (u & 1) ? (uint16_t)(word >> 16) : (uint16_t)(word & 0xffffu);
        return Elem<T>::to_f32(e);
    };
    // additive mask term of that element (masked launches only)
    auto mask_of = [&](int it, int u) -> float {
        const long col = (long)a.row_col[p0 + w + NW * it] * 32 + chunk * 8 + u;
        float v = 0.f;
        if (a.kpm) v += mask_term(a.kpm[z * a.kpm_stride + col], a.kpm_mul);
        if (a.am) v += mask_term(a.am[grow * a.am_stride + col], a.am_mul);
        return v;
    };
    // pass 1: row maximum of x*scale (+ masks)
    float mx = -INFINITY;
    if (!masked && a.scale > 0.f) {              // max commutes with a positive scale: one multiply per lane
#pragma unroll
        for (int it = 0; it < MAXB; ++it)
            if (off[it] >= 0)
#pragma unroll
                for (int u = 0; u < 8; ++u) mx = fmaxf(mx, elem(it, u));
        mx *= a.scale;
    } else {
#pragma unroll
        for (int it = 0; it < MAXB; ++it)
            if (off[it] >= 0)
#pragma unroll
                for (int u = 0; u < 8; ++u) mx = fmaxf(mx, elem(it, u) * a.scale + (masked ? mask_of(it, u) : 0.f));
    }
    mx = fmaxf(mx, __shfl_xor(mx, 1));
    mx = fmaxf(mx, __shfl_xor(mx, 2));
    if (chunk == 0) red[0][w][rl] = mx;
    __syncthreads();
    mx = red[0][0][rl];
#pragma unroll
    for (int ww = 1; ww < NW; ++ww) mx = fmaxf(mx, red[0][ww][rl]);
    // pass 2: exponentials (kept as floats in registers) and their sum; -inf - -inf = NaN, kept
    const float mx2 = mx * LOG2E, scale2 = a.scale * LOG2E;
    float ev[MAXB][8];
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < MAXB; ++it)
        if (off[it] >= 0)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                float arg = elem(it, u) * scale2 - mx2;
                if (masked) arg += mask_of(it, u) * LOG2E;
                ev[it][u] = __builtin_amdgcn_exp2f(arg);
                sum += ev[it][u];
            }
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    if (chunk == 0) red[1][w][rl] = sum;
    __syncthreads();
    sum = red[1][0][rl];
#pragma unroll
    for (int ww = 1; ww < NW; ++ww) sum += red[1][ww][rl];
    const float inv = 1.0f / sum;
    // pass 3: normalise, round once, store
#pragma unroll
    for (int it = 0; it < MAXB; ++it)
        if (off[it] >= 0) {
            uint32_t outw[4];
#pragma unroll
            for (int u2 = 0; u2 < 4; ++u2) {
                T lo = Elem<T>::from_f32(ev[it][2 * u2] * inv);
                T hi = Elem<T>::from_f32(ev[it][2 * u2 + 1] * inv);
                outw[u2] = (uint32_t)*reinterpret_cast<uint16_t*>(&lo) | ((uint32_t)*reinterpret_cast<uint16_t*>(&hi) << 16);
            }
            __builtin_nontemporal_store(uintx4{outw[0], outw[1], outw[2], outw[3]}, reinterpret_cast<uintx4*>(xz + off[it]));
        }
}

// Backward of the block softmax for 32x32 blocks of a 2-byte type, one pass: dx = scale * y * (dy - sum_row(dy * y)).
// Same work split as bs_softmax32_kernel (workgroup per (block-row, 16-row half), wave w takes blocks
// w, w+NW, ...; a lane holds 8 consecutive elements of one row per block): y and dy stay in registers
// in their 2-byte form between the row sum and the result, so HBM sees two reads and one write.
struct RowBwdArgs {
    const void* y; const void* dy; void* dx;
    const int32_t* row_ptr; const int32_t* row_blk;
    long y_sz;
    float scale;
};

template <typename T, int MAXB, int NW>
__global__ __launch_bounds__(64 * NW) void bs_softmax32_bwd_kernel(RowBwdArgs a) {
    __shared__ float red[NW][16];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, rl = lane >> 2, chunk = lane & 3;
    const int brow = blockIdx.x >> 1, row = (blockIdx.x & 1) * 16 + rl;
    const int z = blockIdx.y;
    const int p0 = a.row_ptr[brow], nb = a.row_ptr[brow + 1] - p0;
    const long base = z * a.y_sz + row * 32 + chunk * 8;
    const T* yz = reinterpret_cast<const T*>(a.y) + base;
    const T* dz = reinterpret_cast<const T*>(a.dy) + base;
    T* xz = reinterpret_cast<T*>(a.dx) + base;

    uintx4 ry[MAXB], rd[MAXB];
    int blk[MAXB];
#pragma unroll
    for (int it = 0; it < MAXB; ++it) {
        const int j = w + NW * it;
        blk[it] = -1;
        if (j < nb) {
            blk[it] = a.row_blk[p0 + j];
            ry[it] = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(yz + (long)blk[it] * 1024));
            rd[it] = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(dz + (long)blk[it] * 1024));
        }
    }
    auto elem = [&](uint32_t word, int hi) -> float {
        T e;
        *reinterpret_cast<uint16_t*>(&e) = hi ? (uint16_t)(word >> 16) : (uint16_t)(word & 0xffffu);
        return Elem<T>::to_f32(e);
    };
    float s = 0.f;
#pragma unroll
    for (int it = 0; it < MAXB; ++it)
        if (blk[it] >= 0)
#pragma unroll
            for (int u = 0; u < 8; ++u) s += elem(ry[it][u >> 1], u & 1) * elem(rd[it][u >> 1], u & 1);
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    if (chunk == 0) red[w][rl] = s;
    __syncthreads();
    s = red[0][rl];
#pragma unroll
    for (int ww = 1; ww < NW; ++ww) s += red[ww][rl];
#pragma unroll
    for (int it = 0; it < MAXB; ++it)
        if (blk[it] >= 0) {
            uint32_t outw[4];
#pragma unroll
            for (int u2 = 0; u2 < 4; ++u2) {
                const float lo = a.scale * elem(ry[it][u2], 0) * (elem(rd[it][u2], 0) - s);
                const float hi = a.scale * elem(ry[it][u2], 1) * (elem(rd[it][u2], 1) - s);
                outw[u2] = pack2<T>(lo, hi);
            }
            __builtin_nontemporal_store(uintx4{outw[0], outw[1], outw[2], outw[3]},
                                        reinterpret_cast<uintx4*>(xz + (long)blk[it] * 1024));
        }
}

// rows longer than the register budget: three passes over the row
template <typename T>
__global__ __launch_bounds__(256) void bs_softmax_long_kernel(RowArgs a) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int BLK = 1 << a.blk_shift;
    const long R = (long)blockIdx.x * 4 + w;
    if (R >= (long)a.n_brow * BLK) return;
    const int brow = (int)(R >> a.blk_shift), rl = (int)(R & (BLK - 1));
    const int z = blockIdx.y;
    const int p0 = a.row_ptr[brow], nb = a.row_ptr[brow + 1] - p0;
    const int n = nb << a.blk_shift;
    const int grow = (brow % a.brows_per_head) * BLK + rl;
    T* xz = reinterpret_cast<T*>(a.x) + z * a.x_sz;
    long addr;
    float mx = -INFINITY;
    for (int e = lane; e < n; e += 64) mx = fmaxf(mx, row_value<T>(a, xz, p0, rl, e, z, grow, &addr));
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < n; e += 64) sum += expf(row_value<T>(a, xz, p0, rl, e, z, grow, &addr) - mx);
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    for (int e = lane; e < n; e += 64) {
        const float v = expf(row_value<T>(a, xz, p0, rl, e, z, grow, &addr) - mx) * inv;
        xz[addr] = Elem<T>::from_f32(v);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void bs_rowreduce_kernel(RowArgs a) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int BLK = 1 << a.blk_shift;
    const long R = (long)blockIdx.x * 4 + w;
    if (R >= (long)a.n_brow * BLK) return;
    const int brow = (int)(R >> a.blk_shift), rl = (int)(R & (BLK - 1));
    const int z = blockIdx.y;
    const int p0 = a.row_ptr[brow], nb = a.row_ptr[brow + 1] - p0;
    const int n = nb << a.blk_shift;
    const T* xz = reinterpret_cast<const T*>(a.x) + z * a.x_sz;
    T* out = reinterpret_cast<T*>(a.out) + (long)z * a.n_brow * BLK + R;
    float res = 0.f;
    if (n > 0) {
        if (a.op == 1) {
            float s = 0.f;
            for (int e = lane; e < n; e += 64)
                s += Elem<T>::to_f32(xz[(long)a.row_blk[p0 + (e >> a.blk_shift)] * (BLK * BLK) + rl * BLK + (e & (BLK - 1))]);
            res = wave_sum(s);
        } else {
            float mx = -INFINITY;
            for (int e = lane; e < n; e += 64)
                mx = fmaxf(mx, Elem<T>::to_f32(xz[(long)a.row_blk[p0 + (e >> a.blk_shift)] * (BLK * BLK) + rl * BLK + (e & (BLK - 1))]));
            mx = wave_max(mx);
            float s = 0.f;
            for (int e = lane; e < n; e += 64)
                s += expf(Elem<T>::to_f32(xz[(long)a.row_blk[p0 + (e >> a.blk_shift)] * (BLK * BLK) + rl * BLK + (e & (BLK - 1))]) - mx);
            s = wave_sum(s);
            res = (mx == -INFINITY) ? -INFINITY : mx + logf(s);
        }
    }
    if (lane == 0) *out = Elem<T>::from_f32(res);
}

// ---------------------------------------------------------------------------------------
// host side dispatch
// ---------------------------------------------------------------------------------------
static int blk_shift_of(int blk) {
    switch (blk) { case 16: return 4; case 32: return 5; case 64: return 6; case 128: return 7; default: return -1; }
}

#define BS_DISPATCH_BLK(KERN, T, GRID, ARGS)                                               \
    switch (blk) {                                                                         \
        case 16: hipLaunchKernelGGL((KERN<T, 16>), GRID, dim3(256), 0, st, ARGS); break;   \
        case 32: hipLaunchKernelGGL((KERN<T, 32>), GRID, dim3(256), 0, st, ARGS); break;   \
        case 64: hipLaunchKernelGGL((KERN<T, 64>), GRID, dim3(256), 0, st, ARGS); break;   \
        case 128: hipLaunchKernelGGL((KERN<T, 128>), GRID, dim3(256), 0, st, ARGS); break; \
    }
#define BS_DISPATCH(KERN, GRID, ARGS)                                                      \
    switch (dtype) {                                                                       \
        case F32: BS_DISPATCH_BLK(KERN, float, GRID, ARGS) break;                          \
        case BF16: BS_DISPATCH_BLK(KERN, bf16_t, GRID, ARGS) break;                        \
        case F16: BS_DISPATCH_BLK(KERN, f16_t, GRID, ARGS) break;                          \
    }

static long waves_to_blocks(long waves) { return (waves + 3) / 4; }

}  // namespace flyhip

using namespace flyhip;

static int check_common(const char* who, int blk, int dtype, int Z) {
    FLY_REQUIRE(blk_shift_of(blk) >= 0, "%s: block size %d not in {16,32,64,128}", who, blk);
    FLY_REQUIRE(dtype == F32 || dtype == BF16 || dtype == F16, "%s: unknown dtype code %d", who, dtype);
    FLY_REQUIRE(Z >= 1 && Z <= 65535, "%s: batch %d outside [1, 65535]", who, Z);
    return OK;
}

extern "C" int flyhip_bs_sdd(const void* a, const void* b, void* c, const int32_t* lut, int nnz,
                             const int32_t* row_ptr, const int32_t* row_blk, const int32_t* row_col,
                             int n_brow, int brows_per_head,
                             const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                             int Z, int K, int blk,
                             int64_t a_sz, int64_t a_sh, int64_t a_sm, int64_t a_sk,
                             int64_t b_sz, int64_t b_sh, int64_t b_sn, int64_t b_sk,
                             int dtype, void* stream) {
    int rc = check_common("bs_sdd", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(a && b && c && lut, "bs_sdd: null pointer");
    FLY_REQUIRE(nnz >= 0, "bs_sdd: negative nnz");
    FLY_REQUIRE(K > 0 && K % 16 == 0, "bs_sdd: reduction size %d must be a positive multiple of 16", K);
    if (a_sk == 1) FLY_REQUIRE(((a_sz | a_sh | a_sm) % 4) == 0, "bs_sdd: A strides must be multiples of 4 elements");
    if (b_sk == 1) FLY_REQUIRE(((b_sz | b_sh | b_sn) % 4) == 0, "bs_sdd: B strides must be multiples of 4 elements");
    if (nnz == 0) return OK;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    if (row_ptr && row_blk && row_col && blk == 32 && (dtype == BF16 || dtype == F16) && a_sk == 1 && b_sk == 1 &&
        K % 32 == 0 && K <= 128 && ((a_sz | a_sh | a_sm | b_sz | b_sh | b_sn) % 8) == 0 && n_brow > 0 &&
        brows_per_head > 0) {
        FLY_REQUIRE(n_brow % brows_per_head == 0, "bs_sdd: %d block-rows do not divide into heads of %d", n_brow, brows_per_head);
        const int n_heads = n_brow / brows_per_head;
        if (uni_ptr && uni_inner && uni_blk) {
            const int gph = (brows_per_head + 3) / 4;
            SddUniArgs ua{a, b, c, uni_ptr, uni_inner, uni_blk, nnz, brows_per_head, gph, n_heads, Z,
                          a_sz, a_sh, a_sm, b_sz, b_sh, b_sn, nullptr, nullptr, 1.f};
            const long nwg = unit_grid((long)n_heads * Z, gph);
            ua.n_xcd = machine().xcds;
            FLY_REQUIRE(nwg <= 2147483647L, "bs_sdd: too many workgroups");
            dim3 grid((unsigned)nwg);
#define SDD32U_LAUNCH(T)                                                                         \
            switch (K / 32) {                                                                    \
                case 1: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 1>), grid, dim3(256), 0, st, ua); break; \
                case 2: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 2>), grid, dim3(256), 0, st, ua); break; \
                case 3: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 3>), grid, dim3(256), 0, st, ua); break; \
                default: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 4>), grid, dim3(256), 0, st, ua); break; \
            }
            if (dtype == BF16) { SDD32U_LAUNCH(bf16_t) } else { SDD32U_LAUNCH(f16_t) }
#undef SDD32U_LAUNCH
            return check_launch("bs_sdd32u_kernel");
        }
        SddRowArgs ra{a, b, c, row_ptr, row_blk, row_col, nnz, K, brows_per_head, n_heads, Z, a_sz, a_sh, a_sm, b_sz, b_sh, b_sn};
        const long nwg = unit_grid((long)n_heads * Z, (brows_per_head + 3) / 4);
        ra.n_xcd = machine().xcds;
        FLY_REQUIRE(nwg <= 2147483647L, "bs_sdd: too many workgroups");
        dim3 grid((unsigned)nwg);
#define SDD32_LAUNCH(T)                                                                         \
        switch (K / 32) {                                                                       \
            case 1: hipLaunchKernelGGL((bs_sdd32_kernel<T, 1>), grid, dim3(256), 0, st, ra); break; \
            case 2: hipLaunchKernelGGL((bs_sdd32_kernel<T, 2>), grid, dim3(256), 0, st, ra); break; \
            case 3: hipLaunchKernelGGL((bs_sdd32_kernel<T, 3>), grid, dim3(256), 0, st, ra); break; \
            default: hipLaunchKernelGGL((bs_sdd32_kernel<T, 4>), grid, dim3(256), 0, st, ra); break; \
        }
        if (dtype == BF16) { SDD32_LAUNCH(bf16_t) } else { SDD32_LAUNCH(f16_t) }
#undef SDD32_LAUNCH
        return check_launch("bs_sdd32_kernel");
    }
    SddArgs args{a, b, c, lut, nnz, K, a_sz, a_sh, a_sm, a_sk, b_sz, b_sh, b_sn, b_sk};
    const int tile = blk >= 32 ? 32 : 16, sub = blk / tile;
    const long nblocks = waves_to_blocks((long)nnz * sub * sub);
    FLY_REQUIRE(nblocks <= 2147483647L, "bs_sdd: too many blocks");
    dim3 grid((unsigned)nblocks, Z);
    BS_DISPATCH(bs_sdd_kernel, grid, args)
    return check_launch("bs_sdd_kernel");
}

template <int EPI>
static int launch_sdd_epilogue(const char* what, const void* a_dn, const void* b_dn, const void* p, const float* rowvec, void* c,
                               const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                               int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                               int64_t a_sz, int64_t a_sh, int64_t a_sm, int64_t b_sz, int64_t b_sh, int64_t b_sn,
                               float scale, int dtype, void* stream, const SddUniArgs* second = nullptr) {
    int rc = check_common(what, blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(a_dn && b_dn && (EPI != 1 || p) && (rowvec || (EPI == 3 && second && second->out)) && c && uni_ptr &&
                uni_inner && uni_blk, "%s: null pointer", what);
    FLY_REQUIRE(blk == 32 && (dtype == BF16 || dtype == F16), "%s: needs 32x32 blocks of bf16 / fp16", what);
    FLY_REQUIRE(K % 32 == 0 && K >= 32 && K <= 128, "%s: head dim %d not a multiple of 32 up to 128", what, K);
    FLY_REQUIRE(nnz > 0 && n_heads > 0 && brows_per_head > 0, "%s: bad sizes", what);
    FLY_REQUIRE(((a_sz | a_sh | a_sm | b_sz | b_sh | b_sn) % 8) == 0, "%s: strides must be multiples of 8 elements", what);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    const int gph = (brows_per_head + 3) / 4;
    SddUniArgs ua{a_dn, b_dn, c, uni_ptr, uni_inner, uni_blk, nnz, brows_per_head, gph, n_heads, Z,
                  a_sz, a_sh, a_sm, b_sz, b_sh, b_sn, p, rowvec, scale};
    if (EPI == 3) {
        FLY_REQUIRE(second && second->a2 && second->b2 && second->lse2 && second->p2, "%s: null pointer", what);
        FLY_REQUIRE(((second->a2_sz | second->a2_sh | second->a2_sm | second->b2_sz | second->b2_sh | second->b2_sn) % 8) == 0,
                    "%s: strides must be multiples of 8 elements", what);
        ua.a2 = second->a2; ua.b2 = second->b2; ua.lse2 = second->lse2; ua.p2 = second->p2; ua.scale2 = second->scale2;
        ua.a2_sz = second->a2_sz; ua.a2_sh = second->a2_sh; ua.a2_sm = second->a2_sm;
        ua.b2_sz = second->b2_sz; ua.b2_sh = second->b2_sh; ua.b2_sn = second->b2_sn;
        FLY_REQUIRE(second->dq && ((second->dq_sz | second->dq_sh | second->dq_sm) % 4) == 0,
                    "%s: dq missing or its strides are not multiples of 4 elements", what);
        ua.dq = second->dq; ua.dq_sz = second->dq_sz; ua.dq_sh = second->dq_sh; ua.dq_sm = second->dq_sm;
        FLY_REQUIRE(!second->out || ((second->o_sz | second->o_sh | second->o_sm) % 8) == 0,
                    "%s: out strides must be multiples of 8 elements", what);
        ua.out = second->out; ua.o_sz = second->o_sz; ua.o_sh = second->o_sh; ua.o_sm = second->o_sm;
    }
    const long nwg = unit_grid((long)n_heads * Z, gph);
    ua.n_xcd = machine().xcds;
    FLY_REQUIRE(nwg <= 2147483647L, "%s: too many workgroups", what);
    dim3 grid((unsigned)nwg);
#define SDDS_LAUNCH(T)                                                                                  \
    switch (K / 32) {                                                                                   \
        case 1: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 1, EPI>), grid, dim3(256), 0, st, ua); break;  \
        case 2: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 2, EPI>), grid, dim3(256), 0, st, ua); break;  \
        case 3: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 3, EPI>), grid, dim3(256), 0, st, ua); break;  \
        default: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 4, EPI>), grid, dim3(256), 0, st, ua); break; \
    }
    if constexpr (EPI == 3) {
        if (second->drop_thresh != 0u) {
            ua.drop_seed = second->drop_seed; ua.drop_thresh = second->drop_thresh; ua.drop_scale = second->drop_scale;
            FLY_REQUIRE((long)Z * n_heads * brows_per_head * 32 <= 4294967295L, "%s: more than 2^32 rows", what);
#define SDDS_DROP_LAUNCH(T)                                                                                   \
    switch (K / 32) {                                                                                         \
        case 1: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 1, 3, true>), grid, dim3(256), 0, st, ua); break;    \
        case 2: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 2, 3, true>), grid, dim3(256), 0, st, ua); break;    \
        case 3: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 3, 3, true>), grid, dim3(256), 0, st, ua); break;    \
        default: hipLaunchKernelGGL((bs_sdd32u_kernel<T, 4, 3, true>), grid, dim3(256), 0, st, ua); break;   \
    }
            if (dtype == BF16) { SDDS_DROP_LAUNCH(bf16_t) } else { SDDS_DROP_LAUNCH(f16_t) }
#undef SDDS_DROP_LAUNCH
            return check_launch(what);
        }
    }
    if (dtype == BF16) { SDDS_LAUNCH(bf16_t) } else { SDDS_LAUNCH(f16_t) }
#undef SDDS_LAUNCH
    return check_launch(what);
}

extern "C" int flyhip_bs_sdd_dsoftmax(const void* dout, const void* v, const void* p, const float* delta, void* ds,
                                      const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                                      int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                                      int64_t a_sz, int64_t a_sh, int64_t a_sm,
                                      int64_t b_sz, int64_t b_sh, int64_t b_sn,
                                      float scale, int dtype, void* stream) {
    return launch_sdd_epilogue<1>("bs_sdd_dsoftmax", dout, v, p, delta, ds, uni_ptr, uni_inner, uni_blk, nnz, n_heads,
                                  brows_per_head, Z, K, blk, a_sz, a_sh, a_sm, b_sz, b_sh, b_sn, scale, dtype, stream);
}

extern "C" int flyhip_bs_sdd_prob_dsoftmax_dropout(const void* dout, const void* v, const void* q, const void* k,
                                           const float* delta, const void* out, const float* lse2, void* ds, void* p, void* dq,
                                           const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                                           int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                                           int64_t do_sz, int64_t do_sh, int64_t do_sm,
                                           int64_t v_sz, int64_t v_sh, int64_t v_sn,
                                           int64_t q_sz, int64_t q_sh, int64_t q_sm,
                                           int64_t k_sz, int64_t k_sh, int64_t k_sn,
                                           int64_t dq_sz, int64_t dq_sh, int64_t dq_sm,
                                           int64_t o_sz, int64_t o_sh, int64_t o_sm,
                                           float scale, int dtype, float dropout_p, uint64_t dropout_seed, void* stream);

extern "C" int flyhip_bs_sdd_prob_dsoftmax(const void* dout, const void* v, const void* q, const void* k,
                                           const float* delta, const void* out, const float* lse2, void* ds, void* p, void* dq,
                                           const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                                           int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                                           int64_t do_sz, int64_t do_sh, int64_t do_sm,
                                           int64_t v_sz, int64_t v_sh, int64_t v_sn,
                                           int64_t q_sz, int64_t q_sh, int64_t q_sm,
                                           int64_t k_sz, int64_t k_sh, int64_t k_sn,
                                           int64_t dq_sz, int64_t dq_sh, int64_t dq_sm,
                                           int64_t o_sz, int64_t o_sh, int64_t o_sm,
                                           float scale, int dtype, void* stream) {
    return flyhip_bs_sdd_prob_dsoftmax_dropout(dout, v, q, k, delta, out, lse2, ds, p, dq, uni_ptr, uni_inner, uni_blk, nnz,
                                               n_heads, brows_per_head, Z, K, blk, do_sz, do_sh, do_sm, v_sz, v_sh, v_sn,
                                               q_sz, q_sh, q_sm, k_sz, k_sh, k_sn, dq_sz, dq_sh, dq_sm, o_sz, o_sh, o_sm,
                                               scale, dtype, 0.f, 0, stream);
}

extern "C" int flyhip_bs_sdd_prob_dsoftmax_dropout(const void* dout, const void* v, const void* q, const void* k,
                                           const float* delta, const void* out, const float* lse2, void* ds, void* p, void* dq,
                                           const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                                           int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                                           int64_t do_sz, int64_t do_sh, int64_t do_sm,
                                           int64_t v_sz, int64_t v_sh, int64_t v_sn,
                                           int64_t q_sz, int64_t q_sh, int64_t q_sm,
                                           int64_t k_sz, int64_t k_sh, int64_t k_sn,
                                           int64_t dq_sz, int64_t dq_sh, int64_t dq_sm,
                                           int64_t o_sz, int64_t o_sh, int64_t o_sm,
                                           float scale, int dtype, float dropout_p, uint64_t dropout_seed, void* stream) {
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "bs_sdd_prob_dsoftmax: dropout_p %g not in [0, 1)", (double)dropout_p);
    SddUniArgs second{};
    const DropArgs drop = drop_args(dropout_p, dropout_seed);
    second.drop_seed = drop.seed; second.drop_thresh = drop.thresh; second.drop_scale = drop.scale;
    second.out = out; second.o_sz = o_sz; second.o_sh = o_sh; second.o_sm = o_sm;
    second.dq = dq; second.dq_sz = dq_sz; second.dq_sh = dq_sh; second.dq_sm = dq_sm;
    second.a2 = q; second.b2 = k; second.lse2 = lse2; second.p2 = p; second.scale2 = scale * 1.4426950408889634f;
    second.a2_sz = q_sz; second.a2_sh = q_sh; second.a2_sm = q_sm;
    second.b2_sz = k_sz; second.b2_sh = k_sh; second.b2_sn = k_sn;
    return launch_sdd_epilogue<3>("bs_sdd_prob_dsoftmax", dout, v, nullptr, delta, ds, uni_ptr, uni_inner, uni_blk, nnz,
                                  n_heads, brows_per_head, Z, K, blk, do_sz, do_sh, do_sm, v_sz, v_sh, v_sn, scale, dtype,
                                  stream, &second);
}

// ---------------------------------------------------------------------------------------
// gradients of the one-kernel block-sparse attention without the probabilities in memory
// ---------------------------------------------------------------------------------------
// With P = 2^(scale log2e q.k - lse2[query]) on the nonzero 32 x 32 blocks, g = d out and delta = rowsum(g * out):
// d v = P^T g, dS = P (g v^T - delta), d q = scale dS k, d k = scale dS^T q.  One kernel in two orientations, neither
// of which writes P or dS: a workgroup owns four block-rows (query-major: d q, and delta on the way) or four
// block-columns (key-major: d k and d v), a wave one of them with its two operands in registers (q and g rows; k and v
// rows), and walks the union of their lists (union_table, transposed for key-major), every 32-row tile of the other
// side (K with V; Q with g, lse2 and delta) staged once in LDS for the four waves.  Per block S^T = Y1 . x1 and
// G^T = Y2 . x2 (the tile's rows picked so that a lane's results over the two 16-row blocks are eight consecutive
// inner rows, the contraction slots of what follows), then d x^T[e][outer] += Y^T[e][inner] . {dS, P}[inner][outer]
// with Y^T fragments by transposing LDS reads of the same tiles.
struct AttnBwdArgs {
    const void* q; const void* k; const void* v; const void* go; const void* out;
    const float* lse2; float* delta;                 // (Z, H, 32 * query blocks); delta is written by the query-major launch
    void* dq; void* dk; void* dv;
    const int32_t* uni_ptr; const int32_t* uni_inner; const int32_t* uni_blk;      // of the launch's orientation
    int outer_blocks, inner_blocks, q_blocks, grps_per_head, n_heads, Z;
    long q_sz, q_sh, q_sm, k_sz, k_sh, k_sm, v_sz, v_sh, v_sm, g_sz, g_sh, g_sm, o_sz, o_sh, o_sm;
    long dq_sz, dq_sh, dq_sm, dk_sz, dk_sh, dk_sm, dv_sz, dv_sh, dv_sm;
    float scale;
    int n_xcd;
    // DROP: the forward dropped probabilities by the hash of (seed, row = (z H + head) L + query, key) (drop_keep): d v takes
    // m P and dS = P (m g.v - delta), m = 0 or 1 / (1 - p)
    uint32_t drop_seed, drop_thresh; float drop_scale;
    // the forward's additive masks (flyhip_bs_attn_masks), optional: key_mask (Z, keys) and attn_mask (queries, keys),
    // float32, added to scale * q.k (0 / -inf, or any finite bias)
    const float* key_mask; long km_stride; const float* attn_mask; long am_stride;
};

// (registers for three waves per SIMD: the key-major form at 64 dims takes 176 without the bound, two waves per SIMD,
//  and runs 7 % slower; with the dropout hashes it would spill 24 registers inside the loop at that bound -- 703 us
//  against 365 without dropout -- and keeps two waves; a two-step register prefetch of the tiles costs more registers
//  than it hides latency)
// MASKED: a variant of its own, so that the kernels without masks carry nothing of them (as a kernel-uniform branch the
// mask code cost the key-major form 35 more spilled registers and the query-major form a wave per SIMD)
template <typename T, int E, bool KEYMAJOR, bool DROP = false, bool MASKED = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(KEYMAJOR && (DROP || MASKED) ? 2 : 3, 8))) void bs_attn32_bwd_kernel(const AttnBwdArgs a) {
    static_assert(!(DROP && MASKED), "the forward with masks has no dropout");
    static_assert(sizeof(T) == 2 && E % 32 == 0, "2-byte inputs, whole MFMA steps");
    constexpr int LD = E + 8, KS = E / 32, EB = E / 16;
    constexpr int CPR = E / 8, NCH = (32 * CPR + 255) / 256;        // 16-byte chunks per tile row, per thread
    constexpr float LOG2E = 1.4426950408889634f;
    __shared__ __attribute__((aligned(16))) uint16_t tiles[2][2][32 * LD];      // [stage][Y1 | Y2]
    __shared__ __attribute__((aligned(16))) float rowv[2][3][32];              // key-major: [stage][lse2 | delta | row hash] of the tile's queries
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    int unit, grp;
    if (!unit_of(blockIdx.x, a.n_xcd, a.grps_per_head, a.n_heads * a.Z, unit, grp)) return;
    const int z = unit / a.n_heads, head = unit % a.n_heads;
    const int ug = head * a.grps_per_head + grp;
    const int p0 = a.uni_ptr[ug], n = a.uni_ptr[ug + 1] - p0;
    const int bo = grp * 4 + w;
    const bool have = bo < a.outer_blocks;
    const int bo_c = min(bo, a.outer_blocks - 1);
    const uint16_t* qz = reinterpret_cast<const uint16_t*>(a.q) + z * a.q_sz + head * a.q_sh;
    const uint16_t* kz = reinterpret_cast<const uint16_t*>(a.k) + z * a.k_sz + head * a.k_sh;
    const uint16_t* vz = reinterpret_cast<const uint16_t*>(a.v) + z * a.v_sz + head * a.v_sh;
    const uint16_t* gz = reinterpret_cast<const uint16_t*>(a.go) + z * a.g_sz + head * a.g_sh;
    const uint16_t* x1p = KEYMAJOR ? kz : qz;  const long x1s = KEYMAJOR ? a.k_sm : a.q_sm;     // outer operands
    const uint16_t* x2p = KEYMAJOR ? vz : gz;  const long x2s = KEYMAJOR ? a.v_sm : a.g_sm;
    const uint16_t* y1p = KEYMAJOR ? qz : kz;  const long y1s = KEYMAJOR ? a.q_sm : a.k_sm;     // inner tiles
    const uint16_t* y2p = KEYMAJOR ? gz : vz;  const long y2s = KEYMAJOR ? a.g_sm : a.v_sm;
    const long qvec = ((long)z * a.n_heads + head) * a.q_blocks * 32;                          // row vectors of this (z, head)
    T* d1 = KEYMAJOR ? reinterpret_cast<T*>(a.dk) + z * a.dk_sz + head * a.dk_sh : reinterpret_cast<T*>(a.dq) + z * a.dq_sz + head * a.dq_sh;
    const long d1s = KEYMAJOR ? a.dk_sm : a.dq_sm;
    T* d2 = reinterpret_cast<T*>(a.dv) + z * a.dv_sz + head * a.dv_sh;

    uintx4 x1[2][KS], x2[2][KS];
    float l_own[2] = {0.f, 0.f}, d_own[2] = {0.f, 0.f};
    float km_own[2] = {0.f, 0.f};                     // key-major: the key mask entries of the lane's keys
    uint32_t h_own[2] = {0u, 0u};                     // DROP, query-major: hash of (seed, global row) of the lane's queries
    floatx4 acc1[2][EB], acc2[KEYMAJOR ? 2 : 1][KEYMAJOR ? EB : 1];     // d q | d k, and d v
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
        const long row = (long)bo_c * 32 + 16 * qq + r16;
#pragma unroll
        for (int c = 0; c < KS; ++c) {
            x1[qq][c] = *reinterpret_cast<const uintx4*>(x1p + row * x1s + 32 * c + 8 * g);
            x2[qq][c] = *reinterpret_cast<const uintx4*>(x2p + row * x2s + 32 * c + 8 * g);
        }
        if (MASKED && KEYMAJOR && a.key_mask) km_own[qq] = a.key_mask[z * a.km_stride + row];
        if (!KEYMAJOR) {
            l_own[qq] = a.lse2[qvec + row];
            if (DROP) h_own[qq] = drop_row_hash(a.drop_seed, (uint32_t)(qvec + row));
            // delta of the query, g . out, from the output row in the layout of the gradient row; kept for the key-major launch
            const uint16_t* orow = reinterpret_cast<const uint16_t*>(a.out) + z * a.o_sz + head * a.o_sh + row * a.o_sm;
            float part = 0.f;
#pragma unroll
            for (int c = 0; c < KS; ++c) {
                const uintx4 ov = *reinterpret_cast<const uintx4*>(orow + 32 * c + 8 * g);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    T x, y;
                    *reinterpret_cast<uint16_t*>(&x) = (uint16_t)(x2[qq][c][e >> 1] >> (16 * (e & 1)));
                    *reinterpret_cast<uint16_t*>(&y) = (uint16_t)(ov[e >> 1] >> (16 * (e & 1)));
                    part += Elem<T>::to_f32(x) * Elem<T>::to_f32(y);
                }
            }
            d_own[qq] = group_sum(part);
            if (have && g == 0) a.delta[qvec + row] = d_own[qq];
        }
#pragma unroll
        for (int eb = 0; eb < EB; ++eb) acc1[qq][eb] = Frag<float>::zero();
    }
    if (KEYMAJOR) {
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) acc2[qq][eb] = Frag<float>::zero();
    }

    uintx4 r1[NCH], r2[NCH];
    float rl = 0.f, rd = 0.f;
    uint32_t rh = 0u;
    auto fetch = [&](int inner) __attribute__((always_inline)) {
        const long row0 = (long)inner * 32;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            if (c < 32 * CPR) {
                r1[i] = *reinterpret_cast<const uintx4*>(y1p + (row0 + c / CPR) * y1s + 8 * (c % CPR));
                r2[i] = *reinterpret_cast<const uintx4*>(y2p + (row0 + c / CPR) * y2s + 8 * (c % CPR));
            }
        }
        if (KEYMAJOR && tid < 32) {
            rl = a.lse2[qvec + row0 + tid];
            rd = a.delta[qvec + row0 + tid];
            if (DROP) rh = drop_row_hash(a.drop_seed, (uint32_t)(qvec + row0 + tid));
        }
    };
    auto stash = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            if (c < 32 * CPR) {
                *reinterpret_cast<uintx4*>(&tiles[buf][0][(c / CPR) * LD + 8 * (c % CPR)]) = r1[i];
                *reinterpret_cast<uintx4*>(&tiles[buf][1][(c / CPR) * LD + 8 * (c % CPR)]) = r2[i];
            }
        }
        if (KEYMAJOR && tid < 32) {
            rowv[buf][0][tid] = rl;
            rowv[buf][1][tid] = rd;
            if (DROP) rowv[buf][2][tid] = __uint_as_float(rh);
        }
    };
    const float sc = a.scale * LOG2E;
    const int foff = (8 * (r16 >> 2) + (r16 & 3)) * LD + 8 * g;         // + 4 b LD + 32 c   (elements)
    const int toff = (8 * g + (r16 >> 2)) * LD + 4 * (r16 & 3);         // (+ 4 LD) + 16 eb
    if (n > 0) {
        fetch(a.uni_inner[p0]);
        stash(0);
    }
    __syncthreads();
    for (int s = 0; s < n; ++s) {
        const int cur = s & 1;
        const bool more = s + 1 < n;
        if (more) fetch(a.uni_inner[p0 + s + 1]);
        const bool present = have && a.uni_blk[(long)(p0 + s) * 4 + w] >= 0;      // wave-uniform
        if (present) {
            const uint16_t* Y1 = tiles[cur][0];
            const uint16_t* Y2 = tiles[cur][1];
            floatx4 s1[2][2], gp[2][2];                  // [outer block][inner block b]: scores (unscaled) and g.v
#pragma unroll
            for (int qq = 0; qq < 2; ++qq)
#pragma unroll
                for (int hb = 0; hb < 2; ++hb) { s1[qq][hb] = Frag<float>::zero(); gp[qq][hb] = Frag<float>::zero(); }
#pragma unroll
            for (int hb = 0; hb < 2; ++hb)
#pragma unroll
                for (int c = 0; c < KS; ++c) {
                    const int off = foff + 4 * hb * LD + 32 * c;
                    const uintx4 f1 = *reinterpret_cast<const uintx4*>(Y1 + off);
                    const uintx4 f2 = *reinterpret_cast<const uintx4*>(Y2 + off);
#pragma unroll
                    for (int qq = 0; qq < 2; ++qq) {
                        s1[qq][hb] = mma32<T>(f1, x1[qq][c], s1[qq][hb]);
                        gp[qq][hb] = mma32<T>(f2, x2[qq][c], gp[qq][hb]);
                    }
                }
            floatx4 ln4[2], dl4[2], hh4[2];              // key-major: the tile's queries' lse2, delta and row hashes, by block
            if (KEYMAJOR) {
#pragma unroll
                for (int hb = 0; hb < 2; ++hb) {
                    ln4[hb] = *reinterpret_cast<const floatx4*>(&rowv[cur][0][8 * g + 4 * hb]);
                    dl4[hb] = *reinterpret_cast<const floatx4*>(&rowv[cur][1][8 * g + 4 * hb]);
                    if (DROP) hh4[hb] = *reinterpret_cast<const floatx4*>(&rowv[cur][2][8 * g + 4 * hb]);
                }
            }
            const int inner_cur = a.uni_inner[p0 + s];
            if constexpr (MASKED) {                                     // the masks, in units of the unscaled scores
                const float inv_scale = 1.0f / a.scale;
#pragma unroll
                for (int qq = 0; qq < 2; ++qq)
#pragma unroll
                    for (int hb = 0; hb < 2; ++hb) {
                        const long in0 = (long)inner_cur * 32 + 8 * g + 4 * hb;        // the element's four inner rows
                        const long orow = (long)bo_c * 32 + 16 * qq + r16;             // its outer row
                        floatx4 add = Frag<float>::zero();
                        if (!KEYMAJOR) {
                            if (a.key_mask) add += *reinterpret_cast<const floatx4*>(a.key_mask + z * a.km_stride + in0);
                            if (a.attn_mask) add += *reinterpret_cast<const floatx4*>(a.attn_mask + orow * a.am_stride + in0);
                        } else {
                            if (a.key_mask) add += km_own[qq];
                            if (a.attn_mask) {
#pragma unroll
                                for (int i = 0; i < 4; ++i) add[i] += a.attn_mask[(in0 + i) * a.am_stride + orow];
                            }
                        }
                        s1[qq][hb] += add * inv_scale;
                    }
            }
#pragma unroll
            for (int qq = 0; qq < 2; ++qq)
#pragma unroll
                for (int hb = 0; hb < 2; ++hb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float lrow = KEYMAJOR ? ln4[hb][i] : l_own[qq], drow = KEYMAJOR ? dl4[hb][i] : d_own[qq];
                        const float pr = __builtin_amdgcn_exp2f(fmaf(s1[qq][hb][i], sc, -lrow));   // (a row without scores: lse2 = +inf)
                        if (DROP) {
                            // (query, key) of the element: the inner row 8 g + 4 hb + i of the tile, the outer row 16 qq + r16
                            const uint32_t inner_row = (uint32_t)inner_cur * 32u + 8u * g + 4u * hb + i;
                            const uint32_t outer_row = (uint32_t)bo_c * 32u + 16u * qq + r16;
                            const uint32_t rhash = KEYMAJOR ? __float_as_uint(hh4[hb][i]) : h_own[qq];
                            const float m = drop_keep(rhash, KEYMAJOR ? outer_row : inner_row, a.drop_thresh) ? a.drop_scale : 0.f;
                            s1[qq][hb][i] = m * pr;
                            gp[qq][hb][i] = pr * (m * gp[qq][hb][i] - drow);
                        } else {
                            s1[qq][hb][i] = pr;
                            gp[qq][hb][i] = pr * (gp[qq][hb][i] - drow);
                        }
                    }
            uintx4 pb[KEYMAJOR ? 2 : 1], sb[2];
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                sb[qq] = uintx4{pack2<T>(gp[qq][0][0], gp[qq][0][1]), pack2<T>(gp[qq][0][2], gp[qq][0][3]),
                                pack2<T>(gp[qq][1][0], gp[qq][1][1]), pack2<T>(gp[qq][1][2], gp[qq][1][3])};
                if (KEYMAJOR)
                    pb[qq] = uintx4{pack2<T>(s1[qq][0][0], s1[qq][0][1]), pack2<T>(s1[qq][0][2], s1[qq][0][3]),
                                    pack2<T>(s1[qq][1][0], s1[qq][1][1]), pack2<T>(s1[qq][1][2], s1[qq][1][3])};
            }
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) {
                const uint16_t* p1 = Y1 + toff + 16 * eb;
                const uintx4 t1 = lds_read_tr8(reinterpret_cast<const char*>(p1), reinterpret_cast<const char*>(p1 + 4 * LD));
#pragma unroll
                for (int qq = 0; qq < 2; ++qq) acc1[qq][eb] = mma32<T>(t1, sb[qq], acc1[qq][eb]);
                if (KEYMAJOR) {
                    const uint16_t* p2 = Y2 + toff + 16 * eb;
                    const uintx4 t2 = lds_read_tr8(reinterpret_cast<const char*>(p2), reinterpret_cast<const char*>(p2 + 4 * LD));
#pragma unroll
                    for (int qq = 0; qq < 2; ++qq) acc2[qq][eb] = mma32<T>(t2, pb[qq], acc2[qq][eb]);
                }
            }
        }
        if (more) stash(cur ^ 1);
        __syncthreads();
    }
    if (have) {
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
            const long row = (long)bo * 32 + 16 * qq + r16;
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) store4_f32(d1 + row * d1s + 16 * eb + 4 * g, acc1[qq][eb] * a.scale);
            if (KEYMAJOR) {
#pragma unroll
                for (int eb = 0; eb < EB; ++eb) store4_f32(d2 + row * a.dv_sm + 16 * eb + 4 * g, acc2[qq][eb]);
            }
        }
    }
}

template <typename T, int E, bool KEYMAJOR, bool DROP, bool MASKED = false>
static int launch_attn_bwd_as(const AttnBwdArgs& a, hipStream_t st) {
    AttnBwdArgs args = a;
    args.n_xcd = machine().xcds;
    const long grid = unit_grid((long)a.n_heads * a.Z, a.grps_per_head);
    if (grid > 2147483647L) return fail(ERR_ARG, "bs_attn_bwd: too many workgroups");
    hipLaunchKernelGGL((bs_attn32_bwd_kernel<T, E, KEYMAJOR, DROP, MASKED>), dim3((unsigned)grid), dim3(256), 0, st, args);
    return check_launch("bs_attn32_bwd_kernel");
}
template <typename T, int E, bool KEYMAJOR>
static int launch_attn_bwd(const AttnBwdArgs& a, hipStream_t st) {
    if (a.key_mask != nullptr || a.attn_mask != nullptr) return launch_attn_bwd_as<T, E, KEYMAJOR, false, true>(a, st);
    return a.drop_thresh != 0u ? launch_attn_bwd_as<T, E, KEYMAJOR, true>(a, st) : launch_attn_bwd_as<T, E, KEYMAJOR, false>(a, st);
}

extern "C" int flyhip_bs_attn_bwd(const void* q, const void* k, const void* v, const void* out, const void* grad_out,
                                  const float* lse2, float* delta, void* dq, void* dk, void* dv,
                                  const int32_t* row_ptr, const int32_t* row_inner, const int32_t* row_blk,
                                  const int32_t* col_ptr, const int32_t* col_inner, const int32_t* col_blk,
                                  int n_heads, int brows_per_head, int bcols_per_head, int Z, int E,
                                  int64_t q_sz, int64_t q_sh, int64_t q_sm, int64_t k_sz, int64_t k_sh, int64_t k_sm,
                                  int64_t v_sz, int64_t v_sh, int64_t v_sm, int64_t o_sz, int64_t o_sh, int64_t o_sm,
                                  int64_t g_sz, int64_t g_sh, int64_t g_sm,
                                  int64_t dq_sz, int64_t dq_sh, int64_t dq_sm, int64_t dk_sz, int64_t dk_sh, int64_t dk_sm,
                                  int64_t dv_sz, int64_t dv_sh, int64_t dv_sm,
                                  float scale, int dtype, float dropout_p, uint64_t dropout_seed,
                                  const float* key_mask, int64_t key_mask_stride, const float* attn_mask, int64_t attn_mask_stride,
                                  void* stream) {
    FLY_REQUIRE(q && k && v && out && grad_out && lse2 && delta && dq && dk && dv, "bs_attn_bwd: null pointer");
    FLY_REQUIRE(scale > 0.f, "bs_attn_bwd: scale must be positive");
    FLY_REQUIRE((!key_mask || key_mask_stride % 4 == 0) && (!attn_mask || attn_mask_stride % 4 == 0) &&
                ((reinterpret_cast<uintptr_t>(key_mask) | reinterpret_cast<uintptr_t>(attn_mask)) % 16) == 0,
                "bs_attn_bwd: mask rows must be 16-byte aligned (strides in multiples of 4 floats)");
    FLY_REQUIRE(dropout_p == 0.f || (!key_mask && !attn_mask), "bs_attn_bwd: no dropout together with masks (the forward has none)");
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "bs_attn_bwd: dropout_p %g not in [0, 1)", (double)dropout_p);
    FLY_REQUIRE((long)Z * n_heads * brows_per_head * 32 <= 4294967295L, "bs_attn_bwd: more than 2^32 query rows");
    FLY_REQUIRE(row_ptr && row_inner && row_blk && col_ptr && col_inner && col_blk, "bs_attn_bwd: null table");
    FLY_REQUIRE(n_heads > 0 && brows_per_head > 0 && bcols_per_head > 0 && Z > 0, "bs_attn_bwd: empty problem");
    FLY_REQUIRE(E == 32 || E == 64, "bs_attn_bwd: head dim %d not in {32, 64}", E);
    FLY_REQUIRE(dtype == BF16 || dtype == F16, "bs_attn_bwd supports bfloat16 and float16, got dtype code %d", dtype);
    FLY_REQUIRE(((q_sz | q_sh | q_sm | k_sz | k_sh | k_sm | v_sz | v_sh | v_sm | o_sz | o_sh | o_sm | g_sz | g_sh | g_sm) % 8) == 0,
                "bs_attn_bwd: input strides must be multiples of 8 elements (16-byte loads)");
    FLY_REQUIRE(((dq_sz | dq_sh | dq_sm | dk_sz | dk_sh | dk_sm | dv_sz | dv_sh | dv_sm) % 4) == 0,
                "bs_attn_bwd: output strides must be multiples of 4 elements (8-byte stores)");
    FLY_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                  reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(grad_out)) % 16) == 0 &&
                ((reinterpret_cast<uintptr_t>(dq) | reinterpret_cast<uintptr_t>(dk) | reinterpret_cast<uintptr_t>(dv)) % 8) == 0,
                "bs_attn_bwd: pointers must be 16-byte (inputs) and 8-byte (outputs) aligned");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    AttnBwdArgs a{};
    a.q = q; a.k = k; a.v = v; a.go = grad_out; a.out = out; a.lse2 = lse2; a.delta = delta; a.dq = dq; a.dk = dk; a.dv = dv;
    a.q_blocks = brows_per_head; a.n_heads = n_heads; a.Z = Z; a.scale = scale;
    const DropArgs drop = drop_args(dropout_p, dropout_seed);
    a.drop_seed = drop.seed; a.drop_thresh = drop.thresh; a.drop_scale = drop.scale;
    a.key_mask = key_mask; a.km_stride = key_mask_stride; a.attn_mask = attn_mask; a.am_stride = attn_mask_stride;
    a.q_sz = q_sz; a.q_sh = q_sh; a.q_sm = q_sm; a.k_sz = k_sz; a.k_sh = k_sh; a.k_sm = k_sm; a.v_sz = v_sz; a.v_sh = v_sh; a.v_sm = v_sm;
    a.g_sz = g_sz; a.g_sh = g_sh; a.g_sm = g_sm; a.o_sz = o_sz; a.o_sh = o_sh; a.o_sm = o_sm;
    a.dq_sz = dq_sz; a.dq_sh = dq_sh; a.dq_sm = dq_sm; a.dk_sz = dk_sz; a.dk_sh = dk_sh; a.dk_sm = dk_sm;
    a.dv_sz = dv_sz; a.dv_sh = dv_sh; a.dv_sm = dv_sm;
    for (int km = 0; km < 2; ++km) {                 // query-major first: it leaves delta for the key-major launch
        a.uni_ptr = km ? col_ptr : row_ptr; a.uni_inner = km ? col_inner : row_inner; a.uni_blk = km ? col_blk : row_blk;
        a.outer_blocks = km ? bcols_per_head : brows_per_head;
        a.inner_blocks = km ? brows_per_head : bcols_per_head;
        a.grps_per_head = (a.outer_blocks + 3) / 4;
        int rc;
#define ATTN_BWD_LAUNCH(TT, EE) rc = km ? launch_attn_bwd<TT, EE, true>(a, st) : launch_attn_bwd<TT, EE, false>(a, st)
        if (dtype == BF16) { if (E == 32) ATTN_BWD_LAUNCH(bf16_t, 32); else ATTN_BWD_LAUNCH(bf16_t, 64); }
        else { if (E == 32) ATTN_BWD_LAUNCH(f16_t, 32); else ATTN_BWD_LAUNCH(f16_t, 64); }
#undef ATTN_BWD_LAUNCH
        if (rc) return rc;
    }
    return 0;
}

extern "C" int flyhip_bs_sdd_prob(const void* q, const void* k, const float* lse2, void* p,
                                  const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                                  int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                                  int64_t a_sz, int64_t a_sh, int64_t a_sm,
                                  int64_t b_sz, int64_t b_sh, int64_t b_sn,
                                  float scale, int dtype, void* stream) {
    return launch_sdd_epilogue<2>("bs_sdd_prob", q, k, nullptr, lse2, p, uni_ptr, uni_inner, uni_blk, nnz, n_heads,
                                  brows_per_head, Z, K, blk, a_sz, a_sh, a_sm, b_sz, b_sh, b_sn,
                                  scale * 1.4426950408889634f, dtype, stream);
}

extern "C" int flyhip_bs_sdd_kmajor(const void* a, const void* b, float* c32,
                                    const int32_t* row_ptr, const int32_t* row_blk, const int32_t* row_col,
                                    const int32_t* grp_row0, const int32_t* grp_n, int n_grp, int max_row_nnz,
                                    int brows_per_head, int nnz, int Z, int K, int k_slice, int blk,
                                    int64_t a_sz, int64_t a_sh, int64_t a_sk,
                                    int64_t b_sz, int64_t b_sh, int64_t b_sk,
                                    int dtype, void* stream) {
    int rc = check_common("bs_sdd_kmajor", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(a && b && c32 && row_ptr && row_blk && row_col && grp_row0 && grp_n, "bs_sdd_kmajor: null pointer");
    FLY_REQUIRE(blk == 32 && (dtype == BF16 || dtype == F16), "bs_sdd_kmajor: needs 32x32 blocks of bf16 / fp16");
    FLY_REQUIRE(n_grp > 0 && max_row_nnz > 0 && brows_per_head > 0 && nnz > 0 && K > 0, "bs_sdd_kmajor: bad sizes");
    FLY_REQUIRE(k_slice >= 32 && k_slice % 32 == 0, "bs_sdd_kmajor: k_slice must be a positive multiple of 32");
    FLY_REQUIRE(((a_sz | a_sh | a_sk | b_sz | b_sh | b_sk) % 8) == 0, "bs_sdd_kmajor: strides must be multiples of 8 elements");
    const int chunks = (max_row_nnz + 3) / 4, slices = (K + k_slice - 1) / k_slice;
    FLY_REQUIRE((long)n_grp * chunks <= 2147483647L && slices <= 65535, "bs_sdd_kmajor: too many workgroups");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    SddKArgs args{a, b, c32, row_ptr, row_blk, row_col, grp_row0, grp_n, brows_per_head, K, k_slice, chunks, nnz,
                  a_sz, a_sh, a_sk, b_sz, b_sh, b_sk};
    dim3 grid((unsigned)(n_grp * chunks), slices, Z);
    if (dtype == BF16) hipLaunchKernelGGL((bs_sdd32k_kernel<bf16_t>), grid, dim3(256), 0, st, args);
    else hipLaunchKernelGGL((bs_sdd32k_kernel<f16_t>), grid, dim3(256), 0, st, args);
    return check_launch("bs_sdd32k_kernel");
}

extern "C" int flyhip_bs_dsd(const void* a_sp, const void* b, void* c,
                             const int32_t* seg_ptr, const int32_t* seg_blk, const int32_t* seg_inner,
                             const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                             int n_seg, int rows_per_head, int Z, int N, int blk, int trans_a,
                             int64_t a_sz,
                             int64_t b_sz, int64_t b_sh, int64_t b_sk, int64_t b_sn,
                             int64_t c_sz, int64_t c_sh, int64_t c_sm, int64_t c_sn,
                             int dtype, void* stream) {
    int rc = check_common("bs_dsd", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(a_sp && b && c && seg_ptr && seg_blk && seg_inner, "bs_dsd: null pointer");
    FLY_REQUIRE(n_seg > 0 && rows_per_head > 0 && n_seg % rows_per_head == 0, "bs_dsd: bad segment counts");
    FLY_REQUIRE(N > 0, "bs_dsd: N must be positive");
    if (b_sk == 1) FLY_REQUIRE(((b_sz | b_sh | b_sn) % 4) == 0, "bs_dsd: B strides must be multiples of 4 elements");
    if (c_sn == 1) FLY_REQUIRE(((c_sz | c_sh | c_sm) % 4) == 0, "bs_dsd: C strides must be multiples of 4 elements");
    FLY_REQUIRE(a_sz % 4 == 0, "bs_dsd: sparse batch stride must be a multiple of 4 elements");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    DxdArgs args{a_sp, b, c, seg_ptr, seg_blk, seg_inner, n_seg, rows_per_head, N, trans_a,
                 a_sz, b_sz, b_sh, b_sk, b_sn, c_sz, c_sh, c_sm, c_sn, Z};
    if (blk == 32 && (dtype == BF16 || dtype == F16) && (!trans_a || (uni_ptr && uni_inner && uni_blk)) && b_sn == 1 &&
        c_sn == 1 && N % 8 == 0 &&
        ((a_sz | b_sz | b_sh | b_sk | c_sz | c_sh | c_sm) % 8) == 0) {
        if (uni_ptr && uni_inner && uni_blk) {
            const int gph = (rows_per_head + 3) / 4, n_heads = n_seg / rows_per_head;
            DsdUniArgs ua{a_sp, b, c, uni_ptr, uni_inner, uni_blk, rows_per_head, gph, n_heads, Z, N,
                          a_sz, b_sz, b_sh, b_sk, c_sz, c_sh, c_sm};
            const long nwg = unit_grid((long)n_heads * Z, (long)gph * ((N + 63) / 64));
            ua.n_xcd = machine().xcds;
            FLY_REQUIRE(nwg <= 2147483647L, "bs_dsd: too many workgroups");
            dim3 grid((unsigned)nwg);
            if (dtype == BF16) {
                if (trans_a) hipLaunchKernelGGL((bs_dsd32u_kernel<bf16_t, true>), grid, dim3(256), 0, st, ua);
                else hipLaunchKernelGGL((bs_dsd32u_kernel<bf16_t, false>), grid, dim3(256), 0, st, ua);
            } else {
                if (trans_a) hipLaunchKernelGGL((bs_dsd32u_kernel<f16_t, true>), grid, dim3(256), 0, st, ua);
                else hipLaunchKernelGGL((bs_dsd32u_kernel<f16_t, false>), grid, dim3(256), 0, st, ua);
            }
            return check_launch("bs_dsd32u_kernel");
        }
        const long nwg = unit_grid((long)(n_seg / rows_per_head) * Z, (long)rows_per_head * ((N + 63) / 64));
        args.n_xcd = machine().xcds;
        FLY_REQUIRE(nwg <= 2147483647L, "bs_dsd: too many workgroups");
        dim3 grid((unsigned)nwg);
        if (dtype == BF16) hipLaunchKernelGGL((bs_dsd32_kernel<bf16_t>), grid, dim3(256), 0, st, args);
        else hipLaunchKernelGGL((bs_dsd32_kernel<f16_t>), grid, dim3(256), 0, st, args);
        return check_launch("bs_dsd32_kernel");
    }
    const int tile = blk >= 32 ? 32 : 16;
    const long nblocks = waves_to_blocks((long)n_seg * (blk / tile) * ((N + 31) / 32));
    FLY_REQUIRE(nblocks <= 2147483647L, "bs_dsd: too many blocks");
    dim3 grid((unsigned)nblocks, Z);
    BS_DISPATCH(bs_dsd_kernel, grid, args)
    return check_launch("bs_dsd_kernel");
}

extern "C" int flyhip_bs_dds(const void* a, const void* b_sp, void* c,
                             const int32_t* seg_ptr, const int32_t* seg_blk, const int32_t* seg_inner,
                             const int32_t* grp_row0, const int32_t* grp_n, int n_grp, int max_seg_len,
                             int n_seg, int cols_per_head, int Z, int M, int blk, int trans_b,
                             int64_t a_sz, int64_t a_sh, int64_t a_sm, int64_t a_sk,
                             int64_t b_sz,
                             int64_t c_sz, int64_t c_sh, int64_t c_sm, int64_t c_sn,
                             int dtype, void* stream) {
    int rc = check_common("bs_dds", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(a && b_sp && c && seg_ptr && seg_blk && seg_inner, "bs_dds: null pointer");
    FLY_REQUIRE(n_seg > 0 && cols_per_head > 0 && n_seg % cols_per_head == 0, "bs_dds: bad segment counts");
    FLY_REQUIRE(M > 0, "bs_dds: M must be positive");
    if (a_sk == 1) FLY_REQUIRE(((a_sz | a_sh | a_sm) % 4) == 0, "bs_dds: A strides must be multiples of 4 elements");
    if (c_sn == 1) FLY_REQUIRE(((c_sz | c_sh | c_sm) % 4) == 0, "bs_dds: C strides must be multiples of 4 elements");
    FLY_REQUIRE(b_sz % 4 == 0, "bs_dds: sparse batch stride must be a multiple of 4 elements");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    if (grp_row0 && grp_n && n_grp > 0 && max_seg_len >= 0 && max_seg_len <= DDS_MAX_STEPS && blk == 32 &&
        (dtype == BF16 || dtype == F16) && a_sk == 1 && (long)M * a_sm * 2 < (1L << 32) &&
        c_sn == 1 && ((a_sz | a_sh | a_sm | b_sz | c_sz | c_sh | c_sm) % 8) == 0 && (M + 127) / 128 <= 65535) {
        DdsGroupArgs ga{b_sp, a, c, seg_ptr, seg_blk, seg_inner, grp_row0, grp_n, cols_per_head, M,
                        b_sz, a_sz, a_sh, a_sm, c_sz, c_sh, c_sm};
        const Machine& mach = machine();
        ga.n_xcd = mach.xcds;
        ga.n_grp = n_grp;
        // groups whose weights fit the LDS (four output blocks times the longest reduction list) and enough tokens to
        // amortise bringing them in: the weight-stationary kernel, two workgroups per compute unit
        if (FLY_DDS_STATIONARY == 2 && max_seg_len > 0 && max_seg_len <= DDS_STAT_STEPS && (long)M >= 512L * 8) {
            // one workgroup of eight waves per compute unit: the group's weights and a stage of activations per wave
            // streams of token tiles per group: the count that minimises (rounds of workgroups) x (tiles per workgroup)
            const long tiles = (M + 511) / 512;
            long n_streams = 1, best = -1;
            for (long n = 1; n <= tiles && n * n_grp * Z <= 4L * mach.cus + (long)n_grp * Z; ++n) {
                const long cost = ((n * n_grp * Z + mach.cus - 1) / mach.cus) * ((tiles + n - 1) / n);
                if (best < 0 || cost < best) { best = cost; n_streams = n; }
            }
            const long pairs = n_streams * n_grp;
            const long gx = (pairs + mach.xcds - 1) / mach.xcds * mach.xcds;
            const size_t smem = (size_t)DDS_STAT_STEPS * 8192 + 8 * 8192;
            dim3 grid((unsigned)gx, Z);
#define DDS_DMA(TT, WTT)                                                                                           \
    {                                                                                                              \
        auto kern = bs_dds32d_kernel<TT, WTT>;                                                                     \
        static std::atomic<unsigned long long> lds_set{0};                                                         \
        if (int rc2 = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "bs_dds (staged)")) return rc2; \
        hipLaunchKernelGGL(kern, grid, dim3(512), smem, st, ga, (int)n_streams);                                   \
    }
            if (dtype == BF16) { if (trans_b) DDS_DMA(bf16_t, false) else DDS_DMA(bf16_t, true) }
            else { if (trans_b) DDS_DMA(f16_t, false) else DDS_DMA(f16_t, true) }
#undef DDS_DMA
            return check_launch("bs_dds32d_kernel");
        }
        if (FLY_DDS_STATIONARY == 2 && max_seg_len > DDS_STAT_STEPS && max_seg_len <= DDS_MAX_STEPS && (long)M >= 512L * 8) {
            // longer lists: the same workgroup shape with the weights passing through LDS in chunks
            const long tiles = (M + 511) / 512;
            long n_streams = 1, best = -1;
            for (long n = 1; n <= tiles && n * n_grp * Z <= 4L * mach.cus + (long)n_grp * Z; ++n) {
                const long cost = ((n * n_grp * Z + mach.cus - 1) / mach.cus) * ((tiles + n - 1) / n);
                if (best < 0 || cost < best) { best = cost; n_streams = n; }
            }
            const long pairs = n_streams * n_grp;
            const long gx = (pairs + mach.xcds - 1) / mach.xcds * mach.xcds;
            const size_t smem = (size_t)2 * DDS_CK * 8192 + 8 * 8192;
            dim3 grid((unsigned)gx, Z);
#define DDS_CHUNKED(TT, WTT)                                                                                       \
    {                                                                                                              \
        auto kern = bs_dds32c_kernel<TT, WTT>;                                                                     \
        static std::atomic<unsigned long long> lds_set{0};                                                         \
        if (int rc2 = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "bs_dds (chunked)")) return rc2; \
        hipLaunchKernelGGL(kern, grid, dim3(512), smem, st, ga, (int)n_streams);                                   \
    }
            if (dtype == BF16) { if (trans_b) DDS_CHUNKED(bf16_t, false) else DDS_CHUNKED(bf16_t, true) }
            else { if (trans_b) DDS_CHUNKED(f16_t, false) else DDS_CHUNKED(f16_t, true) }
#undef DDS_CHUNKED
            return check_launch("bs_dds32c_kernel");
        }
        if (FLY_DDS_STATIONARY && max_seg_len > 0 && max_seg_len <= DDS_STAT_STEPS && (long)M >= 256L * 8) {
            const long tiles = (M + 255) / 256;
            long n_streams = 2L * mach.cus / ((long)n_grp * Z);
            if (n_streams < 1) n_streams = 1;
            if (n_streams > tiles) n_streams = tiles;
            const long pairs = n_streams * n_grp;
            const long gx = (pairs + mach.xcds - 1) / mach.xcds * mach.xcds;
            const size_t smem = (size_t)max_seg_len * 8192;
            dim3 grid((unsigned)gx, Z);
#define DDS_STAT(TT, WTT)                                                                                          \
    {                                                                                                              \
        auto kern = bs_dds32s_kernel<TT, WTT, FLY_DDS_DEPTH>;                                                       \
        static std::atomic<unsigned long long> lds_set{0};                                                         \
        if (int rc2 = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "bs_dds (stationary)")) return rc2; \
        hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, ga, (int)n_streams);                                   \
    }
            if (dtype == BF16) { if (trans_b) DDS_STAT(bf16_t, false) else DDS_STAT(bf16_t, true) }
            else { if (trans_b) DDS_STAT(f16_t, false) else DDS_STAT(f16_t, true) }
#undef DDS_STAT
            return check_launch("bs_dds32s_kernel");
        }
        // as many workgroups as are resident together (two fit a CU: 64 KB of tiles each); each walks its share of the
        // token tiles
        const long tiles = (M + 127) / 128;
        long gy = (2L * mach.cus + (long)n_grp * Z - 1) / ((long)n_grp * Z);
        if (gy > tiles) gy = tiles;
        gy = (gy + mach.xcds - 1) / mach.xcds * mach.xcds;   // the kernel deals streams of token tiles to the XCDs
        dim3 grid(n_grp, (unsigned)gy, Z);
        constexpr size_t smem_t = 4 * 128 * 64 * 2;          // two stages of the activation and the weight tile
#define DDS_TILED(TT, WTT)                                                                                         \
    {                                                                                                              \
        auto kern = bs_dds32_kernel<TT, WTT>;                                                                      \
        static std::atomic<unsigned long long> lds_set{0};                                                         \
        if (int rc2 = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem_t, lds_set, "bs_dds (tiled)")) return rc2; \
        hipLaunchKernelGGL(kern, grid, dim3(256), smem_t, st, ga);                                                 \
    }
        if (dtype == BF16) { if (trans_b) DDS_TILED(bf16_t, false) else DDS_TILED(bf16_t, true) }
        else { if (trans_b) DDS_TILED(f16_t, false) else DDS_TILED(f16_t, true) }
#undef DDS_TILED
        return check_launch("bs_dds32_kernel");
    }
    DxdArgs args{b_sp, a, c, seg_ptr, seg_blk, seg_inner, n_seg, cols_per_head, M, trans_b,
                 b_sz, a_sz, a_sh, a_sm, a_sk, c_sz, c_sh, c_sm, c_sn};
    const int tile = blk >= 32 ? 32 : 16;
    const long nblocks = waves_to_blocks((long)((M + 31) / 32) * n_seg * (blk / tile));
    FLY_REQUIRE(nblocks <= 2147483647L, "bs_dds: too many blocks");
    dim3 grid((unsigned)nblocks, Z);
    BS_DISPATCH(bs_dds_kernel, grid, args)
    return check_launch("bs_dds_kernel");
}

template <typename T>
static int launch_softmax(const RowArgs& args, dim3 grid, int max_elems, hipStream_t st) {
    if (sizeof(T) == 2 && args.blk_shift == 5 && max_elems <= 32 * 4 * 16 && (args.x_sz % 8) == 0) {
        dim3 g2(2 * args.n_brow, grid.y);
        const int slots = (max_elems / 32 + 3) / 4;          // blocks per wave with four waves: sizes the register arrays
#define SM32(N) hipLaunchKernelGGL((bs_softmax32_kernel<T, N, 4>), g2, dim3(256), 0, st, args)
#define SM32W(N) hipLaunchKernelGGL((bs_softmax32_kernel<T, N, 8>), g2, dim3(512), 0, st, args)
        if (slots <= 4) SM32(4); else if (slots <= 8) SM32(8);
        else if (slots <= 10) SM32W(5); else if (slots <= 12) SM32W(6); else if (slots <= 14) SM32W(7);
        else SM32W(8);
#undef SM32W
#undef SM32
        return check_launch("bs_softmax32_kernel");
    }
    if (max_elems <= 64 * 8) hipLaunchKernelGGL((bs_softmax_kernel<T, 8>), grid, dim3(256), 0, st, args);
    else if (max_elems <= 64 * 32) hipLaunchKernelGGL((bs_softmax_kernel<T, 32>), grid, dim3(256), 0, st, args);
    else hipLaunchKernelGGL((bs_softmax_long_kernel<T>), grid, dim3(256), 0, st, args);
    return check_launch("bs_softmax_kernel");
}

static int bs_attn_checked(const void* q, const void* k, const void* v, void* out, float* lse2,
                              const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                              int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                              const float* attn_mask, int64_t attn_mask_stride,
                              int Z, int H, int brows_per_head, int D, int blk,
                              int64_t q_sz, int64_t q_sh, int64_t q_sm,
                              int64_t k_sz, int64_t k_sh, int64_t k_sn,
                              int64_t v_sz, int64_t v_sh, int64_t v_sn,
                              int64_t o_sz, int64_t o_sh, int64_t o_sm,
                              float scale, int dtype, void* stream, DropArgs drop) {
    int rc = check_common("bs_attn", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(q && k && v && out && uni_ptr && uni_inner && uni_blk, "bs_attn: null pointer");
    FLY_REQUIRE(blk == 32 && (dtype == BF16 || dtype == F16), "bs_attn: needs 32x32 blocks of bf16 / fp16 (got block %d, dtype %d)", blk, dtype);
    FLY_REQUIRE(D == 32 || D == 64 || D == 128, "bs_attn: head dim %d not in {32,64,128}", D);
    FLY_REQUIRE(rows_per_group == 4 || rows_per_group == 8, "bs_attn: rows_per_group must be 4 or 8");
    FLY_REQUIRE(H > 0 && brows_per_head > 0, "bs_attn: bad sizes");
    FLY_REQUIRE(((q_sz | q_sh | q_sm | k_sz | k_sh | k_sn | v_sz | v_sh | v_sn) % 8) == 0,
                "bs_attn: q / k / v strides must be multiples of 8 elements");
    FLY_REQUIRE(((o_sz | o_sh | o_sm) % 4) == 0, "bs_attn: out strides must be multiples of 4 elements");
    FLY_REQUIRE(!key_mask || key_mask_stride % 4 == 0, "bs_attn: key mask stride must be a multiple of 4");
    FLY_REQUIRE(!attn_mask || attn_mask_stride % 4 == 0, "bs_attn: attention mask stride must be a multiple of 4");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    const int gph = (brows_per_head + rows_per_group - 1) / rows_per_group;
    AttnArgs args{q, k, v, out, uni_ptr, uni_inner, uni_blk, key_mask, key_mask_stride, brows_per_head, gph, H, Z,
                  q_sz, q_sh, q_sm, k_sz, k_sh, k_sn, v_sz, v_sh, v_sn, o_sz, o_sh, o_sm, scale, lse2};
    args.am = attn_mask;
    args.am_stride = attn_mask_stride;
    const long nwg = unit_grid((long)H * Z, gph);
    args.n_xcd = machine().xcds;
    FLY_REQUIRE(nwg <= 2147483647L, "bs_attn: too many workgroups");
    dim3 grid((unsigned)nwg);
    const bool masked = key_mask != nullptr || attn_mask != nullptr || !(scale > 0.f);
    const bool dropping = drop.thresh != 0u;
    args.drop_seed = drop.seed;
    args.drop_thresh = drop.thresh;
    args.drop_scale = drop.scale;
#define ATTN_LAUNCH(T, KS, NW)                                                                                  \
    do {                                                                                                        \
        if (dropping && masked) hipLaunchKernelGGL((bs_attn32_kernel<T, KS, NW, true, true>), grid, dim3(64 * NW), 0, st, args); \
        else if (dropping) hipLaunchKernelGGL((bs_attn32_kernel<T, KS, NW, false, true>), grid, dim3(64 * NW), 0, st, args); \
        else if (masked) hipLaunchKernelGGL((bs_attn32_kernel<T, KS, NW, true>), grid, dim3(64 * NW), 0, st, args);  \
        else hipLaunchKernelGGL((bs_attn32_kernel<T, KS, NW, false>), grid, dim3(64 * NW), 0, st, args);        \
    } while (0)
#define ATTN_KS(T, NW) do { if (D == 32) ATTN_LAUNCH(T, 1, NW); else if (D == 64) ATTN_LAUNCH(T, 2, NW); else ATTN_LAUNCH(T, 4, NW); } while (0)
    if (dtype == BF16) { if (rows_per_group == 4) ATTN_KS(bf16_t, 4); else ATTN_KS(bf16_t, 8); }
    else { if (rows_per_group == 4) ATTN_KS(f16_t, 4); else ATTN_KS(f16_t, 8); }
#undef ATTN_KS
#undef ATTN_LAUNCH
    return check_launch("bs_attn32_kernel");
}

extern "C" int flyhip_bs_attn_masks(const void* q, const void* k, const void* v, void* out, float* lse2,
                              const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                              int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                              const float* attn_mask, int64_t attn_mask_stride,
                              int Z, int H, int brows_per_head, int D, int blk,
                              int64_t q_sz, int64_t q_sh, int64_t q_sm,
                              int64_t k_sz, int64_t k_sh, int64_t k_sn,
                              int64_t v_sz, int64_t v_sh, int64_t v_sn,
                              int64_t o_sz, int64_t o_sh, int64_t o_sm,
                              float scale, int dtype, void* stream) {
    return bs_attn_checked(q, k, v, out, lse2, uni_ptr, uni_inner, uni_blk, rows_per_group, key_mask, key_mask_stride,
                           attn_mask, attn_mask_stride, Z, H, brows_per_head, D, blk, q_sz, q_sh, q_sm, k_sz, k_sh, k_sn,
                           v_sz, v_sh, v_sn, o_sz, o_sh, o_sm, scale, dtype, stream, DropArgs{0u, 0u, 1.f});
}

extern "C" int flyhip_bs_attn_dropout(const void* q, const void* k, const void* v, void* out, float* lse2,
                              const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                              int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                              const float* attn_mask, int64_t attn_mask_stride,
                              int Z, int H, int brows_per_head, int D, int blk,
                              int64_t q_sz, int64_t q_sh, int64_t q_sm,
                              int64_t k_sz, int64_t k_sh, int64_t k_sn,
                              int64_t v_sz, int64_t v_sh, int64_t v_sn,
                              int64_t o_sz, int64_t o_sh, int64_t o_sm,
                              float scale, int dtype, float dropout_p, uint64_t dropout_seed, void* stream) {
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "bs_attn_dropout: dropout_p %g not in [0, 1)", (double)dropout_p);
    FLY_REQUIRE((long)Z * H * brows_per_head * 32 <= 4294967295L, "bs_attn_dropout: more than 2^32 rows");
    return bs_attn_checked(q, k, v, out, lse2, uni_ptr, uni_inner, uni_blk, rows_per_group, key_mask, key_mask_stride,
                           attn_mask, attn_mask_stride, Z, H, brows_per_head, D, blk, q_sz, q_sh, q_sm, k_sz, k_sh, k_sn,
                           v_sz, v_sh, v_sn, o_sz, o_sh, o_sm, scale, dtype, stream, drop_args(dropout_p, dropout_seed));
}

extern "C" int flyhip_bs_attn_lse(const void* q, const void* k, const void* v, void* out, float* lse2,
                              const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                              int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                              int Z, int H, int brows_per_head, int D, int blk,
                              int64_t q_sz, int64_t q_sh, int64_t q_sm,
                              int64_t k_sz, int64_t k_sh, int64_t k_sn,
                              int64_t v_sz, int64_t v_sh, int64_t v_sn,
                              int64_t o_sz, int64_t o_sh, int64_t o_sm,
                              float scale, int dtype, void* stream) {
    return flyhip_bs_attn_masks(q, k, v, out, lse2, uni_ptr, uni_inner, uni_blk, rows_per_group, key_mask, key_mask_stride,
                                nullptr, 0, Z, H, brows_per_head, D, blk, q_sz, q_sh, q_sm, k_sz, k_sh, k_sn, v_sz, v_sh, v_sn,
                                o_sz, o_sh, o_sm, scale, dtype, stream);
}

extern "C" int flyhip_bs_attn(const void* q, const void* k, const void* v, void* out,
                              const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                              int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                              int Z, int H, int brows_per_head, int D, int blk,
                              int64_t q_sz, int64_t q_sh, int64_t q_sm,
                              int64_t k_sz, int64_t k_sh, int64_t k_sn,
                              int64_t v_sz, int64_t v_sh, int64_t v_sn,
                              int64_t o_sz, int64_t o_sh, int64_t o_sm,
                              float scale, int dtype, void* stream) {
    return flyhip_bs_attn_lse(q, k, v, out, nullptr, uni_ptr, uni_inner, uni_blk, rows_per_group, key_mask, key_mask_stride,
                              Z, H, brows_per_head, D, blk, q_sz, q_sh, q_sm, k_sz, k_sh, k_sn, v_sz, v_sh, v_sn,
                              o_sz, o_sh, o_sm, scale, dtype, stream);
}

extern "C" int flyhip_bs_softmax(void* x, const int32_t* row_ptr, const int32_t* row_blk, const int32_t* row_col,
                                 int n_brow, int brows_per_head, int max_row_nnz, int Z, int blk, int64_t x_sz,
                                 float scale, const float* kpm, int64_t kpm_stride, int kpm_mul,
                                 const float* am, int64_t am_stride, int am_mul, int dtype, void* stream) {
    int rc = check_common("bs_softmax", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(x && row_ptr && row_blk && row_col, "bs_softmax: null pointer");
    FLY_REQUIRE(n_brow > 0 && brows_per_head > 0 && n_brow % brows_per_head == 0, "bs_softmax: bad row counts");
    FLY_REQUIRE(max_row_nnz >= 0, "bs_softmax: negative max_row_nnz");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    RowArgs args{x, nullptr, row_ptr, row_blk, row_col, n_brow, brows_per_head, blk_shift_of(blk), x_sz, scale,
                 kpm, kpm_stride, kpm_mul, am, am_stride, am_mul, 0};
    const long nblocks = waves_to_blocks((long)n_brow * blk);
    dim3 grid((unsigned)nblocks, Z);
    const int max_elems = max_row_nnz * blk;   // selects the register-resident or the multi-pass kernel
    switch (dtype) {
        case F32: return launch_softmax<float>(args, grid, max_elems, st);
        case BF16: return launch_softmax<bf16_t>(args, grid, max_elems, st);
        default: return launch_softmax<f16_t>(args, grid, max_elems, st);
    }
}

extern "C" int flyhip_bs_softmax_bwd(const void* y, const void* dy, void* dx,
                                     const int32_t* row_ptr, const int32_t* row_blk,
                                     int n_brow, int max_row_nnz, int Z, int blk, int64_t y_sz,
                                     float scale, int dtype, void* stream) {
    int rc = check_common("bs_softmax_bwd", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(y && dy && dx && row_ptr && row_blk, "bs_softmax_bwd: null pointer");
    FLY_REQUIRE(blk == 32 && (dtype == BF16 || dtype == F16), "bs_softmax_bwd: needs 32x32 blocks of bf16 / fp16");
    FLY_REQUIRE(n_brow > 0 && max_row_nnz >= 0 && max_row_nnz <= 64, "bs_softmax_bwd: at most 64 blocks per block-row (got %d)", max_row_nnz);
    FLY_REQUIRE(y_sz % 8 == 0, "bs_softmax_bwd: batch stride must be a multiple of 8 elements");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    RowBwdArgs args{y, dy, dx, row_ptr, row_blk, y_sz, scale};
    dim3 grid(2 * n_brow, Z);
    const int slots = (max_row_nnz + 3) / 4;
#define SMB(T, N) hipLaunchKernelGGL((bs_softmax32_bwd_kernel<T, N, 4>), grid, dim3(256), 0, st, args)
    // (four waves measured faster than eight here -- 0.68 against 0.77 ms at config 2 -- the opposite of the forward kernel)
#define SMB_T(T) do { if (slots <= 4) SMB(T, 4); else if (slots <= 8) SMB(T, 8); else if (slots <= 13) SMB(T, 13); else SMB(T, 16); } while (0)
    if (dtype == BF16) SMB_T(bf16_t); else SMB_T(f16_t);
#undef SMB_T
#undef SMB
    return check_launch("bs_softmax32_bwd_kernel");
}

extern "C" int flyhip_bs_rowreduce(const void* x, void* out, const int32_t* row_ptr, const int32_t* row_blk,
                                   int n_brow, int Z, int blk, int64_t x_sz, int op, int dtype, void* stream) {
    int rc = check_common("bs_rowreduce", blk, dtype, Z);
    if (rc) return rc;
    FLY_REQUIRE(x && out && row_ptr && row_blk, "bs_rowreduce: null pointer");
    FLY_REQUIRE(op == 0 || op == 1, "bs_rowreduce: op must be 0 (logsumexp) or 1 (sum)");
    FLY_REQUIRE(n_brow > 0, "bs_rowreduce: no rows");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    RowArgs args{const_cast<void*>(x), out, row_ptr, row_blk, nullptr, n_brow, 1, blk_shift_of(blk), x_sz, 1.f,
                 nullptr, 0, 0, nullptr, 0, 0, op};
    dim3 grid((unsigned)waves_to_blocks((long)n_brow * blk), Z);
    switch (dtype) {
        case F32: hipLaunchKernelGGL((bs_rowreduce_kernel<float>), grid, dim3(256), 0, st, args); break;
        case BF16: hipLaunchKernelGGL((bs_rowreduce_kernel<bf16_t>), grid, dim3(256), 0, st, args); break;
        default: hipLaunchKernelGGL((bs_rowreduce_kernel<f16_t>), grid, dim3(256), 0, st, args); break;
    }
    return check_launch("bs_rowreduce_kernel");
}
