// Inputs of the backward band kernels of Scatterbrain-local attention, formed in three launches.
//
// The reference obtains its gradients from autograd through softmax_kernel
// (src/models/attention/feature_maps_sb.py:51-82) and the op sequence of
// src/models/attention/sblocal_attention.py:73-122.  Written out, the backward needs, per (batch, head):
//   psi_i  (T, m)  = Phi(q_i) exp(kappa) / Z_i      phik_s (S, m) = Phi(k_s) exp(-kappa)   (zero past the key length)
//   c_i    = g_i . out_i
//   KV = sum_s phik_s v_s^T,  ksum = sum_s phik_s,  QG = sum_i psi_i g_i^T,  qc = sum_i psi_i c_i
// with Phi_r(x) = exp(+-sqrt(t) p_r.x - t |x|^2 / 2) / sqrt(m), Z_i = exp(log_normalization_i), and kappa the
// largest log-feature of a valid key of the (batch, head), so that no key feature exceeds one.
//   pass 1  sb_prep_kmax_kernel    per 64 keys: max over valid keys and features of the log-feature
//   pass 2  sb_prep_kernel         kappa from pass 1; features (fp32 MFMA projections), c, and this workgroup's
//                                  share of the four sums (fp32 MFMA) as a partial
//   pass 3  sb_prep_reduce_kernel  partials -> KV, ksum, QG, qc
// Everything is float32; nothing here is summed with atomics, so results do not depend on scheduling.
#include "common.h"

namespace flyhip {

struct PrepArgs {
    const float* q; const float* k; const float* v; const float* g; const float* o;   // (BH, rows, DIM), packed
    const float* ln;                 // (BH, T)
    const float* proj;               // (MK/2, DIM), rows >= mh_valid zero
    const int64_t* lens;             // (BH / H) or null
    float* psi; float* phik;         // (BH, T, MK), (BH, S, MK): [exp(+.) | exp(-.)], each half MK/2 wide
    float* c;                        // (BH, T)
    float* kv; float* ksum; float* qg; float* qc;       // (BH, MK, DIM), (BH, MK) twice
    float* pmax;                     // (BH, n_kblk)
    float* part;                     // (BH, n_split_k + n_split_q, MK * (DIM + 1))
    char* qimg; char* kimg;          // tile images for the band kernels on the bf16 matrix pipe (BwdTile), or null
    int BH, H, T, S, mh_valid, n_kblk, n_split_k, n_split_q;
    float temp;
};

constexpr int PREP_ROWS = 64;        // rows per step of a workgroup: 16 per wave
constexpr int PREP_NT = 256;

// 64 rows x W floats in LDS (row stride LD floats) -> their NP-piece images in the two 32-row tiles at `tile0` and
// `tile0 + tile_stride`: chunk c of a row = elements 8c .. 8c + 7, 16 bytes per piece
template <int W, int LD, int NP>
__device__ __forceinline__ void prep_emit_rows(const float* src, char* tile0, long tile_stride, int piece_bytes, int tid) {
    constexpr int CH8 = W / 8, ROWB = 2 * W, TOT = 64 * CH8;
#pragma unroll
    for (int j = 0; j < (TOT + 255) / 256; ++j) {
        const int idx = tid + 256 * j;
        if (TOT % 256 == 0 || idx < TOT) {
            const int row64 = idx / CH8, ch = idx % CH8, row = row64 & 31;
            const float* sp = src + row64 * LD + 8 * ch;
            uintx4 h, m, l;
            if (NP == 3) split3(*reinterpret_cast<const floatx4*>(sp), *reinterpret_cast<const floatx4*>(sp + 4), h, m, l);
            else split2(*reinterpret_cast<const floatx4*>(sp), *reinterpret_cast<const floatx4*>(sp + 4), h, m);
            char* dst = tile0 + (row64 >> 5) * tile_stride + row * ROWB + x3_swz(row, ch, ROWB) * 16;
            *reinterpret_cast<uintx4*>(dst) = h;
            *reinterpret_cast<uintx4*>(dst + piece_bytes) = m;
            if (NP == 3) *reinterpret_cast<uintx4*>(dst + 2 * piece_bytes) = l;
        }
    }
}

// Image of 32 rows of one side (queries: q, g, psi; keys: k, v, phik) for the band kernels on the bf16 matrix
// pipe: every operand as two bf16 pieces (head and rest: 16 to 17 significant bits; the features are rounded to
// 17 bits first, so their pieces are exact), elements of a row in their natural order (both operands of every
// product come from images, so lane g's eight k-slots of a 32-wide MFMA step are simply elements 8g .. 8g + 7 of
// it), 16-byte chunks XOR-swizzled (x3_swz) so that fragment reads of neighbouring rows fall into different LDS
// banks -- the row reads of the score products and the transposed reads of the output products alike.  One image is one LDS stage of the band
// kernel, copied linearly:  [x hi][x lo][y h][y m][y l][features hi][features lo][log2(e) log Z of the 32 rows][c].
// y (the values, resp. d out) comes in three pieces, exact to fp32: df = g.v - g.out is a difference of nearly
// equal numbers wherever one key carries a query's whole weight.
template <int DIM, int MK>
struct BwdTile {
    static constexpr int ROWS = 32;
    static constexpr int X_ROW = 2 * DIM, F_ROW = 2 * MK;                       // bytes per row of a piece
    static constexpr int X_PIECE = ROWS * X_ROW, F_PIECE = ROWS * F_ROW;
    static constexpr int X_OFF = 0, Y_OFF = 2 * X_PIECE, F_OFF = 5 * X_PIECE, S_OFF = F_OFF + 2 * F_PIECE;
    static constexpr int MAIN = S_OFF, BYTES = S_OFF + 2 * ROWS * 4;
    static_assert(MAIN % 1024 == 0, "whole wave loads of 16 bytes per lane");
};

// sqrt(t) P x for the 16 rows of a wave.  prep_load: lane (r16, g) takes elements 16 c + 4 g .. + 3 of input row
// r16 of the wave; prep_project returns in dd[fb][i] the projection of that row on row 16 fb + 4 g + i of P, and
// in sq the row's |x|^2.
template <int DIM>
__device__ __forceinline__ void prep_load(const float* xrow, int g, floatx4 (&xb)[DIM / 16]) {
#pragma unroll
    for (int cc = 0; cc < DIM / 16; ++cc) xb[cc] = *reinterpret_cast<const floatx4*>(xrow + 16 * cc + 4 * g);
}
template <int DIM, int FB>
__device__ __forceinline__ void prep_project(floatx4 (&xb)[DIM / 16], const float* proj, float st, int r16, int g,
                                             floatx4 (&dd)[FB], float& sq) {
    constexpr int EC = DIM / 16;
    const float* pp = proj + r16 * DIM + 4 * g;
    sq = 0.f;
#pragma unroll
    for (int cc = 0; cc < EC; ++cc) {
        sq += xb[cc][0] * xb[cc][0] + xb[cc][1] * xb[cc][1] + xb[cc][2] * xb[cc][2] + xb[cc][3] * xb[cc][3];
        xb[cc] *= st;
    }
    sq = group_sum(sq);
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) dd[fb] = Frag<float>::zero();
#pragma unroll
    for (int cc = 0; cc < EC; ++cc) {
        floatx4 pa[FB];
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) pa[fb] = *reinterpret_cast<const floatx4*>(pp + 16 * fb * DIM + 16 * cc);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int fb = 0; fb < FB; ++fb)
                dd[fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[fb][j], xb[cc][j], dd[fb], 0, 0, 0);
    }
}

template <int DIM, int MK>
__global__ __launch_bounds__(PREP_NT) void sb_prep_kmax_kernel(PrepArgs a) {
    constexpr int FB = MK / 32;
    __shared__ float red[4];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y, b = bh / a.H;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const int row = blockIdx.x * PREP_ROWS + 16 * w + r16;
    const float* xrow = a.k + ((long)bh * a.S + min(row, a.S - 1)) * DIM;
    floatx4 dd[FB], xb[DIM / 16];
    float sq;
    prep_load<DIM>(xrow, g, xb);
    prep_project<DIM, FB>(xb, a.proj, sqrtf(a.temp), r16, g, dd, sq);
    float amax = 0.f;
#pragma unroll
    for (int fb = 0; fb < FB; ++fb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (16 * fb + 4 * g + i < a.mh_valid) amax = fmaxf(amax, fabsf(dd[fb][i]));
    amax = group_max(amax);
    float cs = row < len ? amax - 0.5f * a.temp * sq - 0.5f * logf(2.0f * a.mh_valid) : -INFINITY;
    cs = wave_max(cs);
    if (lane == 0) red[w] = cs;
    __syncthreads();
    if (tid == 0) a.pmax[(long)bh * a.n_kblk + blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// (at least two workgroups per compute unit: the kernel streams, and at 128 features the registers it would like to take
//  leave room for one only; the few it spills instead cost less)
template <int DIM, int MK, bool WRITE_F>     // WRITE_F: the float32 feature arrays are wanted (not only the images)
__global__ __launch_bounds__(PREP_NT) __attribute__((amdgpu_waves_per_eu(2, 8))) void sb_prep_kernel(PrepArgs a) {
    constexpr int MH = MK / 2, FB = MK / 32, RBN = MK / 16, RB = (RBN + 3) / 4, DB = DIM / 16;
    constexpr int LDF = MK + 4, LDY = DIM + 4;
    __shared__ float Fs[PREP_ROWS * LDF];         // features of the current rows
    __shared__ float Ys[PREP_ROWS * LDY];         // their V (keys) or d out (queries)
    __shared__ float red[4];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y, b = bh / a.H;
    const bool key_role = (int)blockIdx.x < a.n_split_k;
    const int sp = key_role ? blockIdx.x : blockIdx.x - a.n_split_k;
    const int n_split = key_role ? a.n_split_k : a.n_split_q;
    const int rows = key_role ? a.S : a.T;
    const int len = key_role ? (a.lens ? min((int)a.lens[b], a.S) : a.S) : a.T;
    const float* X = (key_role ? a.k : a.q) + (long)bh * rows * DIM;
    float* F = WRITE_F ? (key_role ? a.phik : a.psi) : nullptr;
    if (F) F += (long)bh * rows * MK;

    // kappa: the maximum over the key blocks of pass 1 (0 when no key is valid)
    float kappa = -INFINITY;
    for (int i = tid; i < a.n_kblk; i += PREP_NT) kappa = fmaxf(kappa, a.pmax[(long)bh * a.n_kblk + i]);
    kappa = wave_max(kappa);
    if (lane == 0) red[w] = kappa;
    __syncthreads();
    kappa = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (kappa == -INFINITY) kappa = 0.f;
    const float off = 0.5f * logf(2.0f * a.mh_valid), st = sqrtf(a.temp);

    const int n_chunks = (rows + PREP_ROWS - 1) / PREP_ROWS;
    const int per = (n_chunks + n_split - 1) / n_split;
    const int c0 = sp * per, c1 = min(n_chunks, c0 + per);

    floatx4 acc[RB][DB];
#pragma unroll
    for (int x = 0; x < RB; ++x)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[x][db] = Frag<float>::zero();
    floatx4 sp_[FB], sn_[FB];                     // weighted sums of this lane's row of features
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) { sp_[fb] = Frag<float>::zero(); sn_[fb] = Frag<float>::zero(); }

    // one chunk of loads ahead: this thread's pieces of the Y (and out) rows, its wave row of X, that row's log Z
    constexpr int NJ = PREP_ROWS * DIM / 4 / PREP_NT;
    floatx4 yv[NJ], ov[NJ], xn[DIM / 16];
    float ln_n = 0.f;
    auto fetch = [&](int c) __attribute__((always_inline)) {
        const int base = c * PREP_ROWS;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int idx = tid + PREP_NT * j, r = idx / (DIM / 4), c4 = idx % (DIM / 4);
            const long at = ((long)bh * rows + min(base + r, rows - 1)) * DIM + 4 * c4;
            yv[j] = *reinterpret_cast<const floatx4*>((key_role ? a.v : a.g) + at);
            if (!key_role) ov[j] = *reinterpret_cast<const floatx4*>(a.o + at);
        }
        const int row = min(base + 16 * w + r16, rows - 1);
        prep_load<DIM>(X + (long)row * DIM, g, xn);
        if (!key_role) ln_n = a.ln[(long)bh * rows + row];
    };
    if (c0 < c1) fetch(c0);

    for (int c = c0; c < c1; ++c) {
        const int base = c * PREP_ROWS;
        // Y rows -> LDS (rows past the end as zeros); queries: c = g . out on the way, 16 lanes per row
        float* crow = Fs;                         // 64 floats, consumed before the features are written
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int idx = tid + PREP_NT * j, r = idx / (DIM / 4), c4 = idx % (DIM / 4);
            const bool live = base + r < rows;
            floatx4 y = yv[j];
            if (!live) y = Frag<float>::zero();
            *reinterpret_cast<floatx4*>(Ys + r * LDY + 4 * c4) = y;
            if (!key_role) {
                const floatx4 o = ov[j];
                float d = y[0] * o[0] + y[1] * o[1] + y[2] * o[2] + y[3] * o[3];
                if (DIM == 64) {
                    d = row16_sum(d);             // the 16 lanes of a row of 64 floats share a DPP row
                } else {
                    // 8 lanes per row of 32 floats: quad butterflies and the half-row mirror stay inside them
                    d += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(d), 0xB1, 0xf, 0xf, true));
                    d += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(d), 0x4E, 0xf, 0xf, true));
                    d += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(d), 0x141, 0xf, 0xf, true));
                }
                if (c4 == 0) {
                    crow[r] = d;
                    if (live) a.c[(long)bh * rows + base + r] = d;
                }
            }
        }
        floatx4 xb[DIM / 16];
#pragma unroll
        for (int cc = 0; cc < DIM / 16; ++cc) xb[cc] = xn[cc];
        const float ln_row = ln_n;
        __syncthreads();
        if (c + 1 < c1) fetch(c + 1);             // the next chunk's loads fly during this chunk's arithmetic
        const int row = base + 16 * w + r16;
        const bool valid = row < len;
        const float wrow = key_role ? 1.f : crow[16 * w + r16];
        using TL = BwdTile<DIM, MK>;
        char* img = key_role ? a.kimg : a.qimg;
        const int trow = (16 * w + r16) & 31;     // this lane's row inside its 32-row tile
        char* img0 = nullptr;                     // the chunk's first tile
        if (img) {
            img0 = img + ((long)bh * 2 * n_chunks + 2 * c) * TL::BYTES;
            img = img0 + (w >> 1) * TL::BYTES;
            // x of the lane's row: its elements 16 cc + 4 g .. + 3 are half g % 2 of chunk 2 cc + g / 2
#pragma unroll
            for (int cc = 0; cc < DIM / 16; ++cc) {
                const int at = x3_swz(trow, 2 * cc + (g >> 1), TL::X_ROW) * 16 + 8 * (g & 1);
                char* dst = img + TL::X_OFF + trow * TL::X_ROW + at;
                uint2 p0, p1;
                split2_4(xb[cc], p0, p1);
                *reinterpret_cast<uint2*>(dst) = p0;
                *reinterpret_cast<uint2*>(dst + TL::X_PIECE) = p1;
            }
            // y rows from their LDS copy, 16 bytes per piece and thread
            prep_emit_rows<DIM, LDY, 3>(Ys, img0 + TL::Y_OFF, TL::BYTES, TL::X_PIECE, tid);
            if (g == 0) {
                float* tr = reinterpret_cast<float*>(img + TL::S_OFF);
                tr[trow] = key_role ? 0.f : ln_row * 1.4426950408889634f;
                tr[32 + trow] = wrow;
            }
        }
        floatx4 dd[FB];
        float sq;
        prep_project<DIM, FB>(xb, a.proj, st, r16, g, dd, sq);
        float bias;
        if (key_role) bias = -0.5f * a.temp * sq - off - kappa;
        else bias = kappa - ln_row - 0.5f * a.temp * sq - off;
        __syncthreads();                          // every c of this chunk has been read
        float* frow_s = Fs + (16 * w + r16) * LDF;
        floatx4 fblk[WRITE_F ? 2 * FB : 1];       // the row's features: blocks of 16, [exp(+.) | exp(-.)]
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
            floatx4 fp, fn;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = valid && (16 * fb + 4 * g + i < a.mh_valid);
                // (the hardware exponential: its last-bit differences vanish in the rounding to 17 bits below)
                fp[i] = ok ? __expf(dd[fb][i] + bias) : 0.f;
                fn[i] = ok ? __expf(bias - dd[fb][i]) : 0.f;
            }
            if (img) { fp = quant16(fp); fn = quant16(fn); }     // every use sees the features rounded to 17 bits
            sp_[fb] += fp * wrow;
            sn_[fb] += fn * wrow;
            *reinterpret_cast<floatx4*>(frow_s + 16 * fb + 4 * g) = fp;
            *reinterpret_cast<floatx4*>(frow_s + MH + 16 * fb + 4 * g) = fn;
            if (WRITE_F) { fblk[fb] = fp; fblk[FB + fb] = fn; }
        }
        if (WRITE_F && F && row < rows) {
            float* frow_g = F + (long)row * MK;
#pragma unroll
            for (int fb = 0; fb < 2 * FB; ++fb) *reinterpret_cast<floatx4*>(frow_g + 16 * fb + 4 * g) = fblk[fb];
        }
        __syncthreads();
        if (img) prep_emit_rows<MK, LDF, 2>(Fs, img0 + TL::F_OFF, TL::BYTES, TL::F_PIECE, tid);
        // acc[r][d] += sum_rows F[row][r] Y[row][d]; lane ends with element (16 rb + 4g + i, 16 db + r16)
#pragma unroll
        for (int kk = 0; kk < PREP_ROWS / 16; ++kk) {
            floatx4 yb[DB];
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int j = 0; j < 4; ++j) yb[db][j] = Ys[(16 * kk + 4 * g + j) * LDY + 16 * db + r16];
#pragma unroll
            for (int x = 0; x < RB; ++x) {
                const int rb = w + 4 * x;
                if (rb < RBN) {
                    floatx4 fa;
#pragma unroll
                    for (int j = 0; j < 4; ++j) fa[j] = Fs[(16 * kk + 4 * g + j) * LDF + 16 * rb + r16];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int db = 0; db < DB; ++db)
                            acc[x][db] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[j], yb[db][j], acc[x][db], 0, 0, 0);
                }
            }
        }
        __syncthreads();                          // Fs and Ys free for the next chunk
    }

    // the partial: the matrix in accumulator order (tile (rb, db) -> 64 lanes x 4 floats), then the MK sums
    float* part = a.part + ((long)bh * (a.n_split_k + a.n_split_q) + blockIdx.x) * (MK * (DIM + 1));
#pragma unroll
    for (int x = 0; x < RB; ++x) {
        const int rb = w + 4 * x;
        if (rb < RBN) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
                *reinterpret_cast<floatx4*>(part + ((rb * DB + db) * 64 + lane) * 4) = acc[x][db];
        }
    }
    float* sums = Fs;                             // 4 x MK floats
#pragma unroll
    for (int fb = 0; fb < FB; ++fb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float p = row16_sum(sp_[fb][i]), n = row16_sum(sn_[fb][i]);
            if (r16 == 0) {
                sums[w * MK + 16 * fb + 4 * g + i] = p;
                sums[w * MK + MH + 16 * fb + 4 * g + i] = n;
            }
        }
    __syncthreads();
    if (tid < MK) part[MK * DIM + tid] = (sums[tid] + sums[MK + tid]) + (sums[2 * MK + tid] + sums[3 * MK + tid]);
}

// element (r, d) of the matrices (d == DIM: the vectors) = sum over the role's partials, in order
template <int DIM, int MK>
__global__ __launch_bounds__(PREP_NT) void sb_prep_reduce_kernel(PrepArgs a) {
    constexpr int DB = DIM / 16, PER = MK * (DIM + 1);
    const int e = blockIdx.x * PREP_NT + threadIdx.x, role = blockIdx.y, bh = blockIdx.z;
    if (e >= PER) return;
    const int n = role ? a.n_split_q : a.n_split_k;
    const float* part = a.part + ((long)bh * (a.n_split_k + a.n_split_q) + (role ? a.n_split_k : 0)) * PER;
    int src;
    float* dst;
    if (e < MK * DIM) {
        const int r = e / DIM, d = e % DIM;
        src = (((r / 16) * DB + d / 16) * 64 + 16 * ((r % 16) / 4) + d % 16) * 4 + r % 4;
        dst = (role ? a.qg : a.kv) + (long)bh * MK * DIM + e;
    } else {
        src = e;
        dst = (role ? a.qc : a.ksum) + (long)bh * MK + (e - MK * DIM);
    }
    float s = 0.f;
    int i = 0;
    for (; i + 8 <= n; i += 8) {                  // eight loads in flight, summed in order
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = part[(long)(i + j) * PER + src];
#pragma unroll
        for (int j = 0; j < 8; ++j) s += x[j];
    }
    for (; i < n; ++i) s += part[(long)i * PER + src];
    *dst = s;
}

// ---------------------------------------------------------------------------------------
// band terms of the backward pass on the bf16 matrix pipe
// ---------------------------------------------------------------------------------------
// The arithmetic of sblocal_bwd_band_kernel (pair weights a = exp(t q.k - log Z), kb = psi.phik, df = g.v - c,
// dm = a df; five band-limited sums; the finishing epilogue with the per-head matrices and the chain rule through
// the feature map), with every product on v_mfma_f32_16x16x32_bf16 from operands in two bf16 pieces and fp32
// accumulation: three piece products for q.k and the sum over dm; six for (a - kb) g (its low-rank part cancels against Q'^T g) (the rest-times-rest product, 2^-16
// relative, is dropped); six for g.v from three pieces each (exact to fp32: df = g.v - c cancels where one key carries
// a query's weight) and five for phik^T df with df in three pieces; all four for psi.phik, whose operands are exact in two pieces -- the band's low-rank
// weight then cancels against the per-head sums, which the preparation pass forms from the same rounded features.
// The inner side comes as the images of BwdTile, one image = one LDS stage, copied by loads that write LDS
// directly; the outer side's operands are read once from the images of its own rows.  The output products need
// the inner rows transposed (k = inner row): ds_read_b64_tr_b16 delivers that from the row-major pieces -- 16
// lanes pass the addresses of 4 rows x 4 groups of 4 columns and receive, lane l, column l of the 4 rows -- so
// no transposed copy exists anywhere.
struct BwdX3Args {
    const char* oimg; const char* iimg;        // images of the outer and of the inner side
    const float* x1;                           // the outer rows themselves (BH, Lo, E), for the epilogue
    const float* ln; const float* c;           // (BH, T)
    const int64_t* lens;
    float* o1; float* o3;                      // d x1 (BH, Lo, E); d v (BH, S, E), key-major only
    int BH, H, T, S, lc;
    float temp;
    const float* gmat; const float* gvec; const float* proj;
    int n_xcd;
    // small problems: every outer tile's inner range walked in n_parts parts by as many workgroups, whose sums go to
    // part_ws ((tile, part): registers x 256 lanes x 4 floats) and are finished by sblocal_bwd_x3_finish_kernel
    float* part_ws; int n_parts;
    // a block-sparse support instead of a band (LIST kernels; 16 x 16 or 32 x 32 blocks, no key lengths): per (head,
    // 64-row outer tile) the inner 32-row tiles that any of its rows meets on the support, and per entry four masks, one
    // per group of 16 outer rows (a wave): bit 0 / bit 1 = that group meets inner rows 0..15 / 16..31 of the entry's tile
    const int32_t* tl_ptr; const int32_t* tl_inner; const int32_t* tl_blk;
    // long lists: tl_skip (one flag per (head, outer tile)) marks the tiles the main launch leaves out; the launch
    // in parts takes (batch, tl_heavy[j], part) for the n_heavy listed (head, outer tile) indices, then the finish
    const int32_t* tl_skip; const int32_t* tl_heavy; int n_heavy;
    // dropout of the exact weights in the forward (drop_thresh = 0: none): the same mask again from the seed --
    // pair (query i of bh, key s) was kept iff drop_keep(drop_row_hash(drop_seed, bh T + i), s, drop_thresh)
    uint32_t drop_seed, drop_thresh; float drop_scale;
};

// one tile image, global memory -> LDS stage `dst` (linear; each wave load writes 1024 consecutive bytes); TAIL: also
// the 256 bytes behind the MAIN ones (log Z and c of the tile's queries; a full wave load, lanes 16.. repeat them)
template <int MAIN, bool TAIL>
__device__ __forceinline__ void bwd_tile_to_lds(const char* src, char* dst, int tid) {
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
#pragma unroll
    for (int j = 0; j < MAIN / 4096; ++j) dma_to_lds(src + 4096 * j + 16 * tid, dst + 4096 * j + 1024 * w);
    constexpr int FULL = MAIN / 4096 * 4096;
    if (MAIN % 4096 != 0 && w < (MAIN % 4096) / 1024) dma_to_lds(src + FULL + 16 * tid, dst + FULL + 1024 * w);
    if (TAIL && w == 0) dma_to_lds(src + MAIN + 16 * (lane & 15), dst + MAIN);
}

// LDS bytes of the finishing step: gmat (M, D) and the projection (at least 32 rows, E) in three bf16 pieces, gvec
template <int E, int M>
constexpr int bwd_x3_epilogue_bytes() { return 3 * M * 2 * E + 3 * (M / 2 < 32 ? 32 : M / 2) * 2 * E + M * 4; }

// rows x W floats in global memory (row stride W) -> three bf16 pieces in LDS ([h | m | l], `piece` bytes apart, rows
// of 2 W bytes in natural element order, 16-byte chunks swizzled); rows >= rows_valid are written as zeros
template <int W>
__device__ __forceinline__ void bwd_x3_stage3(const float* src, char* dst, int rows, int rows_valid, int piece, int tid) {
    for (int idx = tid; idx < rows * (W / 8); idx += 256) {
        const int r = idx / (W / 8), ch = idx % (W / 8);
        floatx4 x0 = Frag<float>::zero(), x1 = x0;
        if (r < rows_valid) {
            x0 = *reinterpret_cast<const floatx4*>(src + (long)r * W + 8 * ch);
            x1 = *reinterpret_cast<const floatx4*>(src + (long)r * W + 8 * ch + 4);
        }
        uintx4 h, m, l;
        split3(x0, x1, h, m, l);
        char* d = dst + r * (2 * W) + x3_swz(r, ch, 2 * W) * 16;
        *reinterpret_cast<uintx4*>(d) = h;
        *reinterpret_cast<uintx4*>(d + piece) = m;
        *reinterpret_cast<uintx4*>(d + 2 * piece) = l;
    }
}

// The finishing step of an outer tile: the sums over all keys / queries through the per-head matrices, the chain rule
// through the feature map, and the stores; with u_f = x2_f (gmat_f . x3 - c gvec_f - acc2_f),
//   d x1 = t acc1 + sqrt(t) P^T (u+ - u-) - t x1 sum_f u_f,     d v = acc3 + gmat^T x2   (key-major).
// The three products run on the bf16 matrix pipe like the band sums: gmat and P in three pieces (exact), x3 from the
// three pieces of its image, u+ - u- in three pieces, x2 in its two; six, six and five piece products, everything
// above 2^-24 relative, because gmat . x3 is the "all keys" term the band's sum acc2 is subtracted from.  Transposed
// operands (P^T, gmat^T) by ds_read_b64_tr_b16 as in the band loop.  smem: bwd_x3_epilogue_bytes<E, M>() bytes, not in
// use by anyone (the caller's last access to it lies behind a barrier).
template <int E, int M, bool KEYMAJOR>
__device__ __forceinline__ void bwd_x3_epilogue(const BwdX3Args& a, char* smem, int bh, int o, int orow, int Lo,
                                                const char* otile, int trow, float c_o,
                                                floatx4 (&acc1)[E / 16], floatx4 (&acc2)[M / 16], floatx4 (&acc3)[KEYMAJOR ? E / 16 : 1]) {
    using TL = BwdTile<E, M>;
    constexpr int D = E, KS1 = E / 32, EC = E / 16, FC = M / 16, DB = D / 16, MH = M / 2, PR = MH < 32 ? 32 : MH;
    constexpr int G_ROW = 2 * D, G_PIECE = M * G_ROW, P_ROW = 2 * E, P_PIECE = PR * P_ROW;
    const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    char* GMs = smem;                                      // gmat pieces
    char* Ps = GMs + 3 * G_PIECE;                          // projection pieces
    float* GVs = reinterpret_cast<float*>(Ps + 3 * P_PIECE);
    bwd_x3_stage3<D>(a.gmat + (long)bh * M * D, GMs, M, M, G_PIECE, tid);
    bwd_x3_stage3<E>(a.proj, Ps, PR, MH, P_PIECE, tid);
    if (tid < M) GVs[tid] = a.gvec[(long)bh * M + tid];
    // the outer row: x1 in fp32, x3 as the three pieces of its image, its features from their two pieces (exact)
    floatx4 x1[EC], x2[FC];
    uintx4 x3h[KS1], x3m[KS1], x3l[KS1];
#pragma unroll
    for (int c = 0; c < EC; ++c) x1[c] = load4_f32(a.x1 + ((long)bh * Lo + orow) * E + 16 * c + 4 * g);
#pragma unroll
    for (int ks = 0; ks < KS1; ++ks) {
        const char* p = otile + TL::Y_OFF + trow * TL::X_ROW + x3_swz(trow, 4 * ks + g, TL::X_ROW) * 16;
        x3h[ks] = *reinterpret_cast<const uintx4*>(p);
        x3m[ks] = *reinterpret_cast<const uintx4*>(p + TL::X_PIECE);
        x3l[ks] = *reinterpret_cast<const uintx4*>(p + 2 * TL::X_PIECE);
    }
#pragma unroll
    for (int c = 0; c < FC; ++c) {
        const char* p = otile + TL::F_OFF + trow * TL::F_ROW + x3_swz(trow, 2 * c + (g >> 1), TL::F_ROW) * 16 + 8 * (g & 1);
        const uint2 fh = *reinterpret_cast<const uint2*>(p), fl = *reinterpret_cast<const uint2*>(p + TL::F_PIECE);
        x2[c][0] = __uint_as_float(fh.x << 16) + __uint_as_float(fl.x << 16);
        x2[c][1] = __uint_as_float(fh.x & 0xffff0000u) + __uint_as_float(fl.x & 0xffff0000u);
        x2[c][2] = __uint_as_float(fh.y << 16) + __uint_as_float(fl.y << 16);
        x2[c][3] = __uint_as_float(fh.y & 0xffff0000u) + __uint_as_float(fl.y & 0xffff0000u);
    }
    __syncthreads();
    // u^T[f][outer] = sum_d gmat[f][d] x3[d][outer]
    floatx4 u[FC];
#pragma unroll
    for (int c = 0; c < FC; ++c) {
        u[c] = Frag<float>::zero();
#pragma unroll
        for (int ks = 0; ks < KS1; ++ks) {
            const int row = 16 * c + r16;
            const char* p = GMs + row * G_ROW + x3_swz(row, 4 * ks + g, G_ROW) * 16;
            const uintx4 gh = *reinterpret_cast<const uintx4*>(p), gm = *reinterpret_cast<const uintx4*>(p + G_PIECE);
            const uintx4 gl = *reinterpret_cast<const uintx4*>(p + 2 * G_PIECE);
            u[c] = mma_bf16(gl, x3h[ks], u[c]);
            u[c] = mma_bf16(gh, x3l[ks], u[c]);
            u[c] = mma_bf16(gm, x3m[ks], u[c]);
            u[c] = mma_bf16(gm, x3h[ks], u[c]);
            u[c] = mma_bf16(gh, x3m[ks], u[c]);
            u[c] = mma_bf16(gh, x3h[ks], u[c]);
        }
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
    // transposed reads as in the band loop: rows 4g + r16/4 (+ 16) of a 32-row step, columns 4 (r16 % 4) .. + 3 of a block
    const int tr_row = 4 * g + (r16 >> 2), tr_cb = r16 & 3;
    // chain rule through the projection: dp^T[e][outer] = sum_r P[r][e] (u_r - u_{r + M/2}), 32 rows r per step
    floatx4 dp[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) dp[c] = Frag<float>::zero();
#pragma unroll
    for (int ks = 0; ks < PR / 32; ++ks) {
        const floatx4 du0 = u[2 * ks] - u[2 * ks + FC / 2];
        floatx4 du1 = Frag<float>::zero();
        if (2 * ks + 1 < FC / 2) du1 = u[(2 * ks + 1 < FC / 2) ? 2 * ks + 1 : 0] - u[(2 * ks + 1 < FC / 2) ? 2 * ks + 1 + FC / 2 : 0];
        uintx4 dh, dm, dl;
        split3(du0, du1, dh, dm, dl);
#pragma unroll
        for (int eb = 0; eb < EC; ++eb) {
            const int row = 32 * ks + tr_row;
            const char* p = Ps + row * P_ROW + x3_swz(row, 2 * eb + (tr_cb >> 1), P_ROW) * 16 + 8 * (tr_cb & 1);
            const uintx4 ph = lds_read_tr8(p, p + 16 * P_ROW), pm = lds_read_tr8(p + P_PIECE, p + P_PIECE + 16 * P_ROW);
            const uintx4 pl = lds_read_tr8(p + 2 * P_PIECE, p + 2 * P_PIECE + 16 * P_ROW);
            dp[eb] = mma_bf16(pl, dh, dp[eb]);
            dp[eb] = mma_bf16(ph, dl, dp[eb]);
            dp[eb] = mma_bf16(pm, dm, dp[eb]);
            dp[eb] = mma_bf16(pm, dh, dp[eb]);
            dp[eb] = mma_bf16(ph, dm, dp[eb]);
            dp[eb] = mma_bf16(ph, dh, dp[eb]);
        }
    }
    if (KEYMAJOR) {
        // d v^T[d][key] += sum_f gmat[f][d] phik[f][key], 32 features per step
#pragma unroll
        for (int ks = 0; ks < M / 32; ++ks) {
            uintx4 xh, xl;
            split2(x2[2 * ks], x2[2 * ks + 1], xh, xl);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int row = 32 * ks + tr_row;
                const char* p = GMs + row * G_ROW + x3_swz(row, 2 * db + (tr_cb >> 1), G_ROW) * 16 + 8 * (tr_cb & 1);
                const uintx4 gh = lds_read_tr8(p, p + 16 * G_ROW), gm = lds_read_tr8(p + G_PIECE, p + G_PIECE + 16 * G_ROW);
                const uintx4 gl = lds_read_tr8(p + 2 * G_PIECE, p + 2 * G_PIECE + 16 * G_ROW);
                acc3[db] = mma_bf16(gl, xh, acc3[db]);
                acc3[db] = mma_bf16(gm, xl, acc3[db]);
                acc3[db] = mma_bf16(gm, xh, acc3[db]);
                acc3[db] = mma_bf16(gh, xl, acc3[db]);
                acc3[db] = mma_bf16(gh, xh, acc3[db]);
            }
        }
    }
    if (o < Lo) {
        const float st_ = sqrtf(a.temp);
        float* p1 = a.o1 + ((long)bh * Lo + o) * E;
#pragma unroll
        for (int c = 0; c < EC; ++c) store4_f32(p1 + 16 * c + 4 * g, acc1[c] * a.temp + dp[c] * st_ - x1[c] * (a.temp * usum));
        if (KEYMAJOR) {
            float* p3 = a.o3 + ((long)bh * Lo + o) * D;
#pragma unroll
            for (int c = 0; c < DB; ++c) store4_f32(p3 + 16 * c + 4 * g, acc3[c]);
        }
    }
}

template <int E, int M, bool KEYMAJOR, bool PARTS, bool LIST = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void sblocal_bwd_x3_kernel(BwdX3Args a) {
    using TL = BwdTile<E, M>;
    constexpr int NT = 256, TQ = 64, TK = 32, KB = 2;
    constexpr int D = E, KS1 = E / 32, KS2 = M / 32, EC = E / 16, FC = M / 16, DB = D / 16, MH = M / 2;
    constexpr int STAGE = TL::MAIN + 1024;                 // the image and a full wave load for its 256-byte tail
    constexpr float LOG2E = 1.4426950408889634f;
    static_assert(bwd_x3_epilogue_bytes<E, M>() <= 2 * STAGE, "epilogue operands must fit the tile stages");
    extern __shared__ __attribute__((aligned(256))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int Lo = KEYMAJOR ? a.S : a.T, Li = KEYMAJOR ? a.T : a.S;
    const int n_ot = (Lo + TQ - 1) / TQ;
    const int n_parts = PARTS ? a.n_parts : 1;
    const int n_items = (LIST && PARTS ? (a.BH / a.H) * a.n_heavy : a.BH * n_ot) * n_parts;
    const int per_xcd = (n_items + a.n_xcd - 1) / a.n_xcd;
    const int item = (blockIdx.x % a.n_xcd) * per_xcd + blockIdx.x / a.n_xcd;   // neighbouring tiles share a die's L2
    if (item >= n_items) return;                           // workgroup-uniform
    const int part = item % n_parts, tile_id = item / n_parts;
    int ot = tile_id % n_ot, bh = tile_id / n_ot;
    if (LIST && PARTS) {                                   // tile_id = batch entry * n_heavy + index into the long lists
        const int hg = a.tl_heavy[tile_id % a.n_heavy];
        ot = hg % n_ot;
        bh = (tile_id / a.n_heavy) * a.H + hg / n_ot;
    }
    if (LIST && !PARTS && a.tl_skip && a.tl_skip[(bh % a.H) * n_ot + ot]) return;      // walked in parts by another launch
    const int b = bh / a.H;
    const int o0 = ot * TQ, ow0 = o0 + 16 * w, o = ow0 + r16;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi
    const int lo = KEYMAJOR ? -(lc_hi - 1) : -lc_lo, hi = KEYMAJOR ? lc_lo + 1 : lc_hi;     // seen from the outer row
    const int o_limit = KEYMAJOR ? len : a.T, n_limit = KEYMAJOR ? a.T : len;
    const bool ovalid = o < o_limit;
    const int n_oimg = 2 * ((Lo + 63) / 64), n_iimg = 2 * ((Li + 63) / 64);
    const char* itiles = a.iimg + (long)bh * n_iimg * TL::BYTES;

    const int o_last = min(o0 + TQ - 1, o_limit - 1);
    const int n_lo = max(0, o0 + lo), n_hi = min(n_limit, o_last + hi);
    const int kt_lo = n_lo / TK;
    const int kt_hi = (o_last >= o0 && n_hi > n_lo) ? (n_hi + TK - 1) / TK : kt_lo;
    // the inner tiles this workgroup meets: tile_at(i_lo) .. tile_at(i_hi - 1) -- the band's, this part's share of
    // them, or the entries of the outer tile's list
    int e_lo = 0, i_lo = 0, i_hi = kt_hi - kt_lo;
    if (LIST) {
        const int grp = (bh % a.H) * n_ot + ot;
        e_lo = a.tl_ptr[grp];
        i_hi = a.tl_ptr[grp + 1] - e_lo;
    }
    if (PARTS) {
        const int per = (i_hi + n_parts - 1) / n_parts;
        i_lo = min(i_hi, part * per);
        i_hi = min(i_hi, i_lo + per);
    }
    auto tile_at = [&](int i) __attribute__((always_inline)) { return LIST ? a.tl_inner[e_lo + i] : kt_lo + i; };

    if (i_lo < i_hi) bwd_tile_to_lds<TL::MAIN, KEYMAJOR>(itiles + (long)tile_at(i_lo) * TL::BYTES, smem, tid);

    // outer operands (B side: column = outer row, k-slots 8g .. 8g + 7 of every 32-wide step) from the row's image
    const int orow = min(o, Lo - 1), trow = orow & 31;
    const char* otile = a.oimg + ((long)bh * n_oimg + (orow >> 5)) * TL::BYTES;
    uintx4 x1h[KS1], x1l[KS1], x3h[KS1], x3m[KS1], x3l[KS1], x2h[KEYMAJOR ? KS2 : 1], x2l[KEYMAJOR ? KS2 : 1];
#pragma unroll
    for (int ks = 0; ks < KS1; ++ks) {
        const int off = trow * TL::X_ROW + x3_swz(trow, 4 * ks + g, TL::X_ROW) * 16;
        x1h[ks] = *reinterpret_cast<const uintx4*>(otile + TL::X_OFF + off);
        x1l[ks] = *reinterpret_cast<const uintx4*>(otile + TL::X_OFF + TL::X_PIECE + off);
        x3h[ks] = *reinterpret_cast<const uintx4*>(otile + TL::Y_OFF + off);
        x3m[ks] = *reinterpret_cast<const uintx4*>(otile + TL::Y_OFF + TL::X_PIECE + off);
        x3l[ks] = *reinterpret_cast<const uintx4*>(otile + TL::Y_OFF + 2 * TL::X_PIECE + off);
    }
    if (KEYMAJOR) {
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks) {
            const int off = trow * TL::F_ROW + x3_swz(trow, 4 * ks + g, TL::F_ROW) * 16;
            x2h[ks] = *reinterpret_cast<const uintx4*>(otile + TL::F_OFF + off);
            x2l[ks] = *reinterpret_cast<const uintx4*>(otile + TL::F_OFF + TL::F_PIECE + off);
        }
    }
    const float ln_o = KEYMAJOR ? 0.f : a.ln[(long)bh * a.T + orow] * LOG2E, c_o = KEYMAJOR ? 0.f : a.c[(long)bh * a.T + orow];
    const float sc = a.temp * LOG2E;                       // scores leave the MFMA unscaled; exponents are base 2
    const bool drop_on = a.drop_thresh != 0;               // (kernel-uniform)
    const uint32_t drop_row = drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + (KEYMAJOR ? 0 : orow)));   // query-major: the lane's query
    // inner rows this lane's outer row may meet: nmin <= n < nmin + span
    const int nmin = max(o + lo, 0);
    const unsigned span = ovalid ? (unsigned)max(min(o + hi, n_limit) - nmin, 0) : 0u;

    floatx4 acc1[EC], acc2[FC], acc3[KEYMAJOR ? DB : 1];
#pragma unroll
    for (int c = 0; c < EC; ++c) acc1[c] = Frag<float>::zero();
#pragma unroll
    for (int c = 0; c < FC; ++c) acc2[c] = Frag<float>::zero();
#pragma unroll
    for (int c = 0; c < (KEYMAJOR ? DB : 1); ++c) acc3[c] = Frag<float>::zero();

    // transposed reads: this lane passes the address of row 4g + r16/4 (and 16 rows further), columns 4 (r16 % 4) .. + 3
    // of the 16-column block (half (r16 % 4) % 2 of chunk 2c + (r16 % 4) / 2); it receives column r16 of rows
    // 4g .. 4g + 3 (16 + 4g ..): the k-slots of its weights
    const int tr_row = 4 * g + (r16 >> 2), tr_cb = r16 & 3;

    drain_loads();
    __syncthreads();

    for (int it = i_lo; it < i_hi; ++it) {
        const int n_base = tile_at(it) * TK;
        const int cur = (it - i_lo) & 1;
        const char* st = smem + cur * STAGE;
        if (it + 1 < i_hi)                                 // every wave is past the barrier that ended that stage's last use
            bwd_tile_to_lds<TL::MAIN, KEYMAJOR>(itiles + (long)tile_at(it + 1) * TL::BYTES, smem + (cur ^ 1) * STAGE, tid);

        // wave-uniform: does this tile meet the band of any of the wave's 16 outer rows (is the block of the wave's
        // block-row and this block-column part of the support)?
        const int pres = LIST ? a.tl_blk[4 * (e_lo + it) + w] & 3 : 3;      // (LIST: the wave's mask of this entry)
        const bool any = LIST ? pres != 0
                              : !(n_base + TK - 1 - ow0 < lo || n_base - (ow0 + 15) >= hi || n_base >= n_limit || ow0 >= o_limit);
        if (any) {
            floatx4 s1[KB], s2[KB], s3[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) { s1[kb] = Frag<float>::zero(); s2[kb] = Frag<float>::zero(); s3[kb] = Frag<float>::zero(); }
#pragma unroll
            for (int ks = 0; ks < KS1; ++ks)
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    const int row = 16 * kb + r16;
                    const char* p = st + row * TL::X_ROW + x3_swz(row, 4 * ks + g, TL::X_ROW) * 16;
                    const uintx4 yh = *reinterpret_cast<const uintx4*>(p + TL::X_OFF), yl = *reinterpret_cast<const uintx4*>(p + TL::X_OFF + TL::X_PIECE);
                    const uintx4 vh = *reinterpret_cast<const uintx4*>(p + TL::Y_OFF), vm = *reinterpret_cast<const uintx4*>(p + TL::Y_OFF + TL::X_PIECE);
                    const uintx4 vl = *reinterpret_cast<const uintx4*>(p + TL::Y_OFF + 2 * TL::X_PIECE);
                    s1[kb] = mma_bf16(yl, x1h[ks], s1[kb]);
                    s3[kb] = mma_bf16(vl, x3h[ks], s3[kb]);
                    s1[kb] = mma_bf16(yh, x1l[ks], s1[kb]);
                    s3[kb] = mma_bf16(vh, x3l[ks], s3[kb]);
                    s1[kb] = mma_bf16(yh, x1h[ks], s1[kb]);
                    s3[kb] = mma_bf16(vm, x3m[ks], s3[kb]);
                    s3[kb] = mma_bf16(vm, x3h[ks], s3[kb]);
                    s3[kb] = mma_bf16(vh, x3m[ks], s3[kb]);
                    s3[kb] = mma_bf16(vh, x3h[ks], s3[kb]);
                }
            if (KEYMAJOR) {
#pragma unroll
                for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb) {
                        const int row = 16 * kb + r16;
                        const char* p = st + TL::F_OFF + row * TL::F_ROW + x3_swz(row, 4 * ks + g, TL::F_ROW) * 16;
                        const uintx4 fh = *reinterpret_cast<const uintx4*>(p), fl = *reinterpret_cast<const uintx4*>(p + TL::F_PIECE);
                        s2[kb] = mma_bf16(fl, x2l[ks], s2[kb]);
                        s2[kb] = mma_bf16(fl, x2h[ks], s2[kb]);
                        s2[kb] = mma_bf16(fh, x2l[ks], s2[kb]);
                        s2[kb] = mma_bf16(fh, x2h[ks], s2[kb]);
                    }
            }
            // lane holds the pair (outer row o, inner row n_base + 16kb + 4g + i)
            floatx4 wdm[KB], wdf[KB], wak[KB];
            const float* Ss = reinterpret_cast<const float*>(st + TL::S_OFF);
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
                    const bool ok = LIST ? (ovalid && ((pres >> kb) & 1) != 0) : (unsigned)(n - nmin) < span;      // (a present half tile is whole)
                    const float av = ok ? __builtin_amdgcn_exp2f(s1[kb][i] * sc - (KEYMAJOR ? lnq[i] : ln_o)) : 0.f;
                    const float cc = KEYMAJOR ? cq[i] : c_o;
                    const float df = ok ? s3[kb][i] - cc : 0.f;
                    // with dropout D (0 or 1 / (1 - p)) on the exact weight: out = sum (D a - kb) v + ..., and the
                    // normaliser sees no dropout: dm = a (D g.v - c), the weight of g in d v is D a - kb
                    float dk = 1.f;
                    if (drop_on) {
                        const uint32_t rh = KEYMAJOR ? drop_row_hash(a.drop_seed, (uint32_t)(bh * a.T + n)) : drop_row;
                        dk = drop_keep(rh, (uint32_t)(KEYMAJOR ? o : n), a.drop_thresh) ? a.drop_scale : 0.f;
                    }
                    wdm[kb][i] = drop_on ? av * (ok ? dk * s3[kb][i] - cc : 0.f) : av * df;
                    wdf[kb][i] = df;
                    wak[kb][i] = av * dk - (ok ? s2[kb][i] : 0.f);
                }
            }
            uintx4 dmh, dml, dfh, dfm, dfl, akh, akm, akl;
            split2(wdm[0], wdm[1], dmh, dml);
            split3(wdf[0], wdf[1], dfh, dfm, dfl);
            if (KEYMAJOR) split3(wak[0], wak[1], akh, akm, akl);
            // out^T[col][outer] += sum_inner Y[inner][col] w[inner][outer]
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const char* p = st + tr_row * TL::X_ROW + x3_swz(tr_row, 2 * c + (tr_cb >> 1), TL::X_ROW) * 16 + 8 * (tr_cb & 1);
                const uintx4 yh = lds_read_tr8(p + TL::X_OFF, p + TL::X_OFF + 16 * TL::X_ROW);
                const uintx4 yl = lds_read_tr8(p + TL::X_OFF + TL::X_PIECE, p + TL::X_OFF + TL::X_PIECE + 16 * TL::X_ROW);
                acc1[c] = mma_bf16(yl, dmh, acc1[c]);
                acc1[c] = mma_bf16(yh, dml, acc1[c]);
                acc1[c] = mma_bf16(yh, dmh, acc1[c]);
                if (KEYMAJOR) {
                    // (a - kb) g: the band's low-rank part cancels against the per-head sum Q'^T g, so all six products
                    const uintx4 vh = lds_read_tr8(p + TL::Y_OFF, p + TL::Y_OFF + 16 * TL::X_ROW);
                    const uintx4 vm = lds_read_tr8(p + TL::Y_OFF + TL::X_PIECE, p + TL::Y_OFF + TL::X_PIECE + 16 * TL::X_ROW);
                    const uintx4 vl = lds_read_tr8(p + TL::Y_OFF + 2 * TL::X_PIECE, p + TL::Y_OFF + 2 * TL::X_PIECE + 16 * TL::X_ROW);
                    acc3[c] = mma_bf16(vl, akh, acc3[c]);
                    acc3[c] = mma_bf16(vh, akl, acc3[c]);
                    acc3[c] = mma_bf16(vm, akm, acc3[c]);
                    acc3[c] = mma_bf16(vm, akh, acc3[c]);
                    acc3[c] = mma_bf16(vh, akm, acc3[c]);
                    acc3[c] = mma_bf16(vh, akh, acc3[c]);
                }
            }
#pragma unroll
            for (int c = 0; c < FC; ++c) {
                const char* p = st + TL::F_OFF + tr_row * TL::F_ROW + x3_swz(tr_row, 2 * c + (tr_cb >> 1), TL::F_ROW) * 16 + 8 * (tr_cb & 1);
                const uintx4 fh = lds_read_tr8(p, p + 16 * TL::F_ROW);
                const uintx4 fl = lds_read_tr8(p + TL::F_PIECE, p + TL::F_PIECE + 16 * TL::F_ROW);
                acc2[c] = mma_bf16(fl, dfm, acc2[c]);
                acc2[c] = mma_bf16(fh, dfl, acc2[c]);
                acc2[c] = mma_bf16(fl, dfh, acc2[c]);
                acc2[c] = mma_bf16(fh, dfm, acc2[c]);
                acc2[c] = mma_bf16(fh, dfh, acc2[c]);
            }
        }
        drain_loads();                                     // this wave's share of the next tile is in LDS
        __syncthreads();
    }

    if (PARTS) {
        // this part's sums, register by register, 16 bytes per lane
        float* ws = a.part_ws + (long)item * ((EC + FC + (KEYMAJOR ? DB : 0)) * NT * 4) + 4 * tid;
#pragma unroll
        for (int c = 0; c < EC; ++c) *reinterpret_cast<floatx4*>(ws + c * NT * 4) = acc1[c];
#pragma unroll
        for (int c = 0; c < FC; ++c) *reinterpret_cast<floatx4*>(ws + (EC + c) * NT * 4) = acc2[c];
        if (KEYMAJOR) {
#pragma unroll
            for (int c = 0; c < DB; ++c) *reinterpret_cast<floatx4*>(ws + (EC + FC + c) * NT * 4) = acc3[c];
        }
        return;
    }
    bwd_x3_epilogue<E, M, KEYMAJOR>(a, smem, bh, o, orow, Lo, otile, trow, c_o, acc1, acc2, acc3);
}

// the parts of an outer tile summed in order, then its epilogue
template <int E, int M, bool KEYMAJOR>
__global__ __launch_bounds__(256) void sblocal_bwd_x3_finish_kernel(BwdX3Args a) {
    using TL = BwdTile<E, M>;
    constexpr int NT = 256, TQ = 64, D = E, EC = E / 16, FC = M / 16, DB = D / 16, NREG = EC + FC + (KEYMAJOR ? DB : 0);
    extern __shared__ __attribute__((aligned(256))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15;
    const int Lo = KEYMAJOR ? a.S : a.T;
    const int n_ot = (Lo + TQ - 1) / TQ;
    const int tile = blockIdx.x;
    int ot = tile % n_ot, bh = tile / n_ot;
    if (a.tl_heavy) {                                      // tile = batch entry * n_heavy + index into the long lists
        const int hg = a.tl_heavy[tile % a.n_heavy];
        ot = hg % n_ot;
        bh = (tile / a.n_heavy) * a.H + hg / n_ot;
    }
    const int o = ot * TQ + 16 * w + r16, orow = min(o, Lo - 1), trow = orow & 31;
    const int n_oimg = 2 * ((Lo + 63) / 64);
    const char* otile = a.oimg + ((long)bh * n_oimg + (orow >> 5)) * TL::BYTES;
    const float c_o = KEYMAJOR ? 0.f : a.c[(long)bh * a.T + orow];
    floatx4 acc1[EC], acc2[FC], acc3[KEYMAJOR ? DB : 1];
#pragma unroll
    for (int c = 0; c < EC; ++c) acc1[c] = Frag<float>::zero();
#pragma unroll
    for (int c = 0; c < FC; ++c) acc2[c] = Frag<float>::zero();
#pragma unroll
    for (int c = 0; c < (KEYMAJOR ? DB : 1); ++c) acc3[c] = Frag<float>::zero();
    for (int p = 0; p < a.n_parts; ++p) {
        const float* ws = a.part_ws + ((long)tile * a.n_parts + p) * (NREG * NT * 4) + 4 * tid;
#pragma unroll
        for (int c = 0; c < EC; ++c) acc1[c] += *reinterpret_cast<const floatx4*>(ws + c * NT * 4);
#pragma unroll
        for (int c = 0; c < FC; ++c) acc2[c] += *reinterpret_cast<const floatx4*>(ws + (EC + c) * NT * 4);
        if (KEYMAJOR) {
#pragma unroll
            for (int c = 0; c < DB; ++c) acc3[c] += *reinterpret_cast<const floatx4*>(ws + (EC + FC + c) * NT * 4);
        }
    }
    bwd_x3_epilogue<E, M, KEYMAJOR>(a, smem, bh, o, orow, Lo, otile, trow, c_o, acc1, acc2, acc3);
}

// (explicit instantiations: the host stubs of this template are not emitted otherwise)
#define FLY_BWD_X3_INST(EE, MM) \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, false, false>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, true, false>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, false, true>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, true, true>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, false, false, true>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, true, false, true>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, false, true, true>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_kernel<EE, MM, true, true, true>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_finish_kernel<EE, MM, false>(BwdX3Args); \
    template __global__ void sblocal_bwd_x3_finish_kernel<EE, MM, true>(BwdX3Args);
FLY_BWD_X3_INST(32, 32) FLY_BWD_X3_INST(32, 64) FLY_BWD_X3_INST(64, 32) FLY_BWD_X3_INST(64, 64) FLY_BWD_X3_INST(64, 128)
#undef FLY_BWD_X3_INST

// parts per outer tile: as many as fill the machine once, at least two inner tiles each, at most 8
static int bwd_x3_parts(long items, int lc) {
    const int tiles = (64 + lc + 31) / 32 + 1;
    const long fit = machine().slots / std::max(1L, items);
    return (int)std::max(1L, std::min({fit, (long)tiles / 2, 8L}));
}

template <int E, int M, bool KEYMAJOR>
static int launch_bwd_x3(const BwdX3Args& a, long part_ws_floats, hipStream_t st) {
    constexpr size_t smem = 2 * (BwdTile<E, M>::MAIN + 1024);
    constexpr size_t smem_fin = bwd_x3_epilogue_bytes<E, M>();
    constexpr long per_part = (E / 16 + M / 16 + (KEYMAJOR ? E / 16 : 0)) * 256 * 4;      // floats of one part's sums
    const Machine& mach = machine();
    const long tiles = (long)a.BH * (((KEYMAJOR ? a.S : a.T) + 63) / 64);
    int parts = bwd_x3_parts(tiles, a.lc);
    if (!a.part_ws || part_ws_floats < tiles * parts * per_part) parts = 1;
    const long items = tiles * parts;
    const long grid = (items + mach.xcds - 1) / mach.xcds * mach.xcds;
    if (grid > 2147483647L) return fail(ERR_ARG, "sblocal_bwd_x3: too many workgroups");
    BwdX3Args args = a;
    args.n_xcd = mach.xcds;
    args.n_parts = parts;
    if (a.tl_ptr) {
        auto kern = sblocal_bwd_x3_kernel<E, M, KEYMAJOR, false, true>;
        static std::atomic<unsigned long long> lds_set_l{0}, lds_set_lp{0}, lds_set_lf{0};
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set_l, "sblocal_bwd_x3 (lists)")) return rc;
        const long lgrid = (tiles + mach.xcds - 1) / mach.xcds * mach.xcds;
        args.n_parts = 1;
        if (a.n_heavy > 0) {
            // long lists first (they are the longest pieces of work): (batch, long tile, part) workgroups, then their finish
            auto kern_p = sblocal_bwd_x3_kernel<E, M, KEYMAJOR, true, true>;
            auto fin = sblocal_bwd_x3_finish_kernel<E, M, KEYMAJOR>;
            if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern_p), smem, lds_set_lp, "sblocal_bwd_x3 (long lists)")) return rc;
            if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fin), smem_fin, lds_set_lf, "sblocal_bwd_x3_finish")) return rc;
            const long htiles = (long)(a.BH / a.H) * a.n_heavy;
            if (part_ws_floats < htiles * a.n_parts * per_part)
                return fail(ERR_ARG, "sbblocksparse_bwd_pieces: part_ws of %ld floats, %ld needed", part_ws_floats, htiles * a.n_parts * per_part);
            BwdX3Args hargs = args;
            hargs.n_parts = a.n_parts;
            const long hgrid = (htiles * a.n_parts + mach.xcds - 1) / mach.xcds * mach.xcds;
            hipLaunchKernelGGL(kern_p, dim3((unsigned)hgrid), dim3(256), smem, st, hargs);
            if (int rc = check_launch("sblocal_bwd_x3_kernel (long lists)")) return rc;
            hipLaunchKernelGGL(kern, dim3((unsigned)lgrid), dim3(256), smem, st, args);
            if (int rc = check_launch("sblocal_bwd_x3_kernel (lists)")) return rc;
            hipLaunchKernelGGL(fin, dim3((unsigned)htiles), dim3(256), smem_fin, st, hargs);
            return check_launch("sblocal_bwd_x3_finish_kernel (long lists)");
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)lgrid), dim3(256), smem, st, args);
        return check_launch("sblocal_bwd_x3_kernel (lists)");
    }
    if (parts == 1) {
        auto kern = sblocal_bwd_x3_kernel<E, M, KEYMAJOR, false>;
        static std::atomic<unsigned long long> lds_set{0};     // (devices on which this kernel has its LDS limit)
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set, "sblocal_bwd_x3")) return rc;
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), smem, st, args);
        return check_launch("sblocal_bwd_x3_kernel");
    }
    auto kern = sblocal_bwd_x3_kernel<E, M, KEYMAJOR, true>;
    auto fin = sblocal_bwd_x3_finish_kernel<E, M, KEYMAJOR>;
    static std::atomic<unsigned long long> lds_set_p{0}, lds_set_f{0};
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_set_p, "sblocal_bwd_x3 (parts)")) return rc;
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fin), smem_fin, lds_set_f, "sblocal_bwd_x3_finish")) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), smem, st, args);
    if (int rc = check_launch("sblocal_bwd_x3_kernel (parts)")) return rc;
    hipLaunchKernelGGL(fin, dim3((unsigned)tiles), dim3(256), smem_fin, st, args);
    return check_launch("sblocal_bwd_x3_finish_kernel");
}
template <int E, int M>
static int launch_bwd_x3_both(const BwdX3Args& a, long part_ws_floats, bool key_major, hipStream_t st) {
    return key_major ? launch_bwd_x3<E, M, true>(a, part_ws_floats, st) : launch_bwd_x3<E, M, false>(a, part_ws_floats, st);
}

static void prep_splits(int BH, int T, int S, int& n_kblk, int& n_split_k, int& n_split_q) {
    const int kc = (S + PREP_ROWS - 1) / PREP_ROWS, qc = (T + PREP_ROWS - 1) / PREP_ROWS;
    const int want = std::max(1, (machine().slots + 2 * BH - 1) / (2 * BH));       // workgroups per role and (batch, head)
    n_kblk = kc;
    n_split_k = std::min(kc, want);
    n_split_q = std::min(qc, want);
}

template <int DIM, int MK>
static int launch_prep(PrepArgs a, hipStream_t st) {
    hipLaunchKernelGGL((sb_prep_kmax_kernel<DIM, MK>), dim3(a.n_kblk, a.BH), dim3(PREP_NT), 0, st, a);
    if (a.psi || a.phik)
        hipLaunchKernelGGL((sb_prep_kernel<DIM, MK, true>), dim3(a.n_split_k + a.n_split_q, a.BH), dim3(PREP_NT), 0, st, a);
    else
        hipLaunchKernelGGL((sb_prep_kernel<DIM, MK, false>), dim3(a.n_split_k + a.n_split_q, a.BH), dim3(PREP_NT), 0, st, a);
    hipLaunchKernelGGL((sb_prep_reduce_kernel<DIM, MK>), dim3((MK * (DIM + 1) + PREP_NT - 1) / PREP_NT, 2, a.BH),
                       dim3(PREP_NT), 0, st, a);
    return check_launch("sblocal_bwd_prep");
}

}  // namespace flyhip

using namespace flyhip;

extern "C" int64_t flyhip_sblocal_bwd_prep_scratch(int BH, int T, int S, int E, int M) {
    if (BH <= 0 || T <= 0 || S <= 0 || E <= 0 || M <= 0) return -1;
    int n_kblk, nk, nq;
    prep_splits(BH, T, S, n_kblk, nk, nq);
    return (long)BH * n_kblk + (long)BH * (nk + nq) * M * (E + 1);
}

extern "C" int64_t flyhip_sblocal_bwd_image_bytes(int BH, int rows, int E, int M) {
    if (BH <= 0 || rows <= 0 || E <= 0 || M <= 0) return -1;
    const int64_t tile = 32 * (10 * (int64_t)E + 4 * (int64_t)M) + 256;       // BwdTile<E, M>::BYTES
    return (int64_t)BH * 2 * ((rows + PREP_ROWS - 1) / PREP_ROWS) * tile;
}

extern "C" int flyhip_sblocal_bwd_prep(const float* q, const float* k, const float* v, const float* grad_out,
                                       const float* out, const float* log_norm, const float* proj,
                                       const int64_t* key_lengths,
                                       float* psi, float* phik, float* c,
                                       float* kv, float* ksum, float* qg, float* qc,
                                       void* q_images, void* k_images,
                                       float* scratch, int64_t scratch_floats,
                                       int BH, int H, int T, int S, int E, int M, int mh_valid,
                                       float softmax_temp, void* stream) {
    FLY_REQUIRE(q && k && v && grad_out && out && log_norm && proj && c && kv && ksum && qg && qc && scratch,
                "sblocal_bwd_prep: null pointer");
    FLY_REQUIRE((psi && phik) || (q_images && k_images), "sblocal_bwd_prep: neither feature arrays nor images asked for");
    FLY_REQUIRE(!psi == !phik && !q_images == !k_images, "sblocal_bwd_prep: psi / phik and the two image buffers come in pairs");
    FLY_REQUIRE(BH > 0 && H > 0 && BH % H == 0 && T > 0 && S > 0, "sblocal_bwd_prep: empty or inconsistent problem");
    FLY_REQUIRE(softmax_temp > 0.f, "sblocal_bwd_prep: softmax_temp must be positive");
    FLY_REQUIRE(mh_valid >= 1 && 2 * mh_valid <= M, "sblocal_bwd_prep: %d projection rows do not fit %d features", mh_valid, M);
    const int64_t need = flyhip_sblocal_bwd_prep_scratch(BH, T, S, E, M);
    FLY_REQUIRE(scratch_floats >= need, "sblocal_bwd_prep: scratch of %lld floats, %lld needed", (long long)scratch_floats, (long long)need);
    PrepArgs a{q, k, v, grad_out, out, log_norm, proj, key_lengths, psi, phik, c, kv, ksum, qg, qc,
               scratch, scratch + (long)BH * ((S + PREP_ROWS - 1) / PREP_ROWS),
               reinterpret_cast<char*>(q_images), reinterpret_cast<char*>(k_images),
               BH, H, T, S, mh_valid, 0, 0, 0, softmax_temp};
    prep_splits(BH, T, S, a.n_kblk, a.n_split_k, a.n_split_q);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    if (E == 32 && M == 32) return launch_prep<32, 32>(a, st);
    if (E == 32 && M == 64) return launch_prep<32, 64>(a, st);
    if (E == 64 && M == 32) return launch_prep<64, 32>(a, st);
    if (E == 64 && M == 64) return launch_prep<64, 64>(a, st);
    if (E == 64 && M == 128) return launch_prep<64, 128>(a, st);
    return fail(ERR_UNSUPPORTED, "sblocal_bwd_prep: (head dim, features) = (%d, %d) not in "
                                 "{(32,32), (32,64), (64,32), (64,64), (64,128)}", E, M);
}

extern "C" int64_t flyhip_sblocal_bwd_parts_floats(int BH, int T, int S, int E, int M, int local_context) {
    if (BH <= 0 || T <= 0 || S <= 0 || E <= 0 || M <= 0 || local_context < 1) return -1;
    int64_t need = 0;
    for (int km = 0; km < 2; ++km) {
        const long tiles = (long)BH * (((km ? S : T) + 63) / 64);
        const int parts = bwd_x3_parts(tiles, local_context);
        if (parts > 1) need = std::max<int64_t>(need, tiles * parts * (int64_t)((E / 16 + M / 16 + (km ? E / 16 : 0)) * 256 * 4));
    }
    return need;
}

extern "C" int flyhip_sblocal_bwd_pieces(const void* outer_images, const void* inner_images,
                                         const float* x1,
                                         const float* log_norm, const float* c, const int64_t* key_lengths,
                                         const float* gmat, const float* gvec, const float* proj,
                                         float* d1, float* d3, float* part_ws, int64_t part_ws_floats,
                                         int BH, int H, int T, int S, int E, int M, int local_context,
                                         float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                         void* stream) {
    FLY_REQUIRE(outer_images && inner_images && x1 && log_norm && c && gmat && gvec && proj && d1,
                "sblocal_bwd_pieces: null pointer");
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "sblocal_bwd_pieces: dropout probability %g outside [0, 1)", (double)dropout_p);
    FLY_REQUIRE(!key_major || d3, "sblocal_bwd_pieces: the key-major pass needs d3");
    FLY_REQUIRE(BH > 0 && H > 0 && BH % H == 0 && T > 0 && S > 0, "sblocal_bwd_pieces: empty or inconsistent problem");
    FLY_REQUIRE(local_context >= 1, "sblocal_bwd_pieces: local_context must be >= 1");
    FLY_REQUIRE(softmax_temp > 0.f, "sblocal_bwd_pieces: softmax_temp must be positive");
    BwdX3Args a{reinterpret_cast<const char*>(outer_images), reinterpret_cast<const char*>(inner_images), x1,
                log_norm, c, key_lengths, d1, d3, BH, H, T, S, local_context, softmax_temp, gmat, gvec, proj, 0, part_ws, 1,
                nullptr, nullptr, nullptr, nullptr, nullptr, 0};
    const DropArgs dr = drop_args(dropout_p, dropout_seed);
    a.drop_seed = dr.seed; a.drop_thresh = dr.thresh; a.drop_scale = dr.scale;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    const long wsf = part_ws ? (long)part_ws_floats : 0;
    if (E == 32 && M == 32) return launch_bwd_x3_both<32, 32>(a, wsf, key_major != 0, st);
    if (E == 32 && M == 64) return launch_bwd_x3_both<32, 64>(a, wsf, key_major != 0, st);
    if (E == 64 && M == 32) return launch_bwd_x3_both<64, 32>(a, wsf, key_major != 0, st);
    if (E == 64 && M == 64) return launch_bwd_x3_both<64, 64>(a, wsf, key_major != 0, st);
    if (E == 64 && M == 128) return launch_bwd_x3_both<64, 128>(a, wsf, key_major != 0, st);
    return fail(ERR_UNSUPPORTED, "sblocal_bwd_pieces: (head dim, features) = (%d, %d) not in "
                                 "{(32,32), (32,64), (64,32), (64,64), (64,128)}", E, M);
}

extern "C" int64_t flyhip_sbblocksparse_bwd_parts_floats(int B, int n_heavy, int heavy_parts, int E, int M, int key_major) {
    if (B <= 0 || n_heavy < 0 || heavy_parts < 1 || E <= 0 || M <= 0) return -1;
    return (int64_t)B * n_heavy * heavy_parts * ((E / 16 + M / 16 + (key_major ? E / 16 : 0)) * 256 * 4);
}

extern "C" int flyhip_sbblocksparse_bwd_pieces(const void* outer_images, const void* inner_images,
                                               const float* x1, const float* log_norm, const float* c,
                                               const float* gmat, const float* gvec, const float* proj,
                                               float* d1, float* d3,
                                               const int32_t* tl_ptr, const int32_t* tl_inner, const int32_t* tl_blk,
                                               const int32_t* tl_skip, const int32_t* tl_heavy, int n_heavy, int heavy_parts,
                                               float* part_ws, int64_t part_ws_floats,
                                               int BH, int H, int T, int S, int E, int M,
                                               float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                               void* stream) {
    FLY_REQUIRE(outer_images && inner_images && x1 && log_norm && c && gmat && gvec && proj && d1 && tl_ptr && tl_inner && tl_blk,
                "sbblocksparse_bwd_pieces: null pointer");
    FLY_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "sbblocksparse_bwd_pieces: dropout probability %g outside [0, 1)", (double)dropout_p);
    FLY_REQUIRE(!key_major || d3, "sbblocksparse_bwd_pieces: the key-major pass needs d3");
    FLY_REQUIRE(BH > 0 && H > 0 && BH % H == 0 && T > 0 && S > 0, "sbblocksparse_bwd_pieces: empty or inconsistent problem");
    FLY_REQUIRE(T % 16 == 0 && S % 16 == 0, "sbblocksparse_bwd_pieces: sequence lengths %d, %d must be multiples of 16", T, S);
    FLY_REQUIRE(softmax_temp > 0.f, "sbblocksparse_bwd_pieces: softmax_temp must be positive");
    FLY_REQUIRE(n_heavy == 0 || (n_heavy > 0 && tl_skip && tl_heavy && part_ws && heavy_parts >= 2 && heavy_parts <= 64),
                "sbblocksparse_bwd_pieces: long lists need tl_skip, tl_heavy, part_ws and 2..64 parts");
    BwdX3Args a{reinterpret_cast<const char*>(outer_images), reinterpret_cast<const char*>(inner_images), x1,
                log_norm, c, nullptr, d1, d3, BH, H, T, S, 1, softmax_temp, gmat, gvec, proj, 0, part_ws, n_heavy ? heavy_parts : 1,
                tl_ptr, tl_inner, tl_blk, n_heavy ? tl_skip : nullptr, n_heavy ? tl_heavy : nullptr, n_heavy};
    const DropArgs dr = drop_args(dropout_p, dropout_seed);
    a.drop_seed = dr.seed; a.drop_thresh = dr.thresh; a.drop_scale = dr.scale;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (int rc_capture = refuse_capture(st)) return rc_capture;
    const long wsf = part_ws ? (long)part_ws_floats : 0;
    if (E == 32 && M == 32) return launch_bwd_x3_both<32, 32>(a, wsf, key_major != 0, st);
    if (E == 32 && M == 64) return launch_bwd_x3_both<32, 64>(a, wsf, key_major != 0, st);
    if (E == 64 && M == 32) return launch_bwd_x3_both<64, 32>(a, wsf, key_major != 0, st);
    if (E == 64 && M == 64) return launch_bwd_x3_both<64, 64>(a, wsf, key_major != 0, st);
    if (E == 64 && M == 128) return launch_bwd_x3_both<64, 128>(a, wsf, key_major != 0, st);
    return fail(ERR_UNSUPPORTED, "sbblocksparse_bwd_pieces: (head dim, features) = (%d, %d) not in "
                                 "{(32,32), (32,64), (64,32), (64,64), (64,128)}", E, M);
}
