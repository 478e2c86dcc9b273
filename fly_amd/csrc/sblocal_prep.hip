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
    int BH, H, T, S, mh_valid, n_kblk, n_split_k, n_split_q;
    float temp;
};

constexpr int PREP_ROWS = 64;        // rows per step of a workgroup: 16 per wave
constexpr int PREP_NT = 256;

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

template <int DIM, int MK>
__global__ __launch_bounds__(PREP_NT) void sb_prep_kernel(PrepArgs a) {
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
    float* F = (key_role ? a.phik : a.psi) + (long)bh * rows * MK;

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
        floatx4 dd[FB];
        float sq;
        prep_project<DIM, FB>(xb, a.proj, st, r16, g, dd, sq);
        float bias;
        if (key_role) bias = -0.5f * a.temp * sq - off - kappa;
        else bias = kappa - ln_row - 0.5f * a.temp * sq - off;
        __syncthreads();                          // every c of this chunk has been read
        float* frow_s = Fs + (16 * w + r16) * LDF;
        float* frow_g = F + (long)row * MK;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
            floatx4 fp, fn;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = valid && (16 * fb + 4 * g + i < a.mh_valid);
                fp[i] = ok ? expf(dd[fb][i] + bias) : 0.f;
                fn[i] = ok ? expf(bias - dd[fb][i]) : 0.f;
            }
            sp_[fb] += fp * wrow;
            sn_[fb] += fn * wrow;
            *reinterpret_cast<floatx4*>(frow_s + 16 * fb + 4 * g) = fp;
            *reinterpret_cast<floatx4*>(frow_s + MH + 16 * fb + 4 * g) = fn;
            if (row < rows) {
                *reinterpret_cast<floatx4*>(frow_g + 16 * fb + 4 * g) = fp;
                *reinterpret_cast<floatx4*>(frow_g + MH + 16 * fb + 4 * g) = fn;
            }
        }
        __syncthreads();
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
    hipLaunchKernelGGL((sb_prep_kernel<DIM, MK>), dim3(a.n_split_k + a.n_split_q, a.BH), dim3(PREP_NT), 0, st, a);
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

extern "C" int flyhip_sblocal_bwd_prep(const float* q, const float* k, const float* v, const float* grad_out,
                                       const float* out, const float* log_norm, const float* proj,
                                       const int64_t* key_lengths,
                                       float* psi, float* phik, float* c,
                                       float* kv, float* ksum, float* qg, float* qc,
                                       float* scratch, int64_t scratch_floats,
                                       int BH, int H, int T, int S, int E, int M, int mh_valid,
                                       float softmax_temp, void* stream) {
    FLY_REQUIRE(q && k && v && grad_out && out && log_norm && proj && psi && phik && c && kv && ksum && qg && qc && scratch,
                "sblocal_bwd_prep: null pointer");
    FLY_REQUIRE(BH > 0 && H > 0 && BH % H == 0 && T > 0 && S > 0, "sblocal_bwd_prep: empty or inconsistent problem");
    FLY_REQUIRE(softmax_temp > 0.f, "sblocal_bwd_prep: softmax_temp must be positive");
    FLY_REQUIRE(mh_valid >= 1 && 2 * mh_valid <= M, "sblocal_bwd_prep: %d projection rows do not fit %d features", mh_valid, M);
    const int64_t need = flyhip_sblocal_bwd_prep_scratch(BH, T, S, E, M);
    FLY_REQUIRE(scratch_floats >= need, "sblocal_bwd_prep: scratch of %lld floats, %lld needed", (long long)scratch_floats, (long long)need);
    PrepArgs a{q, k, v, grad_out, out, log_norm, proj, key_lengths, psi, phik, c, kv, ksum, qg, qc,
               scratch, scratch + (long)BH * ((S + PREP_ROWS - 1) / PREP_ROWS), BH, H, T, S, mh_valid, 0, 0, 0, softmax_temp};
    prep_splits(BH, T, S, a.n_kblk, a.n_split_k, a.n_split_q);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (E == 32 && M == 32) return launch_prep<32, 32>(a, st);
    if (E == 32 && M == 64) return launch_prep<32, 64>(a, st);
    if (E == 64 && M == 32) return launch_prep<64, 32>(a, st);
    if (E == 64 && M == 64) return launch_prep<64, 64>(a, st);
    if (E == 64 && M == 128) return launch_prep<64, 128>(a, st);
    return fail(ERR_UNSUPPORTED, "sblocal_bwd_prep: (head dim, features) = (%d, %d) not in "
                                 "{(32,32), (32,64), (64,32), (64,64), (64,128)}", E, M);
}
