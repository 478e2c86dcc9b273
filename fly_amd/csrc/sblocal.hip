// Scatterbrain-local attention forward for gfx950.
//
// Three kernels:
//   sb_kfeat_kernel   : per (batch, head, range of 64-key chunks): positive random features of
//                       the keys (projection on fp32 MFMA, wavefront max reductions, exp),
//                       written to HBM once, plus the partial K'^T V / sum K' reductions with an
//                       online rescale to the running maximum.
//   sb_combine_kernel : merges the partial reductions of one (batch, head).
//   sblocal_fwd_kernel: per (batch, head, 64-query tile): query features in registers, then for
//                       each 64-key tile of the band Q K^T and Q' K'^T on MFMA (transposed, so
//                       that every lane owns one query), band/length masking, online softmax with
//                       the low-rank overlap subtracted, P V on MFMA, and the epilogue that adds
//                       the global low-rank term and writes out / log-normaliser.
//
// Layout of an MFMA 16x16 result in a lane (r = lane%16, g = lane/16): element i is
// C[4g+i][r].  All products are formed "transposed" (rows = keys / features / value dims,
// columns = queries) so that r indexes the lane's query and the four register elements index
// consecutive keys/features -- which is exactly the operand layout the next product needs.
#include "common.h"
#include <math.h>

namespace flyhip {

constexpr int CH = 64;     // keys per chunk and per key tile
constexpr int NT = 256;    // threads per workgroup (4 waves)

struct KvArgs {
    const void* k; const void* v; const float* proj; const int64_t* lens;
    float* kfeat; float* chunk_scale; float* kv_part; float* part_max;
    int B, H, S, mh_valid, n_chunks, n_split;
    long k_sb, k_sh, k_ss, v_sb, v_sh, v_ss;
    float temp;
};

struct FwdArgs {
    const void* q; const void* k; const void* v; const float* proj;
    const float* kfeat; const float* chunk_scale; const float* kv; const float* ksum; const float* kmax;
    const int64_t* lens; void* out; float* log_norm;
    int B, H, T, S, mh_valid, lc, n_chunks;
    long q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss;
    float temp;
};

// rows [row0, row0+CH) of a (seq, W) matrix -> LDS tile with leading dimension LD; rows at or
// beyond `limit` are zero filled
template <typename T, int W, int LD>
__device__ __forceinline__ void load_tile(float* dst, const T* src, long row_stride, int row0, int limit, int tid) {
    constexpr int V4 = W / 4;
    for (int idx = tid; idx < CH * V4; idx += NT) {
        int row = idx / V4, c4 = idx % V4;
        floatx4 val = {0.f, 0.f, 0.f, 0.f};
        if (row0 + row < limit) val = load4_f32(src + (long)(row0 + row) * row_stride + 4 * c4);
        *reinterpret_cast<floatx4*>(dst + row * LD + 4 * c4) = val;
    }
}

template <int E, int MH>
__device__ __forceinline__ void load_proj(float* Ps, const float* proj, float scale, int tid) {
    constexpr int V4 = E / 4, LD = E + 4;
    for (int idx = tid; idx < MH * V4; idx += NT) {
        int row = idx / V4, c4 = idx % V4;
        floatx4 val = *reinterpret_cast<const floatx4*>(proj + row * E + 4 * c4);
        val *= scale;
        *reinterpret_cast<floatx4*>(Ps + row * LD + 4 * c4) = val;
    }
}

// ---------------------------------------------------------------------------------------
// key features + partial K'^T V
// ---------------------------------------------------------------------------------------
template <typename T, int E, int D, int M>
__global__ __launch_bounds__(NT) void sb_kfeat_kernel(KvArgs a) {
    constexpr int MH = M / 2, LDK = E + 4, LDV = D + 4, LDF = M + 4;
    constexpr int FB = MH / 16;                  // feature blocks of the projection
    constexpr int RB = (M / 16 + 3) / 4;         // K'^T V row blocks per wave
    extern __shared__ float smem[];
    float* Ps = smem;
    float* Ks = Ps + MH * LDK;
    float* Vs = Ks + CH * LDK;
    float* Fs = Vs + CH * LDV;
    float* red = Fs + CH * LDF;

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H, sp = blockIdx.x;
    const T* kptr = reinterpret_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh;
    const T* vptr = reinterpret_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half = 0.5f * logf(2.0f * a.mh_valid);

    load_proj<E, MH>(Ps, a.proj, sqrtf(a.temp), tid);

    floatx4 kvacc[RB][D / 16];
#pragma unroll
    for (int x = 0; x < RB; ++x)
#pragma unroll
        for (int db = 0; db < D / 16; ++db) kvacc[x][db] = Frag<float>::zero();
    float ksum_acc = 0.f;
    float run_max = -INFINITY;

    const int per = (a.n_chunks + a.n_split - 1) / a.n_split;
    const int c0 = sp * per, c1 = min(a.n_chunks, c0 + per);
    for (int c = c0; c < c1; ++c) {
        const int s_base = c * CH;
        __syncthreads();
        load_tile<T, E, LDK>(Ks, kptr, a.k_ss, s_base, len, tid);
        load_tile<T, D, LDV>(Vs, vptr, a.v_ss, s_base, len, tid);
        __syncthreads();

        // projection of this wave's 16 keys: dd[fb][i] = (sqrt(t) P)[16fb+4g+i] . k[16w+r16]
        floatx4 kb[E / 16];
        float sq = 0.f;
#pragma unroll
        for (int cc = 0; cc < E / 16; ++cc) {
            kb[cc] = *reinterpret_cast<const floatx4*>(Ks + (16 * w + r16) * LDK + 16 * cc + 4 * g);
            sq += kb[cc][0] * kb[cc][0] + kb[cc][1] * kb[cc][1] + kb[cc][2] * kb[cc][2] + kb[cc][3] * kb[cc][3];
        }
        const float diag = 0.5f * a.temp * group_sum(sq);
        floatx4 dd[FB];
        float amax = 0.f;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
            dd[fb] = Frag<float>::zero();
#pragma unroll
            for (int cc = 0; cc < E / 16; ++cc) {
                floatx4 pa = *reinterpret_cast<const floatx4*>(Ps + (16 * fb + r16) * LDK + 16 * cc + 4 * g);
                dd[fb] = Frag<float>::mma(pa, kb[cc], dd[fb]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (16 * fb + 4 * g + i < a.mh_valid) amax = fmaxf(amax, fabsf(dd[fb][i]));
        }
        amax = group_max(amax);
        const bool kvalid = (s_base + 16 * w + r16) < len;
        float cs = kvalid ? (amax - diag - lnm_half) : -INFINITY;
        cs = wave_max(cs);
        if (lane == 0) red[w] = cs;
        __syncthreads();
        const float lmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float new_max = fmaxf(run_max, lmax);
        float* frow_g = a.kfeat + ((long)bh * a.n_chunks * CH + s_base + 16 * w + r16) * M;
        if (new_max == -INFINITY) {   // no valid key yet (workgroup-uniform): features are zero
#pragma unroll
            for (int fb = 0; fb < FB; ++fb) {
                *reinterpret_cast<floatx4*>(frow_g + 16 * fb + 4 * g) = Frag<float>::zero();
                *reinterpret_cast<floatx4*>(frow_g + MH + 16 * fb + 4 * g) = Frag<float>::zero();
            }
            if (tid == 0) a.chunk_scale[(long)bh * a.n_chunks + c] = 0.f;
            continue;
        }
        const float rescale = (run_max == -INFINITY) ? 0.f : expf(run_max - new_max);
        run_max = new_max;
#pragma unroll
        for (int x = 0; x < RB; ++x)
#pragma unroll
            for (int db = 0; db < D / 16; ++db) kvacc[x][db] *= rescale;
        ksum_acc *= rescale;

        const float off = -diag - lnm_half - new_max;
        float* frow_s = Fs + (16 * w + r16) * LDF;
#pragma unroll
        for (int fb = 0; fb < FB; ++fb) {
            floatx4 fp, fn;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = kvalid && (16 * fb + 4 * g + i < a.mh_valid);
                fp[i] = ok ? expf(dd[fb][i] + off) : 0.f;
                fn[i] = ok ? expf(-dd[fb][i] + off) : 0.f;
            }
            *reinterpret_cast<floatx4*>(frow_s + 16 * fb + 4 * g) = fp;
            *reinterpret_cast<floatx4*>(frow_s + MH + 16 * fb + 4 * g) = fn;
            *reinterpret_cast<floatx4*>(frow_g + 16 * fb + 4 * g) = fp;
            *reinterpret_cast<floatx4*>(frow_g + MH + 16 * fb + 4 * g) = fn;
        }
        if (tid == 0) a.chunk_scale[(long)bh * a.n_chunks + c] = new_max;
        __syncthreads();

        // KV[r][d] += sum_keys F[key][r] V[key][d]; lane ends with KV[16rb+4g+i][16db+r16]
#pragma unroll
        for (int x = 0; x < RB; ++x) {
            const int rb = w + 4 * x;
            if (rb < M / 16) {
#pragma unroll
                for (int kk = 0; kk < CH / 16; ++kk) {
                    floatx4 fa;
#pragma unroll
                    for (int j = 0; j < 4; ++j) fa[j] = Fs[(16 * kk + 4 * g + j) * LDF + 16 * rb + r16];
#pragma unroll
                    for (int db = 0; db < D / 16; ++db) {
                        floatx4 vb;
#pragma unroll
                        for (int j = 0; j < 4; ++j) vb[j] = Vs[(16 * kk + 4 * g + j) * LDV + 16 * db + r16];
                        kvacc[x][db] = Frag<float>::mma(fa, vb, kvacc[x][db]);
                    }
                }
            }
        }
        if (tid < M) {
            float s = 0.f;
            for (int row = 0; row < CH; ++row) s += Fs[row * LDF + tid];
            ksum_acc += s;
        }
    }

    float* part = a.kv_part + ((long)bh * a.n_split + sp) * (M * (D + 1));
#pragma unroll
    for (int x = 0; x < RB; ++x) {
        const int rb = w + 4 * x;
        if (rb < M / 16) {
#pragma unroll
            for (int db = 0; db < D / 16; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) part[(16 * rb + 4 * g + i) * D + 16 * db + r16] = kvacc[x][db][i];
        }
    }
    if (tid < M) part[M * D + tid] = ksum_acc;
    if (tid == 0) a.part_max[(long)bh * a.n_split + sp] = run_max;
}

// KV = sum_s exp(part_max_s - kmax) KV_s, same for Ksum; one thread per output element
__global__ void sb_combine_kernel(const float* kv_part, const float* part_max, float* kv, float* ksum,
                                  float* kmax_out, int n_split, int M, int D) {
    const int bh = blockIdx.y;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int per = M * (D + 1);
    float kmax = -INFINITY;
    for (int s = 0; s < n_split; ++s) kmax = fmaxf(kmax, part_max[(long)bh * n_split + s]);
    if (idx == 0) kmax_out[bh] = (kmax == -INFINITY) ? 0.f : kmax;
    if (idx >= per) return;
    float acc = 0.f;
    for (int s = 0; s < n_split; ++s) {
        const float pm = part_max[(long)bh * n_split + s];
        if (pm != -INFINITY) acc += expf(pm - kmax) * kv_part[((long)bh * n_split + s) * per + idx];
    }
    if (idx < M * D) kv[(long)bh * M * D + idx] = acc;
    else ksum[(long)bh * M + idx - M * D] = acc;
}

// ---------------------------------------------------------------------------------------
// fused band kernel
// ---------------------------------------------------------------------------------------
template <typename T, int E, int D, int M>
__global__ __launch_bounds__(NT) void sblocal_fwd_kernel(FwdArgs a) {
    constexpr int MH = M / 2, LDK = E + 4, LDV = D + 4, LDF = M + 4;
    constexpr int FB = MH / 16, EC = E / 16, DB = D / 16, KB = CH / 16;
    extern __shared__ float smem[];
    float* Ks = smem;
    float* Vs = Ks + CH * LDK;
    float* Fs = Vs + CH * LDV;
    float* Ps = smem;                         // only live before the key loop

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const int q0 = blockIdx.x * 64;
    const int iq = q0 + 16 * w + r16;
    const bool qvalid = iq < a.T;
    const T* qptr = reinterpret_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh;
    const T* kptr = reinterpret_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh;
    const T* vptr = reinterpret_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh;
    const int len = a.lens ? min((int)a.lens[b], a.S) : a.S;
    const float lnm_half = 0.5f * logf(2.0f * a.mh_valid);
    const int lc_lo = a.lc / 2, lc_hi = (a.lc + 1) / 2;    // band: -lc_lo <= s - i < lc_hi

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
    load_proj<E, MH>(Ps, a.proj, sqrtf(a.temp), tid);
    __syncthreads();
    floatx4 qf[2 * FB];
    float qmax = 0.f;
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) {
        floatx4 dd = Frag<float>::zero();
#pragma unroll
        for (int c = 0; c < EC; ++c) {
            floatx4 pa = *reinterpret_cast<const floatx4*>(Ps + (16 * fb + r16) * LDK + 16 * c + 4 * g);
            dd = Frag<float>::mma(pa, qr[c], dd);
        }
        qf[fb] = dd;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (16 * fb + 4 * g + i < a.mh_valid) qmax = fmaxf(qmax, fabsf(dd[i]));
    }
    qmax = group_max(qmax);
    const float lsq = -diag_q + qmax - lnm_half;
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) {
        floatx4 dd = qf[fb];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool ok = 16 * fb + 4 * g + i < a.mh_valid;
            qf[fb][i] = ok ? expf(dd[i] - qmax) : 0.f;
            qf[FB + fb][i] = ok ? expf(-dd[i] - qmax) : 0.f;
        }
    }

    const float kmax = a.kmax[bh];
    float m_run = lsq + kmax;       // reference exponent: max(running row max, log-scale of the low-rank part)
    float ze = 0.f, zp = 0.f;       // per-lane partial sums (reduced over g at the end)
    floatx4 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = Frag<float>::zero();

    const int q_last = min(q0 + 63, a.T - 1);
    const int lo = max(0, q0 - lc_lo);
    const int hi = min(len, q_last + lc_hi);
    const int kt_lo = lo / CH;
    const int kt_hi = (hi > lo) ? (hi + CH - 1) / CH : kt_lo;
    const int qw0 = q0 + 16 * w;    // first query of this wave

    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        const int s_base = kt * CH;
        __syncthreads();
        load_tile<T, E, LDK>(Ks, kptr, a.k_ss, s_base, len, tid);
        load_tile<T, D, LDV>(Vs, vptr, a.v_ss, s_base, len, tid);
        load_tile<float, M, LDF>(Fs, a.kfeat + (long)bh * a.n_chunks * CH * M, M, s_base, a.n_chunks * CH, tid);
        __syncthreads();
        const float cscale = a.chunk_scale[(long)bh * a.n_chunks + kt];
        const float beta_k = expf(cscale - kmax);            // <= 1

#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            const int s0 = s_base + 16 * kb;
            // wave-uniform: does this 16-key block touch the band of any of the wave's 16 queries?
            if (s0 + 15 - qw0 < -lc_lo || s0 - (qw0 + 15) >= lc_hi || s0 >= len) continue;
            floatx4 s1 = Frag<float>::zero(), s2 = Frag<float>::zero();
            const float* krow = Ks + (16 * kb + r16) * LDK + 4 * g;
#pragma unroll
            for (int c = 0; c < EC; ++c)
                s1 = Frag<float>::mma(*reinterpret_cast<const floatx4*>(krow + 16 * c), qr[c], s1);
            const float* frow = Fs + (16 * kb + r16) * LDF + 4 * g;
#pragma unroll
            for (int c = 0; c < 2 * FB; ++c)
                s2 = Frag<float>::mma(*reinterpret_cast<const floatx4*>(frow + 16 * c), qf[c], s2);

            // lane now holds the scores of query iq against keys s0 + 4g + i
            bool ok[4];
            float x[4];
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int s = s0 + 4 * g + i;
                const int rel = s - iq;
                ok[i] = qvalid && rel >= -lc_lo && rel < lc_hi && s < len;
                x[i] = a.temp * s1[i];
                if (ok[i]) mx = fmaxf(mx, x[i]);
            }
            mx = group_max(mx);
            if (mx > m_run) {
                const float alpha = expf(m_run - mx);
                m_run = mx;
                ze *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
            }
            const float beta = expf(lsq + cscale - m_run);   // scale of the overlap term, <= 1
            floatx4 p;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = ok[i] ? expf(x[i] - m_run) : 0.f;
                const float ov = ok[i] ? s2[i] : 0.f;
                ze += e;
                zp += ov * beta_k;
                p[i] = e - ov * beta;
            }
            // O^T[d][query] += sum_keys V[key][d] p[key][query]
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                floatx4 va;
#pragma unroll
                for (int i = 0; i < 4; ++i) va[i] = Vs[(16 * kb + 4 * g + i) * LDV + 16 * db + r16];
                oacc[db] = Frag<float>::mma(va, p, oacc[db]);
            }
        }
    }

    // global low-rank term: qkv^T[d][query] = sum_r KV[r][d] q'[query][r],  qk1 = q' . Ksum
    const float* kvp = a.kv + (long)bh * M * D;
    const float* ksp = a.ksum + (long)bh * M;
    floatx4 lacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) lacc[db] = Frag<float>::zero();
    float qk1 = 0.f;
#pragma unroll
    for (int c = 0; c < 2 * FB; ++c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) qk1 += qf[c][j] * ksp[16 * c + 4 * g + j];
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            floatx4 ka;
#pragma unroll
            for (int j = 0; j < 4; ++j) ka[j] = kvp[(16 * c + 4 * g + j) * D + 16 * db + r16];
            lacc[db] = Frag<float>::mma(ka, qf[c], lacc[db]);
        }
    }
    qk1 = group_sum(qk1);
    ze = group_sum(ze);
    zp = group_sum(zp);
    const float gamma = expf(lsq + kmax - m_run);                     // <= 1
    const float Z = ze + gamma * fmaxf(qk1 - zp, 1e-24f);
    const float inv = 1.0f / Z;
    if (qvalid) {
        T* optr = reinterpret_cast<T*>(a.out) + b * a.o_sb + h * a.o_sh + (long)iq * a.o_ss;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            floatx4 o = (oacc[db] + gamma * lacc[db]) * inv;
            store4_f32(optr + 16 * db + 4 * g, o);
        }
        if (g == 0) a.log_norm[(long)bh * a.T + iq] = m_run + logf(Z);
    }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
template <int E, int M> constexpr size_t kfeat_smem() {
    return sizeof(float) * ((M / 2) * (E + 4) + CH * (E + 4) + CH * (E + 4) + CH * (M + 4) + 8);
}
template <int E, int M> constexpr size_t fwd_smem() {
    return sizeof(float) * (CH * (E + 4) + CH * (E + 4) + CH * (M + 4));
}

template <typename T, int E, int M>
static int launch_kfeat(const KvArgs& a, hipStream_t st) {
    auto kern = sb_kfeat_kernel<T, E, E, M>;
    constexpr size_t smem = kfeat_smem<E, M>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return fail(ERR_LAUNCH, "sb_kfeat: LDS attribute: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(kern, dim3(a.n_split, a.B * a.H), dim3(NT), smem, st, a);
    return check_launch("sb_kfeat_kernel");
}

template <typename T, int E, int M>
static int launch_fwd(const FwdArgs& a, hipStream_t st) {
    auto kern = sblocal_fwd_kernel<T, E, E, M>;
    constexpr size_t smem = fwd_smem<E, M>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return fail(ERR_LAUNCH, "sblocal_fwd: LDS attribute: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(kern, dim3((a.T + 63) / 64, a.B * a.H), dim3(NT), smem, st, a);
    return check_launch("sblocal_fwd_kernel");
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

static int plan(int B, int H, int S, int* n_chunks, int* n_split) {
    const int nc = (S + CH - 1) / CH;
    // aim for about 1024 workgroups over the chip, at least one chunk each
    long want = (1024 + (long)B * H - 1) / ((long)B * H);
    if (want < 1) want = 1;
    if (want > nc) want = nc;
    const int per = (nc + (int)want - 1) / (int)want;
    *n_chunks = nc;
    *n_split = (nc + per - 1) / per;
    return OK;
}

}  // namespace flyhip

using namespace flyhip;

extern "C" int flyhip_sb_plan(int B, int H, int S, int* n_chunks, int* n_split) {
    FLY_REQUIRE(B > 0 && H > 0 && S > 0 && n_chunks && n_split, "sb_plan: bad arguments");
    return plan(B, H, S, n_chunks, n_split);
}

static int check_sb_dims(const char* who, int E, int D, int mh, int mh_valid, int dtype,
                         int64_t s0, int64_t s1, int64_t s2) {
    FLY_REQUIRE(E == D, "%s: padded head dims must be equal (E=%d, D=%d)", who, E, D);
    FLY_REQUIRE(mh_valid >= 1 && mh_valid <= mh, "%s: mh_valid=%d outside [1, mh=%d]", who, mh_valid, mh);
    FLY_REQUIRE((s0 % 4) == 0 && (s1 % 4) == 0 && (s2 % 4) == 0,
                "%s: strides must be multiples of 4 elements (16-byte vector access)", who);
    (void)dtype;
    return OK;
}

extern "C" int flyhip_sb_kv_reduce(const void* k, const void* v, const float* proj, const int64_t* key_lengths,
                                   float* kfeat, float* chunk_scale, float* kv_part, float* part_max,
                                   float* kv, float* ksum, float* kmax,
                                   int B, int H, int S, int E, int D, int mh, int mh_valid, int n_split,
                                   int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                   int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                   float softmax_temp, int dtype, void* stream) {
    FLY_REQUIRE(k && v && proj && kfeat && chunk_scale && kv_part && part_max && kv && ksum && kmax,
                "sb_kv_reduce: null pointer");
    FLY_REQUIRE(B > 0 && H > 0 && S > 0, "sb_kv_reduce: empty problem B=%d H=%d S=%d", B, H, S);
    FLY_REQUIRE(softmax_temp > 0.f, "sb_kv_reduce: softmax_temp must be positive");
    int rc = check_sb_dims("sb_kv_reduce", E, D, mh, mh_valid, dtype, k_sb | k_sh, k_ss, v_sb | v_sh | v_ss);
    if (rc) return rc;
    int nc, ns;
    plan(B, H, S, &nc, &ns);
    FLY_REQUIRE(n_split >= 1 && n_split <= nc, "sb_kv_reduce: n_split=%d outside [1, %d]", n_split, nc);
    FLY_REQUIRE((long)B * H <= 65535, "sb_kv_reduce: B*H=%ld exceeds the grid limit 65535", (long)B * H);
    KvArgs a{k, v, proj, key_lengths, kfeat, chunk_scale, kv_part, part_max,
             B, H, S, mh_valid, nc, n_split, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, softmax_temp};
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const int m = 2 * mh;
    rc = dispatch_kfeat(dtype, E, m, a, st);
    if (rc) return rc;
    const int per = m * (D + 1);
    hipLaunchKernelGGL(sb_combine_kernel, dim3((per + 255) / 256, B * H), dim3(256), 0, st,
                       kv_part, part_max, kv, ksum, kmax, n_split, m, D);
    return check_launch("sb_combine_kernel");
}

extern "C" int flyhip_sblocal_fwd(const void* q, const void* k, const void* v, const float* proj,
                                  const float* kfeat, const float* chunk_scale,
                                  const float* kv, const float* ksum, const float* kmax,
                                  const int64_t* key_lengths, void* out, float* log_norm,
                                  int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                                  int local_context,
                                  int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                  int64_t k_sb, int64_t k_sh, int64_t k_ss,
                                  int64_t v_sb, int64_t v_sh, int64_t v_ss,
                                  int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                  float softmax_temp, int dtype, void* stream) {
    FLY_REQUIRE(q && k && v && proj && kfeat && chunk_scale && kv && ksum && kmax && out && log_norm,
                "sblocal_fwd: null pointer");
    FLY_REQUIRE(B > 0 && H > 0 && T > 0 && S > 0, "sblocal_fwd: empty problem");
    FLY_REQUIRE(local_context >= 1, "sblocal_fwd: local_context must be >= 1");
    FLY_REQUIRE(softmax_temp > 0.f, "sblocal_fwd: softmax_temp must be positive");
    int rc = check_sb_dims("sblocal_fwd", E, D, mh, mh_valid, dtype, q_sb | q_sh | q_ss | k_sb | k_sh | k_ss,
                           v_sb | v_sh | v_ss, o_sb | o_sh | o_ss);
    if (rc) return rc;
    FLY_REQUIRE((long)B * H <= 65535, "sblocal_fwd: B*H=%ld exceeds the grid limit 65535", (long)B * H);
    int nc, ns;
    plan(B, H, S, &nc, &ns);
    FwdArgs a{q, k, v, proj, kfeat, chunk_scale, kv, ksum, kmax, key_lengths, out, log_norm,
              B, H, T, S, mh_valid, local_context, nc,
              q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss, softmax_temp};
    return dispatch_fwd(dtype, E, 2 * mh, a, reinterpret_cast<hipStream_t>(stream));
}
