// Shared device/host helpers for the gfx950 kernels: error reporting for the C ABI,
// element-type traits, 16-byte operand loads and the 16x16 MFMA wrappers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <atomic>

namespace flyhip {

// ---------------------------------------------------------------------------------------
// error convention: entry points return 0 or a negative code and leave a message here
// ---------------------------------------------------------------------------------------
enum { OK = 0, ERR_ARG = -1, ERR_UNSUPPORTED = -2, ERR_LAUNCH = -3 };
char* error_buffer();   // thread-local, 512 bytes
inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}
inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return OK;
}
#define FLY_REQUIRE(cond, ...) do { if (!(cond)) return ::flyhip::fail(::flyhip::ERR_ARG, __VA_ARGS__); } while (0)

// ---------------------------------------------------------------------------------------
// facts of the device the calling thread has current, queried from the runtime once per device
// ---------------------------------------------------------------------------------------
struct Machine {
    int cus;       // compute units
    int xcds;      // accelerator dies, each with its own L2; the dispatcher deals consecutive workgroup ids to them in turn
    int slots;     // workgroups of 256 threads that are resident together at two per compute unit
};
const Machine& machine();      // (without a device: the MI355X's 256 compute units on 8 dies)
// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per kernel and device; `done` is the caller's
// per-kernel set of devices already served (one bit each)
int ensure_dynamic_lds(const void* kernel, size_t bytes, std::atomic<unsigned long long>& done, const char* what);

// Every entry point that launches calls this first: a stream under capture into a HIP graph is refused with an error
// (ERR_UNSUPPORTED).  The launchers do things on first use that are not stream operations (the LDS limit of a kernel,
// the address of the built-in scratch array), and a capture of calls of this library has ended in a crash of the host
// process whose cause is not known; until it is, capture is an error here rather than a crash.
int refuse_capture(hipStream_t st);

enum DType { F32 = 0, BF16 = 1, F16 = 2 };

// ---------------------------------------------------------------------------------------
// element types
// ---------------------------------------------------------------------------------------
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
// native 4 x 32-bit vector (arrays of HIP's uint4 struct do not always stay in registers)
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
// two floats -> two bf16 in one 32-bit word (low half = first), round to nearest even in hardware
// (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    floatx2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return (uint16_t)(pack_bf16x2(f, 0.f) & 0xffffu); }

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float to_f32(float x) { return x; }
    static __device__ __forceinline__ float from_f32(float x) { return x; }
};
template <> struct Elem<bf16_t> {
    static __device__ __forceinline__ float to_f32(bf16_t x) { return bf16_to_f32(x.bits); }
    static __device__ __forceinline__ bf16_t from_f32(float x) { bf16_t r; r.bits = f32_to_bf16(x); return r; }
};
template <> struct Elem<f16_t> {
    static __device__ __forceinline__ float to_f32(f16_t x) { return (float)x.v; }
    static __device__ __forceinline__ f16_t from_f32(float x) { f16_t r; r.v = (_Float16)x; return r; }
};

// four consecutive elements -> fp32 (pointer must be aligned to 4 elements)
__device__ __forceinline__ floatx4 load4_f32(const float* p) { return *reinterpret_cast<const floatx4*>(p); }
__device__ __forceinline__ floatx4 load4_f32(const bf16_t* p) {
    uint2 u = *reinterpret_cast<const uint2*>(p);
    floatx4 r;
    r[0] = __uint_as_float(u.x << 16); r[1] = __uint_as_float(u.x & 0xffff0000u);
    r[2] = __uint_as_float(u.y << 16); r[3] = __uint_as_float(u.y & 0xffff0000u);
    return r;
}
__device__ __forceinline__ floatx4 load4_f32(const f16_t* p) {
    halfx4 h = *reinterpret_cast<const halfx4*>(p);
    floatx4 r = {(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
    return r;
}
__device__ __forceinline__ void store4_f32(float* p, floatx4 v) { *reinterpret_cast<floatx4*>(p) = v; }
__device__ __forceinline__ void store4_f32(bf16_t* p, floatx4 v) {
    uint2 u;
    u.x = pack_bf16x2(v[0], v[1]);
    u.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<uint2*>(p) = u;
}
__device__ __forceinline__ void store4_f32(f16_t* p, floatx4 v) {
    halfx4 h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
    *reinterpret_cast<halfx4*>(p) = h;
}

// eight consecutive elements (two accumulator quads) with one 16-byte store for 2-byte types
// (results leave through nontemporal stores: they are written once and read by a later kernel, and on
// the large block-sparse tensors a cached store costs a quarter of the achieved HBM rate)
__device__ __forceinline__ void store8_f32(bf16_t* p, floatx4 a, floatx4 b) {
    __builtin_nontemporal_store(uintx4{pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(b[0], b[1]), pack_bf16x2(b[2], b[3])},
                                reinterpret_cast<uintx4*>(p));
}
__device__ __forceinline__ void store8_f32(f16_t* p, floatx4 a, floatx4 b) {
    typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
    halfx8 h = {(_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3],
                (_Float16)b[0], (_Float16)b[1], (_Float16)b[2], (_Float16)b[3]};
    __builtin_nontemporal_store(h, reinterpret_cast<halfx8*>(p));
}
__device__ __forceinline__ void store8_f32(float* p, floatx4 a, floatx4 b) { store4_f32(p, a); store4_f32(p + 4, b); }

// ---------------------------------------------------------------------------------------
// 16x16 MFMA "k16" step.  A fragment holds, for lane (r = lane%16, g = lane/16), the four
// operand elements k = 4g..4g+3 of row r (A side) or column r (B side) of a 16-wide slice of
// the contraction.  acc holds C[4g+i][r] for i = 0..3.
// ---------------------------------------------------------------------------------------
template <typename T> struct Frag;
template <> struct Frag<float> {
    typedef floatx4 type;
    static __device__ __forceinline__ type zero() { type z = {0.f, 0.f, 0.f, 0.f}; return z; }
    static __device__ __forceinline__ type load(const float* p) { return *reinterpret_cast<const type*>(p); }
    static __device__ __forceinline__ type gather(const float* p, long s) {
        type r = {p[0], p[s], p[2 * s], p[3 * s]}; return r;
    }
    static __device__ __forceinline__ floatx4 mma(type a, type b, floatx4 c) {
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], c, 0, 0, 0);
        return c;
    }
};
template <> struct Frag<bf16_t> {
    typedef shortx4 type;
    static __device__ __forceinline__ type zero() { type z = {0, 0, 0, 0}; return z; }
    static __device__ __forceinline__ type load(const bf16_t* p) { return *reinterpret_cast<const type*>(p); }
    static __device__ __forceinline__ type gather(const bf16_t* p, long s) {
        type r = {(short)p[0].bits, (short)p[s].bits, (short)p[2 * s].bits, (short)p[3 * s].bits}; return r;
    }
    static __device__ __forceinline__ floatx4 mma(type a, type b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
    }
};
template <> struct Frag<f16_t> {
    typedef halfx4 type;
    static __device__ __forceinline__ type zero() { type z = {0, 0, 0, 0}; return z; }
    static __device__ __forceinline__ type load(const f16_t* p) { return *reinterpret_cast<const type*>(p); }
    static __device__ __forceinline__ type gather(const f16_t* p, long s) {
        type r = {p[0].v, p[s].v, p[2 * s].v, p[3 * s].v}; return r;
    }
    static __device__ __forceinline__ floatx4 mma(type a, type b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
    }
};

// 16x16x32 MFMA step for 2-byte types (gfx950): a fragment is the eight contraction elements
// k = 8g..8g+7 of row/column r (one 16-byte load when k is contiguous)
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 halfx8_t __attribute__((ext_vector_type(8)));
template <typename T> struct Frag32;
template <> struct Frag32<bf16_t> {
    static __device__ __forceinline__ floatx4 mma(uint4 a, uint4 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};
template <> struct Frag32<f16_t> {
    static __device__ __forceinline__ floatx4 mma(uint4 a, uint4 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8_t, a), __builtin_bit_cast(halfx8_t, b), c, 0, 0, 0);
    }
};
template <> struct Frag32<float> {     // never used: keeps templates that branch on sizeof(T) compilable
    static __device__ __forceinline__ floatx4 mma(uint4, uint4, floatx4 c) { return c; }
};

// Wait for every outstanding vector-memory load (vmcnt(0); the other counters are left alone).  Placed
// in front of a pipelined loop it tells the compiler's wait-count bookkeeping that the operands
// loaded before the loop have arrived; without it the loop body carries the first iteration's waits
// for them, and those waits -- counters retire in order -- also drain the prefetch the body has
// just issued, every iteration.
__device__ __forceinline__ void drain_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }
// The same for "all but the newest N": in a loop that keeps two register sets of loads in flight,
// placed after the older set has been consumed it records that only the newer set is outstanding,
// so the refill of the older set's registers does not wait for the newer set.
template <int N>
__device__ __forceinline__ void drain_loads_but() {
    static_assert(N >= 0 && N < 64, "vmcnt holds 6 bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

// wave-level butterflies across the four 16-lane groups (lanes r, r+16, r+32, r+48), on the
// gfx950 row-swap instructions: permlane16_swap(v, v) yields {rows 0,0,2,2} and {rows 1,1,3,3},
// permlane32_swap(v, v) yields {low half twice} and {high half twice}; no LDS traffic
__device__ __forceinline__ void rows_pair16(float v, float& a, float& b) {
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void rows_pair32(float v, float& a, float& b) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}
__device__ __forceinline__ float group_max(float v) {
    float a, b;
    rows_pair16(v, a, b); v = fmaxf(a, b);
    rows_pair32(v, a, b); return fmaxf(a, b);
}
__device__ __forceinline__ float group_sum(float v) {
    float a, b;
    rows_pair16(v, a, b); v = a + b;
    rows_pair32(v, a, b); return a + b;
}
// sum over the 16 lanes of a row (lanes with equal lane/16) on DPP: quad butterflies, then the two
// mirrors; every lane of the row ends with the row total
__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));   // quad_perm 1,0,3,2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));   // quad_perm 2,3,0,1
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));  // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));  // row_mirror
    return v;
}
__device__ __forceinline__ float row16_max(float v) {     // as row16_sum; the patterns reach every lane of the row
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// ---- operands as sums of bf16 pieces (float inputs on the bf16 matrix pipe) ----
// one 16x16x32 step on the bf16 matrix pipe: eight k-slots per lane on either side
__device__ __forceinline__ floatx4 mma_bf16(uint4 a, uint4 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ floatx4 mma_bf16(uintx4 a, uintx4 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// chunk c of a row -> the chunk it is stored at
__device__ __forceinline__ int x3_swz(int row, int c, int row_bytes) {
    return row_bytes >= 128 ? (c ^ (row & 7)) : (c ^ ((row >> 1) & 3));
}
// an fp32 value rounded to 17 significant bits (its bf16 head and the bf16 head of the rest then add up to it exactly)
__device__ __forceinline__ float quant16(float x) {
    // (finite x; ties away from zero.  17 significant bits split exactly: the head is rounded to nearest, so the rest is
    //  at most half a unit of its last place, and its sign carries the ninth bit)
    return __uint_as_float((__float_as_uint(x) + 0x40u) & 0xffffff80u);
}
__device__ __forceinline__ floatx4 quant16(floatx4 x) {
    floatx4 r = {quant16(x[0]), quant16(x[1]), quant16(x[2]), quant16(x[3])};
    return r;
}
// eight floats -> bf16 head and remainder (eight k-slots each)
__device__ __forceinline__ void split2(floatx4 x0, floatx4 x1, uintx4& hi, uintx4& lo) {
    hi = uintx4{pack_bf16x2(x0[0], x0[1]), pack_bf16x2(x0[2], x0[3]), pack_bf16x2(x1[0], x1[1]), pack_bf16x2(x1[2], x1[3])};
    floatx4 r0, r1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w0 = hi[i >> 1], w1 = hi[2 + (i >> 1)];
        r0[i] = x0[i] - ((i & 1) ? __uint_as_float(w0 & 0xffff0000u) : __uint_as_float(w0 << 16));
        r1[i] = x1[i] - ((i & 1) ? __uint_as_float(w1 & 0xffff0000u) : __uint_as_float(w1 << 16));
    }
    lo = uintx4{pack_bf16x2(r0[0], r0[1]), pack_bf16x2(r0[2], r0[3]), pack_bf16x2(r1[0], r1[1]), pack_bf16x2(r1[2], r1[3])};
}
// eight floats -> three bf16 pieces whose sum is the value exactly
__device__ __forceinline__ void split3(floatx4 x0, floatx4 x1, uintx4& h, uintx4& m, uintx4& l) {
    h = uintx4{pack_bf16x2(x0[0], x0[1]), pack_bf16x2(x0[2], x0[3]), pack_bf16x2(x1[0], x1[1]), pack_bf16x2(x1[2], x1[3])};
    floatx4 r0, r1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w0 = h[i >> 1], w1 = h[2 + (i >> 1)];
        r0[i] = x0[i] - ((i & 1) ? __uint_as_float(w0 & 0xffff0000u) : __uint_as_float(w0 << 16));
        r1[i] = x1[i] - ((i & 1) ? __uint_as_float(w1 & 0xffff0000u) : __uint_as_float(w1 << 16));
    }
    split2(r0, r1, m, l);
}

// four floats -> bf16 head and rest, four k-slots each
__device__ __forceinline__ void split2_4(floatx4 x, uint2& hi, uint2& lo) {
    hi = make_uint2(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]));
    const floatx4 r = {x[0] - __uint_as_float(hi.x << 16), x[1] - __uint_as_float(hi.x & 0xffff0000u),
                       x[2] - __uint_as_float(hi.y << 16), x[3] - __uint_as_float(hi.y & 0xffff0000u)};
    lo = make_uint2(pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3]));
}

__device__ __forceinline__ void split3_4(floatx4 x, uint2& h, uint2& m, uint2& l) {
    h = make_uint2(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]));
    const floatx4 r = {x[0] - __uint_as_float(h.x << 16), x[1] - __uint_as_float(h.x & 0xffff0000u),
                       x[2] - __uint_as_float(h.y << 16), x[3] - __uint_as_float(h.y & 0xffff0000u)};
    split2_4(r, m, l);
}

// Dropout of attention weights without a stored mask: whether the pair (row, col) is kept is a hash of (seed, row, col),
// so the backward forms the same mask again from the seed.  row_hash depends on the row alone (one query: once per
// lane).  A pair of neighbouring columns (2c, 2c + 1) shares one 32-bit hash -- the pair index enters through a
// multiply-add and the 32-bit finaliser of MurmurHash3 (full avalanche) -- and each column takes one 16-bit half of it:
// the hash is ten vector instructions, and a lane's columns come in consecutive runs.  A pair is
// kept when its half is at least thresh = floor(p 2^16); kept weights are scaled by 1 / (1 - thresh 2^-16).
__device__ __forceinline__ uint32_t drop_mix(uint32_t h) {
    h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
    return h;
}
__device__ __forceinline__ uint32_t drop_row_hash(uint32_t seed, uint32_t row) { return drop_mix(row * 0x9E3779B1u + seed); }
__device__ __forceinline__ bool drop_keep(uint32_t row_hash, uint32_t col, uint32_t thresh) {
    const uint32_t h = drop_mix(row_hash + (col >> 1) * 0x632BE5ABu);
    return ((col & 1u) ? (h >> 16) : (h & 0xffffu)) >= thresh;
}
// host side: the kernels' dropout arguments from a probability and a 64-bit seed (p = 0: thresh = 0 = off)
struct DropArgs { uint32_t seed, thresh; float scale; };
inline DropArgs drop_args(float p, uint64_t seed) {
    DropArgs d{0, 0, 1.f};
    if (p > 0.f) {
        d.seed = (uint32_t)seed ^ ((uint32_t)(seed >> 32) * 0x9E3779B1u);
        const double t = (double)p * 65536.0;
        d.thresh = t >= 65535.0 ? 65535u : (uint32_t)t;
        if (d.thresh == 0) d.thresh = 1;
        d.scale = (float)(1.0 / (1.0 - d.thresh / 65536.0));       // of the probability actually realised: the mean stays exact
    }
    return d;
}

// One wave's 1024 bytes straight from global memory into LDS (lane l's 16 bytes land at wave_base + 16 l), issued as
// assembly: the compiler then does not know of a transfer in flight, and does not drain the load counter in front of
// LDS reads of the other stage (it does so before every transposing read, whose address it cannot tell from the
// transfer's destination, which would leave the prefetch a fraction of a tile to arrive in).  The caller waits for
// its transfers (drain_loads) before the barrier that publishes them.
__device__ __forceinline__ void dma_to_lds(const void* lane_src, const char* wave_base) {
    typedef __attribute__((address_space(3))) const char* lds_ptr;
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr)wave_base);
    // m0 carries the LDS destination of the transfer.  The compiler does not accept m0 in a clobber list (it is a
    // reserved register), so the statement itself puts back what m0 held: whatever the compiler keeps in m0 across
    // this point (LDS-direct reads, register-indexed moves, SGPR spills) survives.  The transfer reads m0 when it is
    // issued, so the restore may follow it directly.
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "v"(lane_src), "s"(base) : "memory");
}

// Transposed operand reads (ds_read_b64_tr_b16): within each group of 16 lanes, lane s passes the address of four
// consecutive 16-bit elements -- row s / 4, columns 4 (s % 4) .. + 3 of a 4 x 16 block -- and lane l receives column l of
// the four rows.
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));
// eight k-slots (inner rows) of one column: two transposed reads of 4 rows each
__device__ __forceinline__ uintx4 lds_read_tr8(const char* p0, const char* p1) {
    typedef __attribute__((address_space(3))) shortx4* lds_ptr;
    const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p0);
    const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p1);
    return __builtin_bit_cast(uintx4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}


}  // namespace flyhip
