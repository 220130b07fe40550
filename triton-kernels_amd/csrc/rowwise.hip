// Row-wise, HBM-bound kernels: RMSNorm (fwd/bwd) and LayerNorm + adaLN modulation.
//
// Layout idea: a row is owned by a group of G adjacent lanes (G = 16, 32 or 64) and lives entirely
// in registers as ITER 16-byte vectors per lane, so each element crosses HBM exactly once in each
// direction and the reduction is a DPP butterfly with no LDS traffic. Rows too long for that
// (more than 64*ITER_MAX vectors) or not 16-byte addressable take a block-per-row kernel that
// re-reads the row from cache.
#include "common.h"

namespace flux {

constexpr int kBlock = 256;

// ------------------------------------------------------------------------------------------------
// Register-resident row helpers
// ------------------------------------------------------------------------------------------------
template <typename T, int G, int ITER>
struct RowRegs {
    static constexpr int VEC = Elem<T>::VEC;
    float x[ITER][VEC];

    // col(it, lane) = (it*G + lane) * VEC
    __device__ __forceinline__ void load(const T* row, int lane, int n, bool row_ok) {
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            int c = (it * G + lane) * VEC;
            if (row_ok && c < n) {
                Vec16<T> v = ld16(row + c);
#pragma unroll
                for (int e = 0; e < VEC; ++e) x[it][e] = Elem<T>::load(v.v[e]);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) x[it][e] = 0.0f;
            }
        }
    }
};

template <typename TS, int VEC>
__device__ __forceinline__ void load_vecf(const TS* p, float (&out)[VEC]) {
    // VEC consecutive elements of a small parameter vector (scale / shift), any alignment >= VEC*sizeof
    if constexpr (sizeof(TS) * VEC == 16) {
        Vec16<TS> v = ld16(p);
#pragma unroll
        for (int e = 0; e < VEC; ++e) out[e] = Elem<TS>::load(v.v[e]);
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) out[e] = Elem<TS>::load(p[e]);
    }
}

// ------------------------------------------------------------------------------------------------
// RMSNorm forward, register-resident.
// ------------------------------------------------------------------------------------------------
// R rows per thread (a block covers R * kBlock / G rows, row j of a thread being kBlock / G rows behind row
// j - 1). One row per thread is what is launched: two rows of one vector each, which put twice the loads
// in flight per wave and halve the number of workgroups, measured 14.7 us against 13.8 us at the Flux shape.
template <typename T, typename TS, int G, int ITER, int R>
__global__ __launch_bounds__(kBlock) void rms_norm_fwd_regs(
    const T* __restrict__ x, const TS* __restrict__ scale, T* __restrict__ y, float* __restrict__ rstd_out,
    int64_t rows, int64_t d1, int64_t d2, int n, int64_t s0, int64_t s1, int64_t s2, float eps) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int ROWS_PER_PASS = kBlock / G;
    const int lane = threadIdx.x % G;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * (ROWS_PER_PASS * R) + threadIdx.x / G;

    // Offset of a row in the strided [d0, d1, d2] view. The host merges dimensions whose strides
    // allow it, so an evenly strided tensor arrives as d1 = 1 and needs no division; other views
    // divide in 32 bits when the row count allows (a 64-bit division costs a hundred instructions,
    // which at one vector per lane is more than the rest of the kernel).
    auto offset_of = [&](int64_t row) -> int64_t {
        if (d1 == 1 && row < d2) return row * s2;
        if (rows <= 0x7fffffffLL) {
            const uint32_t r32 = static_cast<uint32_t>(row), e2 = static_cast<uint32_t>(d2), e1 = static_cast<uint32_t>(d1);
            const uint32_t t = r32 / e2, i2 = r32 - t * e2, i0 = t / e1, i1 = t - i0 * e1;
            return i0 * s0 + i1 * s1 + static_cast<int64_t>(i2) * s2;
        }
        const int64_t i2 = row % d2, t = row / d2;
        return (t / d1) * s0 + (t % d1) * s1 + i2 * s2;
    };
    RowRegs<T, G, ITER> r[R];
    bool row_ok[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int64_t row = row0 + j * ROWS_PER_PASS;
        row_ok[j] = row < rows;
        r[j].load(x + (row_ok[j] ? offset_of(row) : 0), lane, n, row_ok[j]);
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int64_t row = row0 + j * ROWS_PER_PASS;
        float ss = 0.0f;
#pragma unroll
        for (int it = 0; it < ITER; ++it)
#pragma unroll
            for (int e = 0; e < VEC; ++e) ss += r[j].x[it][e] * r[j].x[it][e];
        ss = group_sum<G>(ss);
        const float rstd = rsqrtf(ss / static_cast<float>(n) + eps);

        if (!row_ok[j]) continue;
        if (rstd_out != nullptr && lane == 0) rstd_out[row] = rstd;
        T* yrow = y + row * n;
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            int c = (it * G + lane) * VEC;
            if (c < n) {
                float w[VEC];
                load_vecf<TS, VEC>(scale + c, w);
                Vec16<T> o;
#pragma unroll
                for (int e = 0; e < VEC; ++e) o.v[e] = Elem<T>::store(Elem<T>::round(r[j].x[it][e] * rstd) * w[e]);
                st16(yrow + c, o);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Block-wide sum for the block-per-row kernels.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float block_sum(float v, float* lds /* >= 4 floats + 1 */) {
    v = group_sum<64>(v);
    const int wave = threadIdx.x / 64;
    __syncthreads();
    if (threadIdx.x % 64 == 0) lds[wave] = v;
    __syncthreads();
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) t += lds[w];
    return t;
}

// RMSNorm forward, one block per row, any n and alignment (VEC = 1) or 16-byte rows (VEC = Elem::VEC).
template <typename T, typename TS, int VEC>
__global__ __launch_bounds__(kBlock) void rms_norm_fwd_block(
    const T* __restrict__ x, const TS* __restrict__ scale, T* __restrict__ y, float* __restrict__ rstd_out,
    int64_t rows, int64_t d1, int64_t d2, int n, int64_t s0, int64_t s1, int64_t s2, float eps) {
    __shared__ float lds[8];
    const int64_t row = blockIdx.x;
    int64_t i2 = row % d2;
    int64_t t = row / d2;
    int64_t i1 = t % d1;
    int64_t i0 = t / d1;
    const T* xrow = x + i0 * s0 + i1 * s1 + i2 * s2;
    T* yrow = y + row * n;

    float ss = 0.0f;
    for (int c = threadIdx.x * VEC; c < n; c += kBlock * VEC) {
        if constexpr (VEC == 1) {
            float v = Elem<T>::load(xrow[c]);
            ss += v * v;
        } else {
            Vec16<T> v = ld16(xrow + c);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float f = Elem<T>::load(v.v[e]);
                ss += f * f;
            }
        }
    }
    ss = block_sum(ss, lds);
    const float rstd = rsqrtf(ss / static_cast<float>(n) + eps);
    if (rstd_out != nullptr && threadIdx.x == 0) rstd_out[row] = rstd;
    for (int c = threadIdx.x * VEC; c < n; c += kBlock * VEC) {
        if constexpr (VEC == 1) {
            float v = Elem<T>::load(xrow[c]);
            yrow[c] = Elem<T>::store(Elem<T>::round(v * rstd) * Elem<TS>::load(scale[c]));
        } else {
            Vec16<T> v = ld16(xrow + c);
            float w[VEC];
            load_vecf<TS, VEC>(scale + c, w);
            Vec16<T> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.v[e] = Elem<T>::store(Elem<T>::round(Elem<T>::load(v.v[e]) * rstd) * w[e]);
            st16(yrow + c, o);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// RMSNorm backward: dx = rstd*(dy*w) - rstd^3/n * sum(dy*w*x) * x ;  dscale += sum_rows dy*x*rstd.
// One group of G lanes per row (register-resident); each block reduces its rows' dscale partials in
// registers while its groups walk the block's rows, folds them in LDS and finishes with one atomic
// per column per block. All blocks finish together and their atomics land on the few cache lines of
// dscale, where they are served one at a time: short rows (one vector per lane) therefore run as
// 256 blocks of 1024 threads rather than 1024 blocks of 256.
// ------------------------------------------------------------------------------------------------
template <typename T, typename TS, int G, int ITER, int BLK>
__global__ __launch_bounds__(BLK) void rms_norm_bwd_regs(
    const T* __restrict__ dy, const T* __restrict__ x, const TS* __restrict__ scale, const float* __restrict__ rstd_in,
    T* __restrict__ dx, float* __restrict__ dscale, int64_t rows, int n, int rows_per_group) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int GROUPS = BLK / G;
    const int lane = threadIdx.x % G;
    const int grp = threadIdx.x / G;

    float w[ITER][VEC];
    float dw[ITER][VEC];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        int c = (it * G + lane) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) { w[it][e] = 0.0f; dw[it][e] = 0.0f; }
        if (c < n) load_vecf<TS, VEC>(scale + c, w[it]);
    }

    // A block owns GROUPS * rows_per_group consecutive rows and its groups take them interleaved, so
    // one step of the block reads a contiguous span; U rows per group are requested before the first
    // is used.
    constexpr int U = ITER == 1 ? 4 : (ITER == 2 ? 2 : 1);
    const int64_t block_row0 = static_cast<int64_t>(blockIdx.x) * GROUPS * rows_per_group;
    for (int i0 = 0; i0 < rows_per_group; i0 += U) {
        RowRegs<T, G, ITER> rx[U], rdy[U];
        float rstd[U];
        bool ok[U];
        int64_t row[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            row[u] = block_row0 + static_cast<int64_t>(i0 + u) * GROUPS + grp;
            ok[u] = i0 + u < rows_per_group && row[u] < rows;  // uniform over the group
            const int64_t r = ok[u] ? row[u] : 0;
            rx[u].load(x + r * n, lane, n, ok[u]);
            rdy[u].load(dy + r * n, lane, n, ok[u]);
            rstd[u] = ok[u] ? rstd_in[r] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float dot = 0.0f;
#pragma unroll
            for (int it = 0; it < ITER; ++it)
#pragma unroll
                for (int e = 0; e < VEC; ++e) dot += rdy[u].x[it][e] * w[it][e] * rx[u].x[it][e];
            dot = group_sum<G>(dot);
            const float coef = -rstd[u] * rstd[u] * rstd[u] * dot / static_cast<float>(n);
            if (ok[u]) {
#pragma unroll
                for (int it = 0; it < ITER; ++it) {
                    int c = (it * G + lane) * VEC;
                    if (c < n) {
                        Vec16<T> o;
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            o.v[e] = Elem<T>::store(rstd[u] * rdy[u].x[it][e] * w[it][e] + coef * rx[u].x[it][e]);
                            dw[it][e] += rdy[u].x[it][e] * rx[u].x[it][e] * rstd[u];
                        }
                        st16(dx + row[u] * n + c, o);
                    }
                }
            }
        }
    }
    // Fold the block's GROUPS partial rows in LDS, then one atomic per column per block.
    extern __shared__ float dw_lds[];  // [GROUPS][G*ITER*VEC]
    constexpr int COLS = G * ITER * VEC;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        int c = (it * G + lane) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) dw_lds[grp * COLS + c + e] = dw[it][e];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < n; c += BLK) {
        float t = 0.0f;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) t += dw_lds[g * COLS + c];
        atomicAdd(dscale + c, t);
    }
}

// Block-per-row backward for rows that do not fit the register path.
template <typename T, typename TS>
__global__ __launch_bounds__(kBlock) void rms_norm_bwd_block(
    const T* __restrict__ dy, const T* __restrict__ x, const TS* __restrict__ scale, const float* __restrict__ rstd_in,
    T* __restrict__ dx, float* __restrict__ dscale, int64_t rows, int n) {
    __shared__ float lds[8];
    const int64_t row = blockIdx.x;
    const T* xr = x + row * n;
    const T* dyr = dy + row * n;
    const float rstd = rstd_in[row];
    float dot = 0.0f;
    for (int c = threadIdx.x; c < n; c += kBlock)
        dot += Elem<T>::load(dyr[c]) * Elem<TS>::load(scale[c]) * Elem<T>::load(xr[c]);
    dot = block_sum(dot, lds);
    const float coef = -rstd * rstd * rstd * dot / static_cast<float>(n);
    for (int c = threadIdx.x; c < n; c += kBlock) {
        float g = Elem<T>::load(dyr[c]), xv = Elem<T>::load(xr[c]);
        dx[row * n + c] = Elem<T>::store(rstd * g * Elem<TS>::load(scale[c]) + coef * xv);
        atomicAdd(dscale + c, g * xv * rstd);
    }
}

// ------------------------------------------------------------------------------------------------
// LayerNorm + modulation, register-resident: two-pass statistics on the registers.
// For bf16 storage the normalised value, (1+scale) and the product are each rounded to bf16 before
// the next step, the evaluation order of functional/normalization.py:6-12 on bf16 tensors.
// ------------------------------------------------------------------------------------------------
// Straight-line: rows past the end and columns past n are clamped for the loads (x, scale and shift
// vectors all go out before the first reduction) and masked in the sums; only the stores are
// predicated. FULL = the row fills the lanes exactly (n == G * ITER * VEC), no column masks at all.
// MODLDS: all rows of a workgroup belong to one batch element, and the workgroup prepares that element's
// modulation vectors once, in LDS, as fp32: g = (1 + scale) rounded like the PyTorch op, and shift. Every
// row needs all of both vectors; loaded and converted by each wave for itself (MODLDS = false, the
// general form) that is as many loads as the row itself has and a fifth of the kernel's arithmetic.
template <typename T, int G, int ITER, bool FULL, bool MODLDS>
__global__ __launch_bounds__(kBlock) void ln_mod_fwd_regs(
    const T* __restrict__ x, const T* __restrict__ scale, const T* __restrict__ shift, T* __restrict__ y,
    int64_t rows, int64_t seq, int n, int64_t mod_stride, float eps) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int ROWS_PER_BLOCK = kBlock / G;
    constexpr int NMAX = MODLDS ? G * ITER * VEC : 1;
    __shared__ __attribute__((aligned(16))) float g_lds[NMAX], d_lds[NMAX];
    const int lane = threadIdx.x % G;
    const int64_t row_raw = static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK + threadIdx.x / G;
    const bool row_ok = row_raw < rows;
    const int64_t row = row_ok ? row_raw : rows - 1;
    const int64_t b = row / seq;
    const T* xr = x + row * n;
    const T* sc = scale + b * mod_stride;
    const T* sh = shift + b * mod_stride;

    Vec16<T> xv[ITER], av[ITER], dv[ITER];
    bool in[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int c = (it * G + lane) * VEC;
        in[it] = FULL || c < n;
        const int cl = in[it] ? c : 0;
        xv[it] = ld16(xr + cl);
        if (!MODLDS) {
            av[it] = ld16(sc + cl);
            dv[it] = ld16(sh + cl);
        }
    }
    if (MODLDS) {
        // the first row's batch element is every row's (the host checks that a block does not span two)
        const int64_t b0 = (static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK) / seq;
        for (int c = threadIdx.x * VEC; c < n; c += kBlock * VEC) {
            const Vec16<T> a = ld16(scale + b0 * mod_stride + c), d = ld16(shift + b0 * mod_stride + c);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                g_lds[c + e] = Elem<T>::round(1.0f + Elem<T>::load(a.v[e]));
                d_lds[c + e] = Elem<T>::load(d.v[e]);
            }
        }
    }
    float xf[ITER][VEC];
    float s = 0.0f;
#pragma unroll
    for (int it = 0; it < ITER; ++it)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            xf[it][e] = in[it] ? Elem<T>::load(xv[it].v[e]) : 0.0f;
            s += xf[it][e];
        }
    s = group_sum<G>(s);
    const float mean = s / static_cast<float>(n);
    float q = 0.0f;
#pragma unroll
    for (int it = 0; it < ITER; ++it)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float d = in[it] ? xf[it][e] - mean : 0.0f;
            q += d * d;
        }
    q = group_sum<G>(q);
    const float rstd = rsqrtf(q / static_cast<float>(n) + eps);
    if (MODLDS) __syncthreads();

    T* yrow = y + row * n;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int c = (it * G + lane) * VEC;
        const int cl = in[it] ? c : 0;
        Vec16<T> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float nv = Elem<T>::round((xf[it][e] - mean) * rstd);
            const float g = MODLDS ? g_lds[cl + e] : Elem<T>::round(1.0f + Elem<T>::load(av[it].v[e]));
            const float d = MODLDS ? d_lds[cl + e] : Elem<T>::load(dv[it].v[e]);
            o.v[e] = Elem<T>::store(Elem<T>::round(nv * g) + d);
        }
        if (row_ok && in[it]) st16(yrow + c, o);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void ln_mod_fwd_block(
    const T* __restrict__ x, const T* __restrict__ scale, const T* __restrict__ shift, T* __restrict__ y,
    int64_t rows, int64_t seq, int n, int64_t mod_stride, float eps) {
    __shared__ float lds[8];
    const int64_t row = blockIdx.x;
    const T* xr = x + row * n;
    float s = 0.0f;
    for (int c = threadIdx.x; c < n; c += kBlock) s += Elem<T>::load(xr[c]);
    const float mean = block_sum(s, lds) / static_cast<float>(n);
    float q = 0.0f;
    for (int c = threadIdx.x; c < n; c += kBlock) {
        float d = Elem<T>::load(xr[c]) - mean;
        q += d * d;
    }
    const float rstd = rsqrtf(block_sum(q, lds) / static_cast<float>(n) + eps);
    const int64_t b = row / seq;
    const T* sc = scale + b * mod_stride;
    const T* sh = shift + b * mod_stride;
    for (int c = threadIdx.x; c < n; c += kBlock) {
        float nv = Elem<T>::round((Elem<T>::load(xr[c]) - mean) * rstd);
        float g = Elem<T>::round(1.0f + Elem<T>::load(sc[c]));
        y[row * n + c] = Elem<T>::store(Elem<T>::round(nv * g) + Elem<T>::load(sh[c]));
    }
}

// ------------------------------------------------------------------------------------------------
// Host dispatch
// ------------------------------------------------------------------------------------------------
struct RowPlan {
    int G;     // lanes per row, 0 = use the block kernel
    int ITER;  // vectors per lane
};

static RowPlan plan_row(int n, int vec) {
    if (n % vec != 0) return {0, 0};
    int nv = n / vec;
    if (nv <= 16) return {16, 1};
    if (nv <= 32) return {32, 1};
    if (nv <= 64) return {64, 1};
    int it = (nv + 63) / 64;
    const int allowed[] = {2, 3, 4, 6, 8};
    for (int a : allowed)
        if (it <= a) return {64, a};
    return {0, 0};
}

#define FLUX_DISPATCH_GI(plan, CALL)                                   \
    do {                                                               \
        if (plan.G == 16) { CALL(16, 1); }                             \
        else if (plan.G == 32) { CALL(32, 1); }                        \
        else if (plan.ITER == 1) { CALL(64, 1); }                      \
        else if (plan.ITER == 2) { CALL(64, 2); }                      \
        else if (plan.ITER == 3) { CALL(64, 3); }                      \
        else if (plan.ITER == 4) { CALL(64, 4); }                      \
        else if (plan.ITER == 6) { CALL(64, 6); }                      \
        else { CALL(64, 8); }                                          \
    } while (0)

template <typename T, typename TS>
static int rms_fwd_launch(const void* x, const void* scale, void* y, float* rstd, int64_t d0, int64_t d1, int64_t d2,
                          int n, int64_t s0, int64_t s1, int64_t s2, float eps, hipStream_t st) {
    constexpr int VEC = Elem<T>::VEC;
    const int64_t rows = d0 * d1 * d2;
    const T* xp = static_cast<const T*>(x);
    const TS* sp = static_cast<const TS*>(scale);
    T* yp = static_cast<T*>(y);
    RowPlan plan = plan_row(n, VEC);
    const bool vec_ok = aligned16(x) && aligned16(y) && s0 % VEC == 0 && s1 % VEC == 0 && s2 % VEC == 0 &&
                        (sizeof(TS) * VEC != 16 || aligned16(scale));
    // merge dimensions that are evenly strided: [d0, d1, d2] -> [1, 1, rows] for a contiguous tensor
    if (d0 == 1 || s0 == d1 * s1) { d1 *= d0; d0 = 1; }
    if (d0 == 1 && (d1 == 1 || s1 == d2 * s2)) { d2 *= d1; d1 = 1; }
    if (plan.G != 0 && vec_ok) {
#define CALL(G_, I_)                                                                                          \
    do {                                                                                                      \
        constexpr int R_ = 1;   /* two short rows per thread measured 6 % slower at the Flux shape */            \
        constexpr int RPB_ = (kBlock / G_) * R_;                                                              \
        hipLaunchKernelGGL((rms_norm_fwd_regs<T, TS, G_, I_, R_>), dim3((unsigned)((rows + RPB_ - 1) / RPB_)), \
                           dim3(kBlock), 0, st, xp, sp, yp, rstd, rows, d1, d2, n, s0, s1, s2, eps);           \
    } while (0)
        FLUX_DISPATCH_GI(plan, CALL);
#undef CALL
    } else if (n % VEC == 0 && vec_ok) {
        hipLaunchKernelGGL((rms_norm_fwd_block<T, TS, VEC>), dim3((unsigned)rows), dim3(kBlock), 0, st, xp, sp, yp, rstd,
                           rows, d1, d2, n, s0, s1, s2, eps);
    } else {
        hipLaunchKernelGGL((rms_norm_fwd_block<T, TS, 1>), dim3((unsigned)rows), dim3(kBlock), 0, st, xp, sp, yp, rstd,
                           rows, d1, d2, n, s0, s1, s2, eps);
    }
    return check_launch("flux_rms_norm");
}

template <typename T, typename TS>
static int rms_bwd_launch(const void* dy, const void* x, const void* scale, const float* rstd, void* dx, float* dscale,
                          int64_t rows, int n, hipStream_t st) {
    constexpr int VEC = Elem<T>::VEC;
    const T* dyp = static_cast<const T*>(dy);
    const T* xp = static_cast<const T*>(x);
    const TS* sp = static_cast<const TS*>(scale);
    T* dxp = static_cast<T*>(dx);
    RowPlan plan = plan_row(n, VEC);
    const bool vec_ok = aligned16(dy) && aligned16(x) && aligned16(dx) && (sizeof(TS) * VEC != 16 || aligned16(scale));
    if (plan.G != 0 && plan.ITER <= 4 && vec_ok) {
#define CALL(G_, I_)                                                                                         \
    do {                                                                                                     \
        constexpr int IT = (I_ > 4 ? 4 : I_);                                                                \
        constexpr int BLK = IT == 1 ? 1024 : kBlock;                                                         \
        constexpr int GROUPS = BLK / G_;                                                                     \
        const int64_t want_blocks = IT == 1 ? 256 : 1024;  /* few blocks: few atomics on dscale */           \
        int64_t rpg = (rows + want_blocks * GROUPS - 1) / (want_blocks * GROUPS);                            \
        if (rpg < 1) rpg = 1;                                                                                \
        const unsigned grid = (unsigned)((rows + rpg * GROUPS - 1) / (rpg * GROUPS));                        \
        const size_t lds_bytes = sizeof(float) * BLK * IT * VEC;                                             \
        hipLaunchKernelGGL((rms_norm_bwd_regs<T, TS, G_, IT, BLK>), dim3(grid), dim3(BLK), lds_bytes, st, dyp, xp, sp, \
                           rstd, dxp, dscale, rows, n, (int)rpg);                                            \
    } while (0)
        FLUX_DISPATCH_GI(plan, CALL);
#undef CALL
    } else {
        hipLaunchKernelGGL((rms_norm_bwd_block<T, TS>), dim3((unsigned)rows), dim3(kBlock), 0, st, dyp, xp, sp, rstd, dxp,
                           dscale, rows, n);
    }
    return check_launch("flux_rms_norm_bwd");
}

template <typename T>
static int ln_mod_launch(const void* x, const void* scale, const void* shift, void* y, int64_t batch, int64_t seq, int n,
                         int64_t mod_stride, float eps, hipStream_t st) {
    constexpr int VEC = Elem<T>::VEC;
    const int64_t rows = batch * seq;
    const T* xp = static_cast<const T*>(x);
    const T* scp = static_cast<const T*>(scale);
    const T* shp = static_cast<const T*>(shift);
    T* yp = static_cast<T*>(y);
    RowPlan plan = plan_row(n, VEC);
    const bool vec_ok = aligned16(x) && aligned16(y) && aligned16(scale) && aligned16(shift) && mod_stride % VEC == 0;
    if (plan.G != 0 && vec_ok) {
#define CALL(G_, I_)                                                                                        \
    do {                                                                                                    \
        const dim3 grid_((unsigned)((rows + kBlock / G_ - 1) / (kBlock / G_)));                              \
        /* wave-per-row plans whose blocks stay inside one batch element stage the modulation vectors in LDS */ \
        const bool lds_ = G_ == 64 && (batch == 1 || seq % (kBlock / G_) == 0);                             \
        if (n == G_ * I_ * VEC && lds_)                                                                     \
            hipLaunchKernelGGL((ln_mod_fwd_regs<T, G_, I_, true, G_ == 64>), grid_, dim3(kBlock), 0, st, xp, scp, shp, yp, rows, seq, n, mod_stride, eps);  \
        else if (n == G_ * I_ * VEC)                                                                        \
            hipLaunchKernelGGL((ln_mod_fwd_regs<T, G_, I_, true, false>), grid_, dim3(kBlock), 0, st, xp, scp, shp, yp, rows, seq, n, mod_stride, eps);  \
        else if (lds_)                                                                                      \
            hipLaunchKernelGGL((ln_mod_fwd_regs<T, G_, I_, false, G_ == 64>), grid_, dim3(kBlock), 0, st, xp, scp, shp, yp, rows, seq, n, mod_stride, eps); \
        else                                                                                                \
            hipLaunchKernelGGL((ln_mod_fwd_regs<T, G_, I_, false, false>), grid_, dim3(kBlock), 0, st, xp, scp, shp, yp, rows, seq, n, mod_stride, eps); \
    } while (0)
        FLUX_DISPATCH_GI(plan, CALL);
#undef CALL
    } else {
        hipLaunchKernelGGL((ln_mod_fwd_block<T>), dim3((unsigned)rows), dim3(kBlock), 0, st, xp, scp, shp, yp, rows, seq, n,
                           mod_stride, eps);
    }
    return check_launch("flux_layer_norm_modulation");
}

}  // namespace flux

using namespace flux;

extern "C" int flux_rms_norm(const void* x, const void* scale, void* y, float* rstd, int64_t d0, int64_t d1, int64_t d2,
                             int32_t n, int64_t s0, int64_t s1, int64_t s2, int32_t x_dtype, int32_t scale_dtype,
                             float eps, void* stream) {
    if (!x || !scale || !y) return fail(FLUX_E_NULL, "flux_rms_norm: null pointer");
    if (d0 < 0 || d1 < 0 || d2 < 0 || n <= 0) return fail(FLUX_E_SHAPE, "flux_rms_norm: bad shape [%lld,%lld,%lld,%d]", (long long)d0, (long long)d1, (long long)d2, n);
    if (n > FLUX_MAX_ROW) return fail(FLUX_E_TOO_WIDE, "flux_rms_norm: n = %d exceeds the maximum row length %d", n, FLUX_MAX_ROW);
    if (d0 * d1 * d2 == 0) return FLUX_OK;
    if (d0 * d1 * d2 > 0x7fffffffLL * 4) return fail(FLUX_E_SHAPE, "flux_rms_norm: too many rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == FLUX_BF16 && scale_dtype == FLUX_BF16) return rms_fwd_launch<bf16_t, bf16_t>(x, scale, y, rstd, d0, d1, d2, n, s0, s1, s2, eps, st);
    if (x_dtype == FLUX_BF16 && scale_dtype == FLUX_F32) return rms_fwd_launch<bf16_t, float>(x, scale, y, rstd, d0, d1, d2, n, s0, s1, s2, eps, st);
    if (x_dtype == FLUX_F32 && scale_dtype == FLUX_F32) return rms_fwd_launch<float, float>(x, scale, y, rstd, d0, d1, d2, n, s0, s1, s2, eps, st);
    return fail(FLUX_E_DTYPE, "flux_rms_norm: unsupported dtype pair (%d,%d)", x_dtype, scale_dtype);
}

extern "C" int flux_rms_norm_bwd(const void* dy, const void* x, const void* scale, const float* rstd, void* dx,
                                 float* dscale, int64_t rows, int32_t n, int32_t x_dtype, int32_t scale_dtype,
                                 void* stream) {
    if (!dy || !x || !scale || !rstd || !dx || !dscale) return fail(FLUX_E_NULL, "flux_rms_norm_bwd: null pointer");
    if (rows < 0 || n <= 0) return fail(FLUX_E_SHAPE, "flux_rms_norm_bwd: bad shape [%lld,%d]", (long long)rows, n);
    if (n > FLUX_MAX_ROW) return fail(FLUX_E_TOO_WIDE, "flux_rms_norm_bwd: n = %d exceeds the maximum row length %d", n, FLUX_MAX_ROW);
    if (rows == 0) return FLUX_OK;
    if (rows > 0x7fffffffLL) return fail(FLUX_E_SHAPE, "flux_rms_norm_bwd: too many rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == FLUX_BF16 && scale_dtype == FLUX_BF16) return rms_bwd_launch<bf16_t, bf16_t>(dy, x, scale, rstd, dx, dscale, rows, n, st);
    if (x_dtype == FLUX_BF16 && scale_dtype == FLUX_F32) return rms_bwd_launch<bf16_t, float>(dy, x, scale, rstd, dx, dscale, rows, n, st);
    if (x_dtype == FLUX_F32 && scale_dtype == FLUX_F32) return rms_bwd_launch<float, float>(dy, x, scale, rstd, dx, dscale, rows, n, st);
    return fail(FLUX_E_DTYPE, "flux_rms_norm_bwd: unsupported dtype pair (%d,%d)", x_dtype, scale_dtype);
}

extern "C" int flux_layer_norm_modulation(const void* x, const void* scale, const void* shift, void* y, int64_t batch,
                                          int64_t seq, int32_t n, int64_t mod_batch_stride, int32_t dtype, float eps,
                                          void* stream) {
    if (!x || !scale || !shift || !y) return fail(FLUX_E_NULL, "flux_layer_norm_modulation: null pointer");
    if (batch < 0 || seq < 0 || n <= 0) return fail(FLUX_E_SHAPE, "flux_layer_norm_modulation: bad shape [%lld,%lld,%d]", (long long)batch, (long long)seq, n);
    if (n > FLUX_MAX_ROW) return fail(FLUX_E_TOO_WIDE, "flux_layer_norm_modulation: n = %d exceeds the maximum row length %d", n, FLUX_MAX_ROW);
    if (batch * seq == 0) return FLUX_OK;
    if (batch * seq > 0x7fffffffLL) return fail(FLUX_E_SHAPE, "flux_layer_norm_modulation: too many rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == FLUX_BF16) return ln_mod_launch<bf16_t>(x, scale, shift, y, batch, seq, n, mod_batch_stride, eps, st);
    if (dtype == FLUX_F32) return ln_mod_launch<float>(x, scale, shift, y, batch, seq, n, mod_batch_stride, eps, st);
    return fail(FLUX_E_DTYPE, "flux_layer_norm_modulation: unsupported dtype %d", dtype);
}
