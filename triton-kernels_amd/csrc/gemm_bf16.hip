// Linear layer on the matrix cores:  Y = epilogue(A[M,K] * W[N,K]^T), bf16 operands, fp32 accumulate.
//
// Both operands are K-contiguous, which is exactly what v_mfma_f32_32x32x16_bf16 wants: every lane
// feeds 8 consecutive k of one row. A workgroup of four waves (2 x 2) owns a (64*MI) x (64*NJ) tile
// of Y and each wave a (32*MI) x (32*NJ) sub-tile kept as MI*NJ accumulators of 32x32. The K loop
// moves 64-wide slabs of A and W through a two-stage LDS ring: while the MFMAs consume stage s, the
// slab for the next step lands in stage s^1, either straight from the buffer load (DIRECT) or via
// registers.
//
// LDS slab layout: row r of the slab is 128 bytes = eight 16-byte chunks; chunk c is stored at
// position c ^ (r & 7). Eight lanes that read the same logical chunk of eight consecutive rows then
// touch eight different positions, i.e. all 32 banks once: conflict-free ds_read_b128; the writer
// side stores whole rows, also conflict-free.
//
// The MFMA takes W as its "A" operand and the activations as its "B" operand, so the accumulator
// of a lane holds one activation row m and runs of 4 consecutive output columns n: bias and GELU
// are applied there in fp32 and the result is rounded once, the bf16 tile goes through LDS once more and leaves as full 16-byte
// row segments, where the optional gated residual is applied.
#include "common.h"
#include <stdlib.h>

namespace flux {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct GemmParams {
    const bf16_t* A; const bf16_t* W; const bf16_t* bias;
    bf16_t* Y; bf16_t* Y2;
    const bf16_t* resid; const bf16_t* gate;
    int M, N, K;
    int64_t lda, ldw, ldy, ldy2, ldresid, gate_stride;
    int split_n, y2_col0, rows_per_batch;
    int act, act_begin;
    int tiles_m, tiles_n, group_m;
    int vec_io;  // 1: every output/residual row segment of 8 columns may be accessed as 16 bytes
};

constexpr int kGemmThreads = 256;
constexpr unsigned kRsrcFlags = 0x00020000u;  // raw buffer, 32-bit data format
// A byte offset no buffer of ours reaches (record counts stay below 2^31, and so does k*2 added to
// it): the buffer load returns zeros for it, which is how rows past M/N and the K tail are padded.
constexpr uint32_t kOutOfRange = 0x80000000u;

// LDS-direct buffer loads are counted by vmcnt; the workgroup barrier alone does not wait for them.
__device__ __forceinline__ void wait_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ u32x2 pack4_bf16(float a, float b, float c, float d) {
    u32x2 r;
    r.x = static_cast<uint32_t>(f2bf(a)) | (static_cast<uint32_t>(f2bf(b)) << 16);
    r.y = static_cast<uint32_t>(f2bf(c)) | (static_cast<uint32_t>(f2bf(d)) << 16);
    return r;
}

// XCD-aware tile order. Workgroups are handed to the 8 XCDs round-robin, so workgroup w runs on
// XCD w % 8; giving each XCD one contiguous range of the (grouped) tile sequence makes the ~32 tiles
// resident on an XCD at any time a compact group_m x (32/group_m) patch that shares A and W panels
// in that XCD's L2.
__device__ __forceinline__ bool tile_of_block(const GemmParams& p, int& tm, int& tn) {
    const int total = p.tiles_m * p.tiles_n;
    const int per_xcd = gridDim.x / 8;
    const int t = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (t >= total) return false;
    const int width = p.group_m * p.tiles_n;
    const int group = t / width;
    const int first_m = group * p.group_m;
    const int gsz = min(p.tiles_m - first_m, p.group_m);
    const int in_group = t % width;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
    return true;
}

template <int MI, int NJ, bool DIRECT>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_kernel(GemmParams p) {
    constexpr int BM = 64 * MI, BN = 64 * NJ, BK = 64;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
    constexpr int PA = BM / 32, PB = BN / 32;  // 32-row passes of the 256-thread loader
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    constexpr int C_PITCH = WCOLS * 2, C_CH = WCOLS / 8;  // epilogue tile: bytes per row, 16-byte chunks per row
    static_assert(4 * WROWS * C_PITCH <= 2 * STAGE, "epilogue tile must fit the ring");
    __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE];

    int tm, tn;
    if (!tile_of_block(p, tm, tn)) return;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- loader mapping: thread -> LDS slot (row = pass*32 + tid/8, position tid%8), which holds
    //      logical chunk (tid%8) ^ (row&7) of that row.
    const int lrow = tid >> 3;
    const int lchunk = (tid & 7) ^ (lrow & 7);
    const int rows_a = min(p.M - m0, BM), rows_b = min(p.N - n0, BN);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(p.A + static_cast<int64_t>(m0) * p.lda), 0,
        static_cast<int>(((rows_a - 1) * p.lda + p.K) * 2), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(p.W + static_cast<int64_t>(n0) * p.ldw), 0,
        static_cast<int>(((rows_b - 1) * p.ldw + p.K) * 2), kRsrcFlags);
    uint32_t voff_a[PA], voff_b[PB];
#pragma unroll
    for (int i = 0; i < PA; ++i) {
        const int r = i * 32 + lrow;
        voff_a[i] = r < rows_a ? static_cast<uint32_t>((r * p.lda + lchunk * 8) * 2) : kOutOfRange;
    }
#pragma unroll
    for (int i = 0; i < PB; ++i) {
        const int r = i * 32 + lrow;
        voff_b[i] = r < rows_b ? static_cast<uint32_t>((r * p.ldw + lchunk * 8) * 2) : kOutOfRange;
    }
    const int lds_slot = lrow * 128 + (tid & 7) * 16;  // within a 32-row pass

    u32x4 stage_a[DIRECT ? 1 : PA], stage_b[DIRECT ? 1 : PB];

    auto issue_loads = [&](int kt, int stage) {
        const int k0 = kt * BK;
        const bool kin = k0 + lchunk * 8 < p.K;  // K is a multiple of 8: a chunk is all in or all out
        const uint32_t kb = static_cast<uint32_t>(k0 * 2);
        char* sa = lds + stage * STAGE;
        char* sb = sa + A_BYTES;
#pragma unroll
        for (int i = 0; i < PA; ++i) {
            const uint32_t vo = kin ? voff_a[i] + kb : kOutOfRange;
            if constexpr (DIRECT) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    rsrc_a, (__attribute__((address_space(3))) void*)(sa + i * 4096 + wave * 1024), 16, vo, 0, 0, 0);
            } else {
                stage_a[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, vo, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < PB; ++i) {
            const uint32_t vo = kin ? voff_b[i] + kb : kOutOfRange;
            if constexpr (DIRECT) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    rsrc_b, (__attribute__((address_space(3))) void*)(sb + i * 4096 + wave * 1024), 16, vo, 0, 0, 0);
            } else {
                stage_b[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo, 0, 0);
            }
        }
    };
    auto commit_loads = [&](int stage) {  // register path only
        if constexpr (!DIRECT) {
            char* sa = lds + stage * STAGE;
            char* sb = sa + A_BYTES;
#pragma unroll
            for (int i = 0; i < PA; ++i) *reinterpret_cast<u32x4*>(sa + i * 4096 + lds_slot) = stage_a[i];
#pragma unroll
            for (int i = 0; i < PB; ++i) *reinterpret_cast<u32x4*>(sb + i * 4096 + lds_slot) = stage_b[i];
        }
    };

    // ---- fragment addressing
    const int frow = lane & 31, fhalf = lane >> 5;
    int koff[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) koff[kk] = ((kk * 2 + fhalf) ^ (lane & 7)) * 16;
    const int a_off = (wm * WROWS + frow) * 128;
    const int b_off = A_BYTES + (wn * WCOLS + frow) * 128;

    f32x16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int nk = (p.K + BK - 1) / BK;
    issue_loads(0, 0);
    commit_loads(0);
    if constexpr (DIRECT) wait_vmem();
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) issue_loads(kt + 1, cur ^ 1);
        const char* s = lds + cur * STAGE;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            bf16x8 xa[MI], wb[NJ];
#pragma unroll
            for (int i = 0; i < MI; ++i) xa[i] = *reinterpret_cast<const bf16x8*>(s + a_off + i * 4096 + koff[kk]);
#pragma unroll
            for (int j = 0; j < NJ; ++j) wb[j] = *reinterpret_cast<const bf16x8*>(s + b_off + j * 4096 + koff[kk]);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[j], xa[i], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) commit_loads(cur ^ 1);
        if constexpr (DIRECT) wait_vmem();
        __syncthreads();
    }

    // ---- epilogue phase 1: bias, rounding, GELU in accumulator layout -> bf16 tile in LDS (per wave)
    char* cw = lds + wave * (WROWS * C_PITCH);
    const int wave_n0 = n0 + wn * WCOLS;
    const int wave_m0 = m0 + wm * WROWS;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int nl = j * 32 + g * 8 + fhalf * 4;  // first of 4 consecutive columns, wave-local
            const int n = wave_n0 + nl;
            float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (p.bias != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < p.N) bv[e] = bf2f(p.bias[n + e]);
            }
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t = acc[i][j][g * 4 + e] + bv[e];
                    if (p.act == FLUX_ACT_GELU_TANH && n + e >= p.act_begin) t = gelu_tanh_f32(t);
                    v[e] = t;
                }
                const int row = i * 32 + frow;
                const int slot = (nl >> 3) ^ (row & (C_CH - 1));
                *reinterpret_cast<u32x2*>(cw + row * C_PITCH + slot * 16 + fhalf * 8) = pack4_bf16(v[0], v[1], v[2], v[3]);
            }
        }
    }
    // The tile region is private to the wave (LDS operations of one wave complete in order), but
    // the ring it overlays was shared: the barrier that ended the K loop already ordered every
    // wave's last fragment reads before these writes.
    __builtin_amdgcn_wave_barrier();

    // ---- epilogue phase 2: row-major 16-byte segments, optional gated residual, store
    constexpr int SEGS = WROWS * C_CH;
#pragma unroll 4
    for (int it = 0; it < SEGS / 64; ++it) {
        const int idx = it * 64 + lane;
        const int row = idx / C_CH, ch = idx % C_CH;
        const int m = wave_m0 + row, n = wave_n0 + ch * 8;
        if (m >= p.M || n >= p.N) continue;
        Vec16<bf16_t> y = *reinterpret_cast<const Vec16<bf16_t>*>(cw + row * C_PITCH + ((ch ^ (row & (C_CH - 1))) * 16));
        const bool full = p.vec_io && n + 8 <= p.N;
        if (p.gate != nullptr) {
            const bf16_t* gp = p.gate + static_cast<int64_t>(m / p.rows_per_batch) * p.gate_stride + n;
            const bf16_t* rp = p.resid + static_cast<int64_t>(m) * p.ldresid + n;
            if (full) {
                Vec16<bf16_t> g = ld16(gp), r = ld16(rp);
#pragma unroll
                for (int e = 0; e < 8; ++e) y.v[e] = f2bf(bf2f(r.v[e]) + bf2f(f2bf(bf2f(g.v[e]) * bf2f(y.v[e]))));
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (n + e < p.N) y.v[e] = f2bf(bf2f(rp[e]) + bf2f(f2bf(bf2f(gp[e]) * bf2f(y.v[e]))));
            }
        }
        if (full) {
            bf16_t* dst = n < p.split_n ? p.Y + static_cast<int64_t>(m) * p.ldy + n
                                        : p.Y2 + static_cast<int64_t>(m) * p.ldy2 + (n - p.split_n + p.y2_col0);
            st16(dst, y);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int ne = n + e;
                if (ne < p.N) {
                    bf16_t* dst = ne < p.split_n ? p.Y + static_cast<int64_t>(m) * p.ldy + ne
                                                 : p.Y2 + static_cast<int64_t>(m) * p.ldy2 + (ne - p.split_n + p.y2_col0);
                    *dst = y.v[e];
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Skinny problems (M <= 8, e.g. the Modulation projection of one conditioning vector per batch
// element): HBM-bound on W. One wave per output column streams the W row with 16-byte loads while
// the few activation rows come from cache; the dot products are folded with a wave butterfly.
// ------------------------------------------------------------------------------------------------
template <int MMAX>
__global__ __launch_bounds__(256) void gemv_small_m_kernel(GemmParams p) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= p.N) return;  // whole wave leaves together
    float acc[MMAX];
#pragma unroll
    for (int m = 0; m < MMAX; ++m) acc[m] = 0.0f;
    const bf16_t* wrow = p.W + static_cast<int64_t>(n) * p.ldw;
    for (int k = lane * 8; k < p.K; k += 512) {
        Vec16<bf16_t> w = ld16(wrow + k);
        float wf[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) wf[e] = bf2f(w.v[e]);
#pragma unroll
        for (int m = 0; m < MMAX; ++m) {
            if (m < p.M) {
                Vec16<bf16_t> a = ld16(p.A + static_cast<int64_t>(m) * p.lda + k);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[m] += wf[e] * bf2f(a.v[e]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MMAX; ++m) acc[m] = group_sum<64>(acc[m]);
    if (lane == 0) {
        const float b = p.bias ? bf2f(p.bias[n]) : 0.0f;
        for (int m = 0; m < p.M && m < MMAX; ++m) {
            float t = acc[m] + b;
            if (p.act == FLUX_ACT_GELU_TANH && n >= p.act_begin) t = gelu_tanh_f32(t);
            t = bf2f(f2bf(t));
            if (p.gate != nullptr) {
                const float g = bf2f(p.gate[static_cast<int64_t>(m / p.rows_per_batch) * p.gate_stride + n]);
                const float r = bf2f(p.resid[static_cast<int64_t>(m) * p.ldresid + n]);
                t = r + bf2f(f2bf(g * t));
            }
            bf16_t* dst = n < p.split_n ? p.Y + static_cast<int64_t>(m) * p.ldy + n
                                        : p.Y2 + static_cast<int64_t>(m) * p.ldy2 + (n - p.split_n + p.y2_col0);
            *dst = f2bf(t);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Any-shape kernel for operands the tiled path cannot address with 16-byte loads (K or a leading
// dimension not a multiple of 8, or a misaligned base). One thread per output element.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm_nt_scalar_kernel(GemmParams p) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<int64_t>(p.M) * p.N) return;
    const int m = static_cast<int>(idx / p.N), n = static_cast<int>(idx % p.N);
    const bf16_t* a = p.A + static_cast<int64_t>(m) * p.lda;
    const bf16_t* w = p.W + static_cast<int64_t>(n) * p.ldw;
    float acc = 0.0f;
    for (int k = 0; k < p.K; ++k) acc += bf2f(a[k]) * bf2f(w[k]);
    float t = acc + (p.bias ? bf2f(p.bias[n]) : 0.0f);
    if (p.act == FLUX_ACT_GELU_TANH && n >= p.act_begin) t = gelu_tanh_f32(t);
    t = bf2f(f2bf(t));
    if (p.gate != nullptr) {
        const float g = bf2f(p.gate[static_cast<int64_t>(m / p.rows_per_batch) * p.gate_stride + n]);
        const float r = bf2f(p.resid[static_cast<int64_t>(m) * p.ldresid + n]);
        t = r + bf2f(f2bf(g * t));
    }
    bf16_t* dst = n < p.split_n ? p.Y + static_cast<int64_t>(m) * p.ldy + n
                                : p.Y2 + static_cast<int64_t>(m) * p.ldy2 + (n - p.split_n + p.y2_col0);
    *dst = f2bf(t);
}

template <int MI, int NJ, bool DIRECT>
static void launch_tiled(GemmParams& p, hipStream_t st) {
    constexpr int BM = 64 * MI, BN = 64 * NJ;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    p.group_m = 4;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL((gemm_nt_kernel<MI, NJ, DIRECT>), dim3(grid), dim3(kGemmThreads), 0, st, p);
}

// Selected by FLUX_GEMM_VARIANT for experiments: 0 = automatic.
static int gemm_variant() {
    static int v = [] {
        const char* e = getenv("FLUX_GEMM_VARIANT");
        return e ? atoi(e) : 0;
    }();
    return v;
}

}  // namespace flux

using namespace flux;

extern "C" int flux_linear_bf16(const flux_linear_args* a, void* stream) {
    if (!a) return fail(FLUX_E_NULL, "flux_linear_bf16: null args");
    if (!a->A || !a->W || !a->Y) return fail(FLUX_E_NULL, "flux_linear_bf16: null operand");
    if (a->M < 0 || a->N < 0 || a->K < 0) return fail(FLUX_E_SHAPE, "flux_linear_bf16: negative size");
    if (a->M > 0x7fffffff || a->N > 0x7fffffff || a->K > 0x7fffffff) return fail(FLUX_E_SHAPE, "flux_linear_bf16: size exceeds 2^31");
    if (a->M == 0 || a->N == 0) return FLUX_OK;
    if (a->lda < a->K || a->ldw < a->K) return fail(FLUX_E_SHAPE, "flux_linear_bf16: leading dimension smaller than K");
    if (a->act != FLUX_ACT_NONE && a->act != FLUX_ACT_GELU_TANH) return fail(FLUX_E_UNSUPPORTED, "flux_linear_bf16: unknown activation %d", a->act);
    const bool split = a->Y2 != nullptr && a->split_n < a->N;
    if (split && (a->split_n < 0 || a->y2_col0 < 0)) return fail(FLUX_E_SHAPE, "flux_linear_bf16: bad split");
    if ((a->gate == nullptr) != (a->resid == nullptr)) return fail(FLUX_E_NULL, "flux_linear_bf16: gate and resid go together");
    if (a->gate && a->rows_per_batch <= 0) return fail(FLUX_E_SHAPE, "flux_linear_bf16: rows_per_batch must be positive with a gate");

    GemmParams p;
    p.A = static_cast<const bf16_t*>(a->A); p.W = static_cast<const bf16_t*>(a->W); p.bias = static_cast<const bf16_t*>(a->bias);
    p.Y = static_cast<bf16_t*>(a->Y); p.Y2 = split ? static_cast<bf16_t*>(a->Y2) : nullptr;
    p.resid = static_cast<const bf16_t*>(a->resid); p.gate = static_cast<const bf16_t*>(a->gate);
    p.M = (int)a->M; p.N = (int)a->N; p.K = (int)a->K;
    p.lda = a->lda; p.ldw = a->ldw; p.ldy = a->ldy; p.ldy2 = a->ldy2; p.ldresid = a->ldresid;
    p.gate_stride = a->gate_batch_stride;
    p.split_n = split ? (int)a->split_n : p.N;
    p.y2_col0 = split ? (int)a->y2_col0 : 0;
    p.rows_per_batch = a->gate ? (int)a->rows_per_batch : 1;
    p.act = a->act; p.act_begin = (int)(a->act_begin < 0 ? 0 : (a->act_begin > a->N ? a->N : a->act_begin));
    p.tiles_m = p.tiles_n = 0; p.group_m = 4;
    p.vec_io = aligned16(a->Y) && a->ldy % 8 == 0 &&
               (!split || (aligned16(a->Y2) && a->ldy2 % 8 == 0 && a->split_n % 8 == 0 && a->y2_col0 % 8 == 0)) &&
               (!a->gate || (aligned16(a->gate) && aligned16(a->resid) && a->ldresid % 8 == 0 && a->gate_batch_stride % 8 == 0));

    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p.K == 0) {
        // Degenerate contraction: the scalar kernel's empty K loop leaves bias/epilogue only.
        hipLaunchKernelGGL(gemm_nt_scalar_kernel, dim3((unsigned)(((int64_t)p.M * p.N + 255) / 256)), dim3(256), 0, st, p);
        return check_launch("flux_linear_bf16");
    }
    const bool vec_in = aligned16(a->A) && aligned16(a->W) && a->K % 8 == 0 && a->lda % 8 == 0 && a->ldw % 8 == 0;
    // 32-bit byte offsets inside one tile's rows
    const bool off_ok = a->lda * 2 * 256 < 0x7fffffffLL && a->ldw * 2 * 256 < 0x7fffffffLL;
    if (!vec_in || !off_ok) {
        hipLaunchKernelGGL(gemm_nt_scalar_kernel, dim3((unsigned)(((int64_t)p.M * p.N + 255) / 256)), dim3(256), 0, st, p);
        return check_launch("flux_linear_bf16");
    }
    if (p.M <= 8) {
        hipLaunchKernelGGL((gemv_small_m_kernel<8>), dim3((unsigned)((p.N + 3) / 4)), dim3(256), 0, st, p);
        return check_launch("flux_linear_bf16");
    }
    const int variant = gemm_variant();
    const int64_t big_tiles = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256);
    if (variant == 1) launch_tiled<4, 4, false>(p, st);
    else if (variant == 2) launch_tiled<4, 4, true>(p, st);
    else if (variant == 3) launch_tiled<2, 2, false>(p, st);
    else if (variant == 4) launch_tiled<2, 2, true>(p, st);
    else if (big_tiles >= 192) launch_tiled<4, 4, false>(p, st);
    else launch_tiled<2, 2, false>(p, st);
    return check_launch("flux_linear_bf16");
}
