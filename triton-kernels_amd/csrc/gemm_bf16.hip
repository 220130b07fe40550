// Linear layer on the matrix cores:  Y = epilogue(A[M,K] * W[N,K]^T), bf16 operands, fp32 accumulate.
//
// Both operands are K-contiguous, which is exactly what v_mfma_f32_32x32x16_bf16 wants: every lane
// feeds 8 consecutive k of one row. A workgroup of four waves (2 x 2) owns a (64*MI) x (64*NJ) tile
// of Y and each wave a (32*MI) x (32*NJ) sub-tile kept as MI*NJ accumulators of 32x32. The K loop
// moves 64-wide slabs of A and W through a two-stage LDS ring: while the MFMAs consume stage s, the
// slab for the next step lands in stage s^1 straight from buffer loads that write LDS (no register
// staging).
//
// LDS slab layout: row r of the slab is 128 bytes = eight 16-byte chunks; chunk c is stored at
// position c ^ ((r >> 1) & 7). LDS on gfx950 has 64 banks of 4 bytes, so a ds_read_b128 is served 16
// lanes (256 bytes) per clock: the 16 lanes that read the same logical chunk of 16 consecutive rows
// land on 2 (row parity) x 8 (position) = 16 different 16-byte bank groups, conflict-free. The
// writer side fills whole rows, also conflict-free.
//
// The MFMA takes W as its "A" operand and the activations as its "B" operand, so the accumulator
// of a lane holds one activation row m and runs of 4 consecutive output columns n: bias and GELU
// are applied there in fp32 and the result is rounded once, the bf16 tile goes through LDS once more and leaves as full 16-byte
// row segments, where the optional gated residual is applied.
#include "common.h"
#include <stdlib.h>
#include <type_traits>

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
    int bias_vec;  // 1: bias may be read with 8-byte buffer loads (4-byte aligned base)
    int vec_io;  // 1: every output/residual row segment of 8 columns may be accessed as 16 bytes
};

constexpr int kGemmThreads = 256;
constexpr unsigned kRsrcFlags = 0x00020000u;  // raw buffer, 32-bit data format
// A byte offset no buffer of ours reaches (record counts stay below 2^31, and so does k*2 added to
// it): the buffer load returns zeros for it, which is how rows past M/N and the K tail are padded.
constexpr uint32_t kOutOfRange = 0x80000000u;

// LDS-direct buffer loads are counted by vmcnt; the workgroup barrier alone does not wait for them.

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
// Two floats -> one dword of two bf16 (a in the low half): a single v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ u32x2 pack4_bf16(float a, float b, float c, float d) {
    u32x2 r;
    r.x = pack2_bf16(a, b);
    r.y = pack2_bf16(c, d);
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

// One buffer load of 64 x 16 bytes, written by the memory pipeline straight into LDS at dst
// (+ lane * 16, implied by the instruction). `soff` is the scalar byte offset of the slab inside the
// rows; a vector offset with the top bit set is out of range for the resource and yields zeros.
__device__ __forceinline__ void load_chunk(__amdgpu_buffer_rsrc_t rsrc, char* dst, uint32_t voff, int soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, voff, soff, 0, 0);
}

__device__ __forceinline__ u32x4 load_chunk_reg(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, int soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0);
}

__device__ __forceinline__ void wait_vmem_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Which of a slab's LPS buffer loads goes into issue slot g of SLOTS (-1 = none): spread evenly, so
// the texture-address unit (64 bytes per clock per CU) is never asked for more than it can take and
// the in-order wave does not stall MFMA issue behind a full memory queue.
constexpr int load_at_slot(int g, int slots, int lps) {
    for (int l = 0; l < lps; ++l)
        if (l * slots / lps == g) return l;
    return -1;
}

// Epilogue shared by the tiled kernels. A lane's accumulators hold one activation row and runs of
// 4 consecutive output columns. Per 32-row block: bias and GELU in fp32, one rounding to bf16, the
// block is parked in LDS (a private region per wave, overlaying the ring, which the caller's final
// barrier has retired) and leaves as 16-byte row segments, where the optional gated residual is
// applied. Interior tiles with 16-byte addressable outputs take a branch-free path; edge tiles and
// unaligned outputs take the checked path.
__device__ __forceinline__ float tanh_gelu_fast(float x) {
    // x * sigmoid(2u), u = sqrt(2/pi) (x + 0.044715 x^3), with log2(e) folded into the constants
    const float x2 = x * x;
    const float t = __builtin_fmaf(x2, -0.10294324f, -2.3022082f);
    const float e = __builtin_amdgcn_exp2f(x * t);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

template <int MI, int NJ>
__device__ __forceinline__ void gemm_epilogue_checked(const GemmParams& p, f32x16 (&acc)[MI][NJ], char* lds, int m0, int n0,
                                                   int wave, int lane) {
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    constexpr int C_PITCH = WCOLS * 2, C_CH = WCOLS / 8;  // bytes per row, 16-byte chunks per row
    constexpr int RPI = 64 / C_CH;                         // rows one wave-wide 16-byte access covers
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 31, fhalf = lane >> 5;
    char* cw = lds + wave * (WROWS * C_PITCH);
    const int wave_n0 = n0 + wn * WCOLS;
    const int wave_m0 = m0 + wm * WROWS;

    // bias for the lane's 4*NJ column quads
    float bv[NJ][4][4];
    const bool bias_fast = p.bias != nullptr && p.bias_vec;
    if (bias_fast) {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.bias), 0, p.N * 2, kRsrcFlags);
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x2 raw = __builtin_amdgcn_raw_buffer_load_b64(rb, (wave_n0 + j * 32 + g * 8 + fhalf * 4) * 2, 0, 0);
                bv[j][g][0] = __uint_as_float(raw.x << 16);
                bv[j][g][1] = __uint_as_float(raw.x & 0xffff0000u);
                bv[j][g][2] = __uint_as_float(raw.y << 16);
                bv[j][g][3] = __uint_as_float(raw.y & 0xffff0000u);
            }
    } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int n = wave_n0 + j * 32 + g * 8 + fhalf * 4 + e;
                    bv[j][g][e] = (p.bias != nullptr && n < p.N) ? bf2f(p.bias[n]) : 0.0f;
                }
    }

    // LDS write address of column quad (j, g) in this lane's row, without the 32-row block offset
    int waddr[NJ * 4];
#pragma unroll
    for (int c = 0; c < NJ * 4; ++c) waddr[c] = frow * C_PITCH + ((c ^ (frow & (C_CH - 1))) * 16) + fhalf * 8;
    // read side: lane -> (row within the pass = lane / C_CH, chunk = lane % C_CH)
    const int rrow = lane / C_CH, rch = lane % C_CH;

    const bool gelu_all = p.act == FLUX_ACT_GELU_TANH && wave_n0 >= p.act_begin;
    const bool gelu_some = p.act == FLUX_ACT_GELU_TANH && !gelu_all && wave_n0 + WCOLS > p.act_begin;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        // ---- accumulators of block row i -> bf16 -> LDS
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e] + bv[j][g][e];
                if (gelu_all) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = tanh_gelu_fast(v[e]);
                } else if (gelu_some) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (wave_n0 + j * 32 + g * 8 + fhalf * 4 + e >= p.act_begin) v[e] = tanh_gelu_fast(v[e]);
                }
                *reinterpret_cast<u32x2*>(cw + i * 32 * C_PITCH + waddr[j * 4 + g]) = pack4_bf16(v[0], v[1], v[2], v[3]);
            }
        __builtin_amdgcn_wave_barrier();  // LDS operations of one wave complete in order

        // ---- the 32 rows leave as 16-byte segments
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
            const int row = i * 32 + it * RPI + rrow;
            const int m = wave_m0 + row, n = wave_n0 + rch * 8;
            Vec16<bf16_t> y = *reinterpret_cast<const Vec16<bf16_t>*>(cw + row * C_PITCH + ((rch ^ (row & (C_CH - 1))) * 16));
            if (m >= p.M || n >= p.N) continue;
            const bool full = p.vec_io && n + 8 <= p.N;
            if (p.gate != nullptr) {
                const bf16_t* gp = p.gate + static_cast<int64_t>(m / p.rows_per_batch) * p.gate_stride + n;
                const bf16_t* rp = p.resid + static_cast<int64_t>(m) * p.ldresid + n;
                if (full) {
                    Vec16<bf16_t> gt = ld16(gp), rs = ld16(rp);
#pragma unroll
                    for (int e = 0; e < 8; ++e) y.v[e] = f2bf(bf2f(rs.v[e]) + bf2f(f2bf(bf2f(gt.v[e]) * bf2f(y.v[e]))));
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (n + e < p.N) y.v[e] = f2bf(bf2f(rp[e]) + bf2f(f2bf(bf2f(gp[e]) * bf2f(y.v[e]))));
                }
            }
            if (full && (n + 8 <= p.split_n || n >= p.split_n)) {
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
}

// Branch-free epilogue for interior tiles whose outputs (and residual operands) are 16-byte
// addressable and whose columns all go to one destination. GELU is all-or-nothing for the wave.
// Everything lane-dependent is computed once; per store only a wave-uniform row offset changes, so
// the stores use a scalar base plus a 32-bit lane offset.
template <int MI, int NJ, bool GELU, bool GATE>
__device__ __forceinline__ void gemm_epilogue_fast(const GemmParams& p, f32x16 (&acc)[MI][NJ], char* lds, int m0, int n0,
                                                   int wave, int lane) {
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    constexpr int C_PITCH = WCOLS * 2, C_CH = WCOLS / 8;
    constexpr int RPI = 64 / C_CH;      // rows per wave-wide 16-byte access
    constexpr int NIT = 32 / RPI;       // accesses per 32-row block
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 31, fhalf = lane >> 5;
    char* cw = lds + wave * (WROWS * C_PITCH);
    const int wave_n0 = n0 + wn * WCOLS;
    const int wave_m0 = m0 + wm * WROWS;

    float bv[NJ][4][4];
    if (p.bias != nullptr) {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.bias), 0, p.N * 2, kRsrcFlags);
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x2 raw = __builtin_amdgcn_raw_buffer_load_b64(rb, (wave_n0 + j * 32 + g * 8 + fhalf * 4) * 2, 0, 0);
                bv[j][g][0] = __uint_as_float(raw.x << 16);
                bv[j][g][1] = __uint_as_float(raw.x & 0xffff0000u);
                bv[j][g][2] = __uint_as_float(raw.y << 16);
                bv[j][g][3] = __uint_as_float(raw.y & 0xffff0000u);
            }
    } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) bv[j][g][e] = 0.0f;
    }

    int waddr[NJ * 4];
#pragma unroll
    for (int c = 0; c < NJ * 4; ++c) waddr[c] = frow * C_PITCH + ((c ^ (frow & (C_CH - 1))) * 16) + fhalf * 8;
    const int rrow = lane / C_CH, rch = lane % C_CH;
    // read address for access `it` of a block: row = it*RPI + rrow; the swizzle term repeats every 16 rows
    constexpr int NSW = (16 / RPI) < NIT ? (16 / RPI) : NIT;
    int raddr[NSW];
#pragma unroll
    for (int t = 0; t < NSW; ++t) {
        const int row = t * RPI + rrow;
        raddr[t] = row * C_PITCH + ((rch ^ (row & (C_CH - 1))) * 16);
    }

    const bool to_y = wave_n0 < p.split_n;
    char* dst_u = reinterpret_cast<char*>(to_y ? p.Y + wave_n0 : p.Y2 + (wave_n0 - p.split_n + p.y2_col0));
    const int64_t dst_ld = (to_y ? p.ldy : p.ldy2) * 2;            // bytes
    const uint32_t dst_lane = static_cast<uint32_t>(rrow * dst_ld + rch * 16);
    const char* res_u = nullptr;
    const char* gate_u = nullptr;
    uint32_t res_lane = 0;
    if (GATE) {
        res_u = reinterpret_cast<const char*>(p.resid + wave_n0);
        res_lane = static_cast<uint32_t>(rrow * p.ldresid * 2 + rch * 16);
        gate_u = reinterpret_cast<const char*>(p.gate + wave_n0 + rch * 8);
    }

#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = acc[i][j][g * 4 + e] + bv[j][g][e];
                    if (GELU) v[e] = tanh_gelu_fast(v[e]);
                }
                *reinterpret_cast<u32x2*>(cw + i * 32 * C_PITCH + waddr[j * 4 + g]) = pack4_bf16(v[0], v[1], v[2], v[3]);
            }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int row_u = i * 32 + it * RPI;                 // wave-uniform part of the row
            Vec16<bf16_t> y = *reinterpret_cast<const Vec16<bf16_t>*>(cw + (i * 32 + (it / NSW) * NSW * RPI) * C_PITCH + raddr[it % NSW]);
            const int64_t m_u = wave_m0 + row_u;
            if (GATE) {
                // all rows of one access belong to one batch element when rows_per_batch is a multiple of RPI
                const Vec16<bf16_t> gt = ld16(reinterpret_cast<const bf16_t*>(gate_u) + ((m_u + rrow) / p.rows_per_batch) * p.gate_stride);
                const Vec16<bf16_t> rs = *reinterpret_cast<const Vec16<bf16_t>*>(res_u + m_u * p.ldresid * 2 + res_lane);
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float y0 = bf2f(rs.v[e]) + bf2f(f2bf(bf2f(gt.v[e]) * bf2f(y.v[e])));
                    const float y1 = bf2f(rs.v[e + 1]) + bf2f(f2bf(bf2f(gt.v[e + 1]) * bf2f(y.v[e + 1])));
                    const uint32_t w = pack2_bf16(y0, y1);
                    y.v[e] = static_cast<bf16_t>(w & 0xffffu);
                    y.v[e + 1] = static_cast<bf16_t>(w >> 16);
                }
            }
            *reinterpret_cast<Vec16<bf16_t>*>(dst_u + m_u * dst_ld + dst_lane) = y;
        }
    }
}

template <int MI, int NJ>
__device__ __forceinline__ void gemm_epilogue(const GemmParams& p, f32x16 (&acc)[MI][NJ], char* lds, int m0, int n0,
                                              int wave, int lane) {
    constexpr int BM = 64 * MI, BN = 64 * NJ, WCOLS = 32 * NJ;
    const int wave_n0 = n0 + (wave & 1) * WCOLS;
    const bool gelu_all = p.act == FLUX_ACT_GELU_TANH && wave_n0 >= p.act_begin;
    const bool gelu_none = p.act != FLUX_ACT_GELU_TANH || wave_n0 + WCOLS <= p.act_begin;
    const bool fast = p.vec_io && m0 + BM <= p.M && n0 + BN <= p.N && (gelu_all || gelu_none) &&
                      (wave_n0 + WCOLS <= p.split_n || wave_n0 >= p.split_n) && (p.bias == nullptr || p.bias_vec) &&
                      static_cast<int64_t>(BM) * p.ldy * 2 < 0x7fffffffLL && static_cast<int64_t>(BM) * p.ldy2 * 2 < 0x7fffffffLL;
    if (fast) {
        if (p.gate != nullptr) {
            if (gelu_all) gemm_epilogue_fast<MI, NJ, true, true>(p, acc, lds, m0, n0, wave, lane);
            else gemm_epilogue_fast<MI, NJ, false, true>(p, acc, lds, m0, n0, wave, lane);
        } else {
            if (gelu_all) gemm_epilogue_fast<MI, NJ, true, false>(p, acc, lds, m0, n0, wave, lane);
            else gemm_epilogue_fast<MI, NJ, false, false>(p, acc, lds, m0, n0, wave, lane);
        }
    } else {
        gemm_epilogue_checked<MI, NJ>(p, acc, lds, m0, n0, wave, lane);
    }
}

template <int MI, int NJ, bool STAGED>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_kernel(GemmParams p) {
    constexpr int BM = 64 * MI, BN = 64 * NJ, BK = 64, NS = 2;
    constexpr int ROWB = BK * 2;                 // bytes per slab row
    constexpr int KSUB = BK / 16;                // MFMA K-steps per slab (4)
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int PA = BM / 32, PB = BN / 32;    // loader passes per slab (32 rows = 4096 bytes each)
    constexpr int LPS = PA + PB;                 // buffer loads per thread per slab
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    constexpr int C_PITCH = WCOLS * 2, C_CH = WCOLS / 8;  // epilogue tile: bytes per row, 16-byte chunks per row
    static_assert(4 * WROWS * C_PITCH <= NS * STAGE, "epilogue tile must fit the ring");
    __shared__ __attribute__((aligned(1024))) char lds[NS * STAGE];

    int tm, tn;
    if (!tile_of_block(p, tm, tn)) return;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps LDS bases in SGPRs
    const int wm = wave >> 1, wn = wave & 1;

    // ---- loader mapping: a wave's buffer load drops 64 x 16 bytes into 1 KB of consecutive LDS,
    //      i.e. thread -> LDS slot (row = pass*32 + tid/8, position tid%8), so the thread fetches
    //      logical chunk position ^ ((row>>1)&7) of that row from memory.
    const int lrow = tid >> 3;
    const int lchunk = (tid & 7) ^ ((lrow >> 1) & 7);
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

    const int nk = (p.K + BK - 1) / BK;
    const bool k_ragged = (p.K % BK) != 0;
    // The part of a slab past K is padded with zeros (K is a multiple of 8, so a 16-byte chunk is all
    // in or all out).
    auto slab_kmask = [&](int kt) -> uint32_t {
        return (k_ragged && kt * BK + lchunk * 8 >= p.K) ? kOutOfRange : 0u;
    };
    // Register-staged path: slab data waits in registers (one 16-byte chunk per load) until its ring
    // stage is free, which takes the memory pipeline off the critical path: a load issued in slot g
    // is not needed before slot g of the next slab.
    u32x4 sreg[STAGED ? LPS : 1];
    const int lds_slot = lrow * 128 + (tid & 7) * 16;  // within a 32-row pass
    auto stage_load = [&](int kt, int idx) {   // global -> sreg[idx]; slabs past the end read as zeros
        const uint32_t kmask = (kt >= nk || (k_ragged && kt * BK + lchunk * 8 >= p.K)) ? kOutOfRange : 0u;
        if (idx < PA) sreg[idx] = load_chunk_reg(rsrc_a, voff_a[idx] | kmask, kt * (BK * 2));
        else sreg[idx] = load_chunk_reg(rsrc_b, voff_b[idx - PA] | kmask, kt * (BK * 2));
    };
    auto stage_store = [&](int kt, int idx) {  // sreg[idx] -> ring stage of slab kt
        char* sa = lds + (kt & 1) * STAGE + lds_slot;
        if (idx < PA) *reinterpret_cast<u32x4*>(sa + idx * 4096) = sreg[idx];
        else *reinterpret_cast<u32x4*>(sa + A_BYTES + (idx - PA) * 4096) = sreg[idx];
    };
    // idx-th of the LPS buffer loads of slab kt: first the PA passes of A, then the PB passes of W
    auto issue_load = [&](int kt, uint32_t kmask, int idx) {
        char* sa = lds + (kt & 1) * STAGE + wave * 1024;
        if (idx < PA) load_chunk(rsrc_a, sa + idx * 4096, voff_a[idx] | kmask, kt * (BK * 2));
        else load_chunk(rsrc_b, sa + A_BYTES + (idx - PA) * 4096, voff_b[idx - PA] | kmask, kt * (BK * 2));
    };

    // ---- fragment addressing
    const int frow = lane & 31, fhalf = lane >> 5;
    int koff[KSUB];
#pragma unroll
    for (int kk = 0; kk < KSUB; ++kk) koff[kk] = ((kk * 2 + fhalf) ^ ((frow >> 1) & 7)) * 16;
    const int a_off = (wm * WROWS + frow) * ROWB;
    const int b_off = A_BYTES + (wn * WCOLS + frow) * ROWB;

    f32x16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    bf16x8 xa[2][MI], wb[2][NJ];  // two fragment sets: one feeds the MFMAs while the other is being read
    auto read_frag = [&](int buf, const char* s, int kk, int r) {
        // r-th fragment read of a step, in the order the MFMAs (activation block outer, weight
        // block inner) first need them: x0, w0..w(NJ-1), x1..x(MI-1)
        if (r == 0) xa[buf][0] = *reinterpret_cast<const bf16x8*>(s + a_off + koff[kk]);
        else if (r <= NJ) wb[buf][r - 1] = *reinterpret_cast<const bf16x8*>(s + b_off + (r - 1) * 32 * ROWB + koff[kk]);
        else xa[buf][r - NJ] = *reinterpret_cast<const bf16x8*>(s + a_off + (r - NJ) * 32 * ROWB + koff[kk]);
    };
    auto mfma_one = [&](int buf, int idx) {
        const int i = idx / NJ, j = idx % NJ;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[buf][j], xa[buf][i], acc[i][j], 0, 0, 0);
    };
    constexpr int READS = MI + NJ, MFMAS = MI * NJ, PER = MFMAS / READS;
    static_assert(MFMAS % READS == 0, "MFMAs per fragment read");
    // A slab's loads are issued over three K=16 steps: the step after the barrier that freed the
    // stage (step 3 of the previous slab) and steps 0 and 1; step 2 stays free so that the loads have
    // a few hundred cycles to land before the wait in front of the next barrier.
    constexpr int SLOTS = 3 * READS;
    // One K=16 step in a fixed interleave: every fragment read of the NEXT step is followed by PER
    // MFMAs of the current one, so by the time a fragment is needed it was requested a whole step
    // (>= 256 cycles) earlier; buffer loads of slab `load_kt` are dropped into their issue slots
    // [slot0, slot0 + READS). The scheduling barriers pin this order; the compiler only adds the
    // wait counts.
    auto step = [&](int cur_buf, const char* nxt, int nxt_kk, auto has_next, auto slot0, int load_kt, uint32_t load_kmask) {
#pragma unroll
        for (int r = 0; r < READS; ++r) {
            if constexpr (decltype(has_next)::value) read_frag(cur_buf ^ 1, nxt, nxt_kk, r);
            constexpr int S0 = decltype(slot0)::value;
            if constexpr (S0 >= 0 && !STAGED) {
                const int l = load_at_slot(S0 + r, SLOTS, LPS);
                if (l >= 0) issue_load(load_kt, load_kmask, l);
            }
            if constexpr (S0 >= 0 && STAGED) {
                // load_kt = the slab whose chunk goes from registers to LDS in this slot; the freed
                // register is refilled with the same chunk of the slab after it
                const int l = load_at_slot(S0 + r, 4 * READS, LPS);
                if (l >= 0) {
                    stage_store(load_kt, l);
                    stage_load(load_kt + 1, l);
                }
            }
#pragma unroll
            for (int m = 0; m < PER; ++m) mfma_one(cur_buf, r * PER + m);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    using no_loads = std::integral_constant<int, -1>;
    // One slab with a successor. `more` says whether a slab kt+2 exists, whose first loads go out in
    // the step after the barrier.
    auto slab = [&](int kt, auto more) {
        const char* s = lds + (kt & 1) * STAGE;
        const char* sn = lds + ((kt & 1) ^ 1) * STAGE;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (STAGED) {
            // slots 8..31 move chunks of slab kt+1 into the other stage, the barrier publishes them
            // and frees this slab's stage, whose first chunks (slab kt+2) follow in slots 0..7
            step(0, s, 1, std::true_type{}, std::integral_constant<int, READS>{}, kt + 1, 0u);
            step(1, s, 2, std::true_type{}, std::integral_constant<int, 2 * READS>{}, kt + 1, 0u);
            step(0, s, 3, std::true_type{}, std::integral_constant<int, 3 * READS>{}, kt + 1, 0u);
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            step(1, sn, 0, std::true_type{}, std::integral_constant<int, 0>{}, kt + 2, 0u);
            return;
        }
        const uint32_t kmask1 = slab_kmask(kt + 1);
        step(0, s, 1, std::true_type{}, std::integral_constant<int, READS>{}, kt + 1, kmask1);
        step(1, s, 2, std::true_type{}, std::integral_constant<int, 2 * READS>{}, kt + 1, kmask1);
        step(0, s, 3, std::true_type{}, no_loads{}, 0, 0u);
        wait_vmem_all();   // this wave's share of slab kt+1 has landed ...
        __syncthreads();   // ... and so has everybody else's; all waves are done reading slab kt-1's stage
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (decltype(more)::value)
            step(1, sn, 0, std::true_type{}, std::integral_constant<int, 0>{}, kt + 2, slab_kmask(kt + 2));
        else
            step(1, sn, 0, std::true_type{}, no_loads{}, 0, 0u);
    };

    if constexpr (STAGED) {
        // Prologue: slab 0 through the registers into stage 0; slab 1 into the registers, and its
        // chunks that belong to slots 0..7 already into stage 1.
#pragma unroll
        for (int i = 0; i < LPS; ++i) stage_load(0, i);
#pragma unroll
        for (int i = 0; i < LPS; ++i) stage_store(0, i);
#pragma unroll
        for (int i = 0; i < LPS; ++i) stage_load(1, i);
        __syncthreads();
#pragma unroll
        for (int r = 0; r < READS; ++r) read_frag(0, lds, 0, r);
#pragma unroll
        for (int g = 0; g < READS; ++g) {
            const int l = load_at_slot(g, 4 * READS, LPS);
            if (l >= 0) {
                stage_store(1, l);
                stage_load(2, l);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    } else {
    // Prologue: slab 0 completely, then the first third of slab 1.
        const uint32_t km = slab_kmask(0);
#pragma unroll
        for (int i = 0; i < LPS; ++i) issue_load(0, km, i);
        wait_vmem_all();
        __syncthreads();
#pragma unroll
        for (int r = 0; r < READS; ++r) read_frag(0, lds, 0, r);
        if (nk > 1) {
            const uint32_t km1 = slab_kmask(1);
#pragma unroll
            for (int g = 0; g < READS; ++g) {
                const int l = load_at_slot(g, SLOTS, LPS);
                if (l >= 0) issue_load(1, km1, l);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    int kt = 0;
    for (; kt + 2 < nk; ++kt) slab(kt, std::true_type{});
    if (kt + 1 < nk) {
        slab(kt, std::false_type{});
        ++kt;
    }
    {
        const char* s = lds + (kt & 1) * STAGE;
        step(0, s, 1, std::true_type{}, no_loads{}, 0, 0u);
        step(1, s, 2, std::true_type{}, no_loads{}, 0, 0u);
        step(0, s, 3, std::true_type{}, no_loads{}, 0, 0u);
        step(1, nullptr, 0, std::false_type{}, no_loads{}, 0, 0u);
        __syncthreads();
    }

    gemm_epilogue<MI, NJ>(p, acc, lds, m0, n0, wave, lane);
}

// ------------------------------------------------------------------------------------------------
// Paired-slab variant. The memory path of a CU moves 256-byte granules: asking for the two 128-byte
// halves of a granule one K=64 slab apart (as the kernel above does) fetches every granule twice and
// halves the achievable load rate. Here a thread loads both halves of a granule back to back (the
// same rows, k and k+64) into registers, and the halves enter the two LDS stages when those become
// free: stage 0 always holds the even slab (k % 128 < 64), stage 1 the odd one. One loop iteration
// consumes a K=128 super-slab in eight K=16 steps with two barriers:
//
//   steps 0 1 2 | B1 | 3 4 5 6 | B2 | 7
//   reads stage:  0 0 0   (3 reads 0, prefetches 1)  1 1 1   (7 reads 1, prefetches stage 0 of q+1)
//   H1[l] -> stage 1 : step 7 of the previous iteration (l = 0..LPS/4-1) and steps 0..2   (half 1 of q)
//   H0[l] -> stage 0 : steps 3..6                                                          (half 0 of q+1)
//   right after H1[l] is stored, the pair (H0[l], H1[l]) of the following super-slab is requested;
//   H0[l] is not stored before 4 steps later, H1[l] not before 8.
// ------------------------------------------------------------------------------------------------
template <int MI, int NJ>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_paired_kernel(GemmParams p) {
    constexpr int BM = 64 * MI, BN = 64 * NJ, BK = 64;
    constexpr int ROWB = BK * 2;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int PA = BM / 32, PB = BN / 32;
    constexpr int LPS = PA + PB;                 // 16-byte chunks per thread per K=64 slab
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    static_assert(4 * WROWS * WCOLS * 2 <= 2 * STAGE, "epilogue tile must fit the ring");
    __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE];

    int tm, tn;
    if (!tile_of_block(p, tm, tn)) return;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // loader mapping (as in the kernel above): LDS slot (row = pass*32 + tid/8, position tid%8) holds
    // logical chunk position ^ ((row>>1)&7)
    const int lrow = tid >> 3;
    const int lchunk = (tid & 7) ^ ((lrow >> 1) & 7);
    const int rows_a = min(p.M - m0, BM), rows_b = min(p.N - n0, BN);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(p.A + static_cast<int64_t>(m0) * p.lda), 0,
        static_cast<int>(((rows_a - 1) * p.lda + p.K) * 2), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(p.W + static_cast<int64_t>(n0) * p.ldw), 0,
        static_cast<int>(((rows_b - 1) * p.ldw + p.K) * 2), kRsrcFlags);
    uint32_t voff[LPS];
#pragma unroll
    for (int i = 0; i < LPS; ++i) {
        const int r = (i < PA ? i : i - PA) * 32 + lrow;
        const bool ok = i < PA ? r < rows_a : r < rows_b;
        const int64_t ld = i < PA ? p.lda : p.ldw;
        voff[i] = ok ? static_cast<uint32_t>((r * ld + lchunk * 8) * 2) : kOutOfRange;
    }
    const int lds_slot = lrow * 128 + (tid & 7) * 16;

    const int nq = (p.K + 2 * BK - 1) / (2 * BK);  // K=128 super-slabs
    u32x4 h0[LPS], h1[LPS];
    // Request chunk l of both halves of super-slab q. Chunks at or past K (K is a multiple of 8) and
    // super-slabs past the end read as zeros.
    auto load_pair = [&](int q, int l) {
        const int k0 = q * (2 * BK) + lchunk * 8;
        const uint32_t m0k = k0 >= p.K ? kOutOfRange : 0u;
        const uint32_t m1k = k0 + BK >= p.K ? kOutOfRange : 0u;
        const __amdgpu_buffer_rsrc_t rs = l < PA ? rsrc_a : rsrc_b;
        h0[l] = load_chunk_reg(rs, voff[l] | m0k, q * (4 * BK));
        h1[l] = load_chunk_reg(rs, voff[l] | m1k, q * (4 * BK) + 2 * BK);
    };
    auto store_half = [&](int stage, const u32x4& v, int l) {
        char* dst = lds + stage * STAGE + lds_slot + (l < PA ? l * 4096 : A_BYTES + (l - PA) * 4096);
        *reinterpret_cast<u32x4*>(dst) = v;
    };

    // fragment addressing
    const int frow = lane & 31, fhalf = lane >> 5;
    int koff[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) koff[kk] = ((kk * 2 + fhalf) ^ ((frow >> 1) & 7)) * 16;
    const int a_off = (wm * WROWS + frow) * ROWB;
    const int b_off = A_BYTES + (wn * WCOLS + frow) * ROWB;

    f32x16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    bf16x8 xa[2][MI], wb[2][NJ];
    auto read_frag = [&](int buf, const char* s, int kk, int r) {
        if (r == 0) xa[buf][0] = *reinterpret_cast<const bf16x8*>(s + a_off + koff[kk]);
        else if (r <= NJ) wb[buf][r - 1] = *reinterpret_cast<const bf16x8*>(s + b_off + (r - 1) * 32 * ROWB + koff[kk]);
        else xa[buf][r - NJ] = *reinterpret_cast<const bf16x8*>(s + a_off + (r - NJ) * 32 * ROWB + koff[kk]);
    };
    auto mfma_one = [&](int buf, int idx) {
        const int i = idx / NJ, j = idx % NJ;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[buf][j], xa[buf][i], acc[i][j], 0, 0, 0);
    };
    constexpr int READS = MI + NJ, PER = (MI * NJ) / READS;
    static_assert((MI * NJ) % READS == 0 && LPS % 4 == 0, "schedule shape");
    constexpr int WPS = LPS / 4;  // register->LDS stores per step inside a 4-step window
    // Step `stp` (0..7) of the iteration consuming super-slab q. Fragment reads of the next step are
    // interleaved with this step's MFMAs; the store / load-pair actions sit in the first WPS slots.
    auto step = [&](auto stp_c, int q) {
        constexpr int STP = decltype(stp_c)::value;
        constexpr int cur_buf = STP & 1;
        constexpr int nstp = (STP + 1) & 7;
        const char* nxt = lds + (nstp >> 2) * STAGE;
#pragma unroll
        for (int r = 0; r < READS; ++r) {
            read_frag(cur_buf ^ 1, nxt, nstp & 3, r);
            if (r < WPS) {
                if constexpr (STP == 7) {            // half 1 of q+1, first quarter; then pairs of q+2
                    store_half(1, h1[r], r);
                    load_pair(q + 2, r);
                } else if constexpr (STP <= 2) {     // half 1 of q, remaining quarters; then pairs of q+1
                    const int l = (STP + 1) * WPS + r;
                    store_half(1, h1[l], l);
                    load_pair(q + 1, l);
                } else {                             // steps 3..6: half 0 of q+1
                    const int l = (STP - 3) * WPS + r;
                    store_half(0, h0[l], l);
                }
            }
#pragma unroll
            for (int m = 0; m < PER; ++m) mfma_one(cur_buf, r * PER + m);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Prologue: super-slab 0 through the registers; its half 0 and the first quarter of its half 1 go
    // to LDS, the freed registers take the pairs of super-slab 1.
#pragma unroll
    for (int l = 0; l < LPS; ++l) load_pair(0, l);
#pragma unroll
    for (int l = 0; l < LPS; ++l) store_half(0, h0[l], l);
#pragma unroll
    for (int l = 0; l < WPS; ++l) {
        store_half(1, h1[l], l);
        load_pair(1, l);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < READS; ++r) read_frag(0, lds, 0, r);
    __builtin_amdgcn_sched_barrier(0);

    for (int q = 0; q < nq; ++q) {
        step(std::integral_constant<int, 0>{}, q);
        step(std::integral_constant<int, 1>{}, q);
        step(std::integral_constant<int, 2>{}, q);
        __syncthreads();  // B1: half 1 of q is in stage 1
        __builtin_amdgcn_sched_barrier(0);
        step(std::integral_constant<int, 3>{}, q);
        step(std::integral_constant<int, 4>{}, q);
        step(std::integral_constant<int, 5>{}, q);
        step(std::integral_constant<int, 6>{}, q);
        __syncthreads();  // B2: half 0 of q+1 is in stage 0; stage 1 is free
        __builtin_amdgcn_sched_barrier(0);
        step(std::integral_constant<int, 7>{}, q);
    }
    __syncthreads();
    gemm_epilogue<MI, NJ>(p, acc, lds, m0, n0, wave, lane);
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

template <int MI, int NJ, bool STAGED>
static void launch_tiled(GemmParams& p, hipStream_t st) {
    constexpr int BM = 64 * MI, BN = 64 * NJ;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    p.group_m = 4;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL((gemm_nt_kernel<MI, NJ, STAGED>), dim3(grid), dim3(kGemmThreads), 0, st, p);
}

template <int MI, int NJ>
static void launch_paired(GemmParams& p, hipStream_t st) {
    constexpr int BM = 64 * MI, BN = 64 * NJ;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    p.group_m = 4;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL((gemm_nt_paired_kernel<MI, NJ>), dim3(grid), dim3(kGemmThreads), 0, st, p);
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
    p.bias_vec = a->bias != nullptr && (reinterpret_cast<uintptr_t>(a->bias) & 3u) == 0 && a->N % 4 == 0;
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
    else if (variant == 2) launch_tiled<2, 2, false>(p, st);
    else if (variant == 3) launch_tiled<4, 4, true>(p, st);
    else if (variant == 4) launch_tiled<2, 2, true>(p, st);
    else if (variant == 5) launch_paired<4, 4>(p, st);
    else if (variant == 6) launch_paired<2, 2>(p, st);
    else if (big_tiles >= 192) launch_tiled<4, 4, false>(p, st);
    else launch_tiled<2, 2, false>(p, st);
    return check_launch("flux_linear_bf16");
}
