// Linear layer on the matrix cores:  Y = epilogue(A[M,K] * W[N,K]^T), bf16 operands, fp32 accumulate.
//
// Both operands are K-contiguous, which is exactly what v_mfma_f32_16x16x32_bf16 wants: every lane
// feeds 8 consecutive k of one row. A workgroup of four waves (2 x 2) owns a (64*MI) x (64*MI) tile
// of Y and each wave a (32*MI) x (32*MI) sub-tile kept as (2*MI)^2 accumulators of 16x16. (The
// 16x16x32 shape moves half the accumulator registers per flop of 32x32x16; on a chip that runs
// this kernel at its power limit that is worth more than the extra instruction issues.) The K loop
// moves 64-wide slabs of A and W through a five-unit LDS ring (see the kernel) straight from buffer
// loads that write LDS (no register staging).
//
// LDS slab layout: row r of the slab is 128 bytes = eight 16-byte chunks; chunk c is stored at
// position c ^ ((r >> 1) & 7). LDS on gfx950 has 64 banks of 4 bytes, so a ds_read_b128 is served 16
// lanes (256 bytes) per clock: the 16 lanes that read the same logical chunk of 16 consecutive rows
// land on 2 (row parity) x 8 (position) = 16 different 16-byte bank groups, conflict-free. The
// writer side fills whole rows, also conflict-free.
//
// The MFMA takes W as its "A" operand and the activations as its "B" operand, so the accumulator
// of a lane holds one activation row m and runs of 4 consecutive output columns n: bias and GELU
// are applied there in fp32 and the result is rounded once; the bf16 tile goes through LDS once
// more and leaves as full 16-byte row segments, where the optional gated residual is applied.
#include "common.h"
#include <stdlib.h>
#include <algorithm>
#include <type_traits>

namespace flux {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
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
    int in_silu;  // 1: A passes through x * sigmoid(x), rounded to bf16, on the way in (row-vector and scalar kernels)
    int tiles_m, tiles_n, group_m;
    int bias_vec;  // 1: bias may be read with 8-byte buffer loads (4-byte aligned base)
    int vec_io;  // 1: every output/residual row segment of 8 columns may be accessed as 16 bytes
    // fused QK RMSNorm + RoPE for columns [0, qk_cols): q heads first, then k heads, 128 columns each
    bf16_t* q_out; bf16_t* k_out;
    const bf16_t* q_scale; const bf16_t* k_scale;
    const float* pe;
    int64_t pe_batch_stride;
    int qk_cols, qk_heads, qk_seq_len, qk_out_len, qk_pos0;
    float qk_eps;
};

constexpr int kGemmThreads = 256;
constexpr int kGemmCUs = 256;      // compute units of the one device this library is built for
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
// Tile order of a launch with the q/k epilogue. Its q/k tiles cost more than the others, each XCD
// owns one contiguous range of the tile sequence and works through it alone, and in the natural
// order one XCD would get twice its share of q/k tiles and another none. Here the q/k columns and
// the other columns form two sequences (each grouped like the plain order, so that the tiles
// resident on an XCD still share panels, and the q/k tiles of a patch the same rows of the rotation
// table), and every XCD takes its eighth of the first followed by its eighth of the second.
__device__ __forceinline__ bool tile_of_block_qk(const GemmParams& p, int bn, int& tm, int& tn) {
    const int nq = p.qk_cols / bn;
    const int Q = p.tiles_m * nq, R = p.tiles_m * (p.tiles_n - nq);
    const int per_xcd = gridDim.x / 8;
    const int x = blockIdx.x % 8, i = blockIdx.x / 8;
    const int q0 = x * Q / 8, q1 = (x + 1) * Q / 8;
    int u, cols, col0;
    if (i < q1 - q0) {
        u = q0 + i; cols = nq; col0 = 0;
    } else {
        u = x * per_xcd - q0 + (i - (q1 - q0)); cols = p.tiles_n - nq; col0 = nq;
        if (u >= R) return false;
    }
    const int width = p.group_m * cols;
    const int first_m = (u / width) * p.group_m;
    const int gsz = min(p.tiles_m - first_m, p.group_m);
    const int in_group = u % width;
    tm = first_m + in_group % gsz;
    tn = col0 + in_group / gsz;
    return true;
}

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

__device__ __forceinline__ void wait_vmem_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

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
__device__ __forceinline__ void gemm_epilogue_checked(const GemmParams& p, f32x4 (&acc)[2 * MI][2 * NJ], char* lds, int m0, int n0,
                                                   int wave, int lane) {
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    constexpr int C_PITCH = WCOLS * 2, C_CH = WCOLS / 8;  // bytes per row, 16-byte chunks per row
    constexpr int RPI = 64 / C_CH;                         // rows one wave-wide 16-byte access covers
    constexpr int NQ = 2 * NJ;                             // column quads of a lane: one per 16-column fragment
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 15, fq = lane >> 4;            // accumulator: row frow of a 16-row fragment, columns fq*4..+3
    char* cw = lds + wave * (WROWS * C_PITCH);
    const int wave_n0 = n0 + wn * WCOLS;
    const int wave_m0 = m0 + wm * WROWS;

    // bias for the lane's NQ column quads
    float bv[NQ][4];
    const bool bias_fast = p.bias != nullptr && p.bias_vec;
    if (bias_fast) {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.bias), 0, p.N * 2, kRsrcFlags);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const u32x2 raw = __builtin_amdgcn_raw_buffer_load_b64(rb, (wave_n0 + q * 16 + fq * 4) * 2, 0, 0);
            bv[q][0] = __uint_as_float(raw.x << 16);
            bv[q][1] = __uint_as_float(raw.x & 0xffff0000u);
            bv[q][2] = __uint_as_float(raw.y << 16);
            bv[q][3] = __uint_as_float(raw.y & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = wave_n0 + q * 16 + fq * 4 + e;
                bv[q][e] = (p.bias != nullptr && n < p.N) ? bf2f(p.bias[n]) : 0.0f;
            }
    }

    // LDS write address of column quad q in this lane's row, without the 16-row fragment offset
    int waddr[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) waddr[q] = frow * C_PITCH + (((q * 2 + (fq >> 1)) ^ (frow & (C_CH - 1))) * 16) + (fq & 1) * 8;
    // read side: lane -> (row within the pass = lane / C_CH, chunk = lane % C_CH)
    const int rrow = lane / C_CH, rch = lane % C_CH;

    const bool gelu_all = p.act == FLUX_ACT_GELU_TANH && wave_n0 >= p.act_begin;
    const bool gelu_some = p.act == FLUX_ACT_GELU_TANH && !gelu_all && wave_n0 + WCOLS > p.act_begin;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        // ---- accumulators of block row i (two 16-row fragments) -> bf16 -> LDS
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[2 * i + t][q][e] + bv[q][e];
                if (gelu_all) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = tanh_gelu_fast(v[e]);
                } else if (gelu_some) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (wave_n0 + q * 16 + fq * 4 + e >= p.act_begin) v[e] = tanh_gelu_fast(v[e]);
                }
                *reinterpret_cast<u32x2*>(cw + (i * 32 + t * 16) * C_PITCH + waddr[q]) = pack4_bf16(v[0], v[1], v[2], v[3]);
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
__device__ __forceinline__ void gemm_epilogue_fast(const GemmParams& p, f32x4 (&acc)[2 * MI][2 * NJ], char* lds, int m0, int n0,
                                                   int wave, int lane) {
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    constexpr int C_PITCH = WCOLS * 2, C_CH = WCOLS / 8;
    constexpr int RPI = 64 / C_CH;      // rows per wave-wide 16-byte access
    constexpr int NIT = 32 / RPI;       // accesses per 32-row block
    constexpr int NQ = 2 * NJ;          // column quads of a lane: one per 16-column fragment
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 15, fq = lane >> 4;
    char* cw = lds + wave * (WROWS * C_PITCH);
    const int wave_n0 = n0 + wn * WCOLS;
    const int wave_m0 = m0 + wm * WROWS;

    float bv[NQ][4];
    if (p.bias != nullptr) {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.bias), 0, p.N * 2, kRsrcFlags);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const u32x2 raw = __builtin_amdgcn_raw_buffer_load_b64(rb, (wave_n0 + q * 16 + fq * 4) * 2, 0, 0);
            bv[q][0] = __uint_as_float(raw.x << 16);
            bv[q][1] = __uint_as_float(raw.x & 0xffff0000u);
            bv[q][2] = __uint_as_float(raw.y << 16);
            bv[q][3] = __uint_as_float(raw.y & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[q][e] = 0.0f;
    }

    int waddr[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) waddr[q] = frow * C_PITCH + (((q * 2 + (fq >> 1)) ^ (frow & (C_CH - 1))) * 16) + (fq & 1) * 8;
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
    // Gated residual: the rows of resid this lane adds to are requested a whole 32-row block ahead,
    // into the other half of rs, so that they land while the block in front is converted and stored.
    // (Requested where they are used, every 16-byte store waited for a load round trip of its own,
    // and, the memory counter being in-order, for the store in front of it: 32 round trips in a row
    // per wave.) The tile lies inside one batch element (the caller checks), so the gate vector of
    // this lane's eight columns is loaded once.
    const char* res_u = nullptr;
    uint32_t res_lane = 0;
    Vec16<bf16_t> gt;
    Vec16<bf16_t> rs[2][NIT];
    auto request_resid = [&](int i) {
#pragma unroll
        for (int it = 0; it < NIT; ++it)
            rs[i & 1][it] = *reinterpret_cast<const Vec16<bf16_t>*>(res_u + static_cast<int64_t>(wave_m0 + i * 32 + it * RPI) * p.ldresid * 2 + res_lane);
    };
    if (GATE) {
        res_u = reinterpret_cast<const char*>(p.resid + wave_n0);
        res_lane = static_cast<uint32_t>(rrow * p.ldresid * 2 + rch * 16);
        gt = ld16(p.gate + static_cast<int64_t>(m0 / p.rows_per_batch) * p.gate_stride + wave_n0 + rch * 8);
        request_resid(0);
    }

#pragma unroll
    for (int i = 0; i < MI; ++i) {
        if (GATE) {
            if (i + 1 < MI) request_resid(i + 1);
            __builtin_amdgcn_sched_barrier(0);   // the loads stay in front of the conversion below
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = acc[2 * i + t][q][e] + bv[q][e];
                    if (GELU) v[e] = tanh_gelu_fast(v[e]);
                }
                *reinterpret_cast<u32x2*>(cw + (i * 32 + t * 16) * C_PITCH + waddr[q]) = pack4_bf16(v[0], v[1], v[2], v[3]);
            }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int row_u = i * 32 + it * RPI;                 // wave-uniform part of the row
            Vec16<bf16_t> y = *reinterpret_cast<const Vec16<bf16_t>*>(cw + (i * 32 + (it / NSW) * NSW * RPI) * C_PITCH + raddr[it % NSW]);
            const int64_t m_u = wave_m0 + row_u;
            if (GATE) {
                const Vec16<bf16_t> r = rs[i & 1][it];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float y0 = bf2f(r.v[e]) + bf2f(f2bf(bf2f(gt.v[e]) * bf2f(y.v[e])));
                    const float y1 = bf2f(r.v[e + 1]) + bf2f(f2bf(bf2f(gt.v[e + 1]) * bf2f(y.v[e + 1])));
                    const uint32_t w = pack2_bf16(y0, y1);
                    y.v[e] = static_cast<bf16_t>(w & 0xffffu);
                    y.v[e + 1] = static_cast<bf16_t>(w >> 16);
                }
            }
            *reinterpret_cast<Vec16<bf16_t>*>(dst_u + m_u * dst_ld + dst_lane) = y;
        }
    }
}

// Epilogue for a wave whose 128 columns are one head of q or k: y = A W^T + bias is rounded to bf16
// (the projection's output), RMS-normalised over the head (x * rstd rounded, times scale rounded),
// rotated by the 2x2 matrices of its position and written to [B, heads, out_len, 128]. A lane holds
// 32 of a row's 128 columns; the other 96 are in the lanes 16, 32 and 48 further on, so the sum of
// squares takes two cross-lane steps. RAGGED = false: the tile is interior and lies inside one batch
// element, so its rows are consecutive positions of one (batch, head). RAGGED = true: the tile may run
// past the last row and may hold the last rows of one batch element followed by the first of the next
// (at most one such boundary: sequences are at least a tile long); rows past the end are computed on
// clamped table rows and not stored, rows behind the boundary take their table rows and their
// destination from the next batch element.
template <int MI, int NJ, bool RAGGED>
__device__ __forceinline__ void gemm_epilogue_qk(const GemmParams& p, f32x4 (&acc)[2 * MI][2 * NJ], char* lds, int m0, int n0,
                                                 int wave, int lane) {
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    static_assert(WCOLS == 128, "a wave's columns are one head of 128");
    constexpr int C_PITCH = WCOLS * 2, C_CH = WCOLS / 8;
    constexpr int RPI = 64 / C_CH;
    constexpr int NIT = 32 / RPI;
    constexpr int NQ = 2 * NJ;
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 15, fq = lane >> 4;
    char* cw = lds + wave * (WROWS * C_PITCH);
    const int wave_n0 = n0 + wn * WCOLS;
    const int wave_m0 = m0 + wm * WROWS;
    const int hcol = wave_n0 / WCOLS;
    const bool is_k = hcol >= p.qk_heads;
    const int head = is_k ? hcol - p.qk_heads : hcol;
    const int batch = m0 / p.qk_seq_len;                        // the whole tile is in one batch element
    const int pos_w = p.qk_pos0 + (wave_m0 - batch * p.qk_seq_len);   // output row of the wave's first row

    // bias and scale of this lane's columns stay packed (two bf16 per register) and are unpacked at
    // their use: the epilogue needs its registers for the rotation entries in flight
    u32x2 bvp[NQ], scp[NQ];
    {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(is_k ? p.k_scale : p.q_scale), 0, WCOLS * 2, kRsrcFlags);
#pragma unroll
        for (int q = 0; q < NQ; ++q) scp[q] = __builtin_amdgcn_raw_buffer_load_b64(rs, (q * 16 + fq * 4) * 2, 0, 0);
    }
    if (p.bias != nullptr) {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.bias), 0, p.N * 2, kRsrcFlags);
#pragma unroll
        for (int q = 0; q < NQ; ++q) bvp[q] = __builtin_amdgcn_raw_buffer_load_b64(rb, (wave_n0 + q * 16 + fq * 4) * 2, 0, 0);
    } else {
#pragma unroll
        for (int q = 0; q < NQ; ++q) bvp[q] = u32x2{0u, 0u};
    }
    auto unpack = [](u32x2 v, int e) -> float {
        const uint32_t w = e < 2 ? v.x : v.y;
        return __uint_as_float((e & 1) ? (w & 0xffff0000u) : (w << 16));
    };

    int waddr[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) waddr[q] = frow * C_PITCH + (((q * 2 + (fq >> 1)) ^ (frow & (C_CH - 1))) * 16) + (fq & 1) * 8;
    const int rrow = lane / C_CH, rch = lane % C_CH;
    constexpr int NSW = (16 / RPI) < NIT ? (16 / RPI) : NIT;
    int raddr[NSW];
#pragma unroll
    for (int t = 0; t < NSW; ++t) {
        const int row = t * RPI + rrow;
        raddr[t] = row * C_PITCH + ((rch ^ (row & (C_CH - 1))) * 16);
    }
    // rotation table of this lane's columns: 8 floats per quad, row stride 2 * 128 floats
    const float* pe_lane = p.pe + static_cast<int64_t>(batch) * p.pe_batch_stride + static_cast<int64_t>(pos_w + frow) * (2 * WCOLS) + fq * 8;
    // RAGGED: rows of the wave's sub-tile from `boundary` on belong to the next batch element, whose
    // positions restart: their table row is pe_next floats and their output row out_next bytes further on
    const int boundary = RAGGED ? (batch + 1) * p.qk_seq_len - wave_m0 : WROWS;
    const int64_t pe_next = RAGGED ? p.pe_batch_stride - static_cast<int64_t>(p.qk_seq_len) * (2 * WCOLS) : 0;
    const uint32_t out_next = RAGGED ? static_cast<uint32_t>((static_cast<int64_t>(p.qk_heads) * p.qk_out_len - p.qk_seq_len) * (WCOLS * 2)) : 0u;
    const int rows_valid = RAGGED ? p.M - wave_m0 : WROWS;   // rows of the sub-tile inside the matrix
    if (RAGGED && rows_valid <= 0) return;                   // nothing of this wave's to store (no workgroup barrier follows)
    char* dst_u = reinterpret_cast<char*>((is_k ? p.k_out : p.q_out) +
                                          ((static_cast<int64_t>(batch) * p.qk_heads + head) * p.qk_out_len + pos_w) * WCOLS);
    const uint32_t dst_lane = static_cast<uint32_t>(rrow * (WCOLS * 2) + rch * 16);
    const float inv_d = 1.0f / static_cast<float>(WCOLS);

#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            // the step's rotation entries (from L2) are requested first and land while the sum of
            // squares is formed; the scheduling barrier keeps the compiler from sinking the loads
            // to their uses, where each would be waited for in turn
            f32x4 fr[NQ][2];
            {
                const float* pr = pe_lane + (i * 32 + t * 16) * (2 * WCOLS);
                if (RAGGED) {
                    const int r = min(i * 32 + t * 16 + frow, rows_valid - 1);   // past the end: the last valid row's entries
                    pr = pe_lane + static_cast<int64_t>(r - frow) * (2 * WCOLS) + (r >= boundary ? pe_next : 0);
                }
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    fr[q][0] = *reinterpret_cast<const f32x4*>(pr + q * 32);
                    fr[q][1] = *reinterpret_cast<const f32x4*>(pr + q * 32 + 4);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // roundings to bf16 two values at a time: one v_cvt_pk_bf16_f32, then the halves widened again
            auto round2 = [](float a, float b, float& ra, float& rb) {
                const uint32_t w = pack2_bf16(a, b);
                ra = __uint_as_float(w << 16);
                rb = __uint_as_float(w & 0xffff0000u);
            };
            float x[NQ][4];
            float ss = 0.0f;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
#pragma unroll
                for (int e = 0; e < 4; e += 2)
                    round2(acc[2 * i + t][q][e] + unpack(bvp[q], e), acc[2 * i + t][q][e + 1] + unpack(bvp[q], e + 1), x[q][e], x[q][e + 1]);
#pragma unroll
                for (int e = 0; e < 4; ++e) ss += x[q][e] * x[q][e];
            }
            ss += __shfl_xor(ss, 16);
            ss += __shfl_xor(ss, 32);
            const float rstd = rsqrtf(ss * inv_d + p.qk_eps);
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const f32x4 f0 = fr[q][0];
                const f32x4 f1 = fr[q][1];
                float xn[4];
#pragma unroll
                for (int e = 0; e < 4; e += 2) {
                    float a, b;
                    round2(x[q][e] * rstd, x[q][e + 1] * rstd, a, b);
                    round2(a * unpack(scp[q], e), b * unpack(scp[q], e + 1), xn[e], xn[e + 1]);
                }
                const float o0 = f0[0] * xn[0] + f0[1] * xn[1];
                const float o1 = f0[2] * xn[0] + f0[3] * xn[1];
                const float o2 = f1[0] * xn[2] + f1[1] * xn[3];
                const float o3 = f1[2] * xn[2] + f1[3] * xn[3];
                *reinterpret_cast<u32x2*>(cw + (i * 32 + t * 16) * C_PITCH + waddr[q]) = pack4_bf16(o0, o1, o2, o3);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int row_u = i * 32 + it * RPI;
            const Vec16<bf16_t> y = *reinterpret_cast<const Vec16<bf16_t>*>(cw + (i * 32 + (it / NSW) * NSW * RPI) * C_PITCH + raddr[it % NSW]);
            if (RAGGED) {
                const int r = row_u + rrow;
                if (r < rows_valid)
                    *reinterpret_cast<Vec16<bf16_t>*>(dst_u + static_cast<int64_t>(row_u) * (WCOLS * 2) + (dst_lane + (r >= boundary ? out_next : 0u))) = y;
            } else {
                *reinterpret_cast<Vec16<bf16_t>*>(dst_u + static_cast<int64_t>(row_u) * (WCOLS * 2) + dst_lane) = y;
            }
        }
    }
}

template <int MI, int NJ>
__device__ __forceinline__ void gemm_epilogue(const GemmParams& p, f32x4 (&acc)[2 * MI][2 * NJ], char* lds, int m0, int n0,
                                              int wave, int lane) {
    constexpr int BM = 64 * MI, BN = 64 * NJ, WCOLS = 32 * NJ;
    const int wave_n0 = n0 + (wave & 1) * WCOLS;
    const bool gelu_all = p.act == FLUX_ACT_GELU_TANH && wave_n0 >= p.act_begin;
    const bool gelu_none = p.act != FLUX_ACT_GELU_TANH || wave_n0 + WCOLS <= p.act_begin;
    if constexpr (NJ == 4) {
        if (wave_n0 < p.qk_cols) {   // the host admits the fusion only when the q/k columns are whole tiles
            const bool ragged = m0 + BM > p.M || m0 / p.qk_seq_len != (m0 + BM - 1) / p.qk_seq_len;
            if (ragged) gemm_epilogue_qk<MI, NJ, true>(p, acc, lds, m0, n0, wave, lane);
            else gemm_epilogue_qk<MI, NJ, false>(p, acc, lds, m0, n0, wave, lane);
            return;
        }
    }
    // (with a gate: the fast path loads one gate vector per tile, so the tile must not span batch elements)
    const bool fast = p.vec_io && m0 + BM <= p.M && n0 + BN <= p.N && (gelu_all || gelu_none) &&
                      (p.gate == nullptr || m0 / p.rows_per_batch == (m0 + BM - 1) / p.rows_per_batch) &&
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

// ------------------------------------------------------------------------------------------------
// Tiled kernel: 64*MI x 64*MI output tile per workgroup of four waves (2 x 2, a wave owns
// 32*MI x 32*MI as (2*MI)^2 accumulators of v_mfma_f32_16x16x32_bf16), K in slabs of 64 = two MFMA
// steps of K = 32. With two whole-slab LDS stages the memory pipeline would drain at every barrier
// (the wait in front of it is for ALL outstanding loads). Here LDS is a ring of five units, a unit
// holding one operand's share of a slab (BM rows x 128 bytes): A(kt) lives in unit 2kt % 5 and
// W(kt) in unit (2kt+1) % 5. While slab kt is computed, slab kt+1 and A(kt+2) occupy the other
// three units. The barrier of slab kt sits a quarter into its last step; right behind it the unit
// of A(kt) is free and takes the loads of W(kt+2), one per slot, and the loads of A(kt+3) follow at
// an even pace in front of the next barrier. The wait in front of a barrier only covers W of the
// next slab: the loads of A two slabs ahead stay in flight across it. Every load has more than
// three quarters of a slab of MFMA time to land and the memory pipeline never runs empty.
//
//   slab kt :  step 0            step 1 = [MFMA x PER*BS] wait+barrier [rest, reads step 0 of kt+1]
//   loads   :  ...... A(kt+2) ......................      |  W(kt+2) x PU, one per slot
//
// Ring offsets are wave-uniform scalars that advance by two units per slab.
// ------------------------------------------------------------------------------------------------
template <int K>
using ic = std::integral_constant<int, K>;

template <int N>
__device__ __forceinline__ void wait_loads_and_barrier() {
    // all but the newest N buffer loads of this wave have landed, its LDS reads have returned; the
    // memory clobber keeps LDS accesses on their side of the barrier
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Multiplies K slabs [kb, ke) of the tile at (m0, n0) into acc (cleared first). On return every
// buffer load of the wave has landed and all waves have passed a barrier, so the ring may be
// reused (the epilogue parks its bf16 blocks there).
template <int MI, bool KTAIL>
__device__ __forceinline__ void gemm_tile_slabs(const GemmParams& p, char* lds, int m0, int n0, int kb, int ke,
                                                f32x4 (&acc)[2 * MI][2 * MI]) {
    constexpr int NJ = MI;
    constexpr int FM = 2 * MI, FN = 2 * NJ;      // 16-row fragments per wave and side
    constexpr int BM = 64 * MI, BN = BM, BK = 64;
    constexpr int ROWB = BK * 2, KSUB = BK / 32;
    constexpr int UNIT = BM * ROWB, NU = 5;
    constexpr int PU = BM / 32;                  // buffer loads per thread per unit
    constexpr int NL = 2 * PU;                   // loads per group G(kt) = W(kt+1), A(kt+2)
    constexpr int WROWS = 32 * MI, WCOLS = 32 * NJ;
    constexpr int READS = FM + FN, MFMAS = FM * FN, PER = MFMAS / READS;
    constexpr int BS = READS / 4;                // slots of the last step in front of the barrier
    constexpr int NSLOT = KSUB * READS;          // issue slots per slab
    constexpr int GB = (KSUB - 1) * READS + BS;  // first slot behind the barrier
    constexpr int EARLY = PU;                    // W loads of a group, all issued right behind the previous slab's barrier
    static_assert(MFMAS % READS == 0 && KSUB == 2 && NSLOT == 2 * NL && NSLOT - GB >= PU, "schedule shape");
    static_assert(2 * (NSLOT - GB) >= READS, "the next slab's first fragments are read two per slot behind the barrier");
    static_assert(4 * WROWS * WCOLS * 2 <= NU * UNIT, "epilogue tile must fit the ring");
    (void)BN; (void)WCOLS;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // loader mapping: LDS slot (row = pass*32 + tid/8, position tid%8) holds logical chunk
    // position ^ ((row>>1)&7) of that row
    const int lrow = tid >> 3;
    const int lchunk = (tid & 7) ^ ((lrow >> 1) & 7);
    const int rows_a = min(p.M - m0, BM), rows_b = min(p.N - n0, BN);
    bf16_t* const base_a = const_cast<bf16_t*>(p.A + static_cast<int64_t>(m0) * p.lda);
    bf16_t* const base_b = const_cast<bf16_t*>(p.W + static_cast<int64_t>(n0) * p.ldw);
    const int bytes_a = static_cast<int>(((rows_a - 1) * p.lda + p.K) * 2);
    const int bytes_b = static_cast<int>(((rows_b - 1) * p.ldw + p.K) * 2);
    uint32_t voff_a[PU], voff_b[PU];
#pragma unroll
    for (int i = 0; i < PU; ++i) {
        const int r = i * 32 + lrow;
        voff_a[i] = r < rows_a ? static_cast<uint32_t>((r * p.lda + lchunk * 8) * 2) : kOutOfRange;
        voff_b[i] = r < rows_b ? static_cast<uint32_t>((r * p.ldw + lchunk * 8) * 2) : kOutOfRange;
    }
    // the slab range ends at ke: everything from there on reads as zeros, like the K tail
    const int k_end = min(p.K, ke * BK);
    // Slabs past the end and the part of the last slab past K read as zeros. With a K tail (KTAIL)
    // that is "this thread's chunk starts at or past K" (K is a multiple of 8, so a chunk is all in
    // or all out) and the mask is a per-lane offset bit. Without one a slab is all in or all out,
    // the mask is wave-uniform and selects a buffer resource of zero records instead, which keeps
    // the vector ALU out of the loop.
    auto slab_mask = [&](int kt) -> uint32_t {
        if constexpr (KTAIL) return kt * BK + lchunk * 8 >= k_end ? kOutOfRange : 0u;
        else return kt * BK >= k_end ? kOutOfRange : 0u;
    };
    // ring offsets are wave-uniform byte offsets of a unit inside the ring
    auto load_a = [&](int uoff, int pass, int kt, uint32_t mask) {
        if constexpr (KTAIL) {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_a, 0, bytes_a, kRsrcFlags), lds + uoff + pass * 4096 + wave * 1024,
                       voff_a[pass] | mask, kt * ROWB);
        } else {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_a, 0, mask ? 0 : bytes_a, kRsrcFlags),
                       lds + uoff + pass * 4096 + wave * 1024, voff_a[pass], kt * ROWB);
        }
    };
    auto load_w = [&](int uoff, int pass, int kt, uint32_t mask) {
        if constexpr (KTAIL) {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_b, 0, bytes_b, kRsrcFlags), lds + uoff + pass * 4096 + wave * 1024,
                       voff_b[pass] | mask, kt * ROWB);
        } else {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_b, 0, mask ? 0 : bytes_b, kRsrcFlags),
                       lds + uoff + pass * 4096 + wave * 1024, voff_b[pass], kt * ROWB);
        }
    };

    // fragment addressing
    // v_mfma_f32_16x16x32_bf16 operand: lane holds row lane % 16, k = (lane / 16) * 8 .. +8 of a K=32 step
    const int frow = lane & 15, fq = lane >> 4;
    int koff_a[KSUB], koff_w[KSUB];
#pragma unroll
    for (int kk = 0; kk < KSUB; ++kk) {
        const int ko = ((kk * 4 + fq) ^ ((frow >> 1) & 7)) * 16;
        koff_a[kk] = (wm * WROWS + frow) * ROWB + ko;
        koff_w[kk] = (wn * WCOLS + frow) * ROWB + ko;
    }

#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

    bf16x8 xa[2][FM], wb[2][FN];
    // r-th fragment of K-step kk of the slab whose units start at ua / uw, in the order the MFMAs
    // first need them: x0, w0..w(FN-1), x1..x(FM-1)
    auto read_frag = [&](int buf, int ua, int uw, int kk, int r) {
        const char* pa = lds + (ua + koff_a[kk]);
        const char* pw = lds + (uw + koff_w[kk]);
        if (r == 0) xa[buf][0] = *reinterpret_cast<const bf16x8*>(pa);
        else if (r <= FN) wb[buf][r - 1] = *reinterpret_cast<const bf16x8*>(pw + (r - 1) * 16 * ROWB);
        else xa[buf][r - FN] = *reinterpret_cast<const bf16x8*>(pa + (r - FN) * 16 * ROWB);
    };
    auto mfma_one = [&](int buf, int idx) {
        // boustrophedon over the accumulator grid: from one MFMA to the next only one of the two
        // operands changes, also at the end of a row (about 1 % less time at the power limit)
        const int i = idx / FN, j = (i & 1) ? FN - 1 - idx % FN : idx % FN;
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[buf][j], xa[buf][i], acc[i][j], 0, 0, 0);
    };

    // ua/uw: units of slab kt, ua1/uw1: of slab kt+1, ua2: of A(kt+2); W(kt+2) takes over ua once
    // the barrier has retired it. m2: load mask of slab kt+2; the mask of slab kt+3 is
    // worked out in the shadow of an MFMA so that the loop back-edge carries register moves only.
    auto slab = [&](int kt, int ua, int uw, int ua1, int uw1, int ua2, uint32_t m2, uint32_t& m3) {
        const int uw2 = ua;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NSLOT; ++s) {
            const int stp = s / READS, r = s % READS;
            if (s == GB) {
                wait_loads_and_barrier<PU>();  // slab kt+1 is complete in LDS; this slab's units are free
                __builtin_amdgcn_sched_barrier(0);
            }
            auto slot_reads = [&]() {
                if (stp < KSUB - 1) {
                    read_frag((stp & 1) ^ 1, ua, uw, stp + 1, r);
                } else if (r >= BS) {
                    // two per slot: the last one is requested a few MFMAs before the slab ends, so the
                    // wait at the top of the next slab finds it done
                    const int lo = 2 * (r - BS);
                    for (int f = lo; f < lo + 2 && f < READS; ++f) read_frag(0, ua1, uw1, 0, f);
                }
            };
            // one memory instruction per MFMA interval: the fragment read goes in front of the slot's
            // first MFMA, the buffer load behind it. The slab's first MFMA waits for the fragments
            // requested at the end of the previous slab, and that wait is for every outstanding LDS
            // read: the first read of this slab is therefore issued behind it, not in front.
            if (s != 0) slot_reads();
            mfma_one(stp & 1, r * PER);
            if (s == 0) {
                __builtin_amdgcn_sched_barrier(0);
                slot_reads();
            }
            if (s == 1) m3 = slab_mask(kt + 3);
            __builtin_amdgcn_sched_barrier(0);
            if (s < GB) {
                // A(kt+2): PU loads spread evenly over the slots in front of the barrier
#pragma unroll
                for (int i = 0; i < PU; ++i)
                    if ((i * GB) / PU == s) load_a(ua2, i, kt + 2, m2);
            } else if (s - GB < PU) {
                load_w(uw2, s - GB, kt + 2, m2);   // W(kt+2): one per slot right behind the barrier
            }
#pragma unroll
            for (int m = 1; m < PER; ++m) mfma_one(stp & 1, r * PER + m);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Prologue: slab 0, A(1) and the first loads of G(0); slab 0 must have landed, the rest flies on.
    {
        const uint32_t k0 = slab_mask(kb), k1 = slab_mask(kb + 1);
#pragma unroll
        for (int i = 0; i < PU; ++i) load_a(0, i, kb, k0);
#pragma unroll
        for (int i = 0; i < PU; ++i) load_w(UNIT, i, kb, k0);
#pragma unroll
        for (int i = 0; i < PU; ++i) load_a(2 * UNIT, i, kb + 1, k1);
#pragma unroll
        for (int i = 0; i < EARLY; ++i) load_w(3 * UNIT, i, kb + 1, k1);
        wait_loads_and_barrier<PU + EARLY>();
#pragma unroll
        for (int r = 0; r < READS; ++r) read_frag(0, 0, UNIT, 0, r);
        __builtin_amdgcn_sched_barrier(0);
    }
    static_assert(EARLY <= PU, "loads behind the barrier must all belong to W");

    {
        int ua = 0, uw = UNIT, ua1 = 2 * UNIT, uw1 = 3 * UNIT, ua2 = 4 * UNIT;
        uint32_t m2 = slab_mask(kb + 2);
        for (int kt = kb; kt < ke; ++kt) {
            uint32_t m3;
            slab(kt, ua, uw, ua1, uw1, ua2, m2, m3);
            // the ring advances by two units
            const int t0 = ua, t1 = uw;
            ua = ua1; uw = uw1; ua1 = ua2; uw1 = t0; ua2 = t1;
            m2 = m3;
        }
    }
    // The last slab's trailing loads were masked (they move no data but still write zeros to LDS):
    // retire them before the epilogue reuses the ring.
    wait_vmem_all();
    __syncthreads();
}


template <int MI, bool KTAIL>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_ring_kernel(GemmParams p) {
    constexpr int BM = 64 * MI, BK = 64, NU = 5, UNIT = BM * BK * 2;
    __shared__ __attribute__((aligned(1024))) char lds[NU * UNIT];
    int tm, tn;
    if (p.qk_cols > 0 ? !tile_of_block_qk(p, BM, tm, tn) : !tile_of_block(p, tm, tn)) return;
    const int m0 = tm * BM, n0 = tn * BM;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    f32x4 acc[2 * MI][2 * MI];
    gemm_tile_slabs<MI, KTAIL>(p, lds, m0, n0, 0, (p.K + BK - 1) / BK, acc);
    gemm_epilogue<MI, MI>(p, acc, lds, m0, n0, wave, lane);
}

// ------------------------------------------------------------------------------------------------
// Few tiles: a launch that cannot fill the CUs with 256-wide tiles is bound by the latency of its K
// loop, above all when the weights come from HBM (the first use in a forward pass): a workgroup then
// waits for every slab in turn, and what counts is how many slabs it has in flight. The ring above
// keeps one and a half; this kernel keeps ST - 1 whole slabs (A and W) of a 64*MI-wide tile in LDS
// buffers used round-robin, with one barrier per slab: behind the barrier of slab kt the buffer of slab
// kt - 1 takes slab kt + ST - 1. Fragment reads and MFMAs are left to the compiler's scheduler: the
// loop waits on memory, not on issue slots.
// ------------------------------------------------------------------------------------------------
template <int MI, int ST, bool KTAIL>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_deep_kernel(GemmParams p) {
    constexpr int FM = 2 * MI, FN = 2 * MI;
    constexpr int BM = 64 * MI, BK = 64, ROWB = BK * 2, KSUB = BK / 32;
    constexpr int UNIT = BM * ROWB, SLAB = 2 * UNIT;   // a slab: A rows, then W rows
    constexpr int PU = BM / 32, NL = 2 * PU;           // buffer loads per thread per operand / per slab
    constexpr int WROWS = 32 * MI;
    static_assert(ST >= 3 && (ST - 2) * NL <= 63 && ST * SLAB <= 160 * 1024 && 4 * WROWS * WROWS * 2 <= ST * SLAB, "ring shape");
    __shared__ __attribute__((aligned(1024))) char lds[ST * SLAB];
    int tm, tn;
    if (!tile_of_block(p, tm, tn)) return;
    const int m0 = tm * BM, n0 = tn * BM;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // loader mapping and swizzle as in gemm_tile_slabs
    const int lrow = tid >> 3;
    const int lchunk = (tid & 7) ^ ((lrow >> 1) & 7);
    const int rows_a = min(p.M - m0, BM), rows_b = min(p.N - n0, BM);
    bf16_t* const base_a = const_cast<bf16_t*>(p.A + static_cast<int64_t>(m0) * p.lda);
    bf16_t* const base_b = const_cast<bf16_t*>(p.W + static_cast<int64_t>(n0) * p.ldw);
    const int bytes_a = static_cast<int>(((rows_a - 1) * p.lda + p.K) * 2);
    const int bytes_b = static_cast<int>(((rows_b - 1) * p.ldw + p.K) * 2);
    uint32_t voff_a[PU], voff_b[PU];
#pragma unroll
    for (int i = 0; i < PU; ++i) {
        const int r = i * 32 + lrow;
        voff_a[i] = r < rows_a ? static_cast<uint32_t>((r * p.lda + lchunk * 8) * 2) : kOutOfRange;
        voff_b[i] = r < rows_b ? static_cast<uint32_t>((r * p.ldw + lchunk * 8) * 2) : kOutOfRange;
    }
    const int ke = (p.K + BK - 1) / BK;
    // slabs past the end read as zeros (and keep the count of loads in flight the same to the last slab)
    auto load_slab = [&](int soff, int kt) {
        uint32_t mask;
        if constexpr (KTAIL) mask = kt * BK + lchunk * 8 >= p.K ? kOutOfRange : 0u;
        else mask = kt >= ke ? kOutOfRange : 0u;
        const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(base_a, 0, (!KTAIL && mask) ? 0 : bytes_a, kRsrcFlags);
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(base_b, 0, (!KTAIL && mask) ? 0 : bytes_b, kRsrcFlags);
        const uint32_t lane_mask = KTAIL ? mask : 0u;
#pragma unroll
        for (int i = 0; i < PU; ++i) load_chunk(ra, lds + soff + i * 4096 + wave * 1024, voff_a[i] | lane_mask, kt * ROWB);
#pragma unroll
        for (int i = 0; i < PU; ++i) load_chunk(rb, lds + soff + UNIT + i * 4096 + wave * 1024, voff_b[i] | lane_mask, kt * ROWB);
    };

    const int frow = lane & 15, fq = lane >> 4;
    int koff_a[KSUB], koff_w[KSUB];
#pragma unroll
    for (int kk = 0; kk < KSUB; ++kk) {
        const int ko = ((kk * 4 + fq) ^ ((frow >> 1) & 7)) * 16;
        koff_a[kk] = (wm * WROWS + frow) * ROWB + ko;
        koff_w[kk] = UNIT + (wn * WROWS + frow) * ROWB + ko;
    }
    f32x4 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

#pragma unroll
    for (int s = 0; s < ST - 1; ++s) load_slab(s * SLAB, s);
    int cur = 0, nxt = (ST - 1) * SLAB;
    for (int kt = 0; kt < ke; ++kt) {
        // slab kt has landed (this wave's part: all but the loads of the ST - 2 slabs behind it; the
        // others' by the barrier), and every wave has the fragments of slab kt - 1 in registers
        wait_loads_and_barrier<(ST - 2) * NL>();
        load_slab(nxt, kt + ST - 1);
#pragma unroll
        for (int kk = 0; kk < KSUB; ++kk) {
            bf16x8 xa[FM], wb[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) xa[i] = *reinterpret_cast<const bf16x8*>(lds + cur + koff_a[kk] + i * 16 * ROWB);
#pragma unroll
            for (int j = 0; j < FN; ++j) wb[j] = *reinterpret_cast<const bf16x8*>(lds + cur + koff_w[kk] + j * 16 * ROWB);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[j], xa[i], acc[i][j], 0, 0, 0);
        }
        nxt = cur;
        cur = cur + SLAB == ST * SLAB ? 0 : cur + SLAB;
    }
    wait_vmem_all();
    __syncthreads();
    gemm_epilogue<MI, MI>(p, acc, lds, m0, n0, wave, lane);
}

// ------------------------------------------------------------------------------------------------
// Rectangular tiles: (32*FM) x (32*FN) per workgroup, a wave owns (16*FM) x (16*FN) as FM x FN
// accumulators. One workgroup per CU means a launch costs whole rounds of 256 tiles; 4608 x 3072
// (linear2 of the Flux block) is 216 tiles of 256 x 256, 0.84 of a round with 40 CUs idle, but
// exactly 256 tiles of 288 x 192 (FM = 9, FN = 6: 216 accumulation registers). The main loop is the
// one above with the two operands' slabs in rings of their own, because their units now differ in
// size: three units of A (BM rows x 128 bytes) and two of W (BN rows), 156 KB. While slab kt is
// multiplied, A(kt+1), W(kt+1) and A(kt+2) occupy the other units; behind the barrier of slab kt the
// unit of W(kt) takes W(kt+2), and the loads of A(kt+3) go into the unit of A(kt) in front of the
// next barrier. A step has FM + FN fragment reads for FM * FN MFMAs, which no longer divide: slot r
// issues MFMAs [r * MFMAS / READS, (r + 1) * MFMAS / READS), three or four of them.
// Interior tiles only (the host picks this kernel when both extents divide), one output buffer.
// ------------------------------------------------------------------------------------------------
template <int FM, int FN, bool KTAIL>
__device__ __forceinline__ void gemm_rect_slabs(const GemmParams& p, char* lds, int m0, int n0, int ke, f32x4 (&acc)[FM][FN]) {
    constexpr int BM = 32 * FM, BN = 32 * FN, BK = 64;
    constexpr int ROWB = BK * 2, KSUB = BK / 32;
    constexpr int UNIT_A = BM * ROWB, UNIT_W = BN * ROWB, W0 = 3 * UNIT_A;   // W ring behind the A ring
    constexpr int PA = BM / 32, PW = BN / 32;    // buffer loads per thread per unit of A / W
    constexpr int WROWS = 16 * FM, WCOLS = 16 * FN;
    constexpr int READS = FM + FN, MFMAS = FM * FN;
    constexpr int BS = READS / 4;                // slots of the last step in front of the barrier
    constexpr int NSLOT = KSUB * READS;          // issue slots per slab
    constexpr int GB = (KSUB - 1) * READS + BS;  // first slot behind the barrier
    static_assert(KSUB == 2 && GB >= PA && NSLOT - GB >= PW, "schedule shape");
    static_assert(2 * (NSLOT - GB) >= READS, "the next slab's first fragments are read two per slot behind the barrier");
    static_assert(BM % 32 == 0 && BN % 32 == 0 && (WROWS / 2) % 8 == 0 && (WCOLS / 2) % 8 == 0, "row swizzle must not see the wave offset");
    static_assert(3 * UNIT_A + 2 * UNIT_W <= 160 * 1024, "rings must fit the LDS");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // loader mapping as in the square kernel: LDS slot (row = pass*32 + tid/8, position tid%8) holds
    // logical chunk position ^ ((row>>1)&7) of that row
    const int lrow = tid >> 3;
    const int lchunk = (tid & 7) ^ ((lrow >> 1) & 7);
    bf16_t* const base_a = const_cast<bf16_t*>(p.A + static_cast<int64_t>(m0) * p.lda);
    bf16_t* const base_b = const_cast<bf16_t*>(p.W + static_cast<int64_t>(n0) * p.ldw);
    const int bytes_a = static_cast<int>(((BM - 1) * p.lda + p.K) * 2);
    const int bytes_b = static_cast<int>(((BN - 1) * p.ldw + p.K) * 2);
    uint32_t voff_a[PA], voff_b[PW];
#pragma unroll
    for (int i = 0; i < PA; ++i) voff_a[i] = static_cast<uint32_t>(((i * 32 + lrow) * p.lda + lchunk * 8) * 2);
#pragma unroll
    for (int i = 0; i < PW; ++i) voff_b[i] = static_cast<uint32_t>(((i * 32 + lrow) * p.ldw + lchunk * 8) * 2);
    const int k_end = min(p.K, ke * BK);
    auto slab_mask = [&](int kt) -> uint32_t {
        if constexpr (KTAIL) return kt * BK + lchunk * 8 >= k_end ? kOutOfRange : 0u;
        else return kt * BK >= k_end ? kOutOfRange : 0u;
    };
    auto load_a = [&](int uoff, int pass, int kt, uint32_t mask) {
        if constexpr (KTAIL) {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_a, 0, bytes_a, kRsrcFlags), lds + uoff + pass * 4096 + wave * 1024,
                       voff_a[pass] | mask, kt * ROWB);
        } else {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_a, 0, mask ? 0 : bytes_a, kRsrcFlags),
                       lds + uoff + pass * 4096 + wave * 1024, voff_a[pass], kt * ROWB);
        }
    };
    auto load_w = [&](int uoff, int pass, int kt, uint32_t mask) {
        if constexpr (KTAIL) {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_b, 0, bytes_b, kRsrcFlags), lds + W0 + uoff + pass * 4096 + wave * 1024,
                       voff_b[pass] | mask, kt * ROWB);
        } else {
            load_chunk(__builtin_amdgcn_make_buffer_rsrc(base_b, 0, mask ? 0 : bytes_b, kRsrcFlags),
                       lds + W0 + uoff + pass * 4096 + wave * 1024, voff_b[pass], kt * ROWB);
        }
    };

    const int frow = lane & 15, fq = lane >> 4;
    int koff_a[KSUB], koff_w[KSUB];
#pragma unroll
    for (int kk = 0; kk < KSUB; ++kk) {
        const int ko = ((kk * 4 + fq) ^ ((frow >> 1) & 7)) * 16;
        koff_a[kk] = (wm * WROWS + frow) * ROWB + ko;
        koff_w[kk] = W0 + (wn * WCOLS + frow) * ROWB + ko;
    }
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

    bf16x8 xa[2][FM], wb[2][FN];
    auto read_frag = [&](int buf, int ua, int uw, int kk, int r) {
        const char* pa = lds + (ua + koff_a[kk]);
        const char* pw = lds + (uw + koff_w[kk]);
        if (r == 0) xa[buf][0] = *reinterpret_cast<const bf16x8*>(pa);
        else if (r <= FN) wb[buf][r - 1] = *reinterpret_cast<const bf16x8*>(pw + (r - 1) * 16 * ROWB);
        else xa[buf][r - FN] = *reinterpret_cast<const bf16x8*>(pa + (r - FN) * 16 * ROWB);
    };
    auto mfma_one = [&](int buf, int idx) {
        const int i = idx / FN, j = (i & 1) ? FN - 1 - idx % FN : idx % FN;   // boustrophedon, as above
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[buf][j], xa[buf][i], acc[i][j], 0, 0, 0);
    };

    // ua, ua1, ua2: units of A(kt), A(kt+1), A(kt+2); uw, uw1: of W(kt), W(kt+1); W(kt+2) takes over uw
    // behind the barrier
    auto slab = [&](int kt, int ua, int ua1, int ua2, int uw, int uw1, uint32_t m2, uint32_t& m3) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NSLOT; ++s) {
            const int stp = s / READS, r = s % READS;
            const int lo = r * MFMAS / READS, hi = (r + 1) * MFMAS / READS;
            if (s == GB) {
                wait_loads_and_barrier<PA>();  // W(kt+1) has landed (A(kt+1) before it); this slab's units are free
                __builtin_amdgcn_sched_barrier(0);
            }
            auto slot_reads = [&]() {
                if (stp < KSUB - 1) {
                    read_frag((stp & 1) ^ 1, ua, uw, stp + 1, r);
                } else if (r >= BS) {
                    const int f0 = 2 * (r - BS);
                    for (int f = f0; f < f0 + 2 && f < READS; ++f) read_frag(0, ua1, uw1, 0, f);
                }
            };
            if (s != 0) slot_reads();
            mfma_one(stp & 1, lo);
            if (s == 0) {
                __builtin_amdgcn_sched_barrier(0);
                slot_reads();
            }
            if (s == 1) m3 = slab_mask(kt + 3);
            __builtin_amdgcn_sched_barrier(0);
            if (s < GB) {
#pragma unroll
                for (int i = 0; i < PA; ++i)
                    if ((i * GB) / PA == s) load_a(ua2, i, kt + 2, m2);
            } else if (s - GB < PW) {
                load_w(uw, s - GB, kt + 2, m2);
            }
#pragma unroll
            for (int m = lo + 1; m < hi; ++m) mfma_one(stp & 1, m);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    {
        const uint32_t k0 = slab_mask(0), k1 = slab_mask(1);
#pragma unroll
        for (int i = 0; i < PA; ++i) load_a(0, i, 0, k0);
#pragma unroll
        for (int i = 0; i < PW; ++i) load_w(0, i, 0, k0);
#pragma unroll
        for (int i = 0; i < PA; ++i) load_a(UNIT_A, i, 1, k1);
#pragma unroll
        for (int i = 0; i < PW; ++i) load_w(UNIT_W, i, 1, k1);
        wait_loads_and_barrier<PA + PW>();
#pragma unroll
        for (int r = 0; r < READS; ++r) read_frag(0, 0, 0, 0, r);
        __builtin_amdgcn_sched_barrier(0);
    }
    {
        int ua = 0, ua1 = UNIT_A, ua2 = 2 * UNIT_A, uw = 0, uw1 = UNIT_W;
        uint32_t m2 = slab_mask(2);
        for (int kt = 0; kt < ke; ++kt) {
            uint32_t m3;
            slab(kt, ua, ua1, ua2, uw, uw1, m2, m3);
            const int t0 = ua, t1 = uw;
            ua = ua1; ua1 = ua2; ua2 = t0;
            uw = uw1; uw1 = t1;
            m2 = m3;
        }
    }
    wait_vmem_all();
    __syncthreads();
}

// Epilogue of the rectangular tile: per 16-row fragment row, bias (and GELU) in fp32, one rounding,
// the 16 x WCOLS block parked in LDS and read back as 16-byte row segments: 16 * WCOLS / 8 of them, a
// whole number of wave-wide accesses, lane l of access a taking segment a * 64 + l. With a gate the
// residual rows are requested a fragment row ahead, the gate vectors once (the tile lies in one
// batch element: the host checks).
template <int FM, int FN, bool GELU, bool GATE>
__device__ __forceinline__ void gemm_epilogue_rect(const GemmParams& p, f32x4 (&acc)[FM][FN], char* lds, int m0, int n0, int wave, int lane) {
    constexpr int WROWS = 16 * FM, WCOLS = 16 * FN;
    constexpr int C_CH = WCOLS / 8;               // 16-byte segments per row
    constexpr int C_PITCH = WCOLS * 2 + 16;       // padded: an odd number of 16-byte units spreads the rows over the banks
    constexpr int NACC = 16 * C_CH / 64;          // wave-wide accesses per fragment row
    static_assert(16 * C_CH % 64 == 0, "a fragment row must be a whole number of wave-wide accesses");
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 15, fq = lane >> 4;
    char* cw = lds + wave * (2 * 16 * C_PITCH);   // two fragment rows per wave, used in turn
    const int wave_n0 = n0 + wn * WCOLS;
    const int wave_m0 = m0 + wm * WROWS;

    float bv[FN][4];
    if (p.bias != nullptr) {
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.bias), 0, p.N * 2, kRsrcFlags);
#pragma unroll
        for (int q = 0; q < FN; ++q) {
            const u32x2 raw = __builtin_amdgcn_raw_buffer_load_b64(rb, (wave_n0 + q * 16 + fq * 4) * 2, 0, 0);
            bv[q][0] = __uint_as_float(raw.x << 16);
            bv[q][1] = __uint_as_float(raw.x & 0xffff0000u);
            bv[q][2] = __uint_as_float(raw.y << 16);
            bv[q][3] = __uint_as_float(raw.y & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int q = 0; q < FN; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[q][e] = 0.0f;
    }
    const int waddr = frow * C_PITCH + fq * 8;    // + q * 32: column quad q of this lane's row
    int raddr[NACC];
    uint32_t dst_lane[NACC], res_lane[NACC];
    Vec16<bf16_t> gt[NACC];
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        const int seg = a * 64 + lane, row = seg / C_CH, ch = seg % C_CH;
        raddr[a] = row * C_PITCH + ch * 16;
        dst_lane[a] = static_cast<uint32_t>(row * p.ldy * 2 + ch * 16);
        res_lane[a] = 0;
        if (GATE) {
            res_lane[a] = static_cast<uint32_t>(row * p.ldresid * 2 + ch * 16);
            gt[a] = ld16(p.gate + static_cast<int64_t>(m0 / p.rows_per_batch) * p.gate_stride + wave_n0 + ch * 8);
        }
    }
    char* const dst_u = reinterpret_cast<char*>(p.Y + static_cast<int64_t>(wave_m0) * p.ldy + wave_n0);
    const char* const res_u = GATE ? reinterpret_cast<const char*>(p.resid + static_cast<int64_t>(wave_m0) * p.ldresid + wave_n0) : nullptr;
    Vec16<bf16_t> rs[2][NACC];
    auto request_resid = [&](int i) {
#pragma unroll
        for (int a = 0; a < NACC; ++a)
            rs[i & 1][a] = *reinterpret_cast<const Vec16<bf16_t>*>(res_u + static_cast<int64_t>(i) * 16 * p.ldresid * 2 + res_lane[a]);
    };
    if (GATE) request_resid(0);

#pragma unroll
    for (int i = 0; i < FM; ++i) {
        if (GATE) {
            if (i + 1 < FM) request_resid(i + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        char* const blk = cw + (i & 1) * (16 * C_PITCH);
#pragma unroll
        for (int q = 0; q < FN; ++q) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] = acc[i][q][e] + bv[q][e];
                if (GELU) v[e] = tanh_gelu_fast(v[e]);
            }
            *reinterpret_cast<u32x2*>(blk + waddr + q * 32) = pack4_bf16(v[0], v[1], v[2], v[3]);
        }
        __builtin_amdgcn_wave_barrier();   // LDS operations of one wave complete in order
#pragma unroll
        for (int a = 0; a < NACC; ++a) {
            Vec16<bf16_t> y = *reinterpret_cast<const Vec16<bf16_t>*>(blk + raddr[a]);
            if (GATE) {
                const Vec16<bf16_t> r = rs[i & 1][a];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float y0 = bf2f(r.v[e]) + bf2f(f2bf(bf2f(gt[a].v[e]) * bf2f(y.v[e])));
                    const float y1 = bf2f(r.v[e + 1]) + bf2f(f2bf(bf2f(gt[a].v[e + 1]) * bf2f(y.v[e + 1])));
                    const uint32_t w = pack2_bf16(y0, y1);
                    y.v[e] = static_cast<bf16_t>(w & 0xffffu);
                    y.v[e + 1] = static_cast<bf16_t>(w >> 16);
                }
            }
            *reinterpret_cast<Vec16<bf16_t>*>(dst_u + static_cast<int64_t>(i) * 16 * p.ldy * 2 + dst_lane[a]) = y;
        }
    }
}

template <int FM, int FN, bool KTAIL>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_rect_kernel(GemmParams p) {
    constexpr int BM = 32 * FM, BN = 32 * FN, BK = 64;
    __shared__ __attribute__((aligned(1024))) char lds[(3 * BM + 2 * BN) * BK * 2];
    int tm, tn;
    if (!tile_of_block(p, tm, tn)) return;
    const int m0 = tm * BM, n0 = tn * BN;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    f32x4 acc[FM][FN];
    gemm_rect_slabs<FM, FN, KTAIL>(p, lds, m0, n0, (p.K + BK - 1) / BK, acc);
    const bool gelu = p.act == FLUX_ACT_GELU_TANH;   // all columns or none: the host checks
    if (p.gate != nullptr) {
        if (gelu) gemm_epilogue_rect<FM, FN, true, true>(p, acc, lds, m0, n0, wave, lane);
        else gemm_epilogue_rect<FM, FN, false, true>(p, acc, lds, m0, n0, wave, lane);
    } else {
        if (gelu) gemm_epilogue_rect<FM, FN, true, false>(p, acc, lds, m0, n0, wave, lane);
        else gemm_epilogue_rect<FM, FN, false, false>(p, acc, lds, m0, n0, wave, lane);
    }
}

// ------------------------------------------------------------------------------------------------
// Skinny problems (M <= 8, e.g. the Modulation projection of one conditioning vector per batch
// element): HBM-bound on W. A wave streams the W rows of two output columns with 16-byte loads,
// six in flight per lane, while the few activation rows come from cache; the dot products are
// folded with a wave butterfly. The kernel is instantiated per row count, so it has no row tests.
// ------------------------------------------------------------------------------------------------
constexpr int kGemvCols = 2;  // output columns per wave
constexpr int kGemvSiluLds = 48 * 1024;  // bytes of LDS for the (activated) input rows (bf16)
// 16-byte vectors of a W row a lane requests at once: a whole row of 3072 for one or two activation rows,
// half of that when more rows' products need the registers
constexpr int gemv_depth(int rows) { return rows <= 2 ? 6 : 3; }

// SILU_LDS: the few activation rows are staged in LDS once per workgroup, with the input activation
// x * sigmoid(x) applied on the way (rounded to bf16, as the separate operator would leave it). Every
// wave needs all K values of every row: read from memory inside the K loop they queue behind the W
// loads of the wave (the memory counter is in-order), and the activation, two transcendentals per
// value, would be repeated by each of the N / 2 waves. Rows that do not fit the LDS budget are read
// from memory as they are needed.
// EXACT: K = 512 * U, so every lane has exactly U vectors per row and the K loop runs once, without tests.
template <int MM, bool SILU_LDS, bool EXACT>
__global__ __launch_bounds__(256) void gemv_small_m_kernel(GemmParams p) {
    constexpr int CPW = kGemvCols, U = gemv_depth(MM);  // CPW * U 16-byte loads of W in flight per lane: a whole row of 3072
    extern __shared__ __attribute__((aligned(16))) char act_lds[];
    const int lane = threadIdx.x & 63;
    const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * CPW;
    const bf16_t* wrow[CPW];
#pragma unroll
    for (int c = 0; c < CPW; ++c) wrow[c] = p.W + static_cast<int64_t>(n0 + c < p.N ? n0 + c : (n0 < p.N ? n0 : p.N - 1)) * p.ldw;
    // the first group of W loads goes out before the activation is worked on
    Vec16<bf16_t> w[U][CPW];
    auto request_w = [&](int k0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + u * 512;
            // past the end: a harmless re-read, skipped below
#pragma unroll
            for (int c = 0; c < CPW; ++c) w[u][c] = ld16(wrow[c] + (EXACT || k < p.K ? k : k0));
        }
    };
    if (EXACT || lane * 8 < p.K) request_w(lane * 8);
    if (SILU_LDS) {
        bf16_t* dst = reinterpret_cast<bf16_t*>(act_lds);
        for (int i = threadIdx.x * 8; i < MM * p.K; i += 256 * 8) {   // K is a multiple of 8: a vector stays inside one row
            const int m = i / p.K, k = i - m * p.K;
            const Vec16<bf16_t> a = ld16(p.A + static_cast<int64_t>(m) * p.lda + k);
            Vec16<bf16_t> o = a;
            if (p.in_silu) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float f = bf2f(a.v[e]);
                    o.v[e] = f2bf(f * __builtin_amdgcn_rcpf(1.0f + __expf(-f)));
                }
            }
            *reinterpret_cast<Vec16<bf16_t>*>(dst + i) = o;
        }
        __syncthreads();
    }
    if (n0 >= p.N) return;  // whole wave leaves together (after the barrier)
    float acc[CPW][MM];
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
        for (int m = 0; m < MM; ++m) acc[c][m] = 0.0f;
    for (int k0 = lane * 8; k0 < (EXACT ? 512 : p.K); k0 += 512 * U) {
        if (!EXACT && k0 != lane * 8) request_w(k0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + u * 512;
            if (!EXACT && k >= p.K) break;
            float af[MM][8];
#pragma unroll
            for (int m = 0; m < MM; ++m) {
                Vec16<bf16_t> a;
                if (SILU_LDS) a = *reinterpret_cast<const Vec16<bf16_t>*>(act_lds + (static_cast<size_t>(m) * p.K + k) * 2);
                else a = ld16(p.A + static_cast<int64_t>(m) * p.lda + k);
#pragma unroll
                for (int e = 0; e < 8; ++e) af[m][e] = bf2f(a.v[e]);
                if (!SILU_LDS && p.in_silu) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) af[m][e] = round_bf16(af[m][e] * __builtin_amdgcn_rcpf(1.0f + __expf(-af[m][e])));
                }
            }
#pragma unroll
            for (int c = 0; c < CPW; ++c)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float wf = bf2f(w[u][c].v[e]);
#pragma unroll
                    for (int m = 0; m < MM; ++m) acc[c][m] += wf * af[m][e];
                }
        }
    }
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
        for (int m = 0; m < MM; ++m) acc[c][m] = group_sum<64>(acc[c][m]);
    if (lane == 0) {
#pragma unroll
        for (int c = 0; c < CPW; ++c) {
            const int n = n0 + c;
            if (n >= p.N) break;
            const float b = p.bias ? bf2f(p.bias[n]) : 0.0f;
#pragma unroll
            for (int m = 0; m < MM; ++m) {
                float t = acc[c][m] + b;
                if (p.act == FLUX_ACT_GELU_TANH && n >= p.act_begin) t = gelu_tanh_f32(t);
                t = round_bf16(t);
                if (p.gate != nullptr) {
                    const float g = bf2f(p.gate[static_cast<int64_t>(m / p.rows_per_batch) * p.gate_stride + n]);
                    const float r = bf2f(p.resid[static_cast<int64_t>(m) * p.ldresid + n]);
                    t = r + round_bf16(g * t);
                }
                bf16_t* dst = n < p.split_n ? p.Y + static_cast<int64_t>(m) * p.ldy + n
                                            : p.Y2 + static_cast<int64_t>(m) * p.ldy2 + (n - p.split_n + p.y2_col0);
                *dst = f2bf(t);
            }
        }
    }
}

template <int MM>
static void launch_gemv(const GemmParams& p, hipStream_t st) {
    const unsigned grid = (unsigned)((p.N + 4 * kGemvCols - 1) / (4 * kGemvCols));
    const size_t act_bytes = static_cast<size_t>(MM) * p.K * 2;
    const bool lds = act_bytes <= kGemvSiluLds, exact = p.K == 512 * gemv_depth(MM);
    if (lds && exact) hipLaunchKernelGGL((gemv_small_m_kernel<MM, true, true>), dim3(grid), dim3(256), act_bytes, st, p);
    else if (lds) hipLaunchKernelGGL((gemv_small_m_kernel<MM, true, false>), dim3(grid), dim3(256), act_bytes, st, p);
    else if (exact) hipLaunchKernelGGL((gemv_small_m_kernel<MM, false, true>), dim3(grid), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((gemv_small_m_kernel<MM, false, false>), dim3(grid), dim3(256), 0, st, p);
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
    for (int k = 0; k < p.K; ++k) {
        float x = bf2f(a[k]);
        if (p.in_silu) x = round_bf16(x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)));
        acc += x * bf2f(w[k]);
    }
    float t = acc + (p.bias ? bf2f(p.bias[n]) : 0.0f);
    if (p.act == FLUX_ACT_GELU_TANH && n >= p.act_begin) t = gelu_tanh_f32(t);
    t = round_bf16(t);
    if (p.gate != nullptr) {
        const float g = bf2f(p.gate[static_cast<int64_t>(m / p.rows_per_batch) * p.gate_stride + n]);
        const float r = bf2f(p.resid[static_cast<int64_t>(m) * p.ldresid + n]);
        t = r + round_bf16(g * t);
    }
    bf16_t* dst = n < p.split_n ? p.Y + static_cast<int64_t>(m) * p.ldy + n
                                : p.Y2 + static_cast<int64_t>(m) * p.ldy2 + (n - p.split_n + p.y2_col0);
    *dst = f2bf(t);
}

template <int MI>
static void launch_tiled(GemmParams& p, hipStream_t st) {
    constexpr int BM = 64 * MI;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BM - 1) / BM;
    p.group_m = 4;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    if (p.K % 64 == 0) hipLaunchKernelGGL((gemm_nt_ring_kernel<MI, false>), dim3(grid), dim3(kGemmThreads), 0, st, p);
    else hipLaunchKernelGGL((gemm_nt_ring_kernel<MI, true>), dim3(grid), dim3(kGemmThreads), 0, st, p);
}

template <int MI, int ST>
static void launch_deep(GemmParams& p, hipStream_t st) {
    constexpr int BM = 64 * MI;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BM - 1) / BM;
    p.group_m = 4;
    const int grid = ((p.tiles_m * p.tiles_n + 7) / 8) * 8;
    if (p.K % 64 == 0) hipLaunchKernelGGL((gemm_nt_deep_kernel<MI, ST, false>), dim3(grid), dim3(kGemmThreads), 0, st, p);
    else hipLaunchKernelGGL((gemm_nt_deep_kernel<MI, ST, true>), dim3(grid), dim3(kGemmThreads), 0, st, p);
}

// Rectangular tile shapes the host may pick: 288 x 192 and 256 x 192.
template <int FM, int FN>
static void launch_rect(GemmParams& p, hipStream_t st) {
    constexpr int BM = 32 * FM, BN = 32 * FN;
    p.tiles_m = p.M / BM;
    p.tiles_n = p.N / BN;
    p.group_m = 4;
    const int grid = ((p.tiles_m * p.tiles_n + 7) / 8) * 8;
    if (p.K % 64 == 0) hipLaunchKernelGGL((gemm_nt_rect_kernel<FM, FN, false>), dim3(grid), dim3(kGemmThreads), 0, st, p);
    else hipLaunchKernelGGL((gemm_nt_rect_kernel<FM, FN, true>), dim3(grid), dim3(kGemmThreads), 0, st, p);
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
    if ((a->flags & ~static_cast<int64_t>(FLUX_LINEAR_SHARED_GPU)) != 0) return fail(FLUX_E_UNSUPPORTED, "flux_linear_bf16: unknown flags 0x%llx", (unsigned long long)a->flags);
    if (a->in_act != FLUX_ACT_NONE && a->in_act != FLUX_ACT_SILU) return fail(FLUX_E_UNSUPPORTED, "flux_linear_bf16: unknown input activation %d", a->in_act);
    if (a->in_act == FLUX_ACT_SILU && (a->M > 8 || a->qk != nullptr)) return fail(FLUX_E_UNSUPPORTED, "flux_linear_bf16: input SiLU is for M <= 8 without the qk fusion (M=%lld)", (long long)a->M);
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
    p.in_silu = a->in_act == FLUX_ACT_SILU;
    p.act = a->act; p.act_begin = (int)(a->act_begin < 0 ? 0 : (a->act_begin > a->N ? a->N : a->act_begin));
    p.tiles_m = p.tiles_n = 0; p.group_m = 4;
    p.bias_vec = a->bias != nullptr && (reinterpret_cast<uintptr_t>(a->bias) & 3u) == 0 && a->N % 4 == 0;
    p.vec_io = aligned16(a->Y) && a->ldy % 8 == 0 &&
               (!split || (aligned16(a->Y2) && a->ldy2 % 8 == 0 && a->split_n % 8 == 0 && a->y2_col0 % 8 == 0)) &&
               (!a->gate || (aligned16(a->gate) && aligned16(a->resid) && a->ldresid % 8 == 0 && a->gate_batch_stride % 8 == 0));

    p.q_out = p.k_out = nullptr; p.q_scale = p.k_scale = nullptr; p.pe = nullptr; p.pe_batch_stride = 0;
    p.qk_cols = p.qk_heads = p.qk_seq_len = p.qk_out_len = p.qk_pos0 = 0; p.qk_eps = 0.0f;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a->qk != nullptr) {
        const flux_linear_qk_fusion* f = a->qk;
        if (!f->q_out || !f->k_out || !f->q_scale || !f->k_scale || !f->pe) return fail(FLUX_E_NULL, "flux_linear_bf16: qk fusion with a null pointer");
        const int64_t cols = 2 * f->heads * 128;
        const bool shape_ok = f->heads > 0 && f->seq_len >= 256 && a->M % f->seq_len == 0 && a->N % 256 == 0 &&
                              cols <= a->N && f->pos0 >= 0 && f->pos0 + f->seq_len <= f->out_len && f->out_len < 0x7fffff &&
                              f->heads * f->out_len * 256 < 0x7fffffffLL &&
                              f->pe_batch_stride >= 0 && a->K > 0 && a->K % 8 == 0;
        const bool epi_ok = a->gate == nullptr && p.act_begin >= cols && p.split_n >= cols &&
                            (a->bias == nullptr || p.bias_vec) && p.vec_io;
        const bool ptr_ok = aligned16(f->q_out) && aligned16(f->k_out) && aligned16(f->pe) && f->pe_batch_stride % 4 == 0 &&
                            (reinterpret_cast<uintptr_t>(f->q_scale) & 3u) == 0 && (reinterpret_cast<uintptr_t>(f->k_scale) & 3u) == 0 &&
                            aligned16(a->A) && aligned16(a->W) && a->lda % 8 == 0 && a->ldw % 8 == 0 &&
                            a->lda * 2 * 256 < 0x7fffffffLL && a->ldw * 2 * 256 < 0x7fffffffLL;
        if (!shape_ok || !epi_ok || !ptr_ok)
            return fail(FLUX_E_UNSUPPORTED, "flux_linear_bf16: qk fusion needs N in multiples of 256, sequences of at least 256 rows, "
                                            "aligned operands, no gate, and GELU / split columns behind the k heads");
        p.q_out = static_cast<bf16_t*>(f->q_out); p.k_out = static_cast<bf16_t*>(f->k_out);
        p.q_scale = static_cast<const bf16_t*>(f->q_scale); p.k_scale = static_cast<const bf16_t*>(f->k_scale);
        p.pe = f->pe; p.pe_batch_stride = f->pe_batch_stride;
        p.qk_cols = (int)cols; p.qk_heads = (int)f->heads; p.qk_seq_len = (int)f->seq_len; p.qk_out_len = (int)f->out_len;
        p.qk_pos0 = (int)f->pos0; p.qk_eps = f->eps;
        launch_tiled<4>(p, st);   // a wave's 128 columns are one head
        return check_launch("flux_linear_bf16");
    }
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
        switch (p.M) {
            case 1: launch_gemv<1>(p, st); break;
            case 2: launch_gemv<2>(p, st); break;
            case 3: launch_gemv<3>(p, st); break;
            case 4: launch_gemv<4>(p, st); break;
            case 5: launch_gemv<5>(p, st); break;
            case 6: launch_gemv<6>(p, st); break;
            case 7: launch_gemv<7>(p, st); break;
            default: launch_gemv<8>(p, st); break;
        }
        return check_launch("flux_linear_bf16");
    }
    // 256 x 256 tiles once they fill most of the 256 CUs; below that 128 x 128 tiles (two workgroups
    // per CU) spread the work better than they lose in operand re-reads.
    const int64_t big_tiles = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256);
    const int64_t mid_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
    // 256-wide tiles once they fill most of the chip; below that 128-wide ones (two workgroups per
    // CU); problems with too few of those to give every second CU one are bound by the latency of
    // the K loop and run on 64-wide tiles with a deeper ring, four times as many workgroups.
    // Rectangular tiles (288 x 192 or 256 x 192) when both extents divide and their rounds come out
    // shorter than those of the other tiles. Measured at K = 3072: a round of square tiles 69 us, a
    // round of 288 x 192 tiles 62 us (0.84 of the work at 1.06 times the cost per flop), a launch on
    // 128-wide tiles 0.57 to 0.65 of a square round per wave of 512 workgroups, plus a kernel boundary
    // when it is the tail of a split launch. 4608 x 3072 is 216 square tiles = one round with 40 CUs
    // idle, and 256 tiles of 288 x 192; 4608 x 12288 is 3 square rounds and a tail, or 4 rounds of
    // 288 x 192; 4096 x 3072 is 192 square tiles, and 256 tiles of 256 x 192; 2816 x 3072 is two
    // rounds of 128-wide tiles, the second nearly empty, and 176 tiles of 256 x 192.
    const bool rect_form = !(a->flags & FLUX_LINEAR_SHARED_GPU) && p.vec_io && p.Y2 == nullptr && (p.bias == nullptr || p.bias_vec) &&
                           (p.act == FLUX_ACT_NONE || p.act_begin == 0);
    // cost in square rounds of tiles of rbm x rbn, or a large number where they do not fit
    auto rect_cost = [&](int rbm, int rbn) -> double {
        const bool ok = rect_form && p.M % rbm == 0 && p.N % rbn == 0 && (p.gate == nullptr || p.rows_per_batch % rbm == 0) &&
                        a->lda * 2 * rbm < 0x7fffffffLL && a->ldw * 2 * rbn < 0x7fffffffLL;   // 32-bit byte offsets inside a tile's rows
        if (!ok) return 1e30;
        const int64_t rt = static_cast<int64_t>(p.M / rbm) * (p.N / rbn);
        return static_cast<double>((rt + kGemmCUs - 1) / kGemmCUs) * (rbm * rbn / 65536.0) * 1.06;
    };
    // launches on the cheaper rectangular shape if that costs less than `other` (in square rounds)
    auto rect_if_cheaper = [&](double other) -> bool {
        const double c96 = rect_cost(288, 192), c86 = rect_cost(256, 192);
        if (!(std::min(c96, c86) < 0.97 * other)) return false;
        if (c96 <= c86) launch_rect<9, 6>(p, st);
        else launch_rect<8, 6>(p, st);
        return true;
    };
    if (big_tiles >= 160) {
        // One workgroup per CU: a launch whose last round is mostly empty pays for a whole round
        // (864 tiles of mlp_in at 4608 rows = 3.375 rounds cost 4). When a leading block of whole
        // tile rows fills whole rounds, it is launched on 256-wide tiles and the few rows left over
        // follow on 128-wide ones, two workgroups per CU, in one more short round.
        const int tm = (p.M + 255) / 256, tn = (p.N + 255) / 256;
        const int last = static_cast<int>(big_tiles % kGemmCUs);
        int mb = 0;
        if (big_tiles > kGemmCUs && last != 0 && last < kGemmCUs / 2) {
            for (int c = tm - 1; c >= 1 && mb == 0; --c) {
                const int64_t rest_rows = p.M - static_cast<int64_t>(c) * 256;
                const int64_t rest_tiles = ((rest_rows + 127) / 128) * ((p.N + 127) / 128);
                if (rest_tiles > 2 * kGemmCUs) break;
                const int fill = static_cast<int>((static_cast<int64_t>(c) * tn) % kGemmCUs);
                if ((fill == 0 || fill >= kGemmCUs * 9 / 10) && (p.gate == nullptr || (c * 256) % p.rows_per_batch == 0)) mb = c;
            }
        }
        double sq = static_cast<double>((big_tiles + kGemmCUs - 1) / kGemmCUs);
        if (mb) {
            const int64_t rest_tiles = ((p.M - static_cast<int64_t>(mb) * 256 + 127) / 128) * ((p.N + 127) / 128);
            sq = static_cast<double>((static_cast<int64_t>(mb) * tn + kGemmCUs - 1) / kGemmCUs) +
                 0.65 * static_cast<double>((rest_tiles + 2 * kGemmCUs - 1) / (2 * kGemmCUs)) + 0.1;
        }
        if (rect_if_cheaper(sq)) return check_launch("flux_linear_bf16");
        if (mb == 0) {
            launch_tiled<4>(p, st);
        } else {
            const int row0 = mb * 256;
            GemmParams head = p, tail = p;
            head.M = row0;
            tail.M = p.M - row0;
            tail.A += static_cast<int64_t>(row0) * p.lda;
            tail.Y += static_cast<int64_t>(row0) * p.ldy;
            if (tail.Y2 != nullptr) tail.Y2 += static_cast<int64_t>(row0) * p.ldy2;
            if (tail.resid != nullptr) tail.resid += static_cast<int64_t>(row0) * p.ldresid;
            if (tail.gate != nullptr) tail.gate += static_cast<int64_t>(row0 / p.rows_per_batch) * p.gate_stride;
            launch_tiled<4>(head, st);
            launch_tiled<2>(tail, st);
        }
    }
    // up to one round of 64-wide tiles at two workgroups per CU: the K loop's latency is the whole cost,
    // and the kernel that keeps three slabs in flight wins (3072 x 3072 weights from HBM: 256 rows
    // 39 -> 24 us, 512 rows 44 -> 35 us; from 768 rows on the 128-wide tiles are faster again)
    else if (mid_tiles <= kGemmCUs / 2 && !(a->flags & FLUX_LINEAR_SHARED_GPU)) launch_deep<1, 4>(p, st);   // beside another stream: few, larger workgroups
    else if (!rect_if_cheaper(0.57 * static_cast<double>((mid_tiles + 2 * kGemmCUs - 1) / (2 * kGemmCUs)))) launch_tiled<2>(p, st);
    return check_launch("flux_linear_bf16");
}
