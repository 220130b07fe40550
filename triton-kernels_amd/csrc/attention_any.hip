// Scaled-dot-product attention forward for the head dims the pipelined kernels leave out
// (16, 32 and 256 of the set {16, 32, 64, 128, 256} that kernels/attention.py:184 accepts).
//
// A plain flash-attention loop, one 32-key tile at a time, with no software pipelining beyond a
// register prefetch of the next tile. A workgroup of four waves owns 64 query rows, 16 per wave.
// Everything is computed transposed with v_mfma_f32_16x16x32_bf16 (A: row = lane % 16, 8 k-values
// at (lane / 16) * 8; B: column = lane % 16, the same k-values; C/D: column = lane % 16, rows
// (lane / 16) * 4 .. + 3):
//     S^T = K Q^T      A = K fragment (16 bytes of a key row from LDS), B = Q fragment (registers),
//     O^T += V^T P^T   A = V^T fragment (two transposing LDS reads), B = P^T.
// The lane that holds column q of S^T holds, per 16-key block, keys (lane / 16) * 4 .. + 3: eight
// probabilities of query q per 32-key tile. They are used as the lane's eight k-values of P^T as
// they are; the V^T fragment is read with its keys in the same order, so no data crosses lanes
// between the two products. Row maxima and sums are reduced across the four lanes of a query.
// Scores are scaled in fp32 after the first product (no rounding of a pre-scaled Q), keys past the
// end of the sequence score -inf and their V rows are zero-filled in LDS.
#include "attention_params.h"

#include <math.h>

namespace flux {

typedef __bf16 pbf16x8 __attribute__((ext_vector_type(8)));
typedef float pf32x4 __attribute__((ext_vector_type(4)));
typedef short ps16x4 __attribute__((ext_vector_type(4)));
typedef short ps16x8 __attribute__((ext_vector_type(8)));

constexpr int kPlainKeys = 32;   // keys per tile
constexpr int kPlainRows = 64;   // query rows per workgroup

template <int D>
__global__ __launch_bounds__(256) void attn_fwd_plain_kernel(AttnParams p) {
    constexpr int BN = kPlainKeys;
    constexpr int KS = (D + 31) / 32;           // k-steps of the first product (the last one half empty for D = 16)
    constexpr int DB = D / 16;                  // 16-column blocks of O
    constexpr int RS = D * 2 + 16;              // LDS row stride in bytes: rows 16 bytes apart in bank phase
    constexpr int CPR = D / 8;                  // 16-byte chunks per row
    constexpr int CH = BN * CPR;                // chunks per tile
    constexpr int NCH = (CH + 255) / 256;       // chunks per thread
    static_assert(D % 16 == 0 && D <= 256, "head dim");
    __shared__ __attribute__((aligned(16))) char lds[2 * BN * RS];
    char* const lds_k = lds;
    char* const lds_v = lds + BN * RS;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int L = p.L;
    const int64_t bh = blockIdx.x / p.n_qtiles;
    const int qt = static_cast<int>(blockIdx.x % p.n_qtiles);
    const int64_t b = bh / p.H, h = bh % p.H;
    const bf16_t* qp = p.q + b * p.q_sb + h * p.q_sh;
    const bf16_t* kp = p.k + b * p.k_sb + h * p.k_sh;
    const bf16_t* vp = p.v + b * p.v_sb + h * p.v_sh;
    bf16_t* op = p.o + b * p.o_sb + h * p.o_sh;

    const int qrow_raw = qt * kPlainRows + wave * 16 + l16;
    const bool q_ok = qrow_raw < L;
    const int qrow = q_ok ? qrow_raw : L - 1;

    const uint4 zero4 = make_uint4(0, 0, 0, 0);
    pbf16x8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + g * 8;
        const uint4 raw = d < D ? *reinterpret_cast<const uint4*>(qp + static_cast<int64_t>(qrow) * p.q_sl + d) : zero4;
        qf[ks] = __builtin_bit_cast(pbf16x8, raw);
    }

    uint4 kreg[NCH], vreg[NCH];
    auto gload = [&](int t0) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * 256;
            const int key = t0 + c / CPR, col = (c % CPR) * 8;
            const bool ok = c < CH && key < L;
            kreg[i] = ok ? *reinterpret_cast<const uint4*>(kp + static_cast<int64_t>(key) * p.k_sl + col) : zero4;
            vreg[i] = ok ? *reinterpret_cast<const uint4*>(vp + static_cast<int64_t>(key) * p.v_sl + col) : zero4;
        }
    };
    auto sstore = [&]() {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * 256;
            if (c < CH) {
                const int off = (c / CPR) * RS + (c % CPR) * 16;
                *reinterpret_cast<uint4*>(lds_k + off) = kreg[i];
                *reinterpret_cast<uint4*>(lds_v + off) = vreg[i];
            }
        }
    };

    float m = -INFINITY, lsum = 0.0f;
    pf32x4 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) o[db] = pf32x4{0.0f, 0.0f, 0.0f, 0.0f};

    gload(0);
    for (int t0 = 0; t0 < L; t0 += BN) {
        __syncthreads();  // every wave is done reading the previous tile
        sstore();
        __syncthreads();
        if (t0 + BN < L) gload(t0 + BN);

        // S^T for the two 16-key blocks of the tile
        pf32x4 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            s[kb] = pf32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int d = ks * 32 + g * 8;
                const uint4 raw = d < D ? *reinterpret_cast<const uint4*>(lds_k + (kb * 16 + l16) * RS + d * 2) : zero4;
                s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pbf16x8, raw), qf[ks], s[kb], 0, 0, 0);
            }
        }
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int key = t0 + (j >> 2) * 16 + g * 4 + (j & 3);
            sv[j] = key < L ? s[j >> 2][j & 3] * p.scale_log2 : -INFINITY;
            mx = fmaxf(mx, sv[j]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float mn = fmaxf(m, mx);
        const float alpha = __builtin_amdgcn_exp2f(m - mn);  // 0 on the first tile (m = -inf)
        m = mn;
        float pv[8], ps = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            pv[j] = __builtin_amdgcn_exp2f(sv[j] - mn);
            ps += pv[j];
        }
        lsum = lsum * alpha + ps;
        pbf16x8 pb;
#pragma unroll
        for (int j = 0; j < 8; ++j) pb[j] = static_cast<__bf16>(pv[j]);

        // O^T += V^T P^T: the transposing read hands lane i of a 16-lane group column i of a 4 x 16
        // block whose row r is addressed by lanes 4r .. 4r+3 (8 bytes each): rows are this group's
        // four keys of a 16-key block, columns the 16 head-dim columns of block db.
        const char* vbase = lds_v + (g * 4 + (l16 >> 2)) * RS + (l16 & 3) * 8;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const ps16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ps16x4*)(vbase + db * 32));
            const ps16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ps16x4*)(vbase + 16 * RS + db * 32));
            const ps16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            o[db] *= alpha;
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pbf16x8, a), pb, o[db], 0, 0, 0);
        }
    }

    lsum += __shfl_xor(lsum, 16);
    lsum += __shfl_xor(lsum, 32);
    const float inv = 1.0f / lsum;
    if (q_ok) {
        bf16_t* orow = op + static_cast<int64_t>(qrow) * p.o_sl + g * 4;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            uint2 w;
            w.x = static_cast<uint32_t>(f2bf(o[db][0] * inv)) | (static_cast<uint32_t>(f2bf(o[db][1] * inv)) << 16);
            w.y = static_cast<uint32_t>(f2bf(o[db][2] * inv)) | (static_cast<uint32_t>(f2bf(o[db][3] * inv)) << 16);
            *reinterpret_cast<uint2*>(orow + db * 16) = w;
        }
        if (p.lse != nullptr && g == 0) p.lse[bh * L + qrow] = m + __builtin_amdgcn_logf(lsum);
    }
}

void attn_launch_plain(const AttnParams& p0, int64_t BH, int D, hipStream_t st) {
    AttnParams p = p0;
    p.n_qtiles = (p.L + kPlainRows - 1) / kPlainRows;
    p.total_tiles = static_cast<int>(BH * p.n_qtiles);
    const dim3 grid(static_cast<unsigned>(p.total_tiles)), block(256);
    if (D == 16) hipLaunchKernelGGL(attn_fwd_plain_kernel<16>, grid, block, 0, st, p);
    else if (D == 32) hipLaunchKernelGGL(attn_fwd_plain_kernel<32>, grid, block, 0, st, p);
    else hipLaunchKernelGGL(attn_fwd_plain_kernel<256>, grid, block, 0, st, p);
}

}  // namespace flux
