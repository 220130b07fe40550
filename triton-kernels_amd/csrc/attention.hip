// Non-causal flash-attention forward on the matrix cores (bf16 in, fp32 softmax state, bf16 out).
//
// Everything is computed transposed so that a lane owns one query row for its whole life:
//     S^T[key, q] = K Q^T        (MFMA "A" = K rows from LDS, "B" = Q rows held in registers)
//     O^T[d,   q] = V^T P^T      (MFMA "A" = V^T rows from LDS, "B" = P^T straight from the S^T
//                                 accumulator registers)
// With v_mfma_f32_32x32x16_bf16 the accumulator of lane l holds column q = l % 32 and 16 rows, so
// the running max / sum / rescale of the online softmax are per-lane scalars; the only cross-lane
// step is one exchange between the two half-waves that share a query row. P never touches LDS: the
// 8 accumulator values a lane holds for a 16-key step are exactly the 8 contraction elements the
// "B" operand wants, provided V^T is laid out with the same key order, which the V loader does.
//
// A workgroup of 4 waves handles 128*QB query rows of one (batch, head); each wave 32*QB rows.
// K and V tiles of 64 keys are double-buffered in LDS; V is transposed on the way in (4 keys x 8 d
// per thread, written as eight 8-byte rows of V^T).
#include "common.h"
#include <stdlib.h>

namespace flux {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct AttnParams {
    const bf16_t* q; const bf16_t* k; const bf16_t* v; bf16_t* o; float* lse;
    int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, o_sb, o_sh, o_sl;
    int H, L, n_qtiles, total_tiles;
    float scale_log2;  // sm_scale * log2(e)
};

constexpr unsigned kAttnRsrcFlags = 0x00020000u;
constexpr uint32_t kAttnOutOfRange = 0x80000000u;

__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
    return static_cast<uint32_t>(f2bf(a)) | (static_cast<uint32_t>(f2bf(b)) << 16);
}

template <int D, int QB>
__global__ __launch_bounds__(256) void attn_fwd_kernel(AttnParams p) {
    constexpr int BN = 64;              // keys per tile
    constexpr int KSTEPS = D / 16;      // contraction steps of S^T = K Q^T
    constexpr int DB = D / 32;          // 32-row blocks of O^T
    constexpr int CH = D / 8;           // 16-byte chunks per K row
    constexpr int KROW = D * 2;         // bytes per K row in LDS
    constexpr int K_BYTES = BN * KROW, V_BYTES = D * 128, STAGE = K_BYTES + V_BYTES;
    constexpr int KPASS = BN * CH / 256;  // K loader passes (16-byte chunks per thread)
    constexpr int KROWS_PER_PASS = 256 / CH;
    constexpr int VTHREADS = CH * 16;   // threads that take part in the V loader (4 keys x 8 d each)
    __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE];

    // XCD-aware order: workgroup w runs on XCD w % 8; each XCD gets a contiguous run of
    // (head, q-tile) pairs so the K/V of a head is pulled into one L2 only.
    const int per_xcd = gridDim.x / 8;
    const int vt = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (vt >= p.total_tiles) return;
    const int bh = vt / p.n_qtiles, qt = vt % p.n_qtiles;
    const int b = bh / p.H, h = bh % p.H;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int frow = lane & 31, fhalf = lane >> 5;
    const int q0 = qt * (128 * QB) + wave * (32 * QB);

    const bf16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
    const bf16_t* vbase = p.v + b * p.v_sb + h * p.v_sh;

    // ---- Q fragments ("B" operand): lane holds row q0 + qb*32 + frow, d = (kk*2 + fhalf)*8 .. +8
    bf16x8 qf[QB][KSTEPS];
    {
        const bf16_t* qbase = p.q + b * p.q_sb + h * p.q_sh;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const int row = q0 + qb * 32 + frow;
            const bool ok = row < p.L;
            const bf16_t* rp = qbase + static_cast<int64_t>(ok ? row : 0) * p.q_sl;
#pragma unroll
            for (int kk = 0; kk < KSTEPS; ++kk) {
                u32x4 t = {0u, 0u, 0u, 0u};
                if (ok) t = *reinterpret_cast<const u32x4*>(rp + (kk * 2 + fhalf) * 8);
                qf[qb][kk] = __builtin_bit_cast(bf16x8, t);
            }
        }
    }

    // ---- loader mappings
    const int kl_c = tid % CH, kl_r = tid / CH;             // K: chunk, row within pass
    const int vl_dc = tid % CH, vl_kg = (tid / CH) & 15;    // V: d-chunk, group of 4 keys
    const bool v_active = tid < VTHREADS;
    u32x4 kreg[KPASS], vreg[4];

    auto issue_loads = [&](int key0) {
        const int rows = min(p.L - key0, BN);
        const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<bf16_t*>(kbase + static_cast<int64_t>(key0) * p.k_sl), 0,
            static_cast<int>(((rows - 1) * p.k_sl + D) * 2), kAttnRsrcFlags);
        const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<bf16_t*>(vbase + static_cast<int64_t>(key0) * p.v_sl), 0,
            static_cast<int>(((rows - 1) * p.v_sl + D) * 2), kAttnRsrcFlags);
#pragma unroll
        for (int i = 0; i < KPASS; ++i) {
            const int r = i * KROWS_PER_PASS + kl_r;
            const uint32_t vo = r < rows ? static_cast<uint32_t>((r * p.k_sl + kl_c * 8) * 2) : kAttnOutOfRange;
            kreg[i] = __builtin_amdgcn_raw_buffer_load_b128(rk, vo, 0, 0);
        }
        if (v_active) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = vl_kg * 4 + i;
                const uint32_t vo = r < rows ? static_cast<uint32_t>((r * p.v_sl + vl_dc * 8) * 2) : kAttnOutOfRange;
                vreg[i] = __builtin_amdgcn_raw_buffer_load_b128(rv, vo, 0, 0);
            }
        }
    };
    auto commit_loads = [&](int stage) {
        char* sk = lds + stage * STAGE;
        char* sv = sk + K_BYTES;
#pragma unroll
        for (int i = 0; i < KPASS; ++i) {
            const int r = i * KROWS_PER_PASS + kl_r;
            *reinterpret_cast<u32x4*>(sk + r * KROW + ((kl_c ^ (r & 7)) * 16)) = kreg[i];
        }
        if (v_active) {
            // vreg[i] = V[key 4*kg + i][d = dc*8 .. +8]; emit for each d one 8-byte run of the 4 keys.
            // Key order inside a group of 16 is quads [0,2,1,3]: half-wave h of the MFMA then finds its
            // 8 keys {4h..4h+3, 8+4h..8+4h+3} in one 16-byte unit.
            const int quad = vl_kg & 3;
            const int qpos = (quad == 1) ? 2 : (quad == 2 ? 1 : quad);
            const int u8 = (vl_kg >> 2) * 4 + qpos;  // 8-byte unit inside the 128-byte V^T row
            const int unit = u8 >> 1, half = u8 & 1;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int d = vl_dc * 8 + e;
                const int w = e >> 1;
                uint32_t a0 = vreg[0][w], a1 = vreg[1][w], a2 = vreg[2][w], a3 = vreg[3][w];
                u32x2 out;
                if (e & 1) {
                    out.x = (a0 >> 16) | (a1 & 0xffff0000u);
                    out.y = (a2 >> 16) | (a3 & 0xffff0000u);
                } else {
                    out.x = (a0 & 0xffffu) | (a1 << 16);
                    out.y = (a2 & 0xffffu) | (a3 << 16);
                }
                const int swz = (d & 7) ^ ((d >> 3) & 7);
                *reinterpret_cast<u32x2*>(sv + d * 128 + ((unit ^ swz) * 16) + half * 8) = out;
            }
        }
    };

    // ---- softmax state (per lane = per query row of each q-block)
    float m_run[QB], l_run[QB];
    f32x16 acc[QB][DB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.0f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[qb][db][r] = 0.0f;
    }
    const float c = p.scale_log2;

    const int ntiles = (p.L + BN - 1) / BN;
    issue_loads(0);
    commit_loads(0);
    __syncthreads();

    for (int t = 0; t < ntiles; ++t) {
        const int cur = t & 1;
        const int key0 = t * BN;
        if (t + 1 < ntiles) issue_loads(key0 + BN);
        const char* sk = lds + cur * STAGE;
        const char* sv = sk + K_BYTES;

        // S^T = K Q^T
        f32x16 s[QB][2];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[qb][kb][r] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
            bf16x8 kf[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const int row = kb * 32 + frow;
                kf[kb] = *reinterpret_cast<const bf16x8*>(sk + row * KROW + (((kk * 2 + fhalf) ^ (lane & 7)) * 16));
            }
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
                    s[qb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb], qf[qb][kk], s[qb][kb], 0, 0, 0);
        }

        // ragged tail: keys past L get -inf
        if (key0 + BN > p.L) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * fhalf + (r & 3);
                        if (key >= p.L) s[qb][kb][r] = -INFINITY;
                    }
        }

        // online softmax, P^T packed to bf16 as the "B" operand of the second product
        bf16x8 pf[QB][4];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            float mx = s[qb][0][0];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[qb][kb][r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[qb], mx);
            const float alpha = m_run[qb] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f((m_run[qb] - m_new) * c);
            const float mc = m_new * c;
            m_run[qb] = m_new;
            float sum = 0.0f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                float pv[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    pv[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qb][kb][r], c, -mc));
                    sum += pv[r];
                }
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    u32x4 w;
                    w.x = pack2_bf16(pv[8 * tt + 0], pv[8 * tt + 1]);
                    w.y = pack2_bf16(pv[8 * tt + 2], pv[8 * tt + 3]);
                    w.z = pack2_bf16(pv[8 * tt + 4], pv[8 * tt + 5]);
                    w.w = pack2_bf16(pv[8 * tt + 6], pv[8 * tt + 7]);
                    pf[qb][kb * 2 + tt] = __builtin_bit_cast(bf16x8, w);
                }
            }
            l_run[qb] = l_run[qb] * alpha + sum;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[qb][db][r] *= alpha;
        }

        // O^T += V^T P^T
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int d = db * 32 + frow;
                const int swz = (d & 7) ^ ((d >> 3) & 7);
                const bf16x8 vf = *reinterpret_cast<const bf16x8*>(sv + d * 128 + (((ks * 2 + fhalf) ^ swz) * 16));
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
                    acc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qb][ks], acc[qb][db], 0, 0, 0);
            }
        }

        if (t + 1 < ntiles) commit_loads(cur ^ 1);
        __syncthreads();
    }

    // ---- finish: fold the two half-waves' partial sums, normalise, store
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 32, 64);
        const float inv = 1.0f / l_tot;
        const int row = q0 + qb * 32 + frow;
        if (row < p.L) {
            bf16_t* orow = p.o + b * p.o_sb + h * p.o_sh + static_cast<int64_t>(row) * p.o_sl;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w.x = pack2_bf16(acc[qb][db][g * 4 + 0] * inv, acc[qb][db][g * 4 + 1] * inv);
                    w.y = pack2_bf16(acc[qb][db][g * 4 + 2] * inv, acc[qb][db][g * 4 + 3] * inv);
                    *reinterpret_cast<u32x2*>(orow + db * 32 + g * 8 + fhalf * 4) = w;
                }
            if (p.lse != nullptr && fhalf == 0)
                p.lse[static_cast<int64_t>(bh) * p.L + row] = m_run[qb] * c + __builtin_amdgcn_logf(l_tot);
        }
    }
}

template <int D, int QB>
static void attn_launch(AttnParams& p, int64_t BH, hipStream_t st) {
    const int rows_per_wg = 128 * QB;
    p.n_qtiles = (p.L + rows_per_wg - 1) / rows_per_wg;
    p.total_tiles = static_cast<int>(p.n_qtiles * BH);
    const int grid = ((p.total_tiles + 7) / 8) * 8;
    hipLaunchKernelGGL((attn_fwd_kernel<D, QB>), dim3(grid), dim3(256), 0, st, p);
}

static int attn_variant() {
    static int v = [] {
        const char* e = getenv("FLUX_ATTN_VARIANT");
        return e ? atoi(e) : 0;
    }();
    return v;
}

}  // namespace flux

using namespace flux;

static bool view_ok(const void* ptr, int64_t sb, int64_t sh, int64_t sl) {
    return ptr != nullptr && aligned16(ptr) && sb % 8 == 0 && sh % 8 == 0 && sl % 8 == 0;
}

extern "C" int flux_attention_fwd_bf16(const flux_attn_args* a, void* stream) {
    if (!a) return fail(FLUX_E_NULL, "flux_attention_fwd_bf16: null args");
    if (a->B < 0 || a->H <= 0 || a->L < 0) return fail(FLUX_E_SHAPE, "flux_attention_fwd_bf16: bad shape B=%lld H=%lld L=%lld", (long long)a->B, (long long)a->H, (long long)a->L);
    if (a->D != 64 && a->D != 128) return fail(FLUX_E_UNSUPPORTED, "flux_attention_fwd_bf16: head dim %d not supported (64, 128)", a->D);
    if (!(a->sm_scale >= 0.0f)) return fail(FLUX_E_UNSUPPORTED, "flux_attention_fwd_bf16: sm_scale must be >= 0");
    if (a->B == 0 || a->L == 0) return FLUX_OK;
    if (a->L > 0x7fffffff / 64 || a->B * a->H > 0x7fffffff / 64) return fail(FLUX_E_SHAPE, "flux_attention_fwd_bf16: problem too large");
    if (!view_ok(a->q.ptr, a->q.sb, a->q.sh, a->q.sl) || !view_ok(a->k.ptr, a->k.sb, a->k.sh, a->k.sl) ||
        !view_ok(a->v.ptr, a->v.sb, a->v.sh, a->v.sl) || !view_ok(a->o, a->o_sb, a->o_sh, a->o_sl))
        return fail(FLUX_E_ALIGN, "flux_attention_fwd_bf16: q/k/v/o must be non-null, 16-byte aligned, with strides that are multiples of 8");
    if (a->k.sl * 2 * 64 >= 0x7fffffffLL || a->v.sl * 2 * 64 >= 0x7fffffffLL) return fail(FLUX_E_SHAPE, "flux_attention_fwd_bf16: row stride too large");

    AttnParams p;
    p.q = static_cast<const bf16_t*>(a->q.ptr); p.k = static_cast<const bf16_t*>(a->k.ptr);
    p.v = static_cast<const bf16_t*>(a->v.ptr); p.o = static_cast<bf16_t*>(a->o); p.lse = a->lse;
    p.q_sb = a->q.sb; p.q_sh = a->q.sh; p.q_sl = a->q.sl;
    p.k_sb = a->k.sb; p.k_sh = a->k.sh; p.k_sl = a->k.sl;
    p.v_sb = a->v.sb; p.v_sh = a->v.sh; p.v_sl = a->v.sl;
    p.o_sb = a->o_sb; p.o_sh = a->o_sh; p.o_sl = a->o_sl;
    p.H = (int)a->H; p.L = (int)a->L;
    p.scale_log2 = a->sm_scale * 1.4426950408889634f;
    const int64_t BH = a->B * a->H;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int variant = attn_variant();
    // Two q-blocks per wave halve the LDS traffic per flop; one q-block gives twice the workgroups,
    // which small problems need to fill the chip.
    const bool small = ((a->L + 255) / 256) * BH < 256;
    const int qb = variant == 1 ? 1 : (variant == 2 ? 2 : (small ? 1 : 2));
    if (a->D == 128) {
        if (qb == 1) attn_launch<128, 1>(p, BH, st); else attn_launch<128, 2>(p, BH, st);
    } else {
        if (qb == 1) attn_launch<64, 1>(p, BH, st); else attn_launch<64, 2>(p, BH, st);
    }
    return check_launch("flux_attention_fwd_bf16");
}
