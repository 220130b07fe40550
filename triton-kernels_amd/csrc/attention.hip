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
// "B" operand wants, provided the V^T fragment uses the same key order, which its two transposing
// reads (keys 4h..4h+3 and 8+4h..8+4h+3 of the step) do.
//
// A workgroup of 4 waves handles 128*QB query rows of one (batch, head); each wave 32*QB rows. With
// QB = 1 two workgroups share a CU, so each SIMD interleaves two waves and the softmax VALU work of
// one overlaps the MFMAs of the other. K and V tiles of 64 keys are double-buffered in LDS, both
// row-major, filled by buffer loads that write LDS directly; the V^T fragments are produced by the
// transposing LDS read ds_read_b64_tr_b16.
#include "common.h"
#include <stdlib.h>

namespace flux {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct AttnParams {
    const bf16_t* q; const bf16_t* k; const bf16_t* v; bf16_t* o; float* lse;
    int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, o_sb, o_sh, o_sl;
    int H, L, n_qtiles, total_tiles;
    float scale_log2;  // sm_scale * log2(e)
};

constexpr unsigned kAttnRsrcFlags = 0x00020000u;
constexpr uint32_t kAttnOutOfRange = 0x80000000u;

typedef float f32x2 __attribute__((ext_vector_type(2)));
// Two floats -> one dword of two bf16 (a in the low half): a single v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// One buffer load of 64 x 16 bytes written straight into LDS at dst + lane * 16.
__device__ __forceinline__ void lds_load16(__amdgpu_buffer_rsrc_t rsrc, char* dst, uint32_t voff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, voff, 0, 0, 0);
}
__device__ __forceinline__ void wait_all_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

typedef short s16x4 __attribute__((ext_vector_type(4)));
// ds_read_b64_tr_b16: inside each group of 16 lanes, lanes 4r..4r+3 together supply row r (16
// consecutive 16-bit elements, 8 bytes per lane) of a 4 x 16 matrix; lane i of the group receives
// column i, i.e. the 4 elements (row 0..3)[i].
__device__ __forceinline__ s16x4 lds_read_tr(const char* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
}

template <int D, int QB>
__global__ __launch_bounds__(256, (QB == 1 ? 2 : 1)) void attn_fwd_kernel(AttnParams p) {
    constexpr int BN = 64;              // keys per tile
    constexpr int KSTEPS = D / 16;      // contraction steps of S^T = K Q^T
    constexpr int DB = D / 32;          // 32-row blocks of O^T
    constexpr int CH = D / 8;           // 16-byte chunks per K / V row
    constexpr int ROWB = D * 2;         // bytes per K / V row in LDS
    constexpr int RPW = 64 / CH;        // rows one wave-wide load covers (1 KB)
    constexpr int PASSES = BN / (4 * RPW);  // loads per thread per operand per tile
    constexpr int T_BYTES = BN * ROWB, STAGE = 2 * T_BYTES;
    __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE];

    // XCD-aware order: workgroup w runs on XCD w % 8; each XCD gets a contiguous run of
    // (head, q-tile) pairs so the K/V of a head is pulled into one L2 only.
    const int per_xcd = gridDim.x / 8;
    const int vt = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (vt >= p.total_tiles) return;
    const int bh = vt / p.n_qtiles, qt = vt % p.n_qtiles;
    const int b = bh / p.H, h = bh % p.H;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 31, fhalf = lane >> 5;
    const int q0 = qt * (128 * QB) + wave * (32 * QB);

    const bf16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
    const bf16_t* vbase = p.v + b * p.v_sb + h * p.v_sh;

    // LDS row swizzles (64 banks of 4 bytes; a b128 read is served 16 lanes per clock, a b64 read 32):
    //   K rows are read whole-chunk by 16 lanes on 16 consecutive rows  -> chunk ^ kswz(row)
    //   V rows are read transposed, 4 rows x 64 bytes per clock         -> chunk ^ vswz(row)
    auto kswz = [](int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); };
    auto vswz = [](int row) { return D == 128 ? ((row & 3) * 4) : (((row >> 1) & 1) * 4); };

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

    // ---- loader: thread -> LDS slot (row = pass*4*RPW + wave*RPW + lane/CH, position lane%CH)
    const int l_row = lane / CH, l_pos = lane % CH;
    // Byte offsets of this thread's chunks inside a tile; rows past the end of the sequence fall
    // outside the buffer resource built for the tile and read as zeros.
    uint32_t k_voff[PASSES], v_voff[PASSES];
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
        const int r = i * 4 * RPW + wave * RPW + l_row;
        k_voff[i] = static_cast<uint32_t>((r * p.k_sl + (l_pos ^ kswz(r)) * 8) * 2);
        v_voff[i] = static_cast<uint32_t>((r * p.v_sl + (l_pos ^ vswz(r)) * 8) * 2);
    }
    auto issue_loads = [&](int key0, int stage) {
        const int rows = min(p.L - key0, BN);
        const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<bf16_t*>(kbase + static_cast<int64_t>(key0) * p.k_sl), 0,
            static_cast<int>(((rows - 1) * p.k_sl + D) * 2), kAttnRsrcFlags);
        const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<bf16_t*>(vbase + static_cast<int64_t>(key0) * p.v_sl), 0,
            static_cast<int>(((rows - 1) * p.v_sl + D) * 2), kAttnRsrcFlags);
        char* sk = lds + stage * STAGE + wave * 1024;
        char* sv = sk + T_BYTES;
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            lds_load16(rk, sk + i * 4096, k_voff[i]);
            lds_load16(rv, sv + i * 4096, v_voff[i]);
        }
    };

    // ---- fragment addressing
    // K ("A" of S^T): row kb*32 + frow, chunk kk*2 + fhalf
    const int k_sw = kswz(frow);  // kb*32 does not change the swizzle
    // V^T ("A" of O^T): lane group g = lane/16 -> (half h = g/2 = fhalf, d sub-block g%2); lane j = lane%16
    // supplies 8 bytes of key row 4h + j/4 (+8 for the second read) at d = db*32 + (g%2)*16 + 4*(j%4)
    const int vj = lane & 15, vg = (lane >> 4) & 1;
    const int v_key = 4 * fhalf + (vj >> 2);                  // + 16*ks (+8)
    const int v_chunk = vg * 2 + ((vj & 3) >> 1);             // + db*4
    const int v_in = (vj & 1) * 8;
    const int v_sw = vswz(v_key);                             // unchanged by + 8, + 16*ks
    int k_addr[KSTEPS], v_addr[DB];                           // per-lane parts, the rest are immediates
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) k_addr[kk] = frow * ROWB + (((kk * 2 + fhalf) ^ k_sw) * 16);
#pragma unroll
    for (int db = 0; db < DB; ++db) v_addr[db] = T_BYTES + v_key * ROWB + (((db * 4 + v_chunk) ^ v_sw) * 16) + v_in;

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
    issue_loads(0, 0);
    wait_all_vmem();
    __syncthreads();

    for (int t = 0; t < ntiles; ++t) {
        const int cur = t & 1;
        const int key0 = t * BN;
        if (t + 1 < ntiles) issue_loads(key0 + BN, cur ^ 1);
        const char* sk = lds + cur * STAGE;

        // S^T = K Q^T
        f32x16 s[QB][2];
        const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        __builtin_amdgcn_s_setprio(1);  // the other wave on this SIMD is in its softmax: let the MFMAs go first
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
            bf16x8 kf[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
                kf[kb] = *reinterpret_cast<const bf16x8*>(sk + kb * 32 * ROWB + k_addr[kk]);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
                    s[qb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb], qf[qb][kk], kk == 0 ? zero16 : s[qb][kb], 0, 0, 0);
        }

        __builtin_amdgcn_s_setprio(0);

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
            float mx = fmaxf(s[qb][0][0], s[qb][1][0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, s[qb][0][r]), s[qb][1][r]);  // v_max3_f32
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[qb], mx);
            // The accumulator only needs rescaling when some row's running max moved; after the first
            // few tiles that is rare, so the whole wave skips the multiplies when no lane needs them.
            if (__builtin_amdgcn_ballot_w64(m_new != m_run[qb]) != 0) {
                const float alpha = m_run[qb] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f((m_run[qb] - m_new) * c);
                l_run[qb] *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[qb][db][r] *= alpha;
                m_run[qb] = m_new;
            }
            const float mc = m_new * c;
            float sum = 0.0f;
            const uint32_t ones = 0x3f803f80u;  // (1.0bf16, 1.0bf16)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                uint32_t w[8];
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qb][kb][2 * r], c, -mc));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qb][kb][2 * r + 1], c, -mc));
                    w[r] = pack2_bf16(p0, p1);
                    // row sum from the rounded values, two per instruction: sum += p0*1 + p1*1
                    sum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w[r]), __builtin_bit_cast(bf16x2, ones), sum, false);
                }
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    u32x4 v4 = {w[4 * tt], w[4 * tt + 1], w[4 * tt + 2], w[4 * tt + 3]};
                    pf[qb][kb * 2 + tt] = __builtin_bit_cast(bf16x8, v4);
                }
            }
            l_run[qb] += sum;
        }

        // O^T += V^T P^T ; V^T fragments come out of row-major V through transposing LDS reads
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const char* vp = sk + ks * 16 * ROWB + v_addr[db];
                const s16x4 lo = lds_read_tr(vp);
                const s16x4 hi = lds_read_tr(vp + 8 * ROWB);
                typedef short s16x8 __attribute__((ext_vector_type(8)));
                const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                const bf16x8 vf = __builtin_bit_cast(bf16x8, both);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
                    acc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qb][ks], acc[qb][db], 0, 0, 0);
            }
        }

        __builtin_amdgcn_s_setprio(0);
        wait_all_vmem();   // this wave's part of the next tile has landed
        __syncthreads();   // everybody's has; and everybody is done reading this tile
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
    // One q-block (32 rows) per wave keeps the kernel under 256 registers, so two workgroups share a
    // CU and the two waves on each SIMD overlap softmax with MFMA; two q-blocks per wave halve the LDS
    // traffic per flop but run one wave per SIMD.
    const int qb = variant == 2 ? 2 : 1;
    if (a->D == 128) {
        if (qb == 1) attn_launch<128, 1>(p, BH, st); else attn_launch<128, 2>(p, BH, st);
    } else {
        if (qb == 1) attn_launch<64, 1>(p, BH, st); else attn_launch<64, 2>(p, BH, st);
    }
    return check_launch("flux_attention_fwd_bf16");
}
