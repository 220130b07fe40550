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
// QB = 1 the kernel stays under 256 registers and two workgroups share a CU, so each SIMD has a
// second wave to issue from. K and V tiles of BN keys live row-major in LDS, filled by buffer loads
// that write LDS directly; the V^T fragments are produced by the transposing LDS read
// ds_read_b64_tr_b16 (which tops out near 72 bytes per clock per CU, against ~210 for the 16-byte
// reads of the K fragments, and is what bounds this kernel: every wave re-reads the whole V tile).
//
// The loop is software-pipelined. The body of tile t issues
//     S^T(t+1) = K(t+1) Q^T    while the VALU works through the softmax of S^T(t), and then
//     O^T     += V(t)^T P(t)^T while the softmax finishes (P is consumed one 16-key step at a time),
// as a fixed sequence of slots: one MFMA, a small piece of the softmax, the LDS fragment reads a
// few slots ahead of their use and, now and then, a buffer load of a later tile. Scheduling
// barriers pin that order. K has two LDS buffers and V three, because the one workgroup barrier per
// tile sits in the middle of the body (after the last K fragment read, before the first V fragment
// read): at that point K(t+1) is retired and refilled with K(t+3), while the V buffer being
// refilled is the one read a whole iteration earlier.
#include "common.h"
#include <stdlib.h>
#include <type_traits>

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

typedef float f32x2 __attribute__((ext_vector_type(2)));
// Two floats -> one dword of two bf16 (a in the low half): a single v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ void wait_all_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

typedef short s16x4 __attribute__((ext_vector_type(4)));
// ds_read_b64_tr_b16: inside each group of 16 lanes, lanes 4r..4r+3 together supply row r (16
// consecutive 16-bit elements, 8 bytes per lane) of a 4 x 16 matrix; lane i of the group receives
// column i, i.e. the 4 elements (row 0..3)[i].
__device__ __forceinline__ s16x4 lds_read_tr(const char* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
}

// LDS-writing buffer load issued from inline asm. The compiler's wait-count pass puts
// "s_waitcnt vmcnt(0)" in front of every LDS read it cannot tell apart from the target of an
// outstanding LDS-writing buffer load it knows of (the transposing reads are such reads), which
// would serialise a kernel that keeps such loads in flight all the time. Issued this way the loads
// are invisible to that pass; the kernel waits for them itself in front of its barriers.
// lds_addr: wave-uniform LDS byte address the 64 x 16 bytes go to; rsrc: buffer descriptor.
__device__ __forceinline__ void lds_load16_raw(u32x4 rsrc, uint32_t lds_addr, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc)
                 : "memory");  // m0 is written; nothing else in this file's kernel reads it (LDS ops need no m0 on gfx9+)
}
__device__ __forceinline__ uint32_t lds_addr_of(const char* p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const char*)p));
}

// All but the newest N buffer loads of this wave have landed and its LDS reads have returned, then
// the workgroup barrier; the memory clobber keeps LDS accesses on their side of it.
template <int N>
__device__ __forceinline__ void attn_wait_and_barrier() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Compile-time loop: f(std::integral_constant<int, I>{}) for I in [B, E).
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// Slot of softmax unit g of a tile (see the kernel): units are spread evenly behind the max phase.
constexpr int attn_unit_slot(int g, int qb_count, int nslot, int nunits) {
    return 5 * qb_count + g * (nslot - 9 * qb_count) / nunits;
}
// Every 16-key step of P^T must be complete before the first MFMA that takes it.
constexpr bool attn_units_in_time(int qb_count, int ns, int db_count, int nslot, int ksteps16) {
    for (int ks = 0; ks < ksteps16; ++ks)
        for (int qb = 0; qb < qb_count; ++qb) {
            const int last = ks * 4 * qb_count + qb * 4 + 3;
            if (attn_unit_slot(last, qb_count, nslot, ksteps16 * 4 * qb_count) >= ns + ks * db_count * qb_count + qb) return false;
        }
    return true;
}

template <int D, int QB, int BN>  // BN = keys per tile (32 or 64)
__global__ __launch_bounds__(256, (QB == 1 ? 2 : 1)) void attn_fwd_pipe_kernel(AttnParams p) {
    constexpr int KB = BN / 32;         // 32-key blocks of S^T per tile
    constexpr int PS = BN / 16;         // 16-key steps of P^T per tile
    constexpr int KSTEPS = D / 16;      // contraction steps of S^T = K Q^T
    constexpr int DB = D / 32;          // 32-row blocks of O^T
    constexpr int CH = D / 8;           // 16-byte chunks per K / V row
    constexpr int ROWB = D * 2;         // bytes per K / V row in LDS
    constexpr int RPW = 64 / CH;        // rows one wave-wide load covers (1 KB)
    constexpr int PASSES = BN / (4 * RPW);  // loads per thread per operand per tile
    constexpr int T_BYTES = BN * ROWB;
    constexpr int NKF = KB * KSTEPS;    // K fragments per tile, each feeds QB MFMAs
    constexpr int NVF = PS * DB;        // V^T fragments per tile, each feeds QB MFMAs
    constexpr int NS = NKF * QB;        // MFMAs of S^T
    constexpr int NP = NVF * QB;        // MFMAs of O^T
    constexpr int NSLOT = NS + NP;
    constexpr int KD = 4, KRN = (KD + 2 * QB - 1) / QB;   // K fragments are read KD slots ahead of their first use
    constexpr int VD = 4, VRN = (VD + 2 * QB - 1) / QB;   // V fragments VD slots ahead
    constexpr int BAR = NS - VD;        // slot in front of which the barrier sits
    constexpr int NU = 4 * PS * QB;     // softmax units (two accumulator values each) per tile
    static_assert(NSLOT - KD >= BAR && BAR + 2 * PASSES <= NSLOT && (NKF - 1) * QB - KD < BAR, "slot plan");
    static_assert(attn_units_in_time(QB, NS, DB, NSLOT, PS), "P^T steps must be ready before the MFMAs that take them");
    __shared__ __attribute__((aligned(1024))) char lds[5 * T_BYTES];  // K: 2 buffers, V: 3 buffers
    constexpr int V0 = 2 * T_BYTES;

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

    // LDS row swizzles (64 banks of 4 bytes; a b128 read is served 16 lanes per clock):
    //   K rows are read whole-chunk by 16 lanes on 16 consecutive rows  -> chunk ^ kswz(row)
    //   V rows are read transposed, 4 rows x 64 bytes at a time         -> chunk ^ vswz(row)
    auto kswz = [](int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); };
    auto vswz = [](int row) { return D == 128 ? ((row & 3) * 4) : (((row >> 1) & 1) * 4); };

    // Q fragments ("B" operand): lane holds row q0 + qb*32 + frow, d = (kk*2 + fhalf)*8 .. +8
    bf16x8 qf[QB][KSTEPS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int row = q0 + qb * 32 + frow;
        const bool ok = row < p.L;
        const bf16_t* rp = p.q + b * p.q_sb + h * p.q_sh + static_cast<int64_t>(ok ? row : 0) * p.q_sl;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
            u32x4 t = *reinterpret_cast<const u32x4*>(rp + (kk * 2 + fhalf) * 8);
            if (!ok) t = u32x4{0u, 0u, 0u, 0u};
            qf[qb][kk] = __builtin_bit_cast(bf16x8, t);
        }
    }

    // loader: thread -> LDS slot (row = pass*4*RPW + wave*RPW + lane/CH, position lane%CH)
    const int l_row = lane / CH, l_pos = lane % CH;
    uint32_t k_voff[PASSES], v_voff[PASSES];
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
        const int r = i * 4 * RPW + wave * RPW + l_row;
        k_voff[i] = static_cast<uint32_t>((r * p.k_sl + (l_pos ^ kswz(r)) * 8) * 2);
        v_voff[i] = static_cast<uint32_t>((r * p.v_sl + (l_pos ^ vswz(r)) * 8) * 2);
    }
    // Buffer resource of a 64-key tile starting at key0; keys at or past L are outside it and read
    // as zeros (a tile wholly past L has an empty resource: its base is never dereferenced).
    const int k_row2 = static_cast<int>(p.k_sl * 2), v_row2 = static_cast<int>(p.v_sl * 2);
    auto tile_rsrc = [&](const bf16_t* base, int row2, int key0) -> u32x4 {
        const int rows = min(p.L - key0, BN);
        const int bytes = rows > 0 ? (rows - 1) * row2 + D * 2 : 0;
        const uint64_t addr = reinterpret_cast<uint64_t>(base) + static_cast<uint64_t>(static_cast<int64_t>(key0) * row2);
        u32x4 r;
        r.x = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr));
        r.y = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr >> 32) & 0xffffu);  // stride 0: raw buffer
        r.z = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bytes));
        r.w = kAttnRsrcFlags;
        return r;
    };
    const uint32_t lds_base = lds_addr_of(lds) + wave * 1024;  // this wave's 1 KB inside a 4 KB loader pass

    // fragment addressing
    // K ("A" of S^T): row kb*32 + frow, chunk kk*2 + fhalf; kb*32 does not change the swizzle.
    // V^T ("A" of O^T): lane group g = lane/16 -> (half = g/2 = fhalf, d sub-block g%2); lane j = lane%16
    // supplies 8 bytes of key row 4*fhalf + j/4 (+8 for the second read, +16 per key step) at
    // d = db*32 + (g%2)*16 + 4*(j%4); vswz is unchanged by + 8 and + 16*ks.
    const int k_sw = kswz(frow);
    const int vj = lane & 15, vg = (lane >> 4) & 1;
    const int v_key = 4 * fhalf + (vj >> 2);
    const int v_chunk = vg * 2 + ((vj & 3) >> 1);
    const int v_in = (vj & 1) * 8;
    const int v_sw = vswz(v_key);
    int k_addr[KSTEPS], v_addr[DB];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) k_addr[kk] = frow * ROWB + (((kk * 2 + fhalf) ^ k_sw) * 16);
#pragma unroll
    for (int db = 0; db < DB; ++db) v_addr[db] = v_key * ROWB + (((db * 4 + v_chunk) ^ v_sw) * 16) + v_in;

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
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int ntiles = (p.L + BN - 1) / BN;

    bf16x8 kf[KRN];  // K fragment ring, indexed by fragment number % KRN
    bf16x8 vf[VRN];  // V^T fragment ring
    auto read_k = [&](int kbuf, int n) {  // n-th K fragment of a tile: step n/KB, key block n%KB; kbuf is a constant
        const int kk = n / KB, kb = n % KB;
        kf[n % KRN] = *reinterpret_cast<const bf16x8*>(lds + k_addr[kk] + (kbuf + kb * 32 * ROWB));
    };
    int v_cur_addr[DB];  // v_addr + offset of the V buffer in use, refreshed once per tile
    auto read_v = [&](auto m_c) {  // m-th V^T fragment: key step m/DB, d block m%DB
        constexpr int m = decltype(m_c)::value, ks = m / DB, db = m % DB;
        const char* vp = lds + v_cur_addr[db] + ks * 16 * ROWB;
        const s16x4 lo = lds_read_tr(vp);
        const s16x4 hi = lds_read_tr(vp + 8 * ROWB);
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        vf[m % VRN] = __builtin_bit_cast(bf16x8, both);
    };

    // ---- prologue: K(0), V(0), K(1); S^T(0) without overlap; then K(2), V(1) on their way
    {
        const u32x4 rk0 = tile_rsrc(kbase, k_row2, 0), rv0 = tile_rsrc(vbase, v_row2, 0);
        const u32x4 rk1 = tile_rsrc(kbase, k_row2, BN);
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            lds_load16_raw(rk0, lds_base + i * 4096, k_voff[i]);
            lds_load16_raw(rv0, lds_base + V0 + i * 4096, v_voff[i]);
            lds_load16_raw(rk1, lds_base + T_BYTES + i * 4096, k_voff[i]);
        }
        attn_wait_and_barrier<0>();
    }
    f32x16 sa[QB][KB], sb[QB][KB];  // S^T of the tile in its softmax / of the tile being multiplied
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            const bf16x8 f = *reinterpret_cast<const bf16x8*>(lds + kb * 32 * ROWB + k_addr[kk]);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
                sa[qb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f, qf[qb][kk], kk == 0 ? zero16 : sa[qb][kb], 0, 0, 0);
        }
    }
    attn_wait_and_barrier<0>();  // everybody is done with K(0)
    {
        const u32x4 rk2 = tile_rsrc(kbase, k_row2, 2 * BN), rv1 = tile_rsrc(vbase, v_row2, BN);
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            lds_load16_raw(rk2, lds_base + i * 4096, k_voff[i]);
            lds_load16_raw(rv1, lds_base + V0 + T_BYTES + i * 4096, v_voff[i]);
        }
    }
#pragma unroll
    for (int n = 0; n < NKF; ++n)
        if (n * QB < KD) read_k(T_BYTES, n);  // first fragments of K(1)
    __builtin_amdgcn_sched_barrier(0);

    float mx[QB], mc[QB], sum[QB];
    uint32_t pw[QB][4 * PS];
    bf16x8 pf[QB][PS];

    // One tile. s_cur = S^T(t) (consumed), s_nxt = S^T(t+1) (produced). kcur = LDS offset of K(t+1),
    // which is refilled with K(t+3) behind the barrier; vcur = offset of V(t); vnew = offset of the V
    // buffer that takes V(t+2).
    auto tile = [&](int t, f32x16 (&s_cur)[QB][KB], f32x16 (&s_nxt)[QB][KB], auto kcur_c, int vcur, int vnew) {
        constexpr int kcur = decltype(kcur_c)::value, knext = T_BYTES - kcur;
        const int key0 = t * BN;
#pragma unroll
        for (int db = 0; db < DB; ++db) v_cur_addr[db] = v_addr[db] + vcur;
        if (key0 + BN > p.L) {  // ragged tail: keys past L get -inf
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * fhalf + (r & 3);
                        if (key >= p.L) s_cur[qb][kb][r] = -INFINITY;
                    }
        }
        const u32x4 rk = tile_rsrc(kbase, k_row2, key0 + 3 * BN);
        const u32x4 rv = tile_rsrc(vbase, v_row2, key0 + 2 * BN);
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, NSLOT>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            if constexpr (s == BAR) {
                // K(t+2) and V(t+1) have landed (issued behind the previous barrier); all waves are
                // done reading K(t+1), and V(t-1) was retired an iteration ago
                attn_wait_and_barrier<0>();
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- matrix pipe
            if constexpr (s < NS) {
                constexpr int n = s / QB, qb = s % QB, kk = n / KB, kb = n % KB;
                s_nxt[qb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[n % KRN], qf[qb][kk], kk == 0 ? zero16 : s_nxt[qb][kb], 0, 0, 0);
            } else {
                constexpr int m = (s - NS) / QB, qb = (s - NS) % QB, ks = m / DB, db = m % DB;
                acc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[m % VRN], pf[qb][ks], acc[qb][db], 0, 0, 0);
            }
            // ---- LDS fragment reads for later slots
            static_for<0, NKF>([&](auto n_c) {
                constexpr int n = decltype(n_c)::value;
                if constexpr (n * QB - KD == s) read_k(kcur, n);
                if constexpr (n * QB - KD + NSLOT == s) read_k(knext, n);  // first fragments of K(t+2) for the next tile
            });
            static_for<0, NVF>([&](auto m_c) {
                constexpr int m = decltype(m_c)::value;
                if constexpr (NS + m * QB - VD == s) read_v(m_c);
            });
            // ---- buffer loads of later tiles, one per slot behind the barrier
            if constexpr (s >= BAR && s < BAR + 2 * PASSES) {
                constexpr int i = (s - BAR) / 2;
                if constexpr ((s - BAR) % 2 == 0) lds_load16_raw(rk, lds_base + kcur + i * 4096, k_voff[i]);
                else lds_load16_raw(rv, lds_base + vnew + i * 4096, v_voff[i]);
            }
            // ---- softmax of S^T(t): running max of each q-block over four slots, ...
            if constexpr (s < 4 * QB) {
                constexpr int qb = s / 4;
#pragma unroll
                for (int r = 4 * (s % 4); r < 4 * (s % 4) + 4; ++r) {
                    if (r == 0) mx[qb] = s_cur[qb][0][0];
                    else mx[qb] = fmaxf(mx[qb], s_cur[qb][0][r]);
                    if (KB == 2) mx[qb] = fmaxf(mx[qb], s_cur[qb][1][r]);  // the pairs fuse into v_max3_f32
                }
            }
            // ... the new row maximum and, when it moved, the rescale, ...
            if constexpr (s >= 4 * QB && s < 5 * QB) {
                constexpr int qb = s - 4 * QB;
                mx[qb] = fmaxf(mx[qb], __shfl_xor(mx[qb], 32, 64));
                const float m_new = fmaxf(m_run[qb], mx[qb]);
                // The accumulator only needs rescaling when some row's running max moved; after the
                // first few tiles that is rare, so the whole wave skips the multiplies otherwise.
                if (__builtin_amdgcn_ballot_w64(m_new != m_run[qb]) != 0) {
                    const float alpha = m_run[qb] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f((m_run[qb] - m_new) * c);
                    l_run[qb] *= alpha;
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[qb][db][r] *= alpha;
                    m_run[qb] = m_new;
                }
                mc[qb] = m_new * c;
                sum[qb] = 0.0f;
            }
            // ... and the exponentials, two accumulator values per unit, in the order the MFMAs of
            // O^T take the 16-key steps of P^T (step-major, q-block inside)
            static_for<0, NU>([&](auto g_c) {
                constexpr int g = decltype(g_c)::value;
                if constexpr (attn_unit_slot(g, QB, NSLOT, NU) == s) {
                constexpr int ks = g / (4 * QB), qb = (g / 4) % QB, u = ks * 4 + g % 4;
                constexpr int kb = u / 8, r = (u % 8) * 2;
                // The empty asm ties the unit's inputs to this slot: without it the optimiser is free
                // to hoist all the (mutually independent) exponentials into one clump.
                asm volatile("" : "+v"(s_cur[qb][kb]));
                const float a0 = s_cur[qb][kb][r], a1 = s_cur[qb][kb][r + 1];
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(a0, c, -mc[qb]));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(a1, c, -mc[qb]));
                pw[qb][u] = pack2_bf16(p0, p1);
                // row sum from the rounded values, two per instruction: sum += p0*1 + p1*1
                sum[qb] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pw[qb][u]), __builtin_bit_cast(bf16x2, 0x3f803f80u), sum[qb], false);
                if (u % 4 == 3) {  // a 16-key step of P^T is complete
                    const u32x4 v4 = {pw[qb][u - 3], pw[qb][u - 2], pw[qb][u - 1], pw[qb][u]};
                    pf[qb][u / 4] = __builtin_bit_cast(bf16x8, v4);
                }
                if (u == 4 * PS - 1) l_run[qb] += sum[qb];
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // K buffers alternate (a compile-time constant per tile parity); V buffers rotate through three.
    // Two tiles per trip so that the two S^T accumulators swap roles without register moves.
    int vcur = V0, vnew = V0 + 2 * T_BYTES, vmid = V0 + T_BYTES;  // V(t), buffer for V(t+2), V(t+1)
    auto advance = [&]() {
        const int tv = vcur; vcur = vmid; vmid = vnew; vnew = tv;
    };
    using odd_k = std::integral_constant<int, T_BYTES>;   // K(t+1) of an even tile t sits in the second buffer
    using even_k = std::integral_constant<int, 0>;
    int t = 0;
    for (; t + 1 < ntiles; t += 2) {
        tile(t, sa, sb, odd_k{}, vcur, vnew);
        advance();
        tile(t + 1, sb, sa, even_k{}, vcur, vnew);
        advance();
    }
    if (t < ntiles) tile(t, sa, sb, odd_k{}, vcur, vnew);
    wait_all_vmem();  // loads of tiles past the end are empty but still count

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

template <int D, int QB, int BN>
static void attn_launch_pipe(AttnParams& p, int64_t BH, hipStream_t st) {
    p.n_qtiles = (p.L + 128 * QB - 1) / (128 * QB);
    p.total_tiles = static_cast<int>(p.n_qtiles * BH);
    const int grid = ((p.total_tiles + 7) / 8) * 8;
    hipLaunchKernelGGL((attn_fwd_pipe_kernel<D, QB, BN>), dim3(grid), dim3(256), 0, st, p);
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
    // One q-block (32 rows) per wave keeps the kernel under 256 registers, so two workgroups share a
    // CU and each SIMD has a second wave to issue from while the first waits.
    if (a->D == 128) attn_launch_pipe<128, 1, 64>(p, BH, st);
    else attn_launch_pipe<64, 1, 64>(p, BH, st);
    return check_launch("flux_attention_fwd_bf16");
}
