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
#include "attention_params.h"
#include <stdlib.h>
#include <mutex>
#include <type_traits>

namespace flux {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

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
                 : "memory", "m0");
}
// The same with the LDS address given as a scalar base plus a constant.
template <int OFF>
__device__ __forceinline__ void lds_load16_raw_at(u32x4 rsrc, uint32_t lds_base, uint32_t voff) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_base), "v"(voff), "s"(rsrc), "n"(OFF)
                 : "memory", "scc", "m0");
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

#ifndef FLUX_ATTN_W64_D64_UNIT   // the 32-row kernel belongs to the main unit only
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
            // sm_scale*log2(e) goes into Q once (rounded to bf16), so scores leave the MFMA in the
            // base-2 domain whatever the sign of the scale, and masked keys stay -inf for scale 0
#pragma unroll
            for (int e = 0; e < 4; ++e)
                t[e] = pack2_bf16(__uint_as_float(t[e] << 16) * p.scale_log2, __uint_as_float(t[e] & 0xffff0000u) * p.scale_log2);
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
    constexpr float c = 1.0f;  // the scale is already in Q
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


#endif  // FLUX_ATTN_W64_D64_UNIT

// ------------------------------------------------------------------------------------------------
// Head dim 128, 64 query rows per wave, one wave per SIMD, v_mfma_f32_16x16x32_bf16.
//
// The kernel above gives every wave 32 query rows, so a wave reads a whole K and a whole V tile
// from LDS for 32 rows' worth of MFMA work; at full MFMA rate that is more than the LDS can
// deliver (the transposing V^T reads run at about 70 bytes per clock per CU). Here a wave owns 64
// rows (four 16-row blocks), every K / V^T fragment feeds four MFMAs, and LDS traffic per flop
// halves. The price is the register file: 128 accumulator registers for O^T, 64 for Q, two S^T
// buffers and two P^T buffers need more than 256, so one wave per SIMD runs and the instruction
// stream itself has to keep the matrix pipe fed, the way a GEMM main loop does.
//
//   * Work is cut into sub-tiles of 32 keys. Iteration u issues 16*QB MFMAs (QB = 16-row query
//     blocks per wave, 64 MFMAs for QB = 4): half of them for S^T(u+1) = K(u+1) Q^T, half for
//     O^T += V(u-1)^T P(u-1)^T, while the VALU turns S^T(u) into P^T(u) in the gaps between them:
//     a constexpr schedule (attn_sched) gives every MFMA slot either one exponential or up to two
//     other steps (convert, sums), because a single wave issues one instruction per four cycles
//     and an exponential takes two such issue slots. LDS fragment reads run 3*QB slots ahead.
//   * Q is scaled by sm_scale*log2(e) and rounded to bf16 once; the first MFMA of every S^T
//     accumulator takes "-m" (the row's reference maximum, one register block per 16 rows) as its
//     C operand, so exp2 applies to the MFMA result directly: no multiply, no subtract.
//   * The reference maximum is not the running maximum: it is only moved when a lane's partial sum
//     of a sub-tile reaches 2^40 (which also catches inf and NaN). exp2(s - m) is then simply
//     larger than one for a while, which costs no accuracy in fp32 / bf16 (relative precision),
//     and the common path has no max, no compare per element and no rescale. When the test fires
//     (first sub-tile aside this needs scores to grow by more than 40 in the log2 domain) the
//     whole wave re-bases: true row maxima, accumulators, sums and the S^T blocks in flight are
//     shifted. Row sums are fp32 sums of the unrounded exponentials.
//   * K and V tiles of 64 keys go through two LDS rings of four 16 KB buffers (128 KB). The loop
//     body is unrolled over the four ring positions, so every LDS offset is a compile-time
//     constant; one workgroup barrier per 64 keys, with this wave's own loads of the tile about
//     to be read waited for in front of it. Tiles are fetched with LDS-writing buffer loads
//     through running descriptors (base advanced per tile, rows past the end read as zero).
//   * The ragged tail (keys past L in the last tile) is handled by a second copy of the body that
//     adds a -inf mask to the seed; the common loop carries no such test.
// ------------------------------------------------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));

// MFMAs of this kernel are issued from inline asm so that the register file is laid out by hand.
// Left to the compiler, a kernel with more than 256 registers gets accumulation-register MFMAs for
// everything and a copy in front of every VALU use, or keeps the "a"-constrained operands in vector
// registers and copies them over in front of every MFMA.
//   * The accumulation registers are addressed by number: a[0 : 32*QB-1] = O^T accumulators, block
//     (db, qb) at a[4*(db*QB + qb) ..+3]; the next 16*QB hold the Q fragments, (qb, ks) at
//     a[32*QB + 16*qb + 4*ks ..+3].
//     The compiler never sees them (attn_claim_agprs only makes the kernel descriptor reserve
//     them), so it must not use accumulation registers of its own: the kernel has to fit the 256
//     vector registers without spilling, which tests/test_abi.py checks on the generated code.
//   * S^T, P^T and the LDS fragments are ordinary variables in vector registers (the VALU reads and
//     writes them every slot).
// The hardware does not interlock an MFMA result against a VALU access that follows too closely,
// and the compiler takes an asm statement for an instruction that is complete when the next one
// issues: in the main loop every such pair is half an iteration apart by construction, the rare
// paths (prologue, re-base, epilogue) wait explicitly, and every vector register an MFMA reads or
// writes keeps that role for the whole loop (keep_regs in front of each redefinition), so that the
// compiler cannot hand it to a VALU temporary while an MFMA that uses it is still queued.
#define ATTN_A16(b) "a" #b "0", "a" #b "1", "a" #b "2", "a" #b "3", "a" #b "4", "a" #b "5", "a" #b "6", "a" #b "7", "a" #b "8", "a" #b "9"
template <int N> __device__ __forceinline__ void attn_claim_agprs() {  // a0 .. a(N-1)
    static_assert(N == 96 || N == 144 || N == 192, "clobber lists are spelled out");
    asm volatile("" ::: "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", ATTN_A16(1), ATTN_A16(2), ATTN_A16(3),
                 ATTN_A16(4), ATTN_A16(5), ATTN_A16(6), ATTN_A16(7), ATTN_A16(8), "a90", "a91", "a92", "a93", "a94", "a95");
    if constexpr (N >= 144)
        asm volatile("" ::: "a96", "a97", "a98", "a99", ATTN_A16(10), ATTN_A16(11), ATTN_A16(12), ATTN_A16(13),
                     "a140", "a141", "a142", "a143");
    if constexpr (N == 192)
        asm volatile("" ::: "a144", "a145", "a146", "a147", "a148", "a149", ATTN_A16(15), ATTN_A16(16), ATTN_A16(17), ATTN_A16(18),
                     "a190", "a191");
}
#undef ATTN_A16
// S^T block (vector registers) = K fragment x Q fragment (accumulation registers QLO..QLO+3) + c
template <int QLO>
__device__ __forceinline__ void mfma_s_seed(f32x4& d, const bf16x8& a, const f32x4& c) {
    // "+v" on the destination although the old value is not read: the block keeps its registers
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, a[%3:%4], %2" : "+v"(d) : "v"(a), "v"(c), "n"(QLO), "n"(QLO + 3));
}
// The same with C = 0 as an inline constant. (A register holding zeros would be written by a VALU
// move that the compiler may place right in front of the asm: the MFMA would read it too early.)
template <int QLO>
__device__ __forceinline__ void mfma_s_zero(f32x4& d, const bf16x8& a) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, a[%2:%3], 0" : "+v"(d) : "v"(a), "n"(QLO), "n"(QLO + 3));
}
template <int QLO>
__device__ __forceinline__ void mfma_s_acc(f32x4& d, const bf16x8& a) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, a[%2:%3], %0" : "+v"(d) : "v"(a), "n"(QLO), "n"(QLO + 3));
}
// O^T block (accumulation registers OLO..OLO+3) += V^T fragment x P^T fragment
template <int OLO>
__device__ __forceinline__ void mfma_o_acc(const bf16x8& a, const bf16x8& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" : : "v"(a), "v"(b), "n"(OLO), "n"(OLO + 3));
}
template <int R> __device__ __forceinline__ void acc_write(uint32_t v) {
    asm volatile("v_accvgpr_write_b32 a[%1], %0" : : "v"(v), "n"(R));
}
template <int R> __device__ __forceinline__ float acc_read() {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v) : "n"(R));
    return v;
}
// Marks the old value of x as used here, so that its registers stay reserved up to this point.
template <typename T> __device__ __forceinline__ void keep_regs(T& x) { asm volatile("" : "+v"(x)); }
// Enough wait states for the newest MFMA result to be readable by the VALU (and the other way round).
__device__ __forceinline__ void mfma_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
// Wait states between VALU writes of the four seed blocks and the MFMAs that read them.
__device__ __forceinline__ void mfma_settle_seeds(f32x4 (&b)[4]) {
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]) : : "memory");
}
__device__ __forceinline__ void mfma_settle_seeds(f32x4 (&b)[3]) {
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]) : : "memory");
}
__device__ __forceinline__ void mfma_settle_seeds(f32x4 (&b)[2]) {
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(b[0]), "+v"(b[1]) : : "memory");
}
// The same, and the compiler may not move a use of the S^T blocks in b across it (register-only
// code is otherwise free to float above an asm statement it has no operand in common with).
__device__ __forceinline__ void mfma_settle(f32x4 (&b)[2][4]) {
    asm volatile("s_nop 15\n\ts_nop 15"
                 : "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[0][2]), "+v"(b[0][3]), "+v"(b[1][0]), "+v"(b[1][1]), "+v"(b[1][2]), "+v"(b[1][3])
                 :
                 : "memory");
}
__device__ __forceinline__ void mfma_settle(f32x4 (&b)[2][3]) {
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[0][2]), "+v"(b[1][0]), "+v"(b[1][1]), "+v"(b[1][2]) : : "memory");
}
__device__ __forceinline__ void mfma_settle(f32x4 (&b)[2][2]) {
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[1][0]), "+v"(b[1][1]) : : "memory");
}

template <int N>
__device__ __forceinline__ void attn_vmwait_barrier() {
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// VALU work of one iteration, assigned to the 64 MFMA slots at compile time. A unit is two scores
// of one query block: E0, E1 = their exponentials, C = pack to bf16, A0, A1 = add to the row sum
// (fp32, from the unrounded values: the dot-product instructions that would sum the rounded pair
// run on the matrix pipe and cost a whole MFMA slot each).
// What the schedule is built around, measured on MI355X with one wave per SIMD: beside a 16-cycle
// MFMA the VALU has room for two ordinary instructions or for one exponential, and an instruction
// behind an exponential in the same slot waits for it (and so does the next MFMA). So a slot holds
// either one exponential or up to two other steps; a unit's other steps come two or more slots
// after its exponentials.
enum { ATT_E0, ATT_E1, ATT_C, ATT_A0, ATT_A1, ATT_CHECK };
struct AttnSched {
    int n[64];
    int kind[64][8];
    int arg[64][8];
};
// QB = 16-row query blocks per wave: 16*QB slots, 4*QB units. With one wave per SIMD (QB = 4) a slot
// takes one exponential or two other steps; with two waves per SIMD (QB = 2) the other wave fills
// the gaps, there are fewer slots per step, and three other steps share a slot.
// Head dim 64 has half the MFMAs per score: 8*QB slots for the same 8*QB exponentials, so every slot
// carries one (the first four carry two, which lets the last units finish inside the iteration) and
// up to two other steps behind it.
template <int QB, int D>
constexpr AttnSched attn_sched() {
    constexpr int NS = (D / 8) * QB, NE = 8 * QB, PER = QB >= 3 ? 2 : 3;
    AttnSched S{};
    int qk[160] = {}, qa[160] = {}, qr[160] = {};  // pending steps: kind, argument, first slot allowed
    int head = 0, tail = 0, next_exp = 0;
    for (int s = 0; s < NS; ++s) {
        const bool exp_slot = D == 64 || s < 4 || s % 2 == 1;
        const int exps = !exp_slot ? 0 : (D == 64 && s < 4) ? 2 : 1;
        int added = 0;
        for (int e = 0; e < exps && next_exp < NE; ++e, ++added) {
            const int unit = next_exp / 2, second = next_exp % 2;
            S.kind[s][S.n[s]] = second ? ATT_E1 : ATT_E0; S.arg[s][S.n[s]] = unit; ++S.n[s];
            if (second) {
                qk[tail] = ATT_C; qa[tail] = unit; qr[tail] = s + 2; ++tail;
                qk[tail] = ATT_A0; qa[tail] = unit; qr[tail] = s + 2; ++tail;
                if (unit % 4 != 0) { qk[tail] = ATT_A1; qa[tail] = unit; qr[tail] = s + 2; ++tail; }
            }
            ++next_exp;
        }
        if (D == 64 || added == 0) {
            for (int c = 0; c < PER && head < tail && qr[head] <= s; ++c) {
                S.kind[s][S.n[s]] = qk[head]; S.arg[s][S.n[s]] = qa[head]; ++S.n[s]; ++head;
            }
        }
    }
    while (head < tail) { S.kind[NS - 1][S.n[NS - 1]] = qk[head]; S.arg[NS - 1][S.n[NS - 1]] = qa[head]; ++S.n[NS - 1]; ++head; }
    // The overflow test goes right behind the last add, not into the last slot: the MFMAs and reads
    // of the slots after it then stand between the compare and the branch that takes its result.
    int last = NS - 1;
    while (last > 0 && S.n[last] == 0) --last;
    S.kind[last][S.n[last]] = ATT_CHECK; S.arg[last][S.n[last]] = 0; ++S.n[last];
    return S;
}
template <int QB, int D>
constexpr bool attn_sched_ok(int la) {  // every step exactly once, addresses ready before their first use
    constexpr int NS = (D / 8) * QB;
    const AttnSched S = attn_sched<QB, D>();
    int seen[8][16] = {};
    int exp_at[2][16] = {}, last_use[16] = {};   // position (slot * 8 + place in the slot) of a unit's exponentials and of its last other step
    for (int s = 0; s < NS; ++s) {
        if (S.n[s] > 8) return false;
        for (int c = 0; c < S.n[s]; ++c) {
            const int kind = S.kind[s][c], u = S.arg[s][c];
            seen[kind][u] += 1;
            if (kind == ATT_E0 || kind == ATT_E1) exp_at[kind == ATT_E1][u] = s * 8 + c;
            else if (kind != ATT_CHECK) {
                last_use[u] = s * 8 + c;
                // a step never shares a slot with the exponentials it reads
                if (exp_at[0][u] / 8 == s || exp_at[1][u] / 8 == s) return false;
            }
        }
    }
    // the exponentials of four units are in flight at most: unit u + 4 reuses the registers of unit u
    for (int u = 0; u + 4 < 4 * QB; ++u)
        if (exp_at[0][u + 4] < last_use[u]) return false;
    for (int u = 0; u < 4 * QB; ++u) {
        if (seen[ATT_E0][u] != 1 || seen[ATT_E1][u] != 1 || seen[ATT_C][u] != 1 || seen[ATT_A0][u] != 1) return false;
        if (seen[ATT_A1][u] != (u % 4 != 0)) return false;
    }
    return la > 0 && seen[ATT_CHECK][0] == 1;
}
// Slot of the j-th buffer load of a tile (LPW per wave and tile): behind the barrier (slot BS of the
// first iteration of a body), SP slots apart, continued in the second iteration up to its slot BS.
constexpr int attn_load_slot(int j, int ns, int bs, int sp, bool second) {
    int k = 0;
    for (int s = bs + sp / 2; s < ns; s += sp, ++k)
        if (k == j) return second ? -1 : s;
    for (int s = sp / 2; s < bs; s += sp, ++k)
        if (k == j) return second ? s : -1;
    return -2;  // does not fit
}

// QB = 16-row query blocks per wave, NW = waves per workgroup: 16*QB*NW query rows per workgroup.
//   <4, 4>: 64 rows per wave, 256 per workgroup, one wave per SIMD (248 vector + 192 accumulation registers).
//   <3, 4>: 48 rows per wave, 192 per workgroup: the same code with three quarters of the work per
//           iteration, for the part that evens out the last round (see attn_launch_w64).
//
// Head dim 64 runs the same code with half the MFMAs per iteration (2 + 2 fragments of K, 4 of V^T per
// 32 keys) and the same softmax work, so there the VALU sets the pace: every slot carries an
// exponential. Rows of K and V are 128 bytes, a wave-wide load covers eight of them, and the swizzles
// are those of 128-byte rows (below).
template <int D, int QB, int NW>
__device__ __forceinline__ void attn_w64_tile(const AttnParams& p, char* lds, const int block, const int nblocks) {
    static_assert(NW == 4 && (QB == 3 || QB == 4) && (D == 64 || D == 128), "configurations that have been laid out and measured");
    constexpr int ROWS = 16 * QB * NW;         // query rows per workgroup
    constexpr int KS = D / 32, DBN = D / 16, ROWB = D * 2, TB = 64 * ROWB, HALF = 32 * ROWB;
    constexpr int CH = D / 8, RPL = 64 / CH;   // 16-byte chunks per row; rows a wave-wide load (or store) covers
    constexpr int V0 = 4 * TB;
    constexpr int NSS = 2 * KS * QB, NS = NSS + DBN * QB;  // MFMA slots per iteration; the first NSS are S^T
    constexpr int LA = 3 * QB;                 // look-ahead of the LDS fragment reads in slots: what a ring of four fragments holds
    constexpr int BS = D == 128 ? 10 * QB : 4 * QB;  // slot of the barrier in the first iteration of a body
    constexpr int PP = 64 / (RPL * NW);        // loader passes per tile and operand (a pass = RPL rows per wave)
    constexpr int LPW = 2 * PP;                // buffer loads per wave and body: PP of V(T+2), then PP of K(T+4)
    constexpr int kAccQ = 4 * DBN * QB;        // first accumulation register of the Q fragments
    constexpr int kQRegs = 4 * KS;             // accumulation registers of one query block's fragments
    constexpr AttnSched SCHED = attn_sched<QB, D>();
    static_assert(attn_sched_ok<QB, D>(LA), "VALU schedule");
    static_assert(BS > (2 * KS - 1) * QB - LA && BS < NS - LA, "barrier between the last read of K(T) and the first of K(T+1)");
    static_assert(attn_load_slot(LPW - 1, NS, BS, NS / 8, false) != -2, "load slots");
    constexpr float kRebase = 1.0995116e12f;  // 2^40
    // lds: 8 * TB bytes, K ring of 4 tiles, V ring of 4 tiles
    const int per_xcd = nblocks / 8;
    const int vt = (block % 8) * per_xcd + block / 8;
    if (vt >= p.total_tiles) return;
    const int per_pair = p.cnt_even + p.cnt_odd;
    const int pair = vt / per_pair, rem = vt % per_pair;
    const bool odd = rem >= p.cnt_even;
    const int bh = 2 * pair + odd, qt = odd ? rem - p.cnt_even : rem;
    const int b = bh / p.H, h = bh % p.H;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int q0 = (odd ? p.first_odd : p.first_even) + qt * ROWS + wave * (16 * QB);
    const float c = p.scale_log2;

    const bf16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
    const bf16_t* vbase = p.v + b * p.v_sb + h * p.v_sh;

    // loader: a wave-wide load is RPL rows of ROWB bytes (1 KB); pass i covers rows i*RPL*NW + wave*RPL + lane/CH.
    // 256-byte rows: LDS position pos of row r holds the 16-byte chunk pos ^ (r & 15) of a K row
    // (fragment reads take one chunk of 16 consecutive rows) and chunk pos ^ ((r & 7) << 1) of a V row
    // (transposing reads take 32-byte pieces of 4 consecutive rows in each of four lane groups).
    // 128-byte rows: two rows fill the 256 bytes the banks are wide, so the rows of a pair keep the
    // same position and the pairs differ: chunk pos ^ ((r >> 1) & 7) for K, pos ^ (((r >> 1) & 3) << 1) for V.
    auto k_swz = [](int r) { return D == 128 ? (r & 15) : ((r >> 1) & 7); };
    auto v_swz = [](int r) { return D == 128 ? (r & 7) : ((r >> 1) & 3); };   // in 32-byte units
    const int l_row = lane / CH, l_pos = lane % CH;
    uint32_t k_voff[PP], v_voff[PP];
#pragma unroll
    for (int i = 0; i < PP; ++i) {
        const int r = i * RPL * NW + wave * RPL + l_row;
        k_voff[i] = static_cast<uint32_t>((r * p.k_sl + ((l_pos ^ k_swz(r)) * 8)) * 2);
        v_voff[i] = static_cast<uint32_t>((r * p.v_sl + ((l_pos ^ (v_swz(r) << 1)) * 8)) * 2);
    }
    const int k_row2 = static_cast<int>(p.k_sl * 2), v_row2 = static_cast<int>(p.v_sl * 2);
    auto tile_rsrc = [&](const bf16_t* base, int row2, int key0) -> u32x4 {
        const int rows = min(p.L - key0, 64);
        const int bytes = rows > 0 ? (rows - 1) * row2 + D * 2 : 0;
        const uint64_t addr = reinterpret_cast<uint64_t>(base) + static_cast<uint64_t>(static_cast<int64_t>(key0) * row2);
        u32x4 r;
        r.x = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr));
        r.y = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr >> 32) & 0xffffu);
        r.z = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bytes));
        r.w = kAttnRsrcFlags;
        return r;
    };
    const uint32_t lds_base = lds_addr_of(lds) + wave * 1024;
    auto load_k = [&](int tile, int buf) {
        const u32x4 rs = tile_rsrc(kbase, k_row2, tile * 64);
#pragma unroll
        for (int i = 0; i < PP; ++i) lds_load16_raw(rs, lds_base + buf * TB + i * (NW * 1024), k_voff[i]);
    };
    auto load_v = [&](int tile, int buf) {
        const u32x4 rs = tile_rsrc(vbase, v_row2, tile * 64);
#pragma unroll
        for (int i = 0; i < PP; ++i) lds_load16_raw(rs, lds_base + V0 + buf * TB + i * (NW * 1024), v_voff[i]);
    };

    // The first pass through the loop multiplies P = 0 with whatever the last V buffer holds:
    // make that finite.
    {
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < PP; ++i) *reinterpret_cast<u32x4*>(lds + V0 + 3 * TB + i * (NW * 1024) + tid * 16) = z;
    }
    load_k(0, 0);
    load_v(0, 0);
    load_k(1, 1);

    // Q fragments ("B" operand of S^T): lane holds row q0 + qb*16 + r16, d = ks*32 + g*8 .. +8,
    // scaled by sm_scale*log2(e) and rounded to bf16.
    attn_claim_agprs<(D == 128 ? 48 * QB : 96)>();
    {
        u32x4 qraw[QB][KS];  // all loads in flight before the first conversion
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const int row = q0 + qb * 16 + r16;
            const bool ok = row < p.L;
            const bf16_t* rp = p.q + b * p.q_sb + h * p.q_sh + static_cast<int64_t>(ok ? row : 0) * p.q_sl;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                qraw[qb][ks] = *reinterpret_cast<const u32x4*>(rp + ks * 32 + g * 8);
                if (!ok) qraw[qb][ks] = u32x4{0u, 0u, 0u, 0u};
            }
        }
        static_for<0, QB * KS * 4>([&](auto i_c) {
            constexpr int i = decltype(i_c)::value, qb = i / kQRegs, ks = (i / 4) % KS, e = i % 4;
            const uint32_t t = qraw[qb][ks][e];
            acc_write<kAccQ + i>(pack2_bf16(__uint_as_float(t << 16) * c, __uint_as_float(t & 0xffff0000u) * c));
        });
        static_for<0, kAccQ>([&](auto i_c) { acc_write<decltype(i_c)::value>(0u); });  // O^T = 0
    }

    // fragment addresses, lane part (the ring offset of the sub-tile is added once per iteration,
    // key-block and second-read offsets are immediates)
    // K ("A" of S^T): row kb*16 + r16 of the sub-tile, chunk ks*4 + g.
    // V^T ("A" of O^T): lane group g transposes key rows g*4 .. g*4+3 (first read) and 16 + g*4 ..
    // (second read) of the sub-tile; lane r16 points at row g*4 + r16/4, 8 bytes at d = db*16 + (r16%4)*4.
    int k_addr[KS], v_addr[DBN];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_addr[ks] = r16 * ROWB + (((ks * 4 + g) ^ k_swz(r16)) * 16);
    {
        const int rr = r16 >> 2, cc = r16 & 3, row = g * 4 + rr;
#pragma unroll
        for (int db = 0; db < DBN; ++db) v_addr[db] = V0 + row * ROWB + ((db ^ v_swz(row)) * 32) + cc * 8;
    }

    f32x4 seed[QB];   // -m of the row, in every register of the block: C operand of the first S^T MFMA
    float l_run[QB];
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        seed[qb] = zero4;
        l_run[qb] = 0.0f;
    }
    const int ntiles = (p.L + 63) / 64;

    // Every register an MFMA reads or writes is kept for that purpose through the whole loop
    // (keep_regs in front of each redefinition): see mfma_s_seed.
    bf16x8 kf[4];
    s16x4 vlo[4], vhi[4];
    f32x4 s0[2][QB], s1[2][QB];
    uint32_t pw0[QB][4], pw1[QB][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        kf[i] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        vlo[i] = s16x4{0, 0, 0, 0};
        vhi[i] = s16x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
        for (int w = 0; w < 4; ++w) pw0[qb][w] = pw1[qb][w] = 0u;
        s0[0][qb] = s0[1][qb] = s1[0][qb] = s1[1][qb] = zero4;
    }
    auto read_k = [&](int off, int n) {  // n-th K fragment of the sub-tile at LDS offset off (a constant): key block n/KS, d step n%KS
        keep_regs(kf[n % 4]);
        kf[n % 4] = *reinterpret_cast<const bf16x8*>(lds + k_addr[n % KS] + (off + (n / KS) * 16 * ROWB));
    };
    auto vfrag = [&](int m) {
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        const s16x8 both = {vlo[m][0], vlo[m][1], vlo[m][2], vlo[m][3], vhi[m][0], vhi[m][1], vhi[m][2], vhi[m][3]};
        return __builtin_bit_cast(bf16x8, both);
    };

    // ---- prologue: S^T(0) from the first half of K(0), then the rows' first reference maxima
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    static_for<0, 2 * KS>([&](auto n_c) {
        constexpr int n = decltype(n_c)::value, kb = n / KS, ks = n % KS;
        const bf16x8 f = *reinterpret_cast<const bf16x8*>(lds + k_addr[ks] + kb * 16 * ROWB);
        static_for<0, QB>([&](auto qb_c) {
            constexpr int qb = decltype(qb_c)::value, QA = kAccQ + kQRegs * qb;
            if constexpr (ks == 0) mfma_s_zero<QA>(s0[kb][qb], f);
            else mfma_s_acc<QA + 4 * ks>(s0[kb][qb], f);
        });
    });
    mfma_settle(s0);
    load_k(2, 2);
    load_v(1, 1);
    load_k(3, 3);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int key = kb * 16 + g * 4 + j;
                if (key >= p.L) s0[kb][qb][j] = -INFINITY;
                mx = fmaxf(mx, s0[kb][qb][j]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
#pragma unroll
        for (int j = 0; j < 4; ++j) seed[qb][j] = -mx;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) s0[kb][qb] -= mx;
    }
    mfma_settle_seeds(seed);
#pragma unroll
    for (int n = 0; QB * n < LA; ++n) read_k(HALF, n);  // second half of K(0)
    __builtin_amdgcn_sched_barrier(0);

    // Shift the reference maxima of all rows of the wave (rare). sc = S^T of the sub-tile whose
    // sums tripped the test, sn = the complete S^T of the next one (seeded with the old reference).
    auto rebase = [&](f32x4 (&sc)[2][QB], f32x4 (&sn)[2][QB], uint32_t (&pw)[QB][4], float (&sum)[QB]) {
        mfma_settle(sc);
        mfma_settle(sn);
        static_for<0, QB>([&](auto qb_c) {
            constexpr int qb = decltype(qb_c)::value, QBC = qb;
            float mx = fmaxf(fmaxf(sc[0][qb][0], sc[0][qb][1]), fmaxf(sc[0][qb][2], sc[0][qb][3]));
            mx = fmaxf(mx, fmaxf(fmaxf(sc[1][qb][0], sc[1][qb][1]), fmaxf(sc[1][qb][2], sc[1][qb][3])));
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float d = fmaxf(mx, 0.0f);  // the reference only ever moves up
            const float f = __builtin_amdgcn_exp2f(-d);
            seed[qb] -= d;
            l_run[qb] *= f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                sc[kb][qb] -= d;
                sn[kb][qb] -= d;
            }
            static_for<0, DBN * 4>([&](auto i_c) {
                constexpr int i = decltype(i_c)::value, r = 4 * ((i / 4) * QB + QBC) + i % 4;
                acc_write<r>(__float_as_uint(acc_read<r>() * f));
            });
            float sm = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float p0 = __builtin_amdgcn_exp2f(sc[w / 2][qb][(w % 2) * 2]);
                const float p1 = __builtin_amdgcn_exp2f(sc[w / 2][qb][(w % 2) * 2 + 1]);
                pw[qb][w] = pack2_bf16(p0, p1);
                sm += p0 + p1;
            }
            sum[qb] = sm;
        });
        mfma_settle_seeds(seed);
    };

    // One iteration = 64 slots of (MFMA, fragment reads for later slots, VALU steps of the softmax).
    //   KC:   LDS offset of the K sub-tile of S^T(u+1), KN: that of the iteration after (its first
    //         fragments are read here), VC: offset of the V sub-tile of P(u-1) (relative to V0)
    //   BAR:  this iteration carries the workgroup barrier, behind which tile T+2 of V and T+4 of
    //         K are requested (descriptors rk / rv) into the ring buffers at KLD / VLD, spread over
    //         this iteration and the next one.
    //   RAG:  the sub-tile after this one may reach past the last key (the common loop is built
    //         without that test).
    // All offsets are compile-time constants: the body is unrolled over the four ring positions.
    auto iter = [&](auto bar_c, auto rag_c, auto kc_c, auto kn_c, auto vc_c, auto kld_c, auto vld_c, const u32x4& rk, const u32x4& rv, int u,
                    f32x4 (&sc)[2][QB], f32x4 (&sn)[2][QB], uint32_t (&pc)[QB][4], uint32_t (&pp)[QB][4]) {
        constexpr bool BAR = decltype(bar_c)::value, RAG = decltype(rag_c)::value;
        constexpr int KC = decltype(kc_c)::value, KN = decltype(kn_c)::value, VC = decltype(vc_c)::value;
        constexpr int KLD = decltype(kld_c)::value, VLD = decltype(vld_c)::value;
        bf16x8 ppf[QB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const u32x4 v4 = {pp[qb][0], pp[qb][1], pp[qb][2], pp[qb][3]};
            ppf[qb] = __builtin_bit_cast(bf16x8, v4);
        }
        float sum[QB];
        float e0[4], e1[4];  // exponentials of up to four units in flight
        uint64_t trip = 0;
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, NS>([&](auto i_c) {
            constexpr int i = decltype(i_c)::value;
            if constexpr (BAR && i == BS) {
                // V(T), K(T+1) have landed (everything but the newest 1.5 tiles' loads of this wave); every
                // wave is done with K(T) and V(T-2)
                attn_vmwait_barrier<3 * PP>();
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- matrix pipe
            if constexpr (i < NSS) {
                constexpr int n = i / QB, qb = i % QB, kb = n / KS, ks = n % KS;
                if constexpr (ks == 0) mfma_s_seed<kAccQ + kQRegs * qb>(sn[kb][qb], kf[n % 4], seed[qb]);
                else mfma_s_acc<kAccQ + kQRegs * qb + 4 * ks>(sn[kb][qb], kf[n % 4]);
            } else {
                constexpr int m = (i - NSS) / QB, qb = i % QB;
                mfma_o_acc<4 * (m * QB + qb)>(vfrag(m % 4), ppf[qb]);
            }
            // ---- LDS fragment reads, LA slots ahead of the first MFMA that takes them (K fragment n
            // feeds slots QB*n .. QB*n+QB-1, V^T fragment m slots NSS+QB*m ..; the first K fragments of
            // an iteration are read in the one before)
            static_for<0, 8>([&](auto n_c) {
                constexpr int n = decltype(n_c)::value;
                if constexpr (n < 2 * KS && QB * n - LA == i) read_k(KC, n);
                if constexpr (n < 2 * KS && NS + QB * n - LA == i) read_k(KN, n);
                if constexpr (n < DBN && NSS + QB * n - LA == i) {
                    keep_regs(vlo[n % 4]);
                    vlo[n % 4] = lds_read_tr(lds + v_addr[n % DBN] + VC);
                }
                if constexpr (n < DBN && NSS + 1 + QB * n - LA == i) {
                    keep_regs(vhi[n % 4]);
                    vhi[n % 4] = lds_read_tr(lds + v_addr[n % DBN] + (VC + 16 * ROWB));
                }
            });
            // ---- global loads of later tiles behind the barrier
            // (LPW per tile and wave, NS/8 slots apart: V(T+2) first, then K(T+4))
            static_for<0, LPW>([&](auto j_c) {
                constexpr int j = decltype(j_c)::value;
                if constexpr (attn_load_slot(j, NS, BS, NS / 8, !BAR) == i) {
                    if constexpr (j < PP) lds_load16_raw_at<V0 + VLD + j * NW * 1024>(rv, lds_base, v_voff[j]);
                    else lds_load16_raw_at<KLD + (j - PP) * NW * 1024>(rk, lds_base, k_voff[j - PP]);
                }
            });
            // ---- softmax of S^T(u), the steps that belong to this slot
            // ---- VALU steps of this slot: softmax of S^T(u), LDS addresses
            static_for<0, SCHED.n[i]>([&](auto c_c) {
                constexpr int c = decltype(c_c)::value, kind = SCHED.kind[i][c], k = SCHED.arg[i][c], qb = (k / 4) % QB, w = k % 4;
                if constexpr (kind == ATT_E0 || kind == ATT_E1) {
                    // issued from asm: it stays in its slot, and the compiler adds no wait state in
                    // front of it (nothing reads the result before the next slot but one)
                    const float a = sc[w / 2][qb][(w % 2) * 2 + (kind == ATT_E1)];
                    float e;
                    asm volatile("v_exp_f32 %0, %1" : "=v"(e) : "v"(a));
                    if constexpr (kind == ATT_E0) e0[k % 4] = e;
                    else e1[k % 4] = e;
                } else if constexpr (kind == ATT_C) {
                    keep_regs(pc[qb][w]);  // P^T of the iteration before: read by MFMAs a few slots ago
                    pc[qb][w] = pack2_bf16(e0[k % 4], e1[k % 4]);
                } else if constexpr (kind == ATT_A0) {
                    if constexpr (w == 0) sum[qb] = e0[k % 4] + e1[k % 4];
                    else sum[qb] += e0[k % 4];
                } else if constexpr (kind == ATT_A1) {
                    sum[qb] += e1[k % 4];
                } else {
                    float big = fmaxf(sum[0], sum[1]);
                    if constexpr (QB >= 3) big = fmaxf(big, sum[2]);
                    if constexpr (QB == 4) big = fmaxf(big, sum[3]);
                    trip = __builtin_amdgcn_ballot_w64(!(big < kRebase));
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        // One branch per iteration, off the common path: a reference maximum has to move, or the
        // next sub-tile reaches past the last key.
        if (__builtin_expect((trip != 0) | (RAG && (u + 2) * 32 > p.L), 0)) {
            if (trip != 0) rebase(sc, sn, pc, sum);
            if (RAG && (u + 2) * 32 > p.L) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if ((u + 1) * 32 + kb * 16 + g * 4 + j >= p.L) sn[kb][qb][j] = -INFINITY;
            }
        }
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) l_run[qb] += sum[qb];
        __builtin_amdgcn_sched_barrier(0);
    };

    // Body T: iteration 2T (S^T from the second half of K(T), P V with the second half of V(T-1))
    // and iteration 2T+1 (first half of K(T+1), first half of V(T)). Tile X sits in ring buffer
    // X % 4, so four bodies make one trip of the loop. One more body than there are tiles: the last
    // one only finishes P V. Bodies whose sub-tiles all lie inside the sequence run without the
    // ragged-tail test; the last few take the variant with it.
    // Buffer descriptors of the tiles requested by body T: K(T+4) and V(T+2), advanced by one tile
    // per body; the record count is what is left of the sequence, at most one tile.
    uint64_t k_at = reinterpret_cast<uint64_t>(kbase) + static_cast<uint64_t>(4 * 64) * k_row2;
    uint64_t v_at = reinterpret_cast<uint64_t>(vbase) + static_cast<uint64_t>(2 * 64) * v_row2;
    // rows left from the start of the next tile to request; a tile's record count is formed from at most
    // 64 of them, so it stays in 32 bits however long and widely strided the sequence is
    int k_rows = p.L - 4 * 64, v_rows = p.L - 2 * 64;
    auto next_rsrc = [&](uint64_t& at, int& rows_left, int row2) -> u32x4 {
        const int rows = min(rows_left, 64);
        u32x4 r;
        r.x = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(at));
        r.y = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(at >> 32) & 0xffffu);
        r.z = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(rows > 0 ? (rows - 1) * row2 + D * 2 : 0));
        r.w = kAttnRsrcFlags;
        at += static_cast<uint64_t>(64) * static_cast<uint64_t>(row2);
        rows_left -= 64;
        return r;
    };
    auto body = [&](auto r_c, auto rag_c, int T) -> bool {
        constexpr int r = decltype(r_c)::value, r0 = r * TB, r1 = ((r + 1) & 3) * TB, r2 = ((r + 2) & 3) * TB, r3 = ((r + 3) & 3) * TB;
        using ic = std::integral_constant<int, 0>;
        const u32x4 rk = next_rsrc(k_at, k_rows, k_row2), rv = next_rsrc(v_at, v_rows, v_row2);
        iter(std::true_type{}, rag_c, std::integral_constant<int, r0 + HALF>{}, std::integral_constant<int, r1>{},
             std::integral_constant<int, r3 + HALF>{}, std::integral_constant<int, r0>{}, std::integral_constant<int, r2>{},
             rk, rv, 2 * T, s0, s1, pw0, pw1);
        if (decltype(rag_c)::value && T == ntiles) return false;
        iter(std::false_type{}, rag_c, std::integral_constant<int, r1>{}, std::integral_constant<int, r1 + HALF>{},
             std::integral_constant<int, r0>{}, std::integral_constant<int, r0>{}, std::integral_constant<int, r2>{},
             rk, rv, 2 * T + 1, s1, s0, pw1, pw0);
        return true;
    };
    // bodies 0 .. n_plain-1 never look past the last key: (2T + 3) * 32 <= L, in whole trips of four
    const int n_plain = max(0, (p.L / 32 - 1) / 2) & ~3;
    int T = 0;
    for (; T < n_plain; T += 4) {
        body(std::integral_constant<int, 0>{}, std::false_type{}, T);
        body(std::integral_constant<int, 1>{}, std::false_type{}, T + 1);
        body(std::integral_constant<int, 2>{}, std::false_type{}, T + 2);
        body(std::integral_constant<int, 3>{}, std::false_type{}, T + 3);
    }
    for (;; T += 4) {
        if (!body(std::integral_constant<int, 0>{}, std::true_type{}, T)) break;
        if (!body(std::integral_constant<int, 1>{}, std::true_type{}, T + 1)) break;
        if (!body(std::integral_constant<int, 2>{}, std::true_type{}, T + 2)) break;
        if (!body(std::integral_constant<int, 3>{}, std::true_type{}, T + 3)) break;
    }
    wait_all_vmem();
    mfma_settle();

    // ---- finish: fold the four lane groups' partial sums, normalise, store. A lane holds runs of four
    // columns of sixteen different rows, which would leave as 32-byte pieces; instead the wave parks
    // its rows in LDS (the rings are idle once every wave is past the loop) and they leave as 16-byte
    // pieces of whole rows. 8-byte slot s of row r sits at slot s ^ 2(r mod chunks per row): writes and
    // reads both spread over all banks, and a 16-byte chunk stays contiguous.
    asm volatile("s_barrier" ::: "memory");
    char* const stage = lds + wave * (16 * QB * ROWB);
    static_for<0, QB>([&](auto qb_c) {
        constexpr int qb = decltype(qb_c)::value, QBC = qb;
        float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 16, 64);
        l_tot += __shfl_xor(l_tot, 32, 64);
        const float inv = 1.0f / l_tot;
        const int row = q0 + qb * 16 + r16;
        char* const srow = stage + (qb * 16 + r16) * ROWB;
        static_for<0, DBN>([&](auto db_c) {
            constexpr int db = decltype(db_c)::value, r = 4 * (db * QB + QBC);
            u32x2 w;
            w.x = pack2_bf16(acc_read<r>() * inv, acc_read<r + 1>() * inv);
            w.y = pack2_bf16(acc_read<r + 2>() * inv, acc_read<r + 3>() * inv);
            *reinterpret_cast<u32x2*>(srow + (((db * 4 + g) ^ ((r16 % CH) * 2)) * 8)) = w;
        });
        if (row < p.L && p.lse != nullptr && g == 0)
            p.lse[static_cast<int64_t>(bh) * p.L + row] = -seed[qb][0] + __builtin_amdgcn_logf(l_tot);
    });
    __builtin_amdgcn_wave_barrier();  // LDS operations of one wave complete in order
    {
        bf16_t* const obase = p.o + b * p.o_sb + h * p.o_sh;
        const int chunk = lane % CH;
#pragma unroll
        for (int it = 0; it < 16 * QB / RPL; ++it) {
            const int rl = it * RPL + lane / CH;
            const u32x4 y = *reinterpret_cast<const u32x4*>(stage + rl * ROWB + ((chunk ^ (rl % CH)) * 16));
            const int row = q0 + rl;
            if (row < p.L) *reinterpret_cast<u32x4*>(obase + static_cast<int64_t>(row) * p.o_sl + chunk * 8) = y;
        }
    }
}


constexpr int w64_lds_bytes(int d) { return 8 * 64 * 2 * d; }  // K ring and V ring of four 64-key tiles

// Both tile sizes in one launch: blocks [0, n4) take 256-row tiles of p4, the rest 192-row tiles of
// p3. Workgroups are handed out in order, so the 192-row tiles start on each CU as it finishes its
// 256-row tile, with no launch boundary in between. n4 and the remainder are multiples of eight, so
// a block's XCD is the same counted from either start. A launch of 256-row tiles only has n4 = grid.
template <int D>
__global__ __launch_bounds__(256, 1) void attn_fwd_w64_kernel_pair(AttnParams p4, AttnParams p3, int n4) {
    __shared__ __attribute__((aligned(1024))) char lds[w64_lds_bytes(D)];
    if (static_cast<int>(blockIdx.x) < n4) attn_w64_tile<D, 4, 4>(p4, lds, blockIdx.x, n4);
    else attn_w64_tile<D, 3, 4>(p3, lds, static_cast<int>(blockIdx.x) - n4, static_cast<int>(gridDim.x) - n4);
}

#ifndef FLUX_ATTN_W64_D64_UNIT
template <int D, int QB, int BN>
static void attn_launch_pipe(AttnParams& p, int64_t BH, hipStream_t st) {
    p.n_qtiles = (p.L + 128 * QB - 1) / (128 * QB);
    p.total_tiles = static_cast<int>(p.n_qtiles * BH);
    const int grid = ((p.total_tiles + 7) / 8) * 8;
    hipLaunchKernelGGL((attn_fwd_pipe_kernel<D, QB, BN>), dim3(grid), dim3(256), 0, st, p);
}

#endif

constexpr int64_t kW64MinTiles = 128;

// One workgroup per CU, so a launch of more than one round's worth of equal tiles costs whole
// rounds: 432 tiles of 256 rows on 256 CUs take as long as 512 would. The rows of every (batch, head)
// are therefore cut in two parts: 256-row tiles for the first rows, 192-row tiles for the rest, with
// the cut allowed to differ between the even and the odd member of a (batch, head) pair, chosen so
// that the last workgroup finishes earliest (attn_launch_w64). 110 592 rows of the Flux shape become
// 252 + 240 workgroups, 1.8 tile times instead of 2. The two parts are the two block ranges of one
// launch (attn_fwd_w64_kernel_pair).
constexpr int kAttnCUs = 256;

// Fills in the tile mapping of one part and returns its grid (a multiple of eight, 0 = no tiles).
static int attn_w64_part(AttnParams& p, int64_t BH, int cnt_even, int cnt_odd, int first_even, int first_odd) {
    p.cnt_even = cnt_even; p.cnt_odd = cnt_odd; p.first_even = first_even; p.first_odd = first_odd;
    const int64_t pairs = (BH + 1) / 2;
    p.total_tiles = static_cast<int>(pairs * (cnt_even + cnt_odd));
    if (p.total_tiles == 0) return 0;
    if (BH % 2) p.total_tiles -= cnt_odd;  // the last pair has no odd member: its tiles sit at the very end
    return ((p.total_tiles + 7) / 8) * 8;
}

// When the last 256-row tile has been handed out and all 192-row tiles after it, in units of a fifth
// of a 256-row tile's time (a 192-row tile takes four: 112 and 90 us measured at the Flux shape).
// Workgroups are handed out in order to whichever CU is free.
static int64_t attn_w64_makespan(int64_t n4, int64_t n3) {
    const int64_t q = n4 / kAttnCUs, r = n4 % kAttnCUs;
    const int64_t ta = 5 * q, tb = ta + 5;   // kAttnCUs - r CUs are free at ta, the other r at tb
    const int64_t busy = r ? tb : ta;
    if (n3 == 0) return busy;
    auto taken = [&](int64_t t) {  // 192-row tiles finished by time t
        return (kAttnCUs - r) * (t > ta ? (t - ta) / 4 : 0) + r * (t > tb ? (t - tb) / 4 : 0);
    };
    int64_t lo = ta, hi = tb + 4 * (n3 / kAttnCUs + 2);
    while (lo < hi) {
        const int64_t mid = (lo + hi) / 2;
        if (taken(mid) >= n3) hi = mid;
        else lo = mid + 1;
    }
    return lo > busy ? lo : busy;
}

// The cut that attn_launch_w64 uses for BH (batch, head)s of L rows: ne / no = 256-row tiles of the even
// and the odd member of a pair. The search below evaluates up to a few thousand makespans, so the last
// few answers are kept (a serving loop calls with the same one or two shapes over and over).
static void attn_w64_cut(int64_t BH, int L, int& best_ne, int& best_no) {
    struct Entry { int64_t BH; int L, ne, no; };
    static std::mutex mu;
    static Entry cache[8];
    static int filled = 0, next = 0;
    {
        std::lock_guard<std::mutex> g(mu);
        for (int i = 0; i < filled; ++i)
            if (cache[i].BH == BH && cache[i].L == L) { best_ne = cache[i].ne; best_no = cache[i].no; return; }
    }
    const int n256 = (L + 255) / 256;
    const int64_t tiles = BH * n256;
    const int64_t pairs = BH / 2, lone = BH % 2;   // a last (batch, head) without a partner counts as an even one
    best_ne = n256; best_no = n256;
    int64_t best_t = attn_w64_makespan(tiles, 0), best_n4 = tiles;
    for (int ne = 0; ne <= n256; ++ne)
        for (int no = ne; no <= n256; ++no) {
            const int re = L - min(L, ne * 256), ro = L - min(L, no * 256);
            const int64_t n4 = pairs * (ne + no) + lone * ne;
            const int64_t n3 = pairs * ((re + 191) / 192 + (ro + 191) / 192) + lone * ((re + 191) / 192);
            const int64_t t = attn_w64_makespan(n4, n3);
            if (t < best_t || (t == best_t && n4 > best_n4)) { best_t = t; best_n4 = n4; best_ne = ne; best_no = no; }
        }
    std::lock_guard<std::mutex> g(mu);
    cache[next] = Entry{BH, L, best_ne, best_no};
    next = (next + 1) % 8;
    if (filled < 8) ++filled;
}

template <int D>
static void attn_launch_w64(AttnParams& p, int64_t BH, hipStream_t st) {
    const int n256 = (p.L + 255) / 256;
    const int64_t tiles = BH * n256;
    // More than one round of tiles, and few enough rounds for the last one to matter: choose how many
    // 256-row tiles the even and the odd (batch, head) of a pair get (ne, no; the rest of their rows
    // goes to 192-row tiles) so that the last workgroup finishes earliest; among equals, the most
    // 256-row tiles, which are the more efficient ones.
    if (tiles > kAttnCUs && tiles <= 16 * kAttnCUs && n256 <= 64) {
        int best_ne, best_no;
        attn_w64_cut(BH, p.L, best_ne, best_no);
        if (best_ne < n256 || best_no < n256) {
            const int fe = min(p.L, best_ne * 256), fo = min(p.L, best_no * 256);
            AttnParams p4 = p, p3 = p;
            const int g4 = attn_w64_part(p4, BH, best_ne, best_no, 0, 0);
            const int g3 = attn_w64_part(p3, BH, (p.L - fe + 191) / 192, (p.L - fo + 191) / 192, fe, fo);
            hipLaunchKernelGGL(attn_fwd_w64_kernel_pair<D>, dim3(g4 + g3), dim3(256), 0, st, p4, p3, g4);
            return;
        }
    }
    const int g = attn_w64_part(p, BH, n256, n256, 0, 0);
    if (g > 0) hipLaunchKernelGGL(attn_fwd_w64_kernel_pair<D>, dim3(g), dim3(256), 0, st, p, p, g);
}

// The head-dim-64 instantiation of the 64-row kernels is compiled as a unit of its own
// (attention_d64.hip includes this file with FLUX_ATTN_W64_D64_UNIT defined): the unrolled loop
// bodies take minutes to compile, and the two head dims compile side by side.
void attn_launch_w64_d64(AttnParams& p, int64_t BH, hipStream_t st);
#ifdef FLUX_ATTN_W64_D64_UNIT
void attn_launch_w64_d64(AttnParams& p, int64_t BH, hipStream_t st) { attn_launch_w64<64>(p, BH, st); }
#endif

}  // namespace flux

#ifndef FLUX_ATTN_W64_D64_UNIT
using namespace flux;

static bool view_ok(const void* ptr, int64_t sb, int64_t sh, int64_t sl) {
    return ptr != nullptr && aligned16(ptr) && sb % 8 == 0 && sh % 8 == 0 && sl % 8 == 0;
}

extern "C" int flux_attention_fwd_bf16(const flux_attn_args* a, void* stream) {
    if (!a) return fail(FLUX_E_NULL, "flux_attention_fwd_bf16: null args");
    if (a->B < 0 || a->H <= 0 || a->L < 0) return fail(FLUX_E_SHAPE, "flux_attention_fwd_bf16: bad shape B=%lld H=%lld L=%lld", (long long)a->B, (long long)a->H, (long long)a->L);
    if (a->D != 16 && a->D != 32 && a->D != 64 && a->D != 128 && a->D != 256)
        return fail(FLUX_E_UNSUPPORTED, "flux_attention_fwd_bf16: head dim %d not supported (16, 32, 64, 128, 256)", a->D);
    if (!(a->sm_scale == a->sm_scale)) return fail(FLUX_E_UNSUPPORTED, "flux_attention_fwd_bf16: sm_scale is NaN");
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
    // Head dim 128: 64 rows per wave (256 per workgroup, one workgroup per CU) once there are enough
    // such tiles to occupy the chip; smaller problems get 128-row workgroups, two per CU.
    const int64_t tiles256 = BH * ((a->L + 255) / 256);
    if (a->D != 64 && a->D != 128) {
        if (BH * ((a->L + 63) / 64) > 0x7fffffffLL) return fail(FLUX_E_SHAPE, "flux_attention_fwd_bf16: problem too large");
        attn_launch_plain(p, BH, a->D, st);
    } else if (a->D == 128 && tiles256 >= kW64MinTiles) attn_launch_w64<128>(p, BH, st);
    else if (a->D == 128) attn_launch_pipe<128, 1, 64>(p, BH, st);
    else if (tiles256 >= kW64MinTiles) attn_launch_w64_d64(p, BH, st);
    else attn_launch_pipe<64, 1, 64>(p, BH, st);
    return check_launch("flux_attention_fwd_bf16");
}
#endif  // FLUX_ATTN_W64_D64_UNIT
