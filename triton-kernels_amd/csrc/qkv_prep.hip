// Q/K/V preparation: one streaming pass that gathers q, k, v rows from up to two strided sources
// (txt first, then img) into contiguous [B,H,L,D] tensors, optionally RMS-normalising q and k over
// the head dimension and rotating them with the per-position 2x2 RoPE matrices on the way through.
//
// A row of D elements is owned by D/VEC adjacent lanes (16 lanes for D = 128 in bf16), each holding
// one 16-byte vector = VEC/2 rotation pairs, so the per-row reduction is a DPP butterfly and the
// rotation needs no cross-lane traffic. q and k of the same (b,h,s) are handled by the same lane
// and share the pe registers, and so do four consecutive heads.
#include "common.h"

namespace flux {

constexpr int kPrepBlock = 256;

struct Src {
    const void* txt; int64_t t_sb, t_sh, t_sl;
    const void* img; int64_t i_sb, i_sh, i_sl;
    void* out;
    const void* scale_txt; const void* scale_img;
};

struct PrepParams {
    Src q, k, v;
    const float* pe;
    int64_t pe_sb;
    int64_t H, Lt, L;
    float eps;
    int scale_vec;  // 1: every RMS scale pointer is 16-byte aligned (vector loads)
};

// Row of source s at (b, h0, pos) and the element stride from one head to the next: txt rows first,
// then img rows. Both candidates are formed and one is selected, so there is no branch in front of
// the loads, and the per-head addresses are one multiply-add away.
template <typename T>
__device__ __forceinline__ const T* src_row0(const Src& s, int64_t b, int64_t h0, int64_t pos, int64_t Lt, int64_t& head_stride) {
    const bool is_txt = pos < Lt;
    const T* t = static_cast<const T*>(s.txt) + b * s.t_sb + h0 * s.t_sh + pos * s.t_sl;
    const T* i = static_cast<const T*>(s.img) + b * s.i_sb + h0 * s.i_sh + (pos - Lt) * s.i_sl;
    head_stride = is_txt ? s.t_sh : s.i_sh;
    return is_txt ? t : i;
}

// Heads one thread walks with the same pe / scale registers: the rotation table is read once per
// position and head group instead of once per head, which cuts its share of the L2 traffic from as
// much as q and k together to a quarter of that.
constexpr int kHeadGroup = 4;

// The kernel is straight-line code: rows past the end of the sequence and heads past the last one
// are clamped to the last valid row / head for the loads and only the stores are predicated, so
// every load of a thread (pe, scales, the head group's q and k vectors) is in flight before the
// first one is consumed.
template <typename T, typename TS, int D, bool NORM, bool ROPE>
__global__ __launch_bounds__(kPrepBlock) void qkv_prep_kernel(PrepParams p) {
    constexpr int VEC = Elem<T>::VEC;
    constexpr int G = (D / VEC) < 64 ? (D / VEC) : 64;   // lanes per row
    constexpr int ITER = D / (VEC * G);                   // 16-byte vectors per lane
    constexpr int ROWS = kPrepBlock / G;
    constexpr int HG = ITER == 1 ? kHeadGroup : 1;        // long rows already give a thread enough loads in flight
    static_assert(G * ITER * VEC == D, "head dim must be a multiple of the vector width");
    const int lane = threadIdx.x % G;
    // Consecutive workgroup ids go round the eight XCDs, each with an L2 of its own. The grid is a
    // multiple of eight and XCD x takes the x-th contiguous eighth of the virtual block order, in
    // which the head group moves fastest: all head groups of a stretch of positions run on one XCD,
    // whose L2 then fetches those positions' pe rows (and a fused projection's source rows) once.
    const int64_t groups = (p.H + HG - 1) / HG;
    const int64_t per_xcd = gridDim.x / 8;
    const int64_t vb = static_cast<int64_t>(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (vb >= groups * ((p.L + ROWS - 1) / ROWS)) return;   // padding blocks of the rounded-up grid
    const int64_t pos_raw = (vb / groups) * ROWS + threadIdx.x / G;
    const int64_t b = blockIdx.y, h0 = (vb % groups) * HG;
    const bool ok = pos_raw < p.L;
    const int64_t pos = ok ? pos_raw : p.L - 1;
    const bool is_txt = pos < p.Lt;
    int hd[HG];      // head offset from h0, clamped to the last head
    bool hok[HG];
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        hok[g] = ok && h0 + g < p.H;
        hd[g] = h0 + g < p.H ? g : static_cast<int>(p.H - 1 - h0);
    }
    const int64_t out_row0 = ((b * p.H + h0) * p.L + pos) * D;   // output row of head h0; the next head is L * D further
    const int64_t out_head = p.L * D;

    // pe[pos, pair, a, j]: the lane's vector at column c covers pairs c/2 .. c/2 + VEC/2 - 1
    float f[ITER][VEC * 2];
    if (ROPE) {
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int c = (it * G + lane) * VEC;
            const float* fp = p.pe + b * p.pe_sb + pos * (2 * D) + c * 2;
#pragma unroll
            for (int i = 0; i < VEC * 2 / 4; ++i) {
                Vec16<float> t = ld16(fp + i * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) f[it][i * 4 + e] = t.v[e];
            }
        }
    }

    // v: bit-exact copy
    if (p.v.out != nullptr) {
        int64_t v_hs;
        const T* v_src0 = src_row0<T>(p.v, b, h0, pos, p.Lt, v_hs);
        Vec16<T> vv[HG][ITER];
#pragma unroll
        for (int g = 0; g < HG; ++g) {
            const T* src = v_src0 + hd[g] * v_hs;
#pragma unroll
            for (int it = 0; it < ITER; ++it) vv[g][it] = ld16(src + (it * G + lane) * VEC);
        }
#pragma unroll
        for (int g = 0; g < HG; ++g) {
            T* out = static_cast<T*>(p.v.out) + out_row0 + hd[g] * out_head;
            if (hok[g]) {
#pragma unroll
                for (int it = 0; it < ITER; ++it) st16(out + (it * G + lane) * VEC, vv[g][it]);
            }
        }
    }

    // all q and k loads of the head group go out before the first one is used
    Vec16<T> raw[2][HG][ITER];
    float w[2][ITER][VEC];
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const Src& s = which == 0 ? p.q : p.k;
        if (s.out == nullptr) continue;  // uniform over the grid
        int64_t hs;
        const T* src0 = src_row0<T>(s, b, h0, pos, p.Lt, hs);
#pragma unroll
        for (int g = 0; g < HG; ++g) {
            const T* src = src0 + hd[g] * hs;
#pragma unroll
            for (int it = 0; it < ITER; ++it) raw[which][g][it] = ld16(src + (it * G + lane) * VEC);
        }
        if (NORM) {
            const TS* sc = static_cast<const TS*>(is_txt ? s.scale_txt : s.scale_img);
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                const TS* sp = sc + (it * G + lane) * VEC;
                if (p.scale_vec) {
#pragma unroll
                    for (int i = 0; i < VEC / Elem<TS>::VEC; ++i) {
                        const Vec16<TS> t = ld16(sp + i * Elem<TS>::VEC);
#pragma unroll
                        for (int e = 0; e < Elem<TS>::VEC; ++e) w[which][it][i * Elem<TS>::VEC + e] = Elem<TS>::load(t.v[e]);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) w[which][it][e] = Elem<TS>::load(sp[e]);
                }
            }
        }
    }

#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const Src& s = which == 0 ? p.q : p.k;
        if (s.out == nullptr) continue;
#pragma unroll
        for (int g = 0; g < HG; ++g) {
            T* out = static_cast<T*>(s.out) + out_row0 + hd[g] * out_head;
            if (!NORM && !ROPE) {
                if (hok[g]) {
#pragma unroll
                    for (int it = 0; it < ITER; ++it) st16(out + (it * G + lane) * VEC, raw[which][g][it]);
                }
                continue;
            }
            float x[ITER][VEC];
#pragma unroll
            for (int it = 0; it < ITER; ++it)
#pragma unroll
                for (int e = 0; e < VEC; ++e) x[it][e] = Elem<T>::load(raw[which][g][it].v[e]);
            if (NORM) {
                float ss = 0.0f;
#pragma unroll
                for (int it = 0; it < ITER; ++it)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) ss += x[it][e] * x[it][e];
                ss = group_sum<G>(ss);
                const float rstd = rsqrtf(ss / static_cast<float>(D) + p.eps);
#pragma unroll
                for (int it = 0; it < ITER; ++it)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x[it][e] = Elem<T>::round(Elem<T>::round(x[it][e] * rstd) * w[which][it][e]);
            }
            Vec16<T> o[ITER];
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                if (ROPE) {
#pragma unroll
                    for (int i = 0; i < VEC / 2; ++i) {
                        const float x0 = x[it][2 * i], x1 = x[it][2 * i + 1];
                        o[it].v[2 * i] = Elem<T>::store(f[it][4 * i + 0] * x0 + f[it][4 * i + 1] * x1);
                        o[it].v[2 * i + 1] = Elem<T>::store(f[it][4 * i + 2] * x0 + f[it][4 * i + 3] * x1);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) o[it].v[e] = Elem<T>::store(x[it][e]);
                }
            }
            if (hok[g]) {
#pragma unroll
                for (int it = 0; it < ITER; ++it) st16(out + (it * G + lane) * VEC, o[it]);
            }
        }
    }
}

static bool src_ok(const flux_src4& s, int vec) {
    return s.ptr != nullptr && aligned16(s.ptr) && s.sb % vec == 0 && s.sh % vec == 0 && s.sl % vec == 0;
}

template <typename T, typename TS>
static int prep_launch(const flux_qkv_prep_args& a, hipStream_t st) {
    constexpr int VEC = Elem<T>::VEC;
    const int64_t L = a.Lt + a.Li;
    PrepParams p;
    const flux_src4* txt[3] = {&a.q_txt, &a.k_txt, &a.v_txt};
    const flux_src4* img[3] = {&a.q_img, &a.k_img, &a.v_img};
    void* outs[3] = {a.q_out, a.k_out, a.v_out};
    const void* sc_t[3] = {a.q_scale_txt, a.k_scale_txt, nullptr};
    const void* sc_i[3] = {a.q_scale_img, a.k_scale_img, nullptr};
    Src* dst[3] = {&p.q, &p.k, &p.v};
    const bool norm = a.q_scale_txt || a.q_scale_img || a.k_scale_txt || a.k_scale_img;
    bool any = false;
    for (int i = 0; i < 3; ++i) {
        Src& s = *dst[i];
        s = Src{};
        if (outs[i] == nullptr) continue;
        any = true;
        if (!aligned16(outs[i])) return fail(FLUX_E_ALIGN, "flux_qkv_prep: output %d is not 16-byte aligned", i);
        if (a.Lt > 0 && !src_ok(*txt[i], VEC)) return fail(FLUX_E_ALIGN, "flux_qkv_prep: txt source %d is null or not 16-byte addressable", i);
        if (a.Li > 0 && !src_ok(*img[i], VEC)) return fail(FLUX_E_ALIGN, "flux_qkv_prep: img source %d is null or not 16-byte addressable", i);
        s.txt = txt[i]->ptr; s.t_sb = txt[i]->sb; s.t_sh = txt[i]->sh; s.t_sl = txt[i]->sl;
        s.img = img[i]->ptr; s.i_sb = img[i]->sb; s.i_sh = img[i]->sh; s.i_sl = img[i]->sl;
        s.out = outs[i];
        if (i < 2 && norm) {
            if ((a.Lt > 0 && !sc_t[i]) || (a.Li > 0 && !sc_i[i])) return fail(FLUX_E_NULL, "flux_qkv_prep: RMS scale missing for tensor %d", i);
            s.scale_txt = sc_t[i];
            s.scale_img = sc_i[i];
        }
    }
    if (!any) return FLUX_OK;
    const bool rope = a.pe != nullptr;
    if (rope && !aligned16(a.pe)) return fail(FLUX_E_ALIGN, "flux_qkv_prep: pe is not 16-byte aligned");
    if (rope && a.pe_batch_stride % 4 != 0) return fail(FLUX_E_ALIGN, "flux_qkv_prep: pe batch stride must be a multiple of 4");
    p.pe = a.pe;
    p.pe_sb = a.pe_batch_stride;
    p.H = a.H; p.Lt = a.Lt; p.L = L; p.eps = a.eps;
    p.scale_vec = 1;
    for (int i = 0; i < 2; ++i)
        if ((sc_t[i] && !aligned16(sc_t[i])) || (sc_i[i] && !aligned16(sc_i[i]))) p.scale_vec = 0;

    const int D = a.D;
    const int lanes_per_row = D / VEC < 64 ? D / VEC : 64;
    const int rows_per_block = kPrepBlock / (lanes_per_row > 0 ? lanes_per_row : 1);
    // rows of one 16-byte vector per lane are walked kHeadGroup heads at a time (see the kernel)
    const int64_t hg = (D / VEC <= 64) ? kHeadGroup : 1;
    const int64_t pos_blocks = (L + rows_per_block - 1) / rows_per_block, groups = (a.H + hg - 1) / hg;
    if (a.B > 65535 || pos_blocks * groups > 0x7ffffff0LL) return fail(FLUX_E_SHAPE, "flux_qkv_prep: grid too large (B=%lld, L=%lld, H=%lld)", (long long)a.B, (long long)L, (long long)a.H);
    dim3 grid((unsigned)((pos_blocks * groups + 7) / 8 * 8), (unsigned)a.B);   // the kernel deals blocks out by XCD

#define LAUNCH(D_, N_, R_) hipLaunchKernelGGL((qkv_prep_kernel<T, TS, D_, N_, R_>), grid, dim3(kPrepBlock), 0, st, p)
#define BY_FLAGS(D_)                                   \
    do {                                               \
        if (norm && rope) LAUNCH(D_, true, true);      \
        else if (norm) LAUNCH(D_, true, false);        \
        else if (rope) LAUNCH(D_, false, true);        \
        else LAUNCH(D_, false, false);                 \
    } while (0)
    if (D == 16) BY_FLAGS(16);
    else if (D == 32) BY_FLAGS(32);
    else if (D == 64) BY_FLAGS(64);
    else if (D == 128) BY_FLAGS(128);
    else if (D == 256) BY_FLAGS(256);
    else if (D == 512) BY_FLAGS(512);
    else return fail(FLUX_E_UNSUPPORTED, "flux_qkv_prep: head dim %d not supported (16, 32, 64, 128, 256, 512)", D);
#undef BY_FLAGS
#undef LAUNCH
    return check_launch("flux_qkv_prep");
}

}  // namespace flux

using namespace flux;

extern "C" int flux_qkv_prep(const flux_qkv_prep_args* a, void* stream) {
    if (!a) return fail(FLUX_E_NULL, "flux_qkv_prep: null args");
    if (a->B < 0 || a->H <= 0 || a->Lt < 0 || a->Li < 0 || a->D <= 0) return fail(FLUX_E_SHAPE, "flux_qkv_prep: bad shape B=%lld H=%lld Lt=%lld Li=%lld D=%d", (long long)a->B, (long long)a->H, (long long)a->Lt, (long long)a->Li, a->D);
    if (a->B == 0 || a->Lt + a->Li == 0) return FLUX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a->dtype == FLUX_BF16 && a->scale_dtype == FLUX_BF16) return prep_launch<bf16_t, bf16_t>(*a, st);
    if (a->dtype == FLUX_BF16 && a->scale_dtype == FLUX_F32) return prep_launch<bf16_t, float>(*a, st);
    if (a->dtype == FLUX_F32 && a->scale_dtype == FLUX_F32) return prep_launch<float, float>(*a, st);
    return fail(FLUX_E_DTYPE, "flux_qkv_prep: unsupported dtype pair (%d,%d)", a->dtype, a->scale_dtype);
}
