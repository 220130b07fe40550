// Small element-wise kernels: SiLU, tanh-GELU on a strided [rows, n] view, adaLN scale/shift on an
// already normalised tensor, and the gated residual. All are single-pass streams with 16-byte
// accesses when pointers and strides allow it and a scalar path otherwise.
#include "common.h"

namespace flux {

constexpr int kEwBlock = 256;

template <typename T, int VEC>
struct Pack {
    T v[VEC];
};

template <typename T, int VEC>
__device__ __forceinline__ void ld(const T* p, float (&out)[VEC]) {
    if constexpr (VEC == 1) {
        out[0] = Elem<T>::load(p[0]);
    } else {
        Vec16<T> t = ld16(p);
#pragma unroll
        for (int e = 0; e < VEC; ++e) out[e] = Elem<T>::load(t.v[e]);
    }
}
template <typename T, int VEC>
__device__ __forceinline__ void st(T* p, const float (&in)[VEC]) {
    if constexpr (VEC == 1) {
        p[0] = Elem<T>::store(in[0]);
    } else {
        Vec16<T> t;
#pragma unroll
        for (int e = 0; e < VEC; ++e) t.v[e] = Elem<T>::store(in[e]);
        st16(p, t);
    }
}

enum class Unary { Silu, Gelu };

// y[r, c] = op(x[r, c]) over a [rows, n] view; one thread per VEC columns, grid-stride over rows.
template <typename T, int VEC, Unary OP>
__global__ __launch_bounds__(kEwBlock) void unary_rows_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows,
                                                              int64_t n, int64_t ldx, int64_t ldy) {
    const int64_t nvec = n / VEC;  // VEC == 1 or n % VEC == 0
    const int64_t total = rows * nvec;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * kEwBlock) {
        const int64_t r = i / nvec, c = (i % nvec) * VEC;
        float v[VEC];
        ld<T, VEC>(x + r * ldx + c, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            if (OP == Unary::Silu) v[e] = v[e] * __builtin_amdgcn_rcpf(1.0f + __expf(-v[e]));
            else v[e] = gelu_tanh_f32(v[e]);
        }
        st<T, VEC>(y + r * ldy + c, v);
    }
}

// out = (1 + scale[b]) * x + shift[b]
template <typename T, int VEC>
__global__ __launch_bounds__(kEwBlock) void scale_shift_kernel(const T* __restrict__ x, const T* __restrict__ shift,
                                                               const T* __restrict__ scale, T* __restrict__ out,
                                                               int64_t rows, int64_t seq, int64_t hid, int64_t mod_stride) {
    const int64_t nvec = hid / VEC;
    const int64_t total = rows * nvec;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * kEwBlock) {
        const int64_t r = i / nvec, c = (i % nvec) * VEC;
        const int64_t b = r / seq;
        float xv[VEC], sh[VEC], sc[VEC];
        ld<T, VEC>(x + r * hid + c, xv);
        ld<T, VEC>(shift + b * mod_stride + c, sh);
        ld<T, VEC>(scale + b * mod_stride + c, sc);
#pragma unroll
        for (int e = 0; e < VEC; ++e) xv[e] = (sc[e] + 1.0f) * xv[e] + sh[e];
        st<T, VEC>(out + r * hid + c, xv);
    }
}

// out = x + gate[b] * y
template <typename T, int VEC, bool ROUND>
__global__ __launch_bounds__(kEwBlock) void gate_residual_kernel(const T* __restrict__ x, const T* __restrict__ gate,
                                                                 const T* __restrict__ y, T* __restrict__ out, int64_t rows,
                                                                 int64_t seq, int64_t hid, int64_t gate_stride) {
    const int64_t nvec = hid / VEC;
    const int64_t total = rows * nvec;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * kEwBlock) {
        const int64_t r = i / nvec, c = (i % nvec) * VEC;
        const int64_t b = r / seq;
        float xv[VEC], g[VEC], yv[VEC];
        ld<T, VEC>(x + r * hid + c, xv);
        ld<T, VEC>(gate + b * gate_stride + c, g);
        ld<T, VEC>(y + r * hid + c, yv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float pr = g[e] * yv[e];
            if (ROUND) pr = Elem<T>::round(pr);
            xv[e] = xv[e] + pr;
        }
        st<T, VEC>(out + r * hid + c, xv);
    }
}

static unsigned ew_grid(int64_t work_items) {
    int64_t blocks = (work_items + kEwBlock - 1) / kEwBlock;
    const int64_t cap = 256 * 16;  // 16 resident blocks per CU is plenty for a stream
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return static_cast<unsigned>(blocks);
}

template <typename T, Unary OP>
static int unary_launch(const void* x, void* y, int64_t rows, int64_t n, int64_t ldx, int64_t ldy, hipStream_t st,
                        const char* name) {
    constexpr int VEC = Elem<T>::VEC;
    const T* xp = static_cast<const T*>(x);
    T* yp = static_cast<T*>(y);
    const bool vec_ok = aligned16(x) && aligned16(y) && n % VEC == 0 && ldx % VEC == 0 && ldy % VEC == 0;
    if (vec_ok)
        hipLaunchKernelGGL((unary_rows_kernel<T, VEC, OP>), dim3(ew_grid(rows * (n / VEC))), dim3(kEwBlock), 0, st, xp, yp,
                           rows, n, ldx, ldy);
    else
        hipLaunchKernelGGL((unary_rows_kernel<T, 1, OP>), dim3(ew_grid(rows * n)), dim3(kEwBlock), 0, st, xp, yp, rows, n,
                           ldx, ldy);
    return check_launch(name);
}

}  // namespace flux

using namespace flux;

extern "C" int flux_silu(const void* x, void* y, int64_t numel, int32_t dtype, void* stream) {
    if (!x || !y) return fail(FLUX_E_NULL, "flux_silu: null pointer");
    if (numel < 0) return fail(FLUX_E_SHAPE, "flux_silu: negative size");
    if (numel == 0) return FLUX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == FLUX_BF16) return unary_launch<bf16_t, Unary::Silu>(x, y, 1, numel, numel, numel, st, "flux_silu");
    if (dtype == FLUX_F32) return unary_launch<float, Unary::Silu>(x, y, 1, numel, numel, numel, st, "flux_silu");
    return fail(FLUX_E_DTYPE, "flux_silu: unsupported dtype %d", dtype);
}

extern "C" int flux_gelu_tanh(const void* x, void* y, int64_t rows, int64_t n, int64_t ldx, int64_t ldy, int32_t dtype,
                              void* stream) {
    if (!x || !y) return fail(FLUX_E_NULL, "flux_gelu_tanh: null pointer");
    if (rows < 0 || n < 0) return fail(FLUX_E_SHAPE, "flux_gelu_tanh: negative size");
    if (rows == 0 || n == 0) return FLUX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == FLUX_BF16) return unary_launch<bf16_t, Unary::Gelu>(x, y, rows, n, ldx, ldy, st, "flux_gelu_tanh");
    if (dtype == FLUX_F32) return unary_launch<float, Unary::Gelu>(x, y, rows, n, ldx, ldy, st, "flux_gelu_tanh");
    return fail(FLUX_E_DTYPE, "flux_gelu_tanh: unsupported dtype %d", dtype);
}

template <typename T>
static int scale_shift_launch(const void* x, const void* mod, void* out, int64_t batch, int64_t seq, int64_t hid,
                              int64_t mod_stride, int is_mod1, hipStream_t st) {
    constexpr int VEC = Elem<T>::VEC;
    const T* m = static_cast<const T*>(mod);
    const int chunk = is_mod1 ? 0 : 3;
    const T* shift = m + chunk * hid;
    const T* scale = m + (chunk + 1) * hid;
    const int64_t rows = batch * seq;
    const bool vec_ok = aligned16(x) && aligned16(out) && aligned16(mod) && hid % VEC == 0 && mod_stride % VEC == 0;
    if (vec_ok)
        hipLaunchKernelGGL((scale_shift_kernel<T, VEC>), dim3(ew_grid(rows * (hid / VEC))), dim3(kEwBlock), 0, st,
                           static_cast<const T*>(x), shift, scale, static_cast<T*>(out), rows, seq, hid, mod_stride);
    else
        hipLaunchKernelGGL((scale_shift_kernel<T, 1>), dim3(ew_grid(rows * hid)), dim3(kEwBlock), 0, st,
                           static_cast<const T*>(x), shift, scale, static_cast<T*>(out), rows, seq, hid, mod_stride);
    return check_launch("flux_modulation_scale_shift");
}

extern "C" int flux_modulation_scale_shift(const void* x, const void* mod, void* out, int64_t batch, int64_t seq,
                                           int64_t hid, int64_t mod_row_stride, int32_t is_mod1, int32_t dtype,
                                           void* stream) {
    if (!x || !mod || !out) return fail(FLUX_E_NULL, "flux_modulation_scale_shift: null pointer");
    if (batch < 0 || seq < 0 || hid <= 0) return fail(FLUX_E_SHAPE, "flux_modulation_scale_shift: bad shape");
    if (batch * seq == 0) return FLUX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == FLUX_BF16) return scale_shift_launch<bf16_t>(x, mod, out, batch, seq, hid, mod_row_stride, is_mod1, st);
    if (dtype == FLUX_F32) return scale_shift_launch<float>(x, mod, out, batch, seq, hid, mod_row_stride, is_mod1, st);
    return fail(FLUX_E_DTYPE, "flux_modulation_scale_shift: unsupported dtype %d", dtype);
}

template <typename T>
static int gate_launch(const void* x, const void* gate, const void* y, void* out, int64_t batch, int64_t seq, int64_t hid,
                       int64_t gate_stride, int round_product, hipStream_t st) {
    constexpr int VEC = Elem<T>::VEC;
    const int64_t rows = batch * seq;
    const T* xp = static_cast<const T*>(x);
    const T* gp = static_cast<const T*>(gate);
    const T* yp = static_cast<const T*>(y);
    T* op = static_cast<T*>(out);
    const bool vec_ok = aligned16(x) && aligned16(out) && aligned16(gate) && aligned16(y) && hid % VEC == 0 && gate_stride % VEC == 0;
#define GATE_LAUNCH(V_, R_, ITEMS_) \
    hipLaunchKernelGGL((gate_residual_kernel<T, V_, R_>), dim3(ew_grid(ITEMS_)), dim3(kEwBlock), 0, st, xp, gp, yp, op, rows, seq, hid, gate_stride)
    if (vec_ok) {
        if (round_product) GATE_LAUNCH(VEC, true, rows * (hid / VEC));
        else GATE_LAUNCH(VEC, false, rows * (hid / VEC));
    } else {
        if (round_product) GATE_LAUNCH(1, true, rows * hid);
        else GATE_LAUNCH(1, false, rows * hid);
    }
#undef GATE_LAUNCH
    return check_launch("flux_gate_residual");
}

extern "C" int flux_gate_residual(const void* x, const void* gate, const void* y, void* out, int64_t batch, int64_t seq,
                                  int64_t hid, int64_t gate_batch_stride, int32_t round_product, int32_t dtype,
                                  void* stream) {
    if (!x || !gate || !y || !out) return fail(FLUX_E_NULL, "flux_gate_residual: null pointer");
    if (batch < 0 || seq < 0 || hid <= 0) return fail(FLUX_E_SHAPE, "flux_gate_residual: bad shape");
    if (batch * seq == 0) return FLUX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == FLUX_BF16) return gate_launch<bf16_t>(x, gate, y, out, batch, seq, hid, gate_batch_stride, round_product, st);
    if (dtype == FLUX_F32) return gate_launch<float>(x, gate, y, out, batch, seq, hid, gate_batch_stride, round_product, st);
    return fail(FLUX_E_DTYPE, "flux_gate_residual: unsupported dtype %d", dtype);
}
