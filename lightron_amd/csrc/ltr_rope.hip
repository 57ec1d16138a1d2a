// Rotary position embedding for MI355X (gfx950): one streaming pass, the arithmetic of the reference's
// apply_rotary_emb (layers/layers.py:44-70) - adjacent pairs, fp32 complex multiply, cast back - without the
// fp32 / complex temporaries that the torch formulation writes to HBM.  Bound: HBM (2 x element size per element).
#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>
#include "ltr_attn.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct RopeParams {
    const void *x;
    void *out;
    const float *freqs;
    int H, D8;                 // heads, D / 8
    long long S, n_units;      // n_units = B * S * H * D8, one unit = 8 consecutive elements = 4 complex pairs
    long long xs[3], os[3];
    float sign;                // +1, or -1 for the conjugate
};

// A thread rotates 8 consecutive elements (16 bytes of bf16, 32 of fp32).  Consecutive threads take consecutive
// units of one (b, s, h) row, then the next head: global accesses are fully coalesced for packed layouts and
// the (cos, sin) rows (D * 4 bytes per sequence index) are shared by all heads and batches through L2.
// IDX is the type the unit index is decomposed in: 32-bit when the tensor has fewer than 2^32 units (64-bit
// divisions by run-time values cost several hundred instructions per thread and would make the pass ALU bound).
template <bool BF16, class IDX>
__global__ __launch_bounds__(256) void rope_kernel(const RopeParams p) {
    const IDX u = (IDX)blockIdx.x * 256 + threadIdx.x;
    if (u >= (IDX)p.n_units) return;
    const int c = (int)(u % (IDX)p.D8);
    IDX r = u / (IDX)p.D8;
    const int h = (int)(r % (IDX)p.H);
    r /= (IDX)p.H;
    const long long s = (long long)(r % (IDX)p.S), b = (long long)(r / (IDX)p.S);
    const float *f = p.freqs + (s * p.D8 + c) * 8;   // 4 (cos, sin) pairs
    const f32x4 f0 = *(const f32x4 *)f, f1 = *(const f32x4 *)(f + 4);
    const float cs[4] = {f0[0], f0[2], f1[0], f1[2]};
    const float sn[4] = {f0[1] * p.sign, f0[3] * p.sign, f1[1] * p.sign, f1[3] * p.sign};
    const long long xo = b * p.xs[0] + s * p.xs[1] + h * p.xs[2] + c * 8;
    const long long oo = b * p.os[0] + s * p.os[1] + h * p.os[2] + c * 8;
    float v[8];
    if (BF16) {
        const bf16x8 xv = *(const bf16x8 *)((const __bf16 *)p.x + xo);
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = (float)xv[e];
    } else {
        const f32x4 a = *(const f32x4 *)((const float *)p.x + xo), b4 = *(const f32x4 *)((const float *)p.x + xo + 4);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            v[e] = a[e];
            v[4 + e] = b4[e];
        }
    }
    float o[8];
    {
        // (re + j im)(cos + j sin) with the four products rounded separately (no contraction into fused
        // multiply-adds), as the fp32 complex multiply of the reference on the host does
#pragma clang fp contract(off)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float rr = v[2 * i] * cs[i], ii = v[2 * i + 1] * sn[i];
            const float ri = v[2 * i] * sn[i], ir = v[2 * i + 1] * cs[i];
            o[2 * i] = rr - ii;
            o[2 * i + 1] = ri + ir;
        }
    }
    if (BF16) {
        bf16x8 ov;
#pragma unroll
        for (int e = 0; e < 8; e++) ov[e] = (__bf16)o[e];
        *(bf16x8 *)((__bf16 *)p.out + oo) = ov;
    } else {
        f32x4 a, b4;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            a[e] = o[e];
            b4[e] = o[4 + e];
        }
        *(f32x4 *)((float *)p.out + oo) = a;
        *(f32x4 *)((float *)p.out + oo + 4) = b4;
    }
}

// gfx950 only.  The answer is kept per device in an atomic (two host threads making their first call together both do
// the query and store the same value); a failed query is not remembered.
bool on_gfx950() {
    constexpr int MAX_DEVICES = 64;
    static std::atomic<int> arch[MAX_DEVICES];   // 0 unknown, 1 yes, -1 no
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return false;
    int known = arch[dev].load(std::memory_order_acquire);
    if (known == 0) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return false;
        const char *a = prop.gcnArchName;
        known = (a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0') ? 1 : -1;
        arch[dev].store(known, std::memory_order_release);
    }
    return known == 1;
}

}  // namespace

extern "C" int ltr_rope_apply(const ltr_rope_args *a, void *stream) {
    if (!a || !a->x || !a->out || !a->freqs) return LTR_EINVAL;
    if (a->B < 0 || a->H < 0 || a->S < 0 || a->D <= 0) return LTR_EINVAL;
    if (a->D % 8) return LTR_EUNSUP;
    if (a->io_dtype != LTR_BF16 && a->io_dtype != LTR_F32) return LTR_EUNSUP;
    const int esz = a->io_dtype == LTR_BF16 ? 2 : 4;
    // 16-byte vector accesses: base pointers and every stride
    if (((uintptr_t)a->x | (uintptr_t)a->out | (uintptr_t)a->freqs) & 15) return LTR_EALIGN;
    for (int i = 0; i < 3; i++)
        if ((a->x_stride[i] * esz) % 16 || (a->out_stride[i] * esz) % 16) return LTR_EALIGN;
    const long long n_units = (long long)a->B * a->S * a->H * (a->D / 8);
    if (n_units == 0) return LTR_OK;
    if ((n_units + 255) / 256 > 0x7fffffffLL) return LTR_EINVAL;
    if (!on_gfx950()) return LTR_EDEVICE;
    RopeParams p;
    p.x = a->x;
    p.out = a->out;
    p.freqs = a->freqs;
    p.H = a->H;
    p.D8 = a->D / 8;
    p.S = a->S;
    p.n_units = n_units;
    for (int i = 0; i < 3; i++) {
        p.xs[i] = a->x_stride[i];
        p.os[i] = a->out_stride[i];
    }
    p.sign = (a->flags & LTR_ROPE_CONJ) ? -1.f : 1.f;
    const unsigned grid = (unsigned)((n_units + 255) / 256);
    const bool small = n_units + 256 < 0xffffffffLL;
    hipStream_t st = (hipStream_t)stream;
    // the launch's own status (an error left behind by unrelated earlier work is neither reported as ours nor cleared)
    const void *kernel = a->io_dtype == LTR_BF16
                             ? (small ? (const void *)rope_kernel<true, unsigned> : (const void *)rope_kernel<true, unsigned long long>)
                             : (small ? (const void *)rope_kernel<false, unsigned> : (const void *)rope_kernel<false, unsigned long long>);
    void *args[] = {(void *)&p};
    return hipLaunchKernel(kernel, dim3(grid), dim3(256), args, 0, st) == hipSuccess ? LTR_OK : LTR_ELAUNCH;
}
