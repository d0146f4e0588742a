// Streaming (HBM-bound) residue kernels: add / sub / negate / multiply / multiply-accumulate,
// constant multiplies, the 3-polynomial tensor product and the NTT-domain Galois permutation.
// One workgroup covers 512 consecutive residues of one limb with 16-byte accesses; blockIdx.y
// walks (poly, limb) so every wavefront streams one contiguous 4 KiB run.
#include <algorithm>

#include "hemm_internal.hpp"

namespace {

struct Operand {
    const u64 *p;
    size_t poly_stride;  // elements between polynomials (0 = broadcast one polynomial)
};

enum { OP_ADD = 0, OP_SUB = 1, OP_MUL = 2, OP_NEG = 3, OP_MAC = 4 };

template <int OP>
__global__ __launch_bounds__(256) void binary_kernel(Operand a, Operand b, u64 *__restrict__ out, size_t out_stride,
                                                     const ModQ *__restrict__ modq, LimbList ll, int n_limbs,
                                                     int logN) {
    const int limb = blockIdx.y % n_limbs, poly = blockIdx.y / n_limbs;
    const ModQ m = modq[ll.idx[limb]];
    const size_t e = ((size_t)limb << logN) + ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const ulonglong2 x = *(const ulonglong2 *)(a.p + poly * a.poly_stride + e);
    ulonglong2 y = make_ulonglong2(0, 0);
    if (OP != OP_NEG) y = *(const ulonglong2 *)(b.p + poly * b.poly_stride + e);
    ulonglong2 *o = (ulonglong2 *)(out + poly * out_stride + e);
    ulonglong2 r;
    if (OP == OP_ADD) {
        r.x = addmod(x.x, y.x, m.q);
        r.y = addmod(x.y, y.y, m.q);
    } else if (OP == OP_SUB) {
        r.x = submod(x.x, y.x, m.q);
        r.y = submod(x.y, y.y, m.q);
    } else if (OP == OP_MUL) {
        r.x = mulmod(x.x, y.x, m);
        r.y = mulmod(x.y, y.y, m);
    } else if (OP == OP_NEG) {
        r.x = negmod(x.x, m.q);
        r.y = negmod(x.y, m.q);
    } else {
        ulonglong2 c = *o;
        r.x = addmod(c.x, mulmod(x.x, y.x, m), m.q);
        r.y = addmod(c.y, mulmod(x.y, y.y, m), m.q);
    }
    *o = r;
}

struct ScalarList {
    u64 w[HEMM_MAX_PRIMES], ws[HEMM_MAX_PRIMES];  // per limb: constant and its Shoup quotient
};

// out = a * scalar[limb]; IMAG: scalar is psi^(N/2) and the sign flips on the upper half of the
// bit-reversed index range (factor psi^{(N/2)(2 bitrev(k)+1)} = I * (-1)^{bitrev(k)}).
template <bool IMAG>
__global__ __launch_bounds__(256) void scalar_kernel(Operand a, u64 *__restrict__ out, size_t out_stride,
                                                     const ModQ *__restrict__ modq, LimbList ll, ScalarList sc,
                                                     int n_limbs, int logN) {
    const int limb = blockIdx.y % n_limbs, poly = blockIdx.y / n_limbs;
    const u64 q = modq[ll.idx[limb]].q;
    const size_t k = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const size_t e = ((size_t)limb << logN) + k;
    const ulonglong2 x = *(const ulonglong2 *)(a.p + poly * a.poly_stride + e);
    ulonglong2 r;
    r.x = mul_shoup(x.x, sc.w[limb], sc.ws[limb], q);
    r.y = mul_shoup(x.y, sc.w[limb], sc.ws[limb], q);
    if (IMAG && (k >> (logN - 1))) {
        r.x = negmod(r.x, q);
        r.y = negmod(r.y, q);
    }
    *(ulonglong2 *)(out + poly * out_stride + e) = r;
}

// out = a + re[limb] + im[limb] * (-1)^{bitrev(k) & 1}: the NTT form of the constant polynomial re + im' X^(N/2)
// (im[limb] = im' psi^(N/2), the sign flips on the upper half of the bit-reversed index range), i.e. a complex
// constant in every slot, added without encoding a plaintext.
__global__ __launch_bounds__(256) void scalar_add_kernel(Operand a, u64 *__restrict__ out, size_t out_stride,
                                                         const ModQ *__restrict__ modq, LimbList ll, ScalarList sc,
                                                         int n_limbs, int logN) {
    const int limb = blockIdx.y;
    const u64 q = modq[ll.idx[limb]].q;
    const size_t k = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const size_t e = ((size_t)limb << logN) + k;
    const ulonglong2 x = *(const ulonglong2 *)(a.p + e);
    const u64 im = (k >> (logN - 1)) ? negmod(sc.ws[limb], q) : sc.ws[limb];
    const u64 c = addmod(sc.w[limb], im, q);
    *(ulonglong2 *)(out + e) = make_ulonglong2(addmod(x.x, c, q), addmod(x.y, c, q));
}

// (b1,a1) x (b2,a2) -> (b1 b2, a1 b2 + a2 b1, a1 a2); ACC adds into out.
template <bool ACC>
__global__ __launch_bounds__(256) void tensor_kernel(Operand c1, Operand c2, u64 *__restrict__ out, size_t out_stride,
                                                     const ModQ *__restrict__ modq, int logN) {
    const int limb = blockIdx.y;
    const ModQ m = modq[limb];
    const size_t e = ((size_t)limb << logN) + (size_t)blockIdx.x * 256 + threadIdx.x;
    const u64 b1 = c1.p[e], a1 = c1.p[c1.poly_stride + e];
    const u64 b2 = c2.p[e], a2 = c2.p[c2.poly_stride + e];
    u64 d0 = mulmod(b1, b2, m);
    u128_t t = mul64wide(a1, b2);
    add128(t, mul64wide(a2, b1));
    u64 d1 = barrett128(t, m);
    u64 d2 = mulmod(a1, a2, m);
    if (ACC) {
        d0 = addmod(d0, out[e], m.q);
        d1 = addmod(d1, out[out_stride + e], m.q);
        d2 = addmod(d2, out[2 * out_stride + e], m.q);
    }
    out[e] = d0;
    out[out_stride + e] = d1;
    out[2 * out_stride + e] = d2;
}

// NTT-domain automorphism X -> X^g: out[k] = in[k'], 2 bitrev(k') + 1 = (2 bitrev(k) + 1) g mod 2N.
// Prime independent, so one launch moves every limb of every polynomial.
__global__ __launch_bounds__(256) void galois_kernel(Operand a, u64 *__restrict__ out, size_t out_stride, u32 g,
                                                     int n_limbs, int logN) {
    const int limb = blockIdx.y % n_limbs, poly = blockIdx.y / n_limbs;
    const u32 k = blockIdx.x * 256 + threadIdx.x;
    const u32 mask2n = (2u << logN) - 1;
    const u32 br = __brev(k) >> (32 - logN);
    const u32 e = ((2 * br + 1) * g) & mask2n;
    const u32 kp = __brev(e >> 1) >> (32 - logN);
    const size_t base = (size_t)limb << logN;
    out[poly * out_stride + base + k] = a.p[poly * a.poly_stride + base + kp];
}

}  // namespace

void launch_binary(const hemm_context *c, int op, const u64 *a, size_t a_stride, const u64 *b, size_t b_stride,
                   u64 *out, size_t out_stride, const LimbList &ll, int n_limbs, int n_polys, hipStream_t s) {
    dim3 grid(c->N / 512, n_limbs * n_polys), block(256);
    Operand A{a, a_stride}, B{b, b_stride};
    account(c, TR_POINTWISE, (size_t)(op == OP_NEG ? 2 : op == OP_MAC ? 4 : 3) * n_limbs * n_polys * c->N * 8);
    switch (op) {
        case OP_ADD: hipLaunchKernelGGL(binary_kernel<OP_ADD>, grid, block, 0, s, A, B, out, out_stride, c->d_modq, ll, n_limbs, c->logN); break;
        case OP_SUB: hipLaunchKernelGGL(binary_kernel<OP_SUB>, grid, block, 0, s, A, B, out, out_stride, c->d_modq, ll, n_limbs, c->logN); break;
        case OP_MUL: hipLaunchKernelGGL(binary_kernel<OP_MUL>, grid, block, 0, s, A, B, out, out_stride, c->d_modq, ll, n_limbs, c->logN); break;
        case OP_NEG: hipLaunchKernelGGL(binary_kernel<OP_NEG>, grid, block, 0, s, A, B, out, out_stride, c->d_modq, ll, n_limbs, c->logN); break;
        case OP_MAC: hipLaunchKernelGGL(binary_kernel<OP_MAC>, grid, block, 0, s, A, B, out, out_stride, c->d_modq, ll, n_limbs, c->logN); break;
        default: throw std::invalid_argument("unknown pointwise op");
    }
}

static u64 shoup_host(u64 w, u64 q) { return (u64)((((unsigned __int128)w) << 64) / q); }

// scalars[limb] are plain residues (already reduced mod the limb's prime)
void launch_mul_scalar(const hemm_context *c, const u64 *a, size_t a_stride, const u64 *scalars, u64 *out,
                       size_t out_stride, const LimbList &ll, int n_limbs, int n_polys, hipStream_t s) {
    ScalarList sc;
    for (int j = 0; j < n_limbs; j++) {
        u64 q = c->primes[ll.idx[j]];
        sc.w[j] = scalars[j] % q;
        sc.ws[j] = shoup_host(sc.w[j], q);
    }
    dim3 grid(c->N / 512, n_limbs * n_polys), block(256);
    Operand A{a, a_stride};
    account(c, TR_POINTWISE, (size_t)2 * n_limbs * n_polys * c->N * 8);
    hipLaunchKernelGGL(scalar_kernel<false>, grid, block, 0, s, A, out, out_stride, c->d_modq, ll, sc, n_limbs, c->logN);
}

// out[0 .. words) = 0 (words a multiple of 2): a fill kernel where a memset node would be recorded into a captured graph
__global__ __launch_bounds__(256) void zero_kernel(ulonglong2 *__restrict__ out, size_t pairs) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < pairs; i += (size_t)gridDim.x * 256)
        out[i] = make_ulonglong2(0, 0);
}
void launch_zero(const hemm_context *c, u64 *out, size_t words, hipStream_t s) {
    const size_t pairs = words / 2;
    const unsigned blocks = (unsigned)std::min<size_t>((pairs + 255) / 256, 4096);
    account(c, TR_POINTWISE, words * 8);
    hipLaunchKernelGGL(zero_kernel, dim3(blocks), dim3(256), 0, s, (ulonglong2 *)out, pairs);
}

void launch_mul_imag(const hemm_context *c, const u64 *a, size_t a_stride, u64 *out, size_t out_stride,
                     const LimbList &ll, int n_limbs, int n_polys, hipStream_t s) {
    ScalarList sc;
    for (int j = 0; j < n_limbs; j++) {
        u64 q = c->primes[ll.idx[j]];
        sc.w[j] = h_powmod(c->psi[ll.idx[j]], (u64)c->N / 2, q);
        sc.ws[j] = shoup_host(sc.w[j], q);
    }
    dim3 grid(c->N / 512, n_limbs * n_polys), block(256);
    Operand A{a, a_stride};
    account(c, TR_POINTWISE, (size_t)2 * n_limbs * n_polys * c->N * 8);
    hipLaunchKernelGGL(scalar_kernel<true>, grid, block, 0, s, A, out, out_stride, c->d_modq, ll, sc, n_limbs, c->logN);
}

// re / im: one residue per limb (im may be nullptr); one polynomial
void launch_add_scalar(const hemm_context *c, const u64 *a, const u64 *re, const u64 *im, u64 *out, const LimbList &ll,
                       int n_limbs, hipStream_t s) {
    ScalarList sc;
    for (int j = 0; j < n_limbs; j++) {
        const u64 q = c->primes[ll.idx[j]];
        sc.w[j] = re[j] % q;
        // im' X^(N/2) evaluates to im' psi^(N/2) (2 bitrev(k) + 1 odd): the kernel flips its sign by slot
        sc.ws[j] = im ? h_mulmod(im[j] % q, h_powmod(c->psi[ll.idx[j]], (u64)c->N / 2, q), q) : 0;
    }
    dim3 grid(c->N / 512, n_limbs), block(256);
    Operand A{a, 0};
    account(c, TR_POINTWISE, (size_t)2 * n_limbs * c->N * 8);
    hipLaunchKernelGGL(scalar_add_kernel, grid, block, 0, s, A, out, (size_t)0, c->d_modq, ll, sc, n_limbs, c->logN);
}

void launch_tensor(const hemm_context *c, const u64 *c1, size_t s1, const u64 *c2, size_t s2, u64 *out,
                   size_t out_stride, int nq, bool accumulate, hipStream_t s) {
    dim3 grid(c->N / 256, nq), block(256);
    Operand A{c1, s1}, B{c2, s2};
    account(c, TR_TENSOR, (size_t)(accumulate ? 10 : 7) * nq * c->N * 8);
    if (accumulate)
        hipLaunchKernelGGL(tensor_kernel<true>, grid, block, 0, s, A, B, out, out_stride, c->d_modq, c->logN);
    else
        hipLaunchKernelGGL(tensor_kernel<false>, grid, block, 0, s, A, B, out, out_stride, c->d_modq, c->logN);
}

void launch_galois(const hemm_context *c, const u64 *a, size_t a_stride, u64 *out, size_t out_stride, u64 g,
                   int n_limbs, int n_polys, hipStream_t s) {
    dim3 grid(c->N / 256, n_limbs * n_polys), block(256);
    Operand A{a, a_stride};
    account(c, TR_POINTWISE, (size_t)2 * n_limbs * n_polys * c->N * 8);
    hipLaunchKernelGGL(galois_kernel, grid, block, 0, s, A, out, out_stride, (u32)g, n_limbs, c->logN);
}
