// CKKS encode / decode on the device: the canonical embedding restricted to the orbit zeta^(5^j) and its inverse
// (HEaaN::EnDecoder::encode / decode, EnDecoder.hpp:51,66), in double precision.
//
//   encode: slots z[n] (n = N/2 complex numbers) -> n-point "special" inverse transform (decimation in frequency,
//           stages len = n, n/2, ..., 2, butterfly (a, b) -> (a + b, (a - b) * ksi[M - 5^j * M / 4 len])) -> bit reversal ->
//           coefficient i = round(Re z_i / n * scale), coefficient i + n = round(Im z_i / n * scale) -> residues modulo
//           every limb's prime -> forward NTT.
//   decode: inverse NTT of the first one or two limbs -> centred integer (CRT over two limbs) / scale -> bit reversal ->
//           stages len = 2, 4, ..., n, butterfly (a, b) -> (a + b ksi, a - b ksi), ksi = ksi[5^j * M / 4 len].
//
// Every floating-point operation is a single IEEE operation in a fixed order (no contraction into fused multiply-adds),
// and the root table holds the doubles cos / sin return on the host, so the result does not depend on where the
// transform runs: a host loop over the same butterflies gives the same bits.  Stages whose butterflies stay inside a
// tile of 4096 points run in LDS in one launch; the wider ones are one launch each (three for N = 2^16).
#include <cmath>
#include <mutex>
#include <unordered_map>

#include "hemm_internal.hpp"

#pragma clang fp contract(off)

namespace {

struct EmbTables {
    double2 *ksi = nullptr;   // [M + 1]  exp(2 pi i k / M), M = 2N
    u32 *rot = nullptr;       // [N / 2]  5^j mod M
};
std::mutex g_mu;
std::unordered_map<const hemm_context *, EmbTables> g_tabs;

const EmbTables &tables_of(const hemm_context *c) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_tabs.find(c);
    if (it != g_tabs.end()) return it->second;
    const size_t n = (size_t)c->N / 2, M = 2 * (size_t)c->N;
    std::vector<double2> k(M + 1);
    // separate loops: a cos / sin pair on one value may be merged into one sincos call, which rounds differently
    for (size_t i = 0; i <= M; i++) k[i].x = cos(2.0 * M_PI * (double)i / (double)M);
    for (size_t i = 0; i <= M; i++) k[i].y = sin(2.0 * M_PI * (double)i / (double)M);
    std::vector<u32> r(n);
    u64 g = 1;
    for (size_t j = 0; j < n; j++) {
        r[j] = (u32)g;
        g = g * 5 % M;
    }
    EmbTables t;
    HEMM_HIP(hipMalloc((void **)&t.ksi, k.size() * sizeof(double2)));
    HEMM_HIP(hipMalloc((void **)&t.rot, r.size() * sizeof(u32)));
    HEMM_HIP(hipMemcpy(t.ksi, k.data(), k.size() * sizeof(double2), hipMemcpyHostToDevice));
    HEMM_HIP(hipMemcpy(t.rot, r.data(), r.size() * sizeof(u32), hipMemcpyHostToDevice));
    return g_tabs.emplace(c, t).first->second;
}

__device__ __forceinline__ double2 cmul(const double2 v, const double2 k) {
    return make_double2(v.x * k.x - v.y * k.y, v.x * k.y + v.y * k.x);
}
// one butterfly of stage `len`; a and b are its two points
template <bool DECODE>
__device__ __forceinline__ void butterfly(double2 &a, double2 &b, const u32 j, const u32 len, const u32 M,
                                          const double2 *__restrict__ ksi, const u32 *__restrict__ rot) {
    const u32 lenq = len << 2, gap = M / lenq, r = rot[j] & (lenq - 1);
    if (!DECODE) {
        const double2 k = ksi[(size_t)(lenq - r) * gap];
        const double2 u = make_double2(a.x + b.x, a.y + b.y), v = make_double2(a.x - b.x, a.y - b.y);
        a = u;
        b = cmul(v, k);
    } else {
        const double2 k = ksi[(size_t)r * gap];
        const double2 t = cmul(b, k);
        const double2 u = a;
        a = make_double2(u.x + t.x, u.y + t.y);
        b = make_double2(u.x - t.x, u.y - t.y);
    }
}

// one stage over global memory: a thread owns one butterfly of one message
template <bool DECODE>
__global__ __launch_bounds__(256) void emb_stage_kernel(double2 *__restrict__ z, const u32 n, const u32 len, const u32 M,
                                                        const double2 *__restrict__ ksi, const u32 *__restrict__ rot) {
    const u32 t = blockIdx.x * 256 + threadIdx.x;
    if (t >= n / 2) return;
    const u32 lenh = len >> 1, j = t & (lenh - 1), i = (t / lenh) * len;
    double2 *p = z + (size_t)blockIdx.y * n + i + j;
    double2 a = p[0], b = p[lenh];
    butterfly<DECODE>(a, b, j, len, M, ksi, rot);
    p[0] = a;
    p[lenh] = b;
}

// all stages with len <= tile inside one tile of `tile` consecutive points held in LDS
template <bool DECODE>
__global__ __launch_bounds__(1024) void emb_tile_kernel(double2 *__restrict__ z, const u32 n, const u32 tile, const u32 M,
                                                        const double2 *__restrict__ ksi, const u32 *__restrict__ rot) {
    extern __shared__ double2 s[];
    double2 *p = z + (size_t)blockIdx.y * n + (size_t)blockIdx.x * tile;
    for (u32 e = threadIdx.x; e < tile; e += blockDim.x) s[e] = p[e];
    __syncthreads();
    for (u32 step = 1; step < tile; step <<= 1) {
        const u32 len = DECODE ? step << 1 : tile / step, lenh = len >> 1;
        for (u32 t = threadIdx.x; t < tile / 2; t += blockDim.x) {
            const u32 j = t & (lenh - 1), i = (t / lenh) * len;
            butterfly<DECODE>(s[i + j], s[i + j + lenh], j, len, M, ksi, rot);
        }
        __syncthreads();
    }
    for (u32 e = threadIdx.x; e < tile; e += blockDim.x) p[e] = s[e];
}

__device__ __forceinline__ long long round_half_away(double x) { return (long long)__builtin_round(x); }

// transformed slots -> residues of the rounded coefficients, limb by limb (coefficient form, ready for the NTT)
__global__ __launch_bounds__(256) void emb_lift_kernel(const double2 *__restrict__ z, const u32 n, const int log_n,
                                                       const double scale, const ModQ *__restrict__ modq, LimbList ll,
                                                       const int n_limbs, u64 *__restrict__ out) {
    const u32 i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const double2 v = z[(size_t)blockIdx.y * n + (__brev(i) >> (32 - log_n))];
    const double inv_n = 1.0 / (double)n;   // a power of two: the same value a division by n gives
    const long long c0 = round_half_away(v.x * inv_n * scale), c1 = round_half_away(v.y * inv_n * scale);
    u64 *o = out + (size_t)blockIdx.y * n_limbs * 2 * n;
    for (int j = 0; j < n_limbs; j++) {
        const u64 q = modq[ll.idx[j]].q;
        u64 r0 = (u64)(c0 < 0 ? -c0 : c0) % q, r1 = (u64)(c1 < 0 ? -c1 : c1) % q;
        if (c0 < 0 && r0) r0 = q - r0;
        if (c1 < 0 && r1) r1 = q - r1;
        o[(size_t)j * 2 * n + i] = r0;
        o[(size_t)j * 2 * n + n + i] = r1;
    }
}

// coefficient form of the first limb (or the first two) -> centred value / scale, written in bit-reversed order
__global__ __launch_bounds__(256) void emb_centre_kernel(const u64 *__restrict__ co, const u32 n, const int log_n,
                                                         const int two, const u64 q0, const u64 q1, const u64 q0inv,
                                                         const ModQ *__restrict__ modq, const double scale,
                                                         double2 *__restrict__ z) {
    const u32 i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    double v[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const size_t e = (size_t)h * n + i;
        const u64 l0 = co[e];
        if (!two) {
            v[h] = (l0 > q0 / 2 ? -(double)(q0 - l0) : (double)l0) / scale;
            continue;
        }
        const u64 l1 = co[2 * (size_t)n + e];
        const u64 a = l1 % q1, b = l0 % q1;
        const u64 d = a >= b ? a - b : a + q1 - b;
        const u64 k = mulmod(d, q0inv, modq[1]);
        const unsigned __int128 Q = (unsigned __int128)q0 * q1, x = (unsigned __int128)l0 + (unsigned __int128)q0 * k;
        double w;
        if (x > Q / 2) {
            const unsigned __int128 y = Q - x;
            w = -((double)(u64)(y >> 64) * 18446744073709551616.0 + (double)(u64)y);
        } else
            w = (double)(u64)(x >> 64) * 18446744073709551616.0 + (double)(u64)x;
        v[h] = w / scale;
    }
    z[__brev(i) >> (32 - log_n)] = make_double2(v[0], v[1]);
}

template <bool DECODE>
void run_stages(const hemm_context *c, double2 *z, int n_msgs, hipStream_t s) {
    const EmbTables &t = tables_of(c);
    const u32 n = (u32)c->N / 2, M = 2 * (u32)c->N, tile = n < 4096 ? n : 4096;
    const dim3 wide((n / 2 + 255) / 256, n_msgs), tiles(n / tile, n_msgs);
    const int threads = tile / 2 < 1024 ? (int)(tile / 2) : 1024;
    if (!DECODE) {
        for (u32 len = n; len > tile; len >>= 1)
            hipLaunchKernelGGL(emb_stage_kernel<false>, wide, dim3(256), 0, s, z, n, len, M, t.ksi, t.rot);
        hipLaunchKernelGGL(emb_tile_kernel<false>, tiles, dim3(threads), (size_t)tile * sizeof(double2), s, z, n, tile, M, t.ksi,
                           t.rot);
    } else {
        hipLaunchKernelGGL(emb_tile_kernel<true>, tiles, dim3(threads), (size_t)tile * sizeof(double2), s, z, n, tile, M, t.ksi,
                           t.rot);
        for (u32 len = tile << 1; len <= n; len <<= 1)
            hipLaunchKernelGGL(emb_stage_kernel<true>, wide, dim3(256), 0, s, z, n, len, M, t.ksi, t.rot);
    }
}

}  // namespace

void hemm_embedding_tables_free(const hemm_context *c) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_tabs.find(c);
    if (it == g_tabs.end()) return;
    (void)hipFree(it->second.ksi);
    (void)hipFree(it->second.rot);
    g_tabs.erase(it);
}

// slots: [n_msgs][N/2] complex doubles on the device (clobbered); out: [n_msgs][n_limbs][N] NTT form
void launch_encode(const hemm_context *c, double *slots, double scale, const LimbList &ll, int n_limbs, int n_msgs, u64 *out,
                   hipStream_t s) {
    if (c->N < 16) throw std::invalid_argument("encode needs N >= 16");
    const u32 n = (u32)c->N / 2;
    double2 *z = (double2 *)slots;
    run_stages<false>(c, z, n_msgs, s);
    hipLaunchKernelGGL(emb_lift_kernel, dim3((n + 255) / 256, n_msgs), dim3(256), 0, s, z, n, c->logN - 1, scale, c->d_modq, ll,
                       n_limbs, out);
    account(c, TR_POINTWISE, (size_t)n_msgs * (n_limbs + 1) * c->N * 8);
    LimbList sl;
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) sl.idx[j] = (uint8_t)j;
    launch_ntt_slots(c, out, ll, sl, n_limbs, n_msgs, (size_t)n_limbs * c->N, false, s);
}

// pt: [>= n_limbs][N] NTT form, limbs of chain primes 0 (and 1); work: [n_limbs][N]; slots: [N/2] complex doubles
void launch_decode(const hemm_context *c, const u64 *pt, int n_limbs, double scale, u64 *work, double *slots, hipStream_t s) {
    if (c->N < 16) throw std::invalid_argument("decode needs N >= 16");
    if (n_limbs < 1 || n_limbs > 2) throw std::invalid_argument("decode reads one or two limbs");
    const u32 n = (u32)c->N / 2;
    HEMM_HIP(hipMemcpyAsync(work, pt, (size_t)n_limbs * c->N * 8, hipMemcpyDeviceToDevice, s));
    LimbList ll;
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) ll.idx[j] = (uint8_t)j;
    launch_ntt_slots(c, work, ll, ll, n_limbs, 1, (size_t)n_limbs * c->N, true, s);
    const u64 q0 = c->primes[0], q1 = n_limbs == 2 ? c->primes[1] : 1;
    const u64 q0inv = n_limbs == 2 ? h_invmod(q0 % q1, q1) : 0;
    double2 *z = (double2 *)slots;
    hipLaunchKernelGGL(emb_centre_kernel, dim3((n + 255) / 256), dim3(256), 0, s, work, n, c->logN - 1, n_limbs == 2 ? 1 : 0, q0,
                       q1, q0inv, c->d_modq, scale, z);
    account(c, TR_POINTWISE, (size_t)(n_limbs + 1) * c->N * 8);
    run_stages<true>(c, z, 1, s);
}
