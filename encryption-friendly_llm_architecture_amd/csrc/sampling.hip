// Counter-based samplers on the device.  Every value is a pure function of (stream key, coefficient index):
//   sm64(x)          = splitmix64 finaliser of x + 0x9E3779B97F4A7C15
//   draw(key, i)     = sm64(key + i * 0x9E3779B97F4A7C15)
//   uniform mod q    : attempt t = 0, 1, ... draws draw(sm64(key + t), i) masked to the bit length of q and is
//                      accepted when below q (masked rejection: exactly uniform)
//   error            : centred binomial, popcount of bits 0..20 minus popcount of bits 21..41 of draw(key, i)
// so host code, the CPU oracle and these kernels produce identical keys and encryptions from a seed.
#include "hemm_internal.hpp"

namespace {

__device__ __forceinline__ u64 sm64(u64 x) {
    u64 z = x + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__device__ __forceinline__ u64 draw(u64 key, u64 ctr) { return sm64(key + ctr * 0x9E3779B97F4A7C15ull); }

struct KeyList {
    u64 key[HEMM_MAX_PRIMES];
};

// out[limb][i] uniform in [0, q_limb)
__global__ __launch_bounds__(256) void sample_uniform_kernel(KeyList keys, LimbList ll, const ModQ *__restrict__ modq,
                                                             u64 *__restrict__ out, int logN) {
    const int limb = blockIdx.y;
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    const ModQ m = modq[ll.idx[limb]];
    const u64 mask = m.k >= 64 ? ~0ull : ((1ull << m.k) - 1);
    const u64 key = keys.key[limb];
    u64 x;
    // acceptance is at least 1/2 per attempt; 4096 attempts cannot all fail in practice and bound the loop
    for (u64 t = 0; t < 4096; t++) {
        x = draw(sm64(key + t), i) & mask;
        if (x < m.q) break;
    }
    out[((size_t)limb << logN) + i] = x;
}

// out[limb][i] = e_i mod q_limb for the centred-binomial error e of stream `key`
__global__ __launch_bounds__(256) void sample_error_kernel(u64 key, LimbList ll, const ModQ *__restrict__ modq,
                                                           u64 *__restrict__ out, int logN) {
    const int limb = blockIdx.y;
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    const u64 q = modq[ll.idx[limb]].q;
    const u64 x = draw(key, i);
    const u64 M21 = (1ull << 21) - 1;
    const int e = __popcll(x & M21) - __popcll((x >> 21) & M21);
    out[((size_t)limb << logN) + i] = e >= 0 ? (u64)e : q - (u64)(-e);
}

}  // namespace

void launch_sample_uniform(const hemm_context *c, const u64 *stream_keys, const LimbList &ll, int n_limbs, u64 *out,
                           hipStream_t s) {
    KeyList kl;
    for (int j = 0; j < n_limbs; j++) kl.key[j] = stream_keys[j];
    dim3 grid(c->N / 256, n_limbs), block(256);
    hipLaunchKernelGGL(sample_uniform_kernel, grid, block, 0, s, kl, ll, c->d_modq, out, c->logN);
}

void launch_sample_error(const hemm_context *c, u64 stream_key, const LimbList &ll, int n_limbs, u64 *out, hipStream_t s) {
    dim3 grid(c->N / 256, n_limbs), block(256);
    hipLaunchKernelGGL(sample_error_kernel, grid, block, 0, s, stream_key, ll, c->d_modq, out, c->logN);
}
