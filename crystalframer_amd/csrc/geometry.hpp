// Per-batch geometry shared by every layer of a forward pass, in three launches: the pair list of the
// fully connected crystals (i-major, the complete n x n block of each crystal), the pair vectors, the
// reciprocal lattice and the work order of the atoms (longest rows first).  The reference builds the
// same tensors with framework index arithmetic and a Python loop over crystals
// (models/indexed_latticeformer_encoder.py:15-44,175-245).
#pragma once
#include "device_common.hpp"

namespace cfh {

struct GeometryArgs {
    const float* pos;          // (N, 3)
    const int64_t* batch;      // (N) crystal of each atom, ascending
    const float* tvecs;        // (B, 3, 3) lattice rows
    const int64_t* sizes;      // (B) atoms per crystal
    int64_t* edges;            // (2, E)
    float* rpos;               // (E, 3) pos[j] - pos[i]
    float* recip;              // (B, 3, 3) 2 pi (t_b x t_c) / V, ...
    float* rvlen;              // (B, 3)
    float* vcell;              // (B)
    int64_t* e_start;          // (N + 1)
    int32_t* order;            // (N) atoms by descending crystal size
    int64_t* atom_start;       // (B + 1) scratch / output: first atom of each crystal
    int64_t* pair_start;       // (B + 1) scratch: first pair of each crystal
    int64_t* order_start;      // (B) scratch: first position of each crystal's atoms in `order`
    int32_t N, B;
    int64_t E;
};

constexpr int GEO_THREADS = 1024;
constexpr int GEO_KEYS = 2048;      // crystals of GEO_KEYS - 1 atoms or more share the first place of the order

// Two workgroups.  The second computes the reciprocal lattice; the first the prefix sums over the
// crystals and where each crystal's atoms go in the work order (descending size; equal sizes in crystal
// order when B <= its size, in the order their atomics happen to arrive otherwise).
#pragma clang fp contract(off)      // the framework expressions this replaces round every product and sum
__global__ __launch_bounds__(GEO_THREADS) void geometry_crystals_kernel(const GeometryArgs P) {
    __shared__ long long scan_a[GEO_THREADS], scan_p[GEO_THREADS];
    __shared__ long long carry_a, carry_p;
    __shared__ int hist[GEO_KEYS];
    const int t = threadIdx.x;
    const int T = blockDim.x;              // GEO_THREADS
    if (blockIdx.x == 1) {
        // reciprocal lattice (same operation order as the framework expressions it replaces)
        for (int b = t; b < P.B; b += T) {
            const float* m = P.tvecs + (size_t)b * 9;
            const float v = m[0] * m[4] * m[8] + m[1] * m[5] * m[6] + m[2] * m[3] * m[7] - m[2] * m[4] * m[6]
                            - m[0] * m[5] * m[7] - m[1] * m[3] * m[8];
            const float s = (float)(2.0 * 3.14159265358979323846) / v;
            P.vcell[b] = v;
            for (int r = 0; r < 3; r++) {
                const float* u = m + 3 * ((r + 1) % 3);
                const float* w = m + 3 * ((r + 2) % 3);
                const float cx = u[1] * w[2] - u[2] * w[1], cy = u[2] * w[0] - u[0] * w[2], cz = u[0] * w[1] - u[1] * w[0];
                const float rx = cx * s, ry = cy * s, rz = cz * s;
                P.recip[(size_t)b * 9 + 3 * r + 0] = rx;
                P.recip[(size_t)b * 9 + 3 * r + 1] = ry;
                P.recip[(size_t)b * 9 + 3 * r + 2] = rz;
                P.rvlen[(size_t)b * 3 + r] = sqrtf(rx * rx + ry * ry + rz * rz);
            }
        }
        return;
    }
    const long long n_first = t < P.B ? (long long)P.sizes[t] : 0;      // the first T sizes: used twice below
    if (t == 0) { carry_a = 0; carry_p = 0; }
    __syncthreads();
    // exclusive prefix sums of n and n^2, T crystals at a time: a shuffle scan inside every wavefront, then
    // the totals of the wavefronts before this one
    const int wv = t >> 6, ln = t & 63, nwv = T >> 6;
    for (int b0 = 0; b0 < P.B; b0 += T) {
        const int b = b0 + t;
        const long long n = b0 == 0 ? n_first : (b < P.B ? (long long)P.sizes[b] : 0);
        long long va = n, vp = n * n;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const long long ta = __shfl_up(va, off, 64), tp = __shfl_up(vp, off, 64);
            if (ln >= off) { va += ta; vp += tp; }
        }
        if (ln == 63) { scan_a[wv] = va; scan_p[wv] = vp; }
        __syncthreads();
        long long base_a = carry_a, base_p = carry_p;
        for (int w = 0; w < wv; w++) { base_a += scan_a[w]; base_p += scan_p[w]; }
        if (b < P.B) {
            P.atom_start[b] = base_a + va - n;
            P.pair_start[b] = base_p + vp - n * n;
        }
        __syncthreads();
        if (t == T - 1) { carry_a = base_a + va; carry_p = base_p + vp; }
        __syncthreads();
    }
    (void)nwv;
    if (t == 0) { P.atom_start[P.B] = carry_a; P.pair_start[P.B] = carry_p; }

    // work order
    if (P.B <= T) {
        // rank by (size descending, crystal ascending): atoms of the crystals ranked before this one; the
        // candidates of a crystal are shared by T / (power of two >= B) threads
        int* const sz = reinterpret_cast<int*>(scan_p);
        int* const before = sz + GEO_THREADS;
        __syncthreads();
        sz[t] = (int)n_first;
        before[t] = 0;
        __syncthreads();
        int bp = 64;
        while (bp < P.B) bp <<= 1;
        const int parts = T / bp, part = t / bp, bb = t - part * bp;
        if (bb < P.B && part < parts) {
            const int n = sz[bb];
            const int span = (P.B + parts - 1) / parts;
            const int c0 = part * span, c1 = min(P.B, c0 + span);
            int acc0 = 0, acc1 = 0;
            int c = c0;
            for (; c + 1 < c1; c += 2) {
                const int m0 = sz[c], m1 = sz[c + 1];
                acc0 += (m0 > n || (m0 == n && c < bb)) ? m0 : 0;
                acc1 += (m1 > n || (m1 == n && c + 1 < bb)) ? m1 : 0;
            }
            if (c < c1) { const int m = sz[c]; acc0 += (m > n || (m == n && c < bb)) ? m : 0; }
            atomicAdd(&before[bb], acc0 + acc1);
        }
        __syncthreads();
        if (t < P.B) P.order_start[t] = (long long)before[t];
    } else {
        for (int k = t; k < GEO_KEYS; k += T) hist[k] = 0;
        __syncthreads();
        for (int b = t; b < P.B; b += T) {
            const int n = (int)P.sizes[b];
            atomicAdd(&hist[min(n, GEO_KEYS - 1)], n);
        }
        __syncthreads();
        // hist[k] <- atoms of the crystals with a larger key: exclusive sums from the top key downwards, two
        // keys per thread, a shuffle scan inside every wavefront and the totals of the wavefronts before it
        static_assert(GEO_KEYS == 2 * GEO_THREADS, "two keys per thread");
        {
            int* const wave_total = reinterpret_cast<int*>(scan_a);
            const int k0 = GEO_KEYS - 1 - 2 * t;
            const int h0 = hist[k0], h1 = hist[k0 - 1];
            int incl = h0 + h1;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int up = __shfl_up(incl, off, 64);
                if (ln >= off) incl += up;
            }
            if (ln == 63) wave_total[wv] = incl;
            __syncthreads();
            int base = 0;
            for (int w = 0; w < wv; w++) base += wave_total[w];
            const int excl = base + incl - (h0 + h1);
            hist[k0] = excl;
            hist[k0 - 1] = excl + h0;
        }
        __syncthreads();
        for (int b = t; b < P.B; b += T) {
            const int n = (int)P.sizes[b];
            P.order_start[b] = atomicAdd(&hist[min(n, GEO_KEYS - 1)], n);
        }
    }
}

// One thread per atom: first pair of its row and its place in the work order.
__global__ __launch_bounds__(256) void geometry_atoms_kernel(const GeometryArgs P) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) P.e_start[P.N] = P.pair_start[P.B];
    if (i >= P.N) return;
    const int b = (int)P.batch[i];
    const long long n = (long long)P.sizes[b];
    const long long local = (long long)i - P.atom_start[b];
    P.e_start[i] = P.pair_start[b] + local * n;
    P.order[P.order_start[b] + local] = i;
}

// One thread per pair: its crystal by bisection of the pairs' prefix sums, then (i, j) and the pair vector.
__global__ __launch_bounds__(256) void geometry_pairs_kernel(const GeometryArgs P) {
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= P.E || e >= P.pair_start[P.B]) return;      // never beyond the pairs that exist
    int lo = 0, hi = P.B;                       // pair_start[lo] <= e < pair_start[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (P.pair_start[mid] <= e) lo = mid; else hi = mid;
    }
    const long long n = (long long)P.sizes[lo];
    if (n <= 0) return;
    const long long local = e - P.pair_start[lo];
    const long long il = local / n, jl = local - il * n;
    const long long a0 = P.atom_start[lo];
    const long long i = a0 + il, j = a0 + jl;
    P.edges[e] = i;
    P.edges[P.E + e] = j;
    P.rpos[e * 3 + 0] = P.pos[j * 3 + 0] - P.pos[i * 3 + 0];
    P.rpos[e * 3 + 1] = P.pos[j * 3 + 1] - P.pos[i * 3 + 1];
    P.rpos[e * 3 + 2] = P.pos[j * 3 + 2] - P.pos[i * 3 + 2];
}

}  // namespace cfh
