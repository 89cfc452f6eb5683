// volumerhs: volume right-hand side of a nodal discontinuous-Galerkin Euler solver on hexahedra,
// polynomial order N = 4 (Nq = 5, 125 nodes per element), Float32.
// Replaces the kernel of perf/volumerhs.jl:42-176 launched at :200-201.
//
// Reference mapping: one workgroup of (5,5) work-items per element = 25 of 64 lanes, k walked inside
// the thread, 10 barriers per element.  Here: one lane per node (125 of 128 lanes), two elements per
// 256-thread workgroup.  Every field of an element is a slab of 125 consecutive floats, so each load
// instruction of a wave touches one or two contiguous runs (coalesced).  The 15 metric-weighted
// fluxes of a node go to LDS once, one barrier, then each lane contracts the three 5-point lines
// through its node with the columns of D it needs (held in registers).  All LDS reads are
// conflict-free or broadcasts (strides 1, 5, 25 against 32 banks).
//
// Arithmetic: Float32 throughout like the reference; 1/rho uses v_rcp_f32, which the reference's
// `@fastmath inv` (perf/volumerhs.jl:89-90) also permits; mul+add pairs may contract into FMAs.
#include <cstdlib>

#include "rk_common.hpp"

namespace rk {

constexpr int VR_NQ = 5;
constexpr int VR_NP = VR_NQ * VR_NQ * VR_NQ;   // 125 nodes
constexpr int VR_NSTATE = 5;
constexpr int VR_NVGEO = 14;
constexpr int VR_LANES = 128;                  // lanes reserved per element
constexpr int VR_EPB = 2;                      // elements per workgroup

// state and metric numbering of perf/volumerhs.jl:22-33 (0-based here)
enum { S_RHO = 0, S_U, S_V, S_W, S_E };
enum { G_XIX = 0, G_ETAX, G_ZETAX, G_XIY, G_ETAY, G_ZETAY, G_XIZ, G_ETAZ, G_ZETAZ, G_MJ, G_MJI, G_X, G_Y, G_Z };

__global__ __launch_bounds__(VR_LANES * VR_EPB) void volumerhs_kernel(float* __restrict__ rhs, const float* __restrict__ Q,
                                                                      const float* __restrict__ vgeo, float gravity,
                                                                      const float* __restrict__ D, int64_t nelem) {
    __shared__ float sD[VR_NQ * VR_NQ];
    __shared__ float sF[VR_EPB][VR_NSTATE][VR_NP];
    __shared__ float sG[VR_EPB][VR_NSTATE][VR_NP];
    __shared__ float sH[VR_EPB][VR_NSTATE][VR_NP];

    const int t = threadIdx.x;
    const int el = t / VR_LANES, node = t % VR_LANES;
    const int64_t e = (int64_t)blockIdx.x * VR_EPB + el;
    const bool live = node < VR_NP && e < nelem;
    const int i = node % VR_NQ, j = (node / VR_NQ) % VR_NQ, k = node / (VR_NQ * VR_NQ);

    if (t < VR_NQ * VR_NQ) sD[t] = D[t];

    // rhs and MJI are not needed before the contraction, but loading them here puts their latency under the first
    // round of loads instead of behind the barrier (4000 elements, one round of workgroups: two round trips, not three)
    float MJ = 0.f, MJI = 0.f, rho = 0.f, old[VR_NSTATE] = {0.f, 0.f, 0.f, 0.f, 0.f};
    float* out = rhs + e * (VR_NSTATE * VR_NP) + node;
    if (live) {
        const float* q = Q + e * (VR_NSTATE * VR_NP) + node;
        const float* vg = vgeo + e * (VR_NVGEO * VR_NP) + node;
#pragma unroll
        for (int s = 0; s < VR_NSTATE; ++s) old[s] = out[s * VR_NP];
        MJI = vg[G_MJI * VR_NP];
        rho = q[S_RHO * VR_NP];
        const float U = q[S_U * VR_NP], V = q[S_V * VR_NP], W = q[S_W * VR_NP], E = q[S_E * VR_NP];
        MJ = vg[G_MJ * VR_NP];
        const float xix = vg[G_XIX * VR_NP], xiy = vg[G_XIY * VR_NP], xiz = vg[G_XIZ * VR_NP];
        const float etx = vg[G_ETAX * VR_NP], ety = vg[G_ETAY * VR_NP], etz = vg[G_ETAZ * VR_NP];
        const float zex = vg[G_ZETAX * VR_NP], zey = vg[G_ZETAY * VR_NP], zez = vg[G_ZETAZ * VR_NP];
        const float z = vg[G_Z * VR_NP];

        const float rinv = __builtin_amdgcn_rcpf(rho);
        const float r2inv = 0.5f * rinv;
        const float P = 0.4f * (E - (U * U + V * V + W * W) * r2inv - rho * gravity * z);   // :92

        const float fx[VR_NSTATE] = {U, rinv * U * U + P, rinv * U * V, rinv * U * W, rinv * U * (E + P)};   // :94-98
        const float fy[VR_NSTATE] = {V, rinv * V * U, rinv * V * V + P, rinv * V * W, rinv * V * (E + P)};   // :100-104
        const float fz[VR_NSTATE] = {W, rinv * W * U, rinv * W * V, rinv * W * W + P, rinv * W * (E + P)};   // :106-110
#pragma unroll
        for (int s = 0; s < VR_NSTATE; ++s) {
            sF[el][s][node] = MJ * (xix * fx[s] + xiy * fy[s] + xiz * fz[s]);   // :112-116
            sG[el][s][node] = MJ * (etx * fx[s] + ety * fy[s] + etz * fz[s]);   // :118-122
            sH[el][s][node] = MJ * (zex * fx[s] + zey * fy[s] + zez * fz[s]);   // :124-128
        }
    }
    __syncthreads();
    if (!live) return;

    float Di[VR_NQ], Dj[VR_NQ], Dk[VR_NQ];   // D[n, i], D[n, j], D[n, k]  (column-major: n + 5 * col)
#pragma unroll
    for (int n = 0; n < VR_NQ; ++n) {
        Di[n] = sD[n + VR_NQ * i];
        Dj[n] = sD[n + VR_NQ * j];
        Dk[n] = sD[n + VR_NQ * k];
    }
    const int rowF = VR_NQ * j + VR_NQ * VR_NQ * k;   // + n
    const int rowG = i + VR_NQ * VR_NQ * k;           // + 5 n
    const int rowH = i + VR_NQ * j;                   // + 25 n
#pragma unroll
    for (int s = 0; s < VR_NSTATE; ++s) {
        float r = 0.f;
#pragma unroll
        for (int n = 0; n < VR_NQ; ++n) {
            r += Di[n] * sF[el][s][rowF + n];                      // :148-...
            r += Dj[n] * sG[el][s][rowG + VR_NQ * n];
            r += Dk[n] * sH[el][s][rowH + VR_NQ * VR_NQ * n];      // :131-138
        }
        if (s == S_W) r -= MJ * rho * gravity;                     // :140
        out[s * VR_NP] = old[s] + MJI * r;                         // :166-173
    }
}


// ---- four elements per workgroup, every global access a 16-byte vector ------------------------------------------------
// The kernel above issues 17 four-byte loads and 5 read-modify-writes per lane, and the 500-byte field slabs start at
// 4-byte alignment, so its requests straddle cache lines: 15.35 KB of HBM traffic per element against 13.5 KB of
// algorithmic bytes.  A block of FOUR elements is contiguous and 16-byte aligned in all three arrays (2500 * 4 and
// 7000 * 4 bytes), so here a workgroup of 512 lanes
//   1. copies the block's Q (625 vectors) and vgeo (1750 vectors, minus the ~62 per element that lie wholly inside the
//      unused x and y fields) into LDS with 16-byte non-temporal loads and prefetches the block's rhs (625 vectors, one
//      or two a lane) into registers,
//   2. one lane per node reads its 5 states and 11 metric terms from LDS (consecutive lanes, consecutive words) and
//      forms the 15 metric-weighted fluxes,
//   3. the fluxes replace the staged inputs in LDS, each lane contracts the three 5-point lines through its node with
//      the columns of D (as above) and leaves MJI * r in LDS in the layout of rhs,
//   4. the block of results is added to the prefetched rhs and stored with 16-byte vectors.
// 40 KB of LDS per workgroup: four workgroups (2048 lanes) share a compute unit.
constexpr int VR_EPB4 = 4;
constexpr int VR_QBLK = VR_EPB4 * VR_NSTATE * VR_NP;      // 2500 floats
constexpr int VR_GBLK = VR_EPB4 * VR_NVGEO * VR_NP;       // 7000 floats
constexpr int VR_FLUX = VR_EPB4 * VR_NSTATE * VR_NP;      // per flux direction
static_assert(VR_QBLK % 4 == 0 && VR_GBLK % 4 == 0, "a block of four elements is whole vectors");

__global__ __launch_bounds__(VR_LANES * VR_EPB4) void volumerhs_vec_kernel(float* __restrict__ rhs, const float* __restrict__ Q,
                                                                           const float* __restrict__ vgeo, float gravity,
                                                                           const float* __restrict__ D) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    constexpr int NT = VR_LANES * VR_EPB4;
    __shared__ float sD[VR_NQ * VR_NQ];
    // [0, 7000) vgeo block, [7000, 9500) Q block; later [0, 7500) fluxes F, G, H and [7500, 10000) the results
    __shared__ __attribute__((aligned(16))) float lds[3 * VR_FLUX + VR_QBLK];
    static_assert(VR_GBLK + VR_QBLK <= 3 * VR_FLUX + VR_QBLK, "the staged inputs fit");
    float* sG0 = lds;                 // staged vgeo
    float* sQ0 = lds + VR_GBLK;       // staged Q
    float* sF = lds;
    float* sG = lds + VR_FLUX;
    float* sH = lds + 2 * VR_FLUX;
    float* sR = lds + 3 * VR_FLUX;

    const int t = threadIdx.x;
    const int el = t / VR_LANES, node = t % VR_LANES;
    const int64_t blk = blockIdx.x;
    const f4* gq = (const f4*)(Q + blk * VR_QBLK);
    const f4* gv = (const f4*)(vgeo + blk * VR_GBLK);
    f4* gr = (f4*)(rhs + blk * VR_QBLK);
    constexpr int NQV = VR_QBLK / 4, NGV = VR_GBLK / 4;     // 625, 1750 vectors

    // 1. stage
    const bool second = t + NT < NQV;
    const f4 r0 = load_nt(gr + t);
    f4 r1 = {0.f, 0.f, 0.f, 0.f};
    if (second) r1 = load_nt(gr + t + NT);
    {
        const f4 q0 = load_nt(gq + t);
        f4 q1 = {0.f, 0.f, 0.f, 0.f};
        if (second) q1 = load_nt(gq + t + NT);
        f4 g[(NGV + NT - 1) / NT];
#pragma unroll
        for (int u = 0; u < (NGV + NT - 1) / NT; ++u) {
            const int v = t + u * NT;
            // floats [4v, 4v + 4) of the block; unused: fields x and y of each element, floats 1375 .. 1624 of its 1750
            const int f0 = 4 * v, w = f0 % (VR_NVGEO * VR_NP);
            const bool used = v < NGV && !(w >= G_X * VR_NP && w + 4 <= G_Z * VR_NP);
            g[u] = f4{0.f, 0.f, 0.f, 0.f};
            if (used) g[u] = load_nt(gv + v);
        }
        ((f4*)sQ0)[t] = q0;
        if (second) ((f4*)sQ0)[t + NT] = q1;
#pragma unroll
        for (int u = 0; u < (NGV + NT - 1) / NT; ++u) {
            const int v = t + u * NT;
            if (v < NGV) ((f4*)sG0)[v] = g[u];
        }
    }
    if (t < VR_NQ * VR_NQ) sD[t] = D[t];
    __syncthreads();

    // 2. fluxes of this lane's node
    const bool live = node < VR_NP;
    const int i = node % VR_NQ, j = (node / VR_NQ) % VR_NQ, k = node / (VR_NQ * VR_NQ);
    float MJ = 0.f, MJI = 0.f, rho = 1.f;
    float F[VR_NSTATE], G[VR_NSTATE], H[VR_NSTATE];
#pragma unroll
    for (int s = 0; s < VR_NSTATE; ++s) F[s] = G[s] = H[s] = 0.f;
    if (live) {
        const float* q = sQ0 + el * (VR_NSTATE * VR_NP) + node;
        const float* vg = sG0 + el * (VR_NVGEO * VR_NP) + node;
        rho = q[S_RHO * VR_NP];
        const float U = q[S_U * VR_NP], V = q[S_V * VR_NP], W = q[S_W * VR_NP], E = q[S_E * VR_NP];
        MJ = vg[G_MJ * VR_NP];
        MJI = vg[G_MJI * VR_NP];
        const float xix = vg[G_XIX * VR_NP], xiy = vg[G_XIY * VR_NP], xiz = vg[G_XIZ * VR_NP];
        const float etx = vg[G_ETAX * VR_NP], ety = vg[G_ETAY * VR_NP], etz = vg[G_ETAZ * VR_NP];
        const float zex = vg[G_ZETAX * VR_NP], zey = vg[G_ZETAY * VR_NP], zez = vg[G_ZETAZ * VR_NP];
        const float z = vg[G_Z * VR_NP];

        const float rinv = __builtin_amdgcn_rcpf(rho);
        const float r2inv = 0.5f * rinv;
        const float P = 0.4f * (E - (U * U + V * V + W * W) * r2inv - rho * gravity * z);   // :92

        const float fx[VR_NSTATE] = {U, rinv * U * U + P, rinv * U * V, rinv * U * W, rinv * U * (E + P)};   // :94-98
        const float fy[VR_NSTATE] = {V, rinv * V * U, rinv * V * V + P, rinv * V * W, rinv * V * (E + P)};   // :100-104
        const float fz[VR_NSTATE] = {W, rinv * W * U, rinv * W * V, rinv * W * W + P, rinv * W * (E + P)};   // :106-110
#pragma unroll
        for (int s = 0; s < VR_NSTATE; ++s) {
            F[s] = MJ * (xix * fx[s] + xiy * fy[s] + xiz * fz[s]);   // :112-116
            G[s] = MJ * (etx * fx[s] + ety * fy[s] + etz * fz[s]);   // :118-122
            H[s] = MJ * (zex * fx[s] + zey * fy[s] + zez * fz[s]);   // :124-128
        }
    }
    __syncthreads();          // every lane has read its staged inputs: the fluxes may take their place
    if (live) {
#pragma unroll
        for (int s = 0; s < VR_NSTATE; ++s) {
            const int o = (el * VR_NSTATE + s) * VR_NP + node;
            sF[o] = F[s];
            sG[o] = G[s];
            sH[o] = H[s];
        }
    }
    __syncthreads();

    // 3. contraction with D; MJI * r goes to LDS in the layout of rhs
    if (live) {
        float Di[VR_NQ], Dj[VR_NQ], Dk[VR_NQ];   // D[n, i], D[n, j], D[n, k]  (column-major: n + 5 * col)
#pragma unroll
        for (int n = 0; n < VR_NQ; ++n) {
            Di[n] = sD[n + VR_NQ * i];
            Dj[n] = sD[n + VR_NQ * j];
            Dk[n] = sD[n + VR_NQ * k];
        }
        const int rowF = VR_NQ * j + VR_NQ * VR_NQ * k;   // + n
        const int rowG = i + VR_NQ * VR_NQ * k;           // + 5 n
        const int rowH = i + VR_NQ * j;                   // + 25 n
#pragma unroll
        for (int s = 0; s < VR_NSTATE; ++s) {
            const int o = (el * VR_NSTATE + s) * VR_NP;
            float r = 0.f;
#pragma unroll
            for (int n = 0; n < VR_NQ; ++n) {
                r += Di[n] * sF[o + rowF + n];                         // :148-...
                r += Dj[n] * sG[o + rowG + VR_NQ * n];
                r += Dk[n] * sH[o + rowH + VR_NQ * VR_NQ * n];         // :131-138
            }
            if (s == S_W) r -= MJ * rho * gravity;                     // :140
            sR[o + node] = MJI * r;                                    // :166-173
        }
    }
    __syncthreads();

    // 4. rhs += results, 16 bytes a store
    store_nt(gr + t, r0 + ((const f4*)sR)[t]);
    if (second) store_nt(gr + t + NT, r1 + ((const f4*)sR)[t + NT]);
}

__global__ __launch_bounds__(256) void findall_scatter_kernel(const uint8_t* __restrict__ bools, const int64_t* __restrict__ indices,
                                                              int64_t* __restrict__ ys, int ndim, int64_t n,
                                                              int64_t s0, int64_t s1, int64_t s2, int64_t s3, int64_t s4, int64_t s5,
                                                              int64_t s6, int64_t s7) {
    const int64_t shape[RK_MAX_DIMS] = {s0, s1, s2, s3, s4, s5, s6, s7};
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n || !bools[i]) return;
    const int64_t b = indices[i] - 1;    // new position
    if (ndim <= 1) { ys[b] = i + 1; return; }
    int64_t rem = i;
    for (int d = 0; d < ndim; ++d) {
        ys[b * ndim + d] = rem % shape[d] + 1;
        rem /= shape[d];
    }
}

}  // namespace rk

using namespace rk;

// Fewest elements for which the four-element kernel is used (RK_VOLUMERHS_VEC_MIN).
static int64_t vec_min_elements() {
    static const int64_t v = [] {
        const char* e = std::getenv("RK_VOLUMERHS_VEC_MIN");
        const long long x = e ? std::atoll(e) : 0;
        return (int64_t)(x >= VR_EPB4 ? x : 32768);
    }();
    return v;
}

extern "C" int32_t rk_volumerhs_f32(float* rhs, const float* Q, const float* vgeo, float gravity, const float* D,
                                    int64_t nelem, void* stream) {
    if (nelem < 0) return RK_ERR_INVALID_ARGUMENT;
    if (nelem == 0) return RK_SUCCESS;
    if (rhs == nullptr || Q == nullptr || vgeo == nullptr || D == nullptr) return RK_ERR_INVALID_ARGUMENT;
    // whole blocks of four elements with 16-byte accesses when the arrays are aligned for them; the up to three elements
    // that remain (or everything, for unaligned arrays) with the lane-per-node kernel and its 4-byte accesses
    // Few elements (the 4000 of the small benchmark case: every workgroup of either kernel is resident at once) are bound by the latency
    // of one workgroup, and the lane-per-node kernel with its single barrier is the shorter one: 10.7 against 14.5 us.
    int64_t done = 0;
    if (is_aligned(rhs, 16) && is_aligned(Q, 16) && is_aligned(vgeo, 16) && nelem >= vec_min_elements()) {
        const int64_t nblk = nelem / VR_EPB4;
        if (nblk > 0x7fffffff) return RK_ERR_TOO_LARGE;
        volumerhs_vec_kernel<<<(unsigned)nblk, VR_LANES * VR_EPB4, 0, (hipStream_t)stream>>>(rhs, Q, vgeo, gravity, D);
        RK_LAUNCH_CHECK();
        done = nblk * VR_EPB4;
    }
    const int64_t rest = nelem - done;
    if (rest > 0) {
        const int64_t blocks = (rest + VR_EPB - 1) / VR_EPB;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        volumerhs_kernel<<<(unsigned)blocks, VR_LANES * VR_EPB, 0, (hipStream_t)stream>>>(
            rhs + done * (VR_NSTATE * VR_NP), Q + done * (VR_NSTATE * VR_NP), vgeo + done * (VR_NVGEO * VR_NP), gravity, D, rest);
        RK_LAUNCH_CHECK();
    }
    return RK_SUCCESS;
}

extern "C" int32_t rk_findall_scatter(const uint8_t* bools, const int64_t* indices, int64_t* ys, int ndim, const int64_t* shape,
                                      void* stream) {
    if (ndim < 0 || ndim > RK_MAX_DIMS || (ndim > 0 && shape == nullptr)) return RK_ERR_INVALID_ARGUMENT;
    int64_t n = 1, s[RK_MAX_DIMS];
    for (int d = 0; d < RK_MAX_DIMS; ++d) {
        s[d] = d < ndim ? shape[d] : 1;
        if (s[d] < 0) return RK_ERR_INVALID_ARGUMENT;
        n *= s[d];
    }
    if (n == 0) return RK_SUCCESS;
    if (bools == nullptr || indices == nullptr || ys == nullptr) return RK_ERR_INVALID_ARGUMENT;
    const int64_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
    findall_scatter_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(bools, indices, ys, ndim, n, s[0], s[1], s[2], s[3], s[4],
                                                                             s[5], s[6], s[7]);
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}
