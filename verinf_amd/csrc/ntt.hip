// Batched Goldilocks NTT and coset low-degree extension for gfx950.
//
// A transform is one or more passes over digits of its length (ntt_pass.hpp): gather a tile of T columns x L points,
// transform the L-point columns, multiply by the inter-pass twiddles precomputed in HBM and scatter.  Digits of
// 32..256 points run in k_ntt_fast (two register-blocked 16 / 2..16-point transforms with one LDS crossing,
// ntt_fast.hpp), 512 points in k_ntt_512, and the last inverse pass of an LDE together with the first forward pass in
// k_lde_mid (the coefficients never leave the registers); k_ntt_pass, radix-2 levels in LDS, is left with digits
// below 32 points.  Whole rows of 2^10 .. 2^12 points are one launch of k_ntt_row (a 4..16-point digit, then a
// 256-point one, both crossings in LDS).  The host side (ntt_plan.hpp) decides the digit split, owns the cached tables and strings
// passes together into
//   * vi_ntt_batched  -- in-place natural-order transform of (m, n) rows
//     (prover/cuda_primitives.py:388-409);
//   * vi_coset_lde    -- values at w_K^c -> codeword on shift*<w_N>
//     (layergkr/gpu.py:141-203), with the zero-extension fused into the first
//     gather and the rho = N/K cosets written interleaved by the last pass, so the
//     padded (m, N) buffer of the reference recipe is never materialised.
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.hpp"
#include "ntt_plan.hpp"

using namespace ntt;

__global__ __launch_bounds__(NTHREADS) void k_ntt_pass(const PassArgs A) {
    __shared__ u64 lds[LDS_WORDS];
    const int tid = threadIdx.x;
    const i64 tile = blockIdx.x;
    u64 reg[EPT];
    ph_load(A, tile, tid, reg);
    const int n_loop = (!A.is_final && A.loop_cosets) ? (1 << A.log_rho) : 1;
    for (int t = 0; t < n_loop; ++t) {
        ph_stage(A, tile, tid, t, reg, lds);
        __syncthreads();
        for (int s = 0; s < A.a; ++s) {
            ph_level(A, tid, s, lds);
            __syncthreads();
        }
        ph_store(A, tile, tid, t, lds);
        __syncthreads();
    }
}

// Register-blocked pass for digits of 2^5 .. 2^8 points (ntt_fast.hpp): one LDS
// crossing, shift-only butterflies, 16 elements per thread held in registers.
// FIN: compiled for the final (transposing) pass only, without the strided passes' addressing (110 instead of
// 120 registers).  The strided passes keep the run-time flag: compiled with it fixed to 0 they took 128
// registers and spilled.
// UNI: compiled for passes whose tiles are all addressed by scalar bases plus 32-bit thread offsets (pass_uniform).
// HALF: the first pass over source rows at most half as wide as the transform (upper_half_zero): eight of a thread's
// sixteen inputs are zero, so they are not loaded and the first butterfly level of stage 1 is skipped.
// SGL: a single-pass transform over whole tiles of contiguous rows (pass_uniform): stage 2 stores along output rows.
template <int A2, bool INV, bool FIN, bool UNI, bool HALF = false, bool SGL = false>
__global__ __launch_bounds__(NTHREADS, 4) void k_ntt_fast(const PassArgs A_in) {
    PassArgs A = A_in;
    if (FIN) A.is_final = 1;
    static_assert(!SGL || (FIN && UNI && !HALF), "whole-tile single-pass transforms are uniform final passes");
    __shared__ u64 lds[SGL ? SglLds<A2>::WORDS : TILE + (16 << A2)];
    __shared__ u64 twi[16 << A2];
    const int tid = threadIdx.x;
    // A pass that expands one source tile into rho cosets runs rho workgroups per tile, the coset being the low
    // bits of the workgroup id, so that the workgroups that read the same coefficients run at about the same time
    // (3.394 vs 3.420 ms against the coset as grid.y); each of them re-reads the tile.  A loop over the cosets
    // inside one workgroup was slower: every address becomes loop-invariant, ~50 more live registers, spills.
    const bool expand = !A.is_final && A.loop_cosets;
    const i64 n_tiles = expand ? (i64)(gridDim.x >> A.log_rho) : (i64)gridDim.x;
    i64 tile = expand ? (i64)(blockIdx.x >> A.log_rho) : (i64)blockIdx.x;
    int t = expand ? (int)(blockIdx.x & ((1u << A.log_rho) - 1)) : 0;
    if (expand && (n_tiles & 7) == 0) {
        // Workgroup ids are dealt to the 8 XCDs in turn.  Taking the XCD from the low three id bits and (tile, coset)
        // from the rest puts the rho workgroups of a tile on consecutive slots of ONE XCD, so that all but the first
        // find the coefficients in that XCD's L2 (3.46-3.50 vs 3.49-3.53 ms).  A bijection of [0, 8 * n_tiles/8 * rho).
        const u32 xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        t = (int)(slot & ((1u << A.log_rho) - 1));
        tile = (i64)(slot >> A.log_rho) * 8 + xcd;
    }
    // the inner twiddle rows this thread copies into LDS are requested first, the tile after them
    const int lt = TILE_LOG - A.a;
    const int lane = tid & 63, first = ((tid & ~63) >> lt) * 16, count = lt >= 6 ? 16 : (16 << (6 - lt));
    u64 tw_mine[(16 << A2) / NTHREADS > 0 ? (16 << A2) / NTHREADS : 1];
    u64 tw_wave = 0;
    if (!A.is_final) {
        // strided pass: a wavefront uses only the table rows of its own n2 values (at most 64 words), so each
        // wavefront fills just those and no workgroup barrier is needed before stage 1
        if (lane < count) tw_wave = A.twi[first + lane];
    } else {
#pragma unroll
        for (int i = 0; i < (int)(sizeof(tw_mine) / sizeof(u64)); ++i)
            tw_mine[i] = (tid + i * NTHREADS < (16 << A2)) ? A.twi[tid + i * NTHREADS] : 0;
    }
    u64 reg[16], pw[16];
    u32 ok;
    if (A.pre) fast_pre_load<A2, UNI>(A, tile, tid, t, pw);
    // A tile that only this workgroup reads is fetched with the streaming hint, like the stores: in a strided pass
    // (except the one whose rho workgroups per tile share it through the L2), and in the final pass over 256-point
    // digits.  Measured per kind of pass on two boxes: strided passes 0 to -0.2 % on the 2^16 -> 2^18 extension and
    // -2.5 % on transforms of 2^20 points; final passes -0.3 to -1 % on the 2^16 -> 2^18 extension and -0.6 % on
    // transforms of 2^16 points, but +1 % on the 2^14 -> 2^16 extension (128-point digits) and +6 % on transforms of
    // 2^20 points (64-point digits).
    constexpr bool STREAM = UNI && (!FIN || A2 == 4);
    if (STREAM && !expand) fast_load<A2, UNI, HALF, STREAM>(A, tile, tid, reg, ok);
    else fast_load<A2, UNI, HALF>(A, tile, tid, reg, ok);
    if (!A.is_final) {
        if (lane < count) twi[first + lane] = tw_wave;
        __builtin_amdgcn_wave_barrier();
    } else {
#pragma unroll
        for (int i = 0; i < (int)(sizeof(tw_mine) / sizeof(u64)); ++i)
            if (tid + i * NTHREADS < (16 << A2)) twi[twi_slot<A2, FIN>((tid + i * NTHREADS) >> 4, (tid + i * NTHREADS) & 15)] = tw_mine[i];
        __syncthreads();
    }
    fast_stage1<A2, INV, HALF, FIN, SGL>(A, tile, tid, t, ok, reg, pw, twi, lds);
    __syncthreads();
    fast_stage2<A2, INV, UNI, SGL>(A, tile, tid, t, lds);
}


// 512-point rows: one pass, 16 x 32 (fast_stage2_512); eight rows (or row-coset pairs) per workgroup
template <bool INV, bool UNI>
__global__ __launch_bounds__(NTHREADS, 4) void k_ntt_512(const PassArgs A_in) {
    PassArgs A = A_in;
    A.is_final = 1;
    constexpr int A2 = 5;
    __shared__ u64 lds[UNI ? SglLds<A2>::WORDS : TILE + (16 << A2)];
    __shared__ u64 twi[16 << A2];
    const int tid = threadIdx.x;
    const i64 tile = blockIdx.x;
    u64 tw_mine[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) tw_mine[i] = A.twi[tid + i * NTHREADS];
    u64 reg[16], pw[16];
    u32 ok;
    if (A.pre) fast_pre_load<A2, false>(A, tile, tid, 0, pw);      // never in a uniform pass
    fast_load<A2, UNI, false, UNI>(A, tile, tid, reg, ok);             // whole tiles: streaming (rows of 2^9 0.249 -> 0.240 ms)
#pragma unroll
    for (int i = 0; i < 2; ++i) twi[twi_slot<A2, true>((tid + i * NTHREADS) >> 4, (tid + i * NTHREADS) & 15)] = tw_mine[i];
    __syncthreads();
    fast_stage1<A2, INV, false, true, UNI>(A, tile, tid, 0, ok, reg, pw, twi, lds);
    __syncthreads();
    fast_stage2_512<INV, UNI>(A, tile, tid, lds);
}

// Rows of 2^10 .. 2^12 points: the whole transform in one launch (row_stage0), 16 >> A0 rows per workgroup.  The
// tile crosses LDS twice (first digit -> last digit, and inside the last digit) and HBM not at all in between.
// UNI: the last digit's stores through scalar-base addressing (rows of 2^12 points: a tile is one whole row).
template <int A0, bool INV, bool UNI>
__global__ __launch_bounds__(NTHREADS, 4) void k_ntt_row(const PassArgs P0, const PassArgs P1_in) {
    PassArgs P1 = P1_in;
    P1.is_final = 1;
    __shared__ u64 lds[TILE + 256];                        // 16 columns of ROW_ST words, then 256 rows of 17
    __shared__ u64 twi[256];
    static_assert(16 * ROW_ST <= TILE + 256, "the columns of the first digit fit the exchange buffer of the last");
    const int tid = threadIdx.x;
    const i64 tile = blockIdx.x;
    const u64 tw_mine = P1.twi[tid];
    row_stage0<A0, INV>(P0, tile, tid, lds);
    twi[twi_slot<4, true>(tid >> 4, tid & 15)] = tw_mine;
    __syncthreads();
    u64 reg[16];
    row_gather(lds, tid, reg);
    __syncthreads();                                       // every thread has its inputs: the buffer is free again
    fast_stage1<4, INV, false, true>(P1, tile, tid, 0, 0xFFFFu, reg, reg, twi, lds);
    __syncthreads();
    fast_stage2<4, INV, UNI>(P1, tile, tid, 0, lds);
}

// The last inverse pass and the first forward pass of a coset extension in one launch (fused_stage2_inv): the
// coefficients stay in registers between the two, so they are neither written to nor read back from HBM (unless the
// caller wants them), and the rho cosets are expanded by a loop inside the workgroup.
// Four workgroups per CU (128 registers, 39 KB of LDS each): with three the kernel was 8 % slower.
#ifndef VI_MID_MIN_WG
#define VI_MID_MIN_WG 4
#endif
// MRG: the coset factors split into shift^i (once), a power of two per input, and factors carried by the twiddle
// tables of each coset (ntt_plan.hpp, append_coset_merged).
template <int A2, bool MRG>
__global__ __launch_bounds__(NTHREADS, VI_MID_MIN_WG) void k_lde_mid(const PassArgs Ai_in, const PassArgs Af_in) {
    PassArgs Ai = Ai_in, Af = Af_in;
    Ai.is_final = 1;
    Af.is_final = 0;
    __shared__ u64 lds[TILE + (16 << A2)];
    __shared__ u64 twi_i[16 << A2];
    __shared__ u64 twi_f[16 << A2];                        // MRG: the inner twiddles of the coset in hand
    const int tid = threadIdx.x;
    const i64 tile = blockIdx.x;
    constexpr int PER = (16 << A2) / NTHREADS > 0 ? (16 << A2) / NTHREADS : 1;
    const u64 *src_f = MRG ? Af.twim : Af.twi;
    u64 ti[PER], tf[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const bool in = tid + i * NTHREADS < (16 << A2);
        ti[i] = in ? Ai.twi[tid + i * NTHREADS] : 0;
        tf[i] = in ? src_f[tid + i * NTHREADS] : 0;
    }
    u64 reg[16], coef[16];
    u32 ok;
    fast_load<A2, true, false, A2 == 4>(Ai, tile, tid, reg, ok);      // streaming where it measured faster, see k_ntt_fast
#pragma unroll
    for (int i = 0; i < PER; ++i)
        if (tid + i * NTHREADS < (16 << A2)) {
            twi_i[twi_slot<A2, true>((tid + i * NTHREADS) >> 4, (tid + i * NTHREADS) & 15)] = ti[i];
            twi_f[tid + i * NTHREADS] = tf[i];
        }
    __syncthreads();
    fast_stage1<A2, true, false, true>(Ai, tile, tid, 0, ok, reg, reg, twi_i, lds);   // no pre-multipliers on the inverse side
    __syncthreads();
    fused_stage2_inv<A2>(Ai, tile, tid, lds, coef);
    if (MRG) fused_twist<A2>(Af, tile, tid, coef);
    const int rho = 1 << Af.log_rho;
    for (int t = 0; t < rho; ++t) {
        __syncthreads();                                   // every thread is done reading the tile of the step before
        fused_stage1_fwd<A2, MRG>(Af, tile, tid, t, coef, twi_f, lds);
        __syncthreads();
        fused_stage2_fwd<A2, MRG>(Af, tile, tid, t, lds);
        // stage 1 of this coset is over everywhere, so its inner twiddles make way for the next coset's (fetched and
        // stored in one place: held in registers across either stage they cost the kernel its fourth workgroup per CU)
        if (MRG && t + 1 < rho) {
#pragma unroll
            for (int i = 0; i < PER; ++i)
                if (tid + i * NTHREADS < (16 << A2)) twi_f[tid + i * NTHREADS] = src_f[((size_t)(t + 1) << Af.a) + tid + i * NTHREADS];
        }
    }
}

namespace {

struct DeviceTables {
    Tables T;
    std::vector<void *> owned;
};

std::mutex g_mu;
std::map<std::tuple<int, int, int>, DeviceTables *> g_tables;        // (device, logn, inverse + 2 * row split)
std::map<std::pair<int, int>, u64 *> g_twl;                          // (device, inverse)
std::map<std::tuple<int, int, int, u64>, u64 *> g_pre;               // (device, logK, logN, shift)

int upload(const std::vector<u64> &h, u64 **out) {
    void *d = nullptr;
    VI_HIP(hipMalloc(&d, h.size() * sizeof(u64)));
    hipError_t e = hipMemcpy(d, h.data(), h.size() * sizeof(u64), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(d);
        return vi::fail(VI_EHIP, "upload of a twiddle table: %s", hipGetErrorString(e));
    }
    *out = (u64 *)d;
    return VI_OK;
}

int get_twl(int dev, int inv, const u64 **out) {
    auto key = std::make_pair(dev, inv);
    auto it = g_twl.find(key);
    if (it == g_twl.end()) {
        u64 *d = nullptr;
        int rc = upload(make_twl(inv), &d);
        if (rc) return rc;
        it = g_twl.emplace(key, d).first;
    }
    *out = it->second;
    return VI_OK;
}

// tables of one (logn, direction) on the current device; built on first use (which allocates and copies
// synchronously; later calls with the same length only look the tables up)
// row: the tables of the single-launch split of a short row (row_split) instead of split_digits
int get_tables(int logn, int inv, const Tables **out, bool row = false) {
    int dev = 0;
    VI_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_mu);
    auto key = std::make_tuple(dev, logn, inv + (row ? 2 : 0));
    auto it = g_tables.find(key);
    if (it == g_tables.end()) {
        const Split rs = row_split(logn);
        HostTables H = make_tables(logn, inv, row ? &rs : nullptr);
        DeviceTables *D = new DeviceTables();
        D->T.sp = H.sp;
        D->T.logn = logn;
        D->T.scale = H.scale;
        D->T.inverse = inv;
        int rc = VI_OK;
        for (int q = 0; q < 4; ++q) D->T.twi[q] = nullptr;
        for (int q = 0; q < 3; ++q) D->T.tw[q] = nullptr;
        for (int q = 0; q < 4 && !rc; ++q) {
            if (H.twi[q].empty()) continue;
            u64 *d = nullptr;
            rc = upload(H.twi[q], &d);
            if (!rc) { D->T.twi[q] = d; D->owned.push_back(d); }
        }
        for (int q = 0; q < 3 && !rc; ++q) {
            if (H.tw[q].empty()) continue;
            u64 *d = nullptr;
            rc = upload(H.tw[q], &d);
            if (!rc) { D->T.tw[q] = d; D->owned.push_back(d); }
        }
        if (!rc) rc = get_twl(dev, inv, &D->T.twl);
        if (rc) {                                          // give back what was uploaded before the failure
            for (void *p : D->owned) (void)hipFree(p);
            delete D;
            return rc;
        }
        it = g_tables.emplace(key, D).first;
    }
    *out = &it->second->T;
    return VI_OK;
}

// Coset multiplier tables are N words each and depend on the shift: the most recently used MAX_PRE per process are
// kept, the least recently used one is freed when a new one is needed (hipFree waits for the kernels that may still
// read it).
constexpr size_t MAX_PRE = 16;
u64 g_pre_clock = 0;
std::map<std::tuple<int, int, int, u64>, u64> g_pre_used;            // key -> time of last use

int get_pre(int logK, int logN, u64 shift, const u64 **out) {
    int dev = 0;
    VI_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_mu);
    auto key = std::make_tuple(dev, logK, logN, shift);
    auto it = g_pre.find(key);
    if (it == g_pre.end()) {
        if (g_pre.size() >= MAX_PRE) {
            auto oldest = g_pre_used.begin();
            for (auto u = g_pre_used.begin(); u != g_pre_used.end(); ++u)
                if (u->second < oldest->second) oldest = u;
            auto victim = g_pre.find(oldest->first);
            int vdev = std::get<0>(victim->first);
            if (vdev != dev) VI_HIP(hipSetDevice(vdev));
            hipError_t e = hipFree(victim->second);
            if (vdev != dev) VI_HIP(hipSetDevice(dev));
            if (e != hipSuccess) return vi::fail(VI_EHIP, "hipFree of a coset table: %s", hipGetErrorString(e));
            g_pre.erase(victim);
            g_pre_used.erase(oldest);
        }
        u64 *d = nullptr;
        std::vector<u64> h = make_coset_pre(logK, logN, shift);
        if (coset_mergeable(logK, logN)) append_coset_merged(logK, logN, h);
        int rc = upload(h, &d);
        if (rc) return rc;
        it = g_pre.emplace(key, d).first;
    }
    g_pre_used[key] = ++g_pre_clock;
    *out = it->second;
    return VI_OK;
}

template <int A2, bool UNI>
void launch_fast_u(const PassArgs &A, dim3 grid, dim3 block, hipStream_t s) {
    switch ((A.inverse ? 2 : 0) + (A.is_final ? 1 : 0)) {
        case 0: hipLaunchKernelGGL((k_ntt_fast<A2, false, false, UNI>), grid, block, 0, s, A); break;
        case 1: hipLaunchKernelGGL((k_ntt_fast<A2, false, true, UNI>), grid, block, 0, s, A); break;
        case 2: hipLaunchKernelGGL((k_ntt_fast<A2, true, false, UNI>), grid, block, 0, s, A); break;
        default: hipLaunchKernelGGL((k_ntt_fast<A2, true, true, UNI>), grid, block, 0, s, A); break;
    }
}

template <int A2>
void launch_fast_a(const PassArgs &A_in, dim3 grid, dim3 block, hipStream_t s) {
    PassArgs A = A_in;
    A.uniform = pass_uniform(A, &A.n1_valid) ? 1 : 0;
    if (A.uniform && A.inverse && upper_half_zero(A))
        hipLaunchKernelGGL((k_ntt_fast<A2, true, false, true, true>), grid, block, 0, s, A);
    else if (A.uniform && A.is_final && A.ndig == 0) {     // single-pass transform over whole tiles
        if (A.inverse) hipLaunchKernelGGL((k_ntt_fast<A2, true, true, true, false, true>), grid, block, 0, s, A);
        else hipLaunchKernelGGL((k_ntt_fast<A2, false, true, true, false, true>), grid, block, 0, s, A);
    } else if (A.uniform) launch_fast_u<A2, true>(A, grid, block, s);
    else launch_fast_u<A2, false>(A, grid, block, s);
}

void launch_fast(const PassArgs &A, dim3 grid, dim3 block, hipStream_t s) {
    switch (A.a - FAST_A1) {
        case 1: launch_fast_a<1>(A, grid, block, s); break;
        case 2: launch_fast_a<2>(A, grid, block, s); break;
        case 3: launch_fast_a<3>(A, grid, block, s); break;
        default: launch_fast_a<4>(A, grid, block, s); break;
    }
}

int launch_fused(const PassArgs &Ai_in, const PassArgs &Af_in, hipStream_t s) {
    PassArgs Ai = Ai_in, Af = Af_in;
    Ai.uniform = Af.uniform = 1;
    Ai.n1_valid = Af.n1_valid = 16;
    const i64 tiles = pass_tiles(Ai);
    if (tiles > 0x7FFFFFFF) return vi::fail(VI_EINVAL, "ntt pass: %lld tiles exceed the grid limit", (long long)tiles);
    dim3 grid((unsigned)tiles), block(NTHREADS);
    if (Af.twm && Af.twim && Af.merge_unit > 0) {
        switch (Ai.a - FAST_A1) {
            case 1: hipLaunchKernelGGL((k_lde_mid<1, true>), grid, block, 0, s, Ai, Af); break;
            case 2: hipLaunchKernelGGL((k_lde_mid<2, true>), grid, block, 0, s, Ai, Af); break;
            case 3: hipLaunchKernelGGL((k_lde_mid<3, true>), grid, block, 0, s, Ai, Af); break;
            default: hipLaunchKernelGGL((k_lde_mid<4, true>), grid, block, 0, s, Ai, Af); break;
        }
    } else {
        switch (Ai.a - FAST_A1) {
            case 1: hipLaunchKernelGGL((k_lde_mid<1, false>), grid, block, 0, s, Ai, Af); break;
            case 2: hipLaunchKernelGGL((k_lde_mid<2, false>), grid, block, 0, s, Ai, Af); break;
            case 3: hipLaunchKernelGGL((k_lde_mid<3, false>), grid, block, 0, s, Ai, Af); break;
            default: hipLaunchKernelGGL((k_lde_mid<4, false>), grid, block, 0, s, Ai, Af); break;
        }
    }
    VI_LAUNCH_CHECK("k_lde_mid");
    return VI_OK;
}

int launch_passes(const std::vector<PassArgs> &passes, hipStream_t s) {
    for (size_t q = 0; q < passes.size(); ++q) {
        const PassArgs &A = passes[q];
        i64 tiles = pass_tiles(A);
        if (tiles <= 0) continue;
        if (A.fuse_next && q + 1 < passes.size() && passes_fusable(A, passes[q + 1])) {
            int rc = launch_fused(A, passes[q + 1], s);
            if (rc) return rc;
            ++q;
            continue;
        }
        if (tiles > 0x7FFFFFFF) return vi::fail(VI_EINVAL, "ntt pass: %lld tiles exceed the grid limit", (long long)tiles);
        dim3 grid((unsigned)tiles), block(NTHREADS);
        if (fast_ok(A.a) && A.twi) {
            if (!A.is_final && A.loop_cosets) grid.x <<= A.log_rho;       // tiles * rho <= 2^31 by max_rows_per_launch
            launch_fast(A, grid, block, s);
        } else if (fast512_ok(A.a) && A.twi && A.is_final) {
            PassArgs U = A;
            U.is_final = 1;
            U.uniform = pass_uniform(U, &U.n1_valid) ? 1 : 0;
            switch ((U.inverse ? 2 : 0) + U.uniform) {
                case 0: hipLaunchKernelGGL((k_ntt_512<false, false>), grid, block, 0, s, U); break;
                case 1: hipLaunchKernelGGL((k_ntt_512<false, true>), grid, block, 0, s, U); break;
                case 2: hipLaunchKernelGGL((k_ntt_512<true, false>), grid, block, 0, s, U); break;
                default: hipLaunchKernelGGL((k_ntt_512<true, true>), grid, block, 0, s, U); break;
            }
        } else {
            hipLaunchKernelGGL(k_ntt_pass, grid, block, 0, s, A);
        }
        VI_LAUNCH_CHECK("k_ntt_pass");
    }
    return VI_OK;
}

// VI_NTT_ROW=0 (read once per process): rows of 2^10 .. 2^12 points as two launches through a workspace, like longer rows
bool row_launch_on() {
    static const bool on = []() { const char *e = getenv("VI_NTT_ROW"); return !(e && e[0] == '0'); }();
    return on;
}

int launch_row(const PassArgs &P0, const PassArgs &P1, hipStream_t s) {
    const i64 tiles = pass_tiles(P1);
    if (tiles > 0x7FFFFFFF) return vi::fail(VI_EINVAL, "ntt pass: %lld tiles exceed the grid limit", (long long)tiles);
    dim3 grid((unsigned)tiles), block(NTHREADS);
    int nv = 16;
    const bool uni = pass_uniform(P1, &nv) && nv == 16;
    switch (P0.a * 2 + (P0.inverse ? 1 : 0)) {
        case 4: hipLaunchKernelGGL((k_ntt_row<2, false, false>), grid, block, 0, s, P0, P1); break;
        case 5: hipLaunchKernelGGL((k_ntt_row<2, true, false>), grid, block, 0, s, P0, P1); break;
        case 6: hipLaunchKernelGGL((k_ntt_row<3, false, false>), grid, block, 0, s, P0, P1); break;
        case 7: hipLaunchKernelGGL((k_ntt_row<3, true, false>), grid, block, 0, s, P0, P1); break;
        case 8:
            if (uni) hipLaunchKernelGGL((k_ntt_row<4, false, true>), grid, block, 0, s, P0, P1);
            else hipLaunchKernelGGL((k_ntt_row<4, false, false>), grid, block, 0, s, P0, P1);
            break;
        case 9:
            if (uni) hipLaunchKernelGGL((k_ntt_row<4, true, true>), grid, block, 0, s, P0, P1);
            else hipLaunchKernelGGL((k_ntt_row<4, true, false>), grid, block, 0, s, P0, P1);
            break;
        default: return vi::fail(VI_EINVAL, "k_ntt_row: first digit of 2^%d points", P0.a);
    }
    VI_LAUNCH_CHECK("k_ntt_row");
    return VI_OK;
}

// rows per launch so that grids stay below 2^31 tiles
i64 max_rows_per_launch(int logn) { return ((i64)1 << 40) >> logn; }

// rows per chunk of a coset extension: within the grid limit, and small enough that the coset planes of the forward
// intermediate stay inside the 2^29-element window the final pass's scalar-base addressing covers (a larger chunk
// would still be correct, on the per-element path)
i64 max_lde_chunk(int logK, int logN) {
    i64 cap = max_rows_per_launch(logN);
    const i64 K = (i64)1 << logK, rho = (i64)1 << (logN - logK);
    if (rho > 1 && logK <= 26) {
        const i64 fit = (((i64)1 << 29) - K - 1) / ((rho - 1) * K);
        if (fit >= 8 && fit < cap) cap = fit;
    }
    return cap;
}

}  // namespace

extern "C" {

size_t vi_ntt_workspace_bytes(int64_t m, int64_t n) {
    if (m <= 0 || !vi::is_pow2(n) || n < 2) return 0;
    if (row_launch_on() && row_single_ok(vi::ilog2(n))) return 0;
    return split_digits(vi::ilog2(n)).p > 1 ? (size_t)m * (size_t)n * sizeof(u64) : 0;
}

int vi_ntt_batched(uint64_t *rows, int64_t m, int64_t n, int inverse, void *ws, size_t ws_bytes,
                   void *stream) {
    if (m < 0) return vi::fail(VI_EINVAL, "vi_ntt_batched: m = %lld", (long long)m);
    if (!vi::is_pow2(n) || n < 2 || n > ((int64_t)1 << 32))
        return vi::fail(VI_EINVAL, "vi_ntt_batched: row length must be a power of 2 in [2, 2^32], got %lld", (long long)n);
    if (m == 0) return VI_OK;
    if (!rows) return vi::fail(VI_EINVAL, "vi_ntt_batched: null rows");
    const int logn = vi::ilog2(n);
    const Tables *T = nullptr;
    if (row_launch_on() && row_single_ok(logn)) {
        int rc = get_tables(logn, inverse ? 1 : 0, &T, true);
        if (rc) return rc;
        const i64 cap = max_rows_per_launch(logn);
        for (i64 lo = 0; lo < m; lo += cap) {
            PassArgs P0, P1;
            build_row_passes(*T, rows + lo * n, (m - lo < cap) ? (m - lo) : cap, P0, P1);
            rc = launch_row(P0, P1, (hipStream_t)stream);
            if (rc) return rc;
        }
        return VI_OK;
    }
    int rc = get_tables(logn, inverse ? 1 : 0, &T);
    if (rc) return rc;
    i64 chunk = m;
    if (T->sp.p > 1) {
        i64 fit = (i64)(ws_bytes / ((size_t)n * sizeof(u64)));
        if (!ws || fit < 1)
            return vi::fail(VI_ENOMEM, "vi_ntt_batched: n = %lld needs a workspace of at least %zu bytes (one row)",
                            (long long)n, (size_t)n * sizeof(u64));
        if (fit < chunk) chunk = fit;
    }
    if (chunk > max_rows_per_launch(logn)) chunk = max_rows_per_launch(logn);
    for (i64 lo = 0; lo < m; lo += chunk) {
        i64 cnt = (m - lo < chunk) ? (m - lo) : chunk;
        std::vector<PassArgs> passes;
        build_ntt_passes(*T, rows + lo * n, (u64 *)ws, cnt, passes);
        rc = launch_passes(passes, (hipStream_t)stream);
        if (rc) return rc;
    }
    return VI_OK;
}

size_t vi_coset_lde_min_workspace_bytes(int64_t K, int64_t N) {
    if (!vi::is_pow2(K) || !vi::is_pow2(N) || K < 2 || N < K) return 0;
    return (size_t)lde_ws_elems(vi::ilog2(K), vi::ilog2(N), 1) * sizeof(u64);
}

size_t vi_coset_lde_workspace_bytes(int64_t m, int64_t K, int64_t N) {
    size_t one = vi_coset_lde_min_workspace_bytes(K, N);
    if (!one || m <= 0) return 0;
    // A launch should hold many workgroups per CU (no partially filled last round) and the chunk count should be
    // low: measured on 1024 x 2^16 -> 2^18, 80 / 160 / 320 / 640 / 1280 / 2560 MiB of scratch give
    // 4.87 / 4.09 / 3.85 / 3.64 / 3.57 / 3.63 ms.  1.25 GiB is small change next to 288 GB of HBM.
    const size_t target = (size_t)1280 << 20;
    size_t rows = target / one;
    if (rows < 8) rows = 8;
    if ((int64_t)rows > m) rows = (size_t)m;
    return rows * one;
}

int64_t vi_coset_lde_launches(int64_t m, int64_t K, int64_t N, size_t ws_bytes) {
    size_t one = vi_coset_lde_min_workspace_bytes(K, N);
    if (!one || m <= 0 || ws_bytes < one) return 0;
    i64 chunk = (i64)(ws_bytes / one);
    if (chunk > m) chunk = m;
    if (chunk > max_lde_chunk(vi::ilog2(K), vi::ilog2(N))) chunk = max_lde_chunk(vi::ilog2(K), vi::ilog2(N));
    const i64 n_chunks = (m + chunk - 1) / chunk;         // balancing keeps the chunk count
    chunk = (m + n_chunks - 1) / n_chunks;
    // the pass list of one chunk, planned with placeholder addresses (only their being null or not matters)
    const int logK = vi::ilog2(K), logN = vi::ilog2(N);
    Tables Ti{}, Tf{};
    Ti.sp = Tf.sp = split_digits(logK);
    Ti.logn = Tf.logn = logK;
    Ti.inverse = 1;
    Ti.scale = Tf.scale = 1;
    u64 *dummy = (u64 *)(uintptr_t)4096;
    std::vector<PassArgs> passes;
    build_lde_passes(Ti, Tf, dummy, logN, dummy, K, K, dummy, N, dummy, chunk, passes);
    i64 per_chunk = 0;
    for (size_t q = 0; q < passes.size(); ++q) {
        if (passes[q].fuse_next && q + 1 < passes.size() && passes_fusable(passes[q], passes[q + 1])) ++q;
        ++per_chunk;
    }
    return n_chunks * per_chunk;
}

namespace {

// m rows of `cols` zeros (row pitch `stride`)
__global__ __launch_bounds__(NTHREADS) void k_zero_rows(u64 *dst, i64 m, i64 cols, i64 stride) {
    const i64 total = m * cols;
    for (i64 e = (i64)blockIdx.x * NTHREADS + threadIdx.x; e < total; e += (i64)gridDim.x * NTHREADS)
        dst[(e / cols) * stride + (e % cols)] = 0;
}

int zero_rows(u64 *dst, i64 m, i64 cols, i64 stride, hipStream_t s) {
    i64 blocks = (m * cols + NTHREADS - 1) / NTHREADS;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(k_zero_rows, dim3((unsigned)blocks), dim3(NTHREADS), 0, s, dst, m, cols, stride);
    VI_LAUNCH_CHECK("k_zero_rows");
    return VI_OK;
}

// values (or coefficients) -> optional coefficients -> optional codewords, chunked over rows
int coset_lde_impl(const char *who, const uint64_t *in, int64_t m, int64_t width, int64_t in_stride, int64_t K,
                   int64_t N, uint64_t shift, uint64_t *out, int64_t out_stride, uint64_t *coeffs,
                   int64_t coeffs_stride, bool in_is_coeffs, void *ws, size_t ws_bytes, void *stream) {
    if (!vi::is_pow2(K) || !vi::is_pow2(N) || K < 2 || N < K || N > ((int64_t)1 << 32))
        return vi::fail(VI_EINVAL, "%s: need powers of two with 2 <= K <= N <= 2^32, got K=%lld N=%lld", who,
                        (long long)K, (long long)N);
    if (m < 0 || width < 0 || width > K || in_stride < width || (out && out_stride < N) || (coeffs && coeffs_stride < K))
        return vi::fail(VI_EINVAL, "%s: bad shape m=%lld width=%lld in_stride=%lld out_stride=%lld coeffs_stride=%lld", who,
                        (long long)m, (long long)width, (long long)in_stride, (long long)out_stride, (long long)coeffs_stride);
    if (shift == 0 || shift >= gl::P) return vi::fail(VI_EINVAL, "%s: shift must be in [1, p)", who);
    if (m == 0) return VI_OK;
    if ((!in && width > 0) || (!out && !coeffs)) return vi::fail(VI_EINVAL, "%s: null pointer", who);
    if (width == 0) {
        // the empty message is the zero polynomial; the kernels are not run on it (they read word 0 of the
        // source in place of every element that does not exist, and here there is no word 0)
        int rc = VI_OK;
        if (coeffs && !in_is_coeffs) rc = zero_rows(coeffs, m, K, coeffs_stride, (hipStream_t)stream);
        if (!rc && out) rc = zero_rows(out, m, N, out_stride, (hipStream_t)stream);
        return rc;
    }
    const int logK = vi::ilog2(K), logN = vi::ilog2(N);
    size_t one = (size_t)lde_ws_elems(logK, logN, 1) * sizeof(u64);
    i64 chunk = (i64)(ws_bytes / one);
    if (!ws || chunk < 1)
        return vi::fail(VI_ENOMEM, "%s: workspace of %zu bytes is below the one-row minimum %zu", who, ws_bytes, one);
    if (chunk > m) chunk = m;
    if (chunk > max_lde_chunk(logK, logN)) chunk = max_lde_chunk(logK, logN);
    chunk = (m + ((m + chunk - 1) / chunk) - 1) / ((m + chunk - 1) / chunk);   // same chunk count, even sizes
    const Tables *Ti = nullptr, *Tf = nullptr;
    const u64 *pre = nullptr;
    int rc = get_tables(logK, 1, &Ti);
    if (!rc) rc = get_tables(logK, 0, &Tf);
    if (!rc) rc = get_pre(logK, logN, shift, &pre);
    if (rc) return rc;
    // the split form of the coset factors: its tables lie behind the N words of pre
    static const bool use_merged = []() { const char *e = getenv("VI_LDE_MERGED"); return !e || e[0] != '0'; }();
    const u64 *merged = (use_merged && coset_mergeable(logK, logN)) ? pre + N : nullptr;
    for (i64 lo = 0; lo < m; lo += chunk) {
        i64 cnt = (m - lo < chunk) ? (m - lo) : chunk;
        std::vector<PassArgs> passes;
        build_lde_passes(*Ti, *Tf, pre, logN, in + lo * in_stride, width, in_stride, out ? out + lo * out_stride : nullptr,
                         out_stride, (u64 *)ws, cnt, passes, coeffs ? coeffs + lo * coeffs_stride : nullptr, coeffs_stride,
                         in_is_coeffs, true, merged);
        rc = launch_passes(passes, (hipStream_t)stream);
        if (rc) return rc;
    }
    return VI_OK;
}

}  // namespace

int vi_coset_lde(const uint64_t *in, int64_t m, int64_t width, int64_t in_stride, int64_t K,
                 int64_t N, uint64_t shift, uint64_t *out, int64_t out_stride, void *ws,
                 size_t ws_bytes, void *stream) {
    if (m > 0 && !out) return vi::fail(VI_EINVAL, "vi_coset_lde: null pointer");
    return coset_lde_impl("vi_coset_lde", in, m, width, in_stride, K, N, shift, out, out_stride, nullptr, 0, false, ws,
                          ws_bytes, stream);
}

int vi_coset_lde_coeffs(const uint64_t *in, int64_t m, int64_t width, int64_t in_stride, int64_t K, int64_t N,
                        uint64_t shift, uint64_t *coeffs, int64_t coeffs_stride, uint64_t *out, int64_t out_stride,
                        void *ws, size_t ws_bytes, void *stream) {
    if (m > 0 && !coeffs) return vi::fail(VI_EINVAL, "vi_coset_lde_coeffs: null coeffs");
    if (coeffs == in && coeffs_stride != in_stride)
        return vi::fail(VI_EINVAL, "vi_coset_lde_coeffs: in-place use needs equal strides");
    return coset_lde_impl("vi_coset_lde_coeffs", in, m, width, in_stride, K, N, shift, out, out_stride, coeffs,
                          coeffs_stride, false, ws, ws_bytes, stream);
}

int vi_coset_extend(const uint64_t *coeffs, int64_t m, int64_t width, int64_t coeffs_stride, int64_t K, int64_t N,
                    uint64_t shift, uint64_t *out, int64_t out_stride, void *ws, size_t ws_bytes, void *stream) {
    if (m > 0 && !out) return vi::fail(VI_EINVAL, "vi_coset_extend: null pointer");
    return coset_lde_impl("vi_coset_extend", coeffs, m, width, coeffs_stride, K, N, shift, out, out_stride, nullptr, 0,
                          true, ws, ws_bytes, stream);
}

}  // extern "C"
