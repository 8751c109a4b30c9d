// CPU build of the NTT / LDE pass logic (verinf_amd/csrc/ntt_pass.hpp, ntt_plan.hpp).
// Runs every workgroup phase as a plain loop over thread ids, so the index maps,
// twiddle tables and pass sequencing of the HIP kernels can be checked against the
// oracle without a GPU.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../verinf_amd/csrc/ntt_plan.hpp"

using namespace ntt;

namespace {

struct Owned {
    HostTables H;
    std::vector<u64> twl;
    Tables T;
};

Owned *make_owned(int logn, int inv, bool row = false) {
    Owned *o = new Owned();
    const Split rs = row_split(logn);
    o->H = make_tables(logn, inv, row ? &rs : nullptr);
    o->twl = make_twl(inv);
    o->T.sp = o->H.sp;
    o->T.logn = logn;
    for (int q = 0; q < 3; ++q) o->T.tw[q] = o->H.tw[q].empty() ? nullptr : o->H.tw[q].data();
    for (int q = 0; q < 4; ++q) o->T.twi[q] = o->H.twi[q].empty() ? nullptr : o->H.twi[q].data();
    o->T.inverse = inv;
    o->T.twl = o->twl.data();
    o->T.scale = o->H.scale;
    return o;
}

int g_use_fast = 1;

template <int A2, bool INV, bool UNI, bool HALF = false, bool SGL = false>
void run_fast_u(const PassArgs &A) {
    i64 tiles = pass_tiles(A);
    std::vector<u64> lds(SGL ? SglLds<A2>::WORDS : fast_lds_words(A.a));
    std::vector<u64> regs((size_t)NTHREADS * 16);
    std::vector<u32> oks(NTHREADS);
    int n_loop = (!A.is_final && A.loop_cosets) ? (1 << A.log_rho) : 1;
    for (i64 tile = 0; tile < tiles; ++tile) {
        for (int tid = 0; tid < NTHREADS; ++tid)
            fast_load<A2, UNI, HALF>(A, tile, tid, *reinterpret_cast<u64(*)[16]>(&regs[(size_t)tid * 16]), oks[tid]);
        for (int t = 0; t < n_loop; ++t) {
            for (int tid = 0; tid < NTHREADS; ++tid)
            {
                u64 pw[16] = {};
                if (A.pre) fast_pre_load<A2, UNI>(A, tile, tid, t, pw);
                fast_stage1<A2, INV, HALF, false, SGL>(A, tile, tid, t, oks[tid], *reinterpret_cast<const u64(*)[16]>(&regs[(size_t)tid * 16]),
                                                       pw, A.twi, lds.data());
            }
            for (int tid = 0; tid < NTHREADS; ++tid) fast_stage2<A2, INV, UNI, SGL>(A, tile, tid, t, lds.data());
        }
    }
}

int g_allow_uniform = 1;
long g_single_uniform_runs = 0;             // single-pass transforms that ran with scalar-base addressing
int g_allow_merged = 1;
int g_allow_half = 1;
long g_half_runs = 0;                       // first passes that skipped the zero half of their inputs
long g_merged_runs = 0;                     // fused launches that took the split form of the coset factors

// the same choice the HIP launcher makes: scalar-base addressing when the pass qualifies
template <int A2, bool INV>
void run_fast(const PassArgs &A_in) {
    PassArgs A = A_in;
    A.uniform = (g_allow_uniform && pass_uniform(A, &A.n1_valid)) ? 1 : 0;
    if (A.uniform && A.is_final && A.ndig == 0) {          // the launcher's choice of the whole-tile form
        ++g_single_uniform_runs;
        run_fast_u<A2, INV, true, false, true>(A);
        return;
    }
    if (INV && A.uniform && g_allow_half && upper_half_zero(A)) { ++g_half_runs; run_fast_u<A2, INV, true, true>(A); }
    else if (A.uniform) run_fast_u<A2, INV, true>(A);
    else run_fast_u<A2, INV, false>(A);
}

// the fused launch of the last inverse and the first forward pass, phase by phase like the kernel
template <int A2>
void run_fused(const PassArgs &Ai_in, const PassArgs &Af_in) {
    PassArgs Ai = Ai_in, Af = Af_in;
    Ai.uniform = Af.uniform = 1;
    Ai.n1_valid = Af.n1_valid = 16;
    const i64 tiles = pass_tiles(Ai);
    std::vector<u64> lds(fast_lds_words(Ai.a));
    std::vector<u64> regs((size_t)NTHREADS * 16), coef((size_t)NTHREADS * 16);
    std::vector<u32> oks(NTHREADS);
    auto R = [&](std::vector<u64> &v, int tid) -> u64(&)[16] { return *reinterpret_cast<u64(*)[16]>(&v[(size_t)tid * 16]); };
    for (i64 tile = 0; tile < tiles; ++tile) {
        u64 pw[16] = {};
        for (int tid = 0; tid < NTHREADS; ++tid) fast_load<A2, true>(Ai, tile, tid, R(regs, tid), oks[tid]);
        for (int tid = 0; tid < NTHREADS; ++tid)
            fast_stage1<A2, true>(Ai, tile, tid, 0, oks[tid], R(regs, tid), pw, Ai.twi, lds.data());
        for (int tid = 0; tid < NTHREADS; ++tid) fused_stage2_inv<A2>(Ai, tile, tid, lds.data(), R(coef, tid));
        const bool mrg = Af.twm && Af.twim && Af.merge_unit > 0;       // the launcher's choice of k_lde_mid<A2, MRG>
        if (mrg && tile == 0) ++g_merged_runs;
        if (mrg)
            for (int tid = 0; tid < NTHREADS; ++tid) fused_twist<A2>(Af, tile, tid, R(coef, tid));
        for (int t = 0; t < (1 << Af.log_rho); ++t) {
            for (int tid = 0; tid < NTHREADS; ++tid) {
                if (mrg) fused_stage1_fwd<A2, true>(Af, tile, tid, t, R(coef, tid), Af.twim + ((size_t)t << Af.a), lds.data());
                else fused_stage1_fwd<A2, false>(Af, tile, tid, t, R(coef, tid), Af.twi, lds.data());
            }
            for (int tid = 0; tid < NTHREADS; ++tid) {
                if (mrg) fused_stage2_fwd<A2, true>(Af, tile, tid, t, lds.data());
                else fused_stage2_fwd<A2, false>(Af, tile, tid, t, lds.data());
            }
        }
    }
}

int g_allow_fusion = 1;
int g_allow_row = 1;
long g_row_runs = 0;                        // transforms of short rows that ran as the single launch

// the single launch for rows of 2^10 .. 2^12 points, phase by phase like k_ntt_row
template <int A0, bool INV, bool UNI = false>
void run_row(const PassArgs &P0, const PassArgs &P1_in) {
    PassArgs P1 = P1_in;
    P1.is_final = 1;
    const i64 tiles = pass_tiles(P1);
    std::vector<u64> lds(TILE + 256), twi(256);
    std::vector<u64> regs((size_t)NTHREADS * 16);
    auto R = [&](int tid) -> u64(&)[16] { return *reinterpret_cast<u64(*)[16]>(&regs[(size_t)tid * 16]); };
    for (int tid = 0; tid < NTHREADS; ++tid) twi[twi_slot<4, true>(tid >> 4, tid & 15)] = P1.twi[tid];
    ++g_row_runs;
    for (i64 tile = 0; tile < tiles; ++tile) {
        for (int tid = 0; tid < NTHREADS; ++tid) row_stage0<A0, INV>(P0, tile, tid, lds.data());
        for (int tid = 0; tid < NTHREADS; ++tid) row_gather(lds.data(), tid, R(tid));
        for (int tid = 0; tid < NTHREADS; ++tid)
            fast_stage1<4, INV, false, true>(P1, tile, tid, 0, 0xFFFFu, R(tid), R(tid), twi.data(), lds.data());
        for (int tid = 0; tid < NTHREADS; ++tid) fast_stage2<4, INV, UNI>(P1, tile, tid, 0, lds.data());
    }
}

// runs passes[q] (and passes[q + 1] with it when the two fuse); returns how many passes it consumed
int run_passes_at(const std::vector<PassArgs> &passes, size_t q);

template <bool INV, bool UNI>
void run_512_u(const PassArgs &A) {
    i64 tiles = pass_tiles(A);
    std::vector<u64> lds(UNI ? SglLds<5>::WORDS : fast_lds_words(A.a));
    std::vector<u64> regs((size_t)NTHREADS * 16);
    std::vector<u32> oks(NTHREADS);
    for (i64 tile = 0; tile < tiles; ++tile) {
        for (int tid = 0; tid < NTHREADS; ++tid)
            fast_load<5, UNI>(A, tile, tid, *reinterpret_cast<u64(*)[16]>(&regs[(size_t)tid * 16]), oks[tid]);
        for (int tid = 0; tid < NTHREADS; ++tid) {
            u64 pw[16] = {};
            if (A.pre) fast_pre_load<5, false>(A, tile, tid, 0, pw);
            fast_stage1<5, INV, false, false, UNI>(A, tile, tid, 0, oks[tid], *reinterpret_cast<const u64(*)[16]>(&regs[(size_t)tid * 16]), pw,
                                                   A.twi, lds.data());
        }
        for (int tid = 0; tid < NTHREADS; ++tid) fast_stage2_512<INV, UNI>(A, tile, tid, lds.data());
    }
}

// the launcher's choice: contiguous whole tiles through scalar-base addressing
template <bool INV>
void run_512(const PassArgs &A_in) {
    PassArgs A = A_in;
    A.is_final = 1;
    A.uniform = (g_allow_uniform && pass_uniform(A, &A.n1_valid)) ? 1 : 0;
    if (A.uniform) ++g_single_uniform_runs;
    if (A.uniform) run_512_u<INV, true>(A);
    else run_512_u<INV, false>(A);
}

void run_pass(const PassArgs &A) {
    if (g_use_fast && fast512_ok(A.a) && A.is_final && A.twi) {
        if (A.inverse) run_512<true>(A);
        else run_512<false>(A);
        return;
    }
    if (g_use_fast && fast_ok(A.a)) {
        switch ((A.a - FAST_A1) * 2 + (A.inverse ? 1 : 0)) {
            case 2: run_fast<1, false>(A); return;
            case 3: run_fast<1, true>(A); return;
            case 4: run_fast<2, false>(A); return;
            case 5: run_fast<2, true>(A); return;
            case 6: run_fast<3, false>(A); return;
            case 7: run_fast<3, true>(A); return;
            case 8: run_fast<4, false>(A); return;
            case 9: run_fast<4, true>(A); return;
        }
    }
    i64 tiles = pass_tiles(A);
    std::vector<u64> lds(LDS_WORDS);
    std::vector<u64> regs((size_t)NTHREADS * EPT);
    int n_loop = (!A.is_final && A.loop_cosets) ? (1 << A.log_rho) : 1;
    for (i64 tile = 0; tile < tiles; ++tile) {
        for (int tid = 0; tid < NTHREADS; ++tid)
            ph_load(A, tile, tid, *reinterpret_cast<u64(*)[EPT]>(&regs[(size_t)tid * EPT]));
        for (int t = 0; t < n_loop; ++t) {
            for (int tid = 0; tid < NTHREADS; ++tid)
                ph_stage(A, tile, tid, t, *reinterpret_cast<const u64(*)[EPT]>(&regs[(size_t)tid * EPT]), lds.data());
            for (int s = 0; s < A.a; ++s)
                for (int tid = 0; tid < NTHREADS; ++tid) ph_level(A, tid, s, lds.data());
            for (int tid = 0; tid < NTHREADS; ++tid) ph_store(A, tile, tid, t, lds.data());
        }
    }
}

int run_passes_at(const std::vector<PassArgs> &passes, size_t q) {
    const PassArgs &A = passes[q];
    if (g_use_fast && g_allow_uniform && g_allow_fusion && A.fuse_next && q + 1 < passes.size() &&
        passes_fusable(A, passes[q + 1])) {
        switch (A.a - FAST_A1) {
            case 1: run_fused<1>(A, passes[q + 1]); break;
            case 2: run_fused<2>(A, passes[q + 1]); break;
            case 3: run_fused<3>(A, passes[q + 1]); break;
            default: run_fused<4>(A, passes[q + 1]); break;
        }
        return 2;
    }
    run_pass(A);
    return 1;
}

void run_all(const std::vector<PassArgs> &passes) {
    for (size_t q = 0; q < passes.size();) q += run_passes_at(passes, q);
}

}  // namespace

extern "C" {

void emu_set_fast(int on) { g_use_fast = on; }
void emu_set_uniform(int on) { g_allow_uniform = on; }
void emu_set_fusion(int on) { g_allow_fusion = on; }
void emu_set_merged(int on) { g_allow_merged = on; }
long emu_merged_runs() { return g_merged_runs; }
void emu_set_half(int on) { g_allow_half = on; }
long emu_half_runs() { return g_half_runs; }
u64 emu_mul(u64 a, u64 b) { return gl::mul(a, b); }
u64 emu_add(u64 a, u64 b) { return gl::add(a, b); }
u64 emu_sub(u64 a, u64 b) { return gl::sub(a, b); }
u64 emu_mul_pow2(u64 x, unsigned s) { return gl::mul_pow2(x, s); }
u64 emu_inv(u64 x) { return gl::inv(x); }

long emu_single_uniform_runs() { return g_single_uniform_runs; }
void emu_set_row(int on) { g_allow_row = on; }
long emu_row_runs() { return g_row_runs; }

int emu_ntt_batched(u64 *buf, long m, int logn, int inverse) {
    if (g_use_fast && g_allow_row && row_single_ok(logn)) {
        Owned *o = make_owned(logn, inverse, true);
        PassArgs P0, P1;
        build_row_passes(o->T, buf, m, P0, P1);
        int nv = 16;
        const bool uni = g_allow_uniform && pass_uniform(P1, &nv) && nv == 16;
        switch (P0.a * 2 + (inverse ? 1 : 0)) {
            case 4: run_row<2, false>(P0, P1); break;
            case 5: run_row<2, true>(P0, P1); break;
            case 6: run_row<3, false>(P0, P1); break;
            case 7: run_row<3, true>(P0, P1); break;
            case 8:                                        // the launcher's choice: scalar-base stores when the last digit qualifies
                if (uni) run_row<4, false, true>(P0, P1);
                else run_row<4, false>(P0, P1);
                break;
            default:
                if (uni) run_row<4, true, true>(P0, P1);
                else run_row<4, true>(P0, P1);
                break;
        }
        delete o;
        return 1;
    }
    Owned *o = make_owned(logn, inverse);
    std::vector<u64> ws(o->T.sp.p > 1 ? (size_t)m << logn : 1);
    std::vector<PassArgs> passes;
    build_ntt_passes(o->T, buf, ws.data(), m, passes);
    run_all(passes);
    delete o;
    return (int)passes.size();
}

int emu_coset_lde(const u64 *in, long m, long w, long in_stride, int logK, int logN, u64 shift,
                  u64 *out) {
    Owned *oi = make_owned(logK, 1), *of = make_owned(logK, 0);
    std::vector<u64> pre = make_coset_pre(logK, logN, shift);
    const bool mergeable = g_allow_merged && coset_mergeable(logK, logN);
    if (mergeable) append_coset_merged(logK, logN, pre);
    const u64 *merged = mergeable ? pre.data() + ((size_t)1 << logN) : nullptr;
    std::vector<u64> ws((size_t)lde_ws_elems(logK, logN, m));
    std::vector<PassArgs> passes;
    build_lde_passes(oi->T, of->T, pre.data(), logN, in, w, in_stride, out, (i64)1 << logN, ws.data(), m,
                     passes, nullptr, 0, false, g_use_fast && g_allow_uniform && g_allow_fusion,
                     merged);
    run_all(passes);
    delete oi;
    delete of;
    return (int)passes.size();
}
// mode 0: values -> coeffs (+ out if not null); mode 1: coefficients -> out
int emu_coset_lde_ex(const u64 *in, long m, long w, long in_stride, int logK, int logN, u64 shift,
                     u64 *coeffs, long coeffs_stride, u64 *out, int in_is_coeffs) {
    Owned *oi = make_owned(logK, 1), *of = make_owned(logK, 0);
    std::vector<u64> pre = make_coset_pre(logK, logN, shift);
    const bool mergeable = g_allow_merged && coset_mergeable(logK, logN);
    if (mergeable) append_coset_merged(logK, logN, pre);
    const u64 *merged = mergeable ? pre.data() + ((size_t)1 << logN) : nullptr;
    std::vector<u64> ws((size_t)lde_ws_elems(logK, logN, m));
    std::vector<PassArgs> passes;
    build_lde_passes(oi->T, of->T, pre.data(), logN, in, w, in_stride, out, (i64)1 << logN, ws.data(), m,
                     passes, coeffs, coeffs_stride, in_is_coeffs != 0, g_use_fast && g_allow_uniform && g_allow_fusion,
                     merged);
    run_all(passes);
    delete oi;
    delete of;
    return (int)passes.size();
}
}
