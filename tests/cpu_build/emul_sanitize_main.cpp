// Driver for the sanitizer build of the CPU emulation: runs the NTT and LDE pass logic over a list of shapes with
// heap buffers of exactly the sizes the entry points document, so that AddressSanitizer / UBSan see any access
// outside them (a wrong index map would otherwise only show as a GPU fault).  Results are checked by properties
// that need no second implementation: inverse(forward(x)) = x, and chunk-independence of the LDE.
#include "emul_ntt.cpp"

#include <cstring>

static u64 rnd_state = 88172645463325252ull;
static u64 rnd() {
    rnd_state ^= rnd_state << 13; rnd_state ^= rnd_state >> 7; rnd_state ^= rnd_state << 17;
    return rnd_state % gl::P;
}

// a heap block of exactly `words` words (one byte when there are none, which no index map may touch as a word)
static u64 *exact(size_t words) { return (u64 *)malloc(words ? words * 8 : 1); }

static int check_ntt(int logn, long m) {
    size_t n = (size_t)m << logn;
    u64 *a = exact(n), *b = exact(n);
    for (size_t i = 0; i < n; ++i) a[i] = b[i] = rnd();
    emu_ntt_batched(a, m, logn, 0);
    emu_ntt_batched(a, m, logn, 1);
    int bad = memcmp(a, b, n * 8) != 0;
    if (bad) printf("ntt round trip differs: logn=%d m=%ld\n", logn, m);
    free(a); free(b);
    return bad;
}

// width < K, strided input rows, every row count around the tile and chunk boundaries
static int check_lde(int logK, int logN, long m, long w, long in_stride) {
    size_t K = (size_t)1 << logK, N = (size_t)1 << logN;
    size_t in_words = m ? (size_t)(m - 1) * in_stride + w : 0;
    u64 *in = exact(in_words), *out = exact((size_t)m * N);
    u64 *co = exact((size_t)m * K), *out2 = exact((size_t)m * N);
    for (size_t i = 0; i < in_words; ++i) in[i] = rnd();
    int bad = 0;
    if (w > 0) {
        emu_coset_lde(in, m, w, in_stride, logK, logN, 7, out);
        // values -> coefficients, then coefficients -> codewords: the same codewords
        emu_coset_lde_ex(in, m, w, in_stride, logK, logN, 7, co, (long)K, nullptr, 0);
        emu_coset_lde_ex(co, m, (long)K, (long)K, logK, logN, 7, nullptr, 0, out2, 1);
        bad = memcmp(out, out2, (size_t)m * N * 8) != 0;
        if (bad) printf("lde two-step differs: logK=%d logN=%d m=%ld w=%ld\n", logK, logN, m, w);
    }
    free(in); free(out); free(co); free(out2);
    return bad;
}

int main() {
    int bad = 0;
    const int sizes[][2] = {{1, 3}, {2, 5}, {4, 300}, {5, 129}, {6, 65}, {7, 33}, {8, 17}, {9, 9}, {10, 5}, {11, 3},
                            {12, 3}, {13, 2}, {14, 3}, {15, 1}, {16, 2}, {17, 1}, {18, 1}};
    for (auto &s : sizes) bad += check_ntt(s[0], s[1]);
    for (int fast = 0; fast < 2; ++fast) {
        emu_set_fast(fast);
        bad += check_ntt(8, 17);
        bad += check_ntt(10, 5);
    }
    emu_set_fast(1);
    // rows of 2^10 .. 2^12 points: the single launch (tiles of 4, 2 and 1 rows, the last one partly empty) and the two passes
    for (int row = 0; row < 2; ++row) {
        emu_set_row(row);
        bad += check_ntt(10, 7);
        bad += check_ntt(10, 1);
        bad += check_ntt(11, 1);
        bad += check_ntt(11, 4);
        bad += check_ntt(12, 1);
    }
    emu_set_row(1);
    // single-pass transforms over whole tiles (scalar-base addressing) and over a batch that ends inside a tile
    const int whole[][2] = {{5, 128}, {6, 64}, {7, 64}, {8, 16}, {8, 32}, {9, 8}, {9, 16}, {8, 15}, {9, 7}};
    for (auto &s : whole) bad += check_ntt(s[0], s[1]);
    const long lde[][5] = {
        // logK logN m width in_stride
        {4, 6, 3, 16, 16},   {4, 6, 3, 9, 11},    {5, 7, 130, 32, 32}, {6, 8, 65, 33, 64},   {8, 10, 17, 256, 300},
        {8, 10, 16, 1, 1},   {9, 11, 9, 300, 512}, {10, 12, 5, 1024, 1024}, {10, 12, 4, 513, 600}, {10, 10, 3, 1000, 1024},
        {12, 14, 3, 4096, 4096}, {12, 14, 2, 2048, 4096}, {12, 15, 1, 4095, 4095}, {13, 15, 2, 8192, 8200},
        {14, 16, 2, 8192, 16384}, {14, 16, 1, 16384, 16384}, {16, 18, 1, 65536, 65536}, {16, 17, 1, 40000, 40000},
        {16, 16, 1, 65536, 65536}, {8, 10, 0, 256, 256}, {12, 14, 2, 5, 8}, {14, 16, 2, 100, 128}, {14, 16, 2, 2816, 2816},
        {16, 18, 1, 4097, 4100}, {16, 18, 1, 4095, 4095}, {12, 14, 3, 257, 257},
    };
    // per-element addressing, scalar-base addressing where it applies, the fused middle launch of the LDE, and that
    // launch with the coset factors split into shifts and per-coset twiddle tables
    for (int mode = 0; mode < 4; ++mode) {
        emu_set_uniform(mode >= 1);
        emu_set_fusion(mode >= 2);
        emu_set_merged(mode >= 3);
        for (auto &s : lde) bad += check_lde((int)s[0], (int)s[1], s[2], s[3], s[4]);
        bad += check_ntt(12, 3);
        bad += check_ntt(18, 1);
    }
    printf(bad ? "FAIL %d\n" : "OK\n", bad);
    return bad ? 1 : 0;
}
