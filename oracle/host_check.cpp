// host_check.cpp -- test infrastructure: a host-only harness over the library's CPU-side code (the data layer
// of fasted_amd/csrc/point_table.hpp, the tile order and LDS swizzles of fasted_amd/csrc/tile_order.hpp) and
// over the CPU checker (fasted_oracle.c), built with the address and undefined-behaviour sanitizers by
// `make -C oracle asan`.  The reference's own provision for this is a pair of commented compute-sanitizer
// lines (source/run.sh:74-76); sanitizers here run on host code only.  Exit status 0 = every check held and
// the sanitizers stayed silent.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <set>
#include <string>
#include <vector>

#include "../fasted_amd/csrc/point_table.hpp"
#include "../fasted_amd/csrc/tile_order.hpp"

extern "C" {
uint16_t oracle_f32_to_f16(float value);
float oracle_f16_to_f32(uint16_t h);
void oracle_quantize(const double* in, size_t n, uint16_t* out);
void oracle_exponential_points(int n, int d, double lambda, double max_value, double* out);
void oracle_sum_squared_rz(const uint16_t* pts, size_t n, size_t d, float* sums);
void oracle_sum_squared_rn(const uint16_t* pts, size_t n, size_t d, float* sums);
void oracle_sum_squared_f64(const uint16_t* pts, size_t n, size_t d, double* sums);
int oracle_raster_coord(unsigned long long idx, unsigned long long chunk_rows, unsigned long long chunk_cols,
                        unsigned int raster_size, int tile_m, int tile_n, int* row, int* col);
long long oracle_pairs_get_space(unsigned long long* found, unsigned long long* stored, unsigned long long max_pairs,
                                 unsigned long long n);
unsigned long long oracle_self_join_f64(const uint16_t* pts, size_t n, size_t d, double eps, int* out_q, int* out_c,
                                        unsigned long long cap);
unsigned long long oracle_self_join_f32(const uint16_t* pts, size_t n, size_t d, double eps, const float* sums,
                                        int* out_q, int* out_c, unsigned long long cap);
void oracle_pair_distances_f64(const uint16_t* pts, size_t d, const int* q, const int* c, size_t npairs, double* dist);
void oracle_pair_stats(const int* lq, const int* lc, size_t nl, const int* rq, const int* rc, size_t nr,
                       unsigned long long stats[5], int* only_q, int* only_c, int* only_side, size_t only_cap);
}

static int g_failures = 0;
#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) {                                                           \
            std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            ++g_failures;                                                        \
        }                                                                        \
    } while (0)

static void check_quantisation() {
    // every finite half survives half -> float -> (library and checker) half; the library and the checker agree
    // on doubles around ties
    for (unsigned h = 0; h < 65536; ++h) {
        const float f = oracle_f16_to_f32((uint16_t)h);
        if (std::isnan(f)) continue;
        CHECK(oracle_f32_to_f16(f) == h);
        CHECK(fasted::quantize_half((double)f) == h);
    }
    const double probes[] = {0.01198196413320991, 1.00048828125, 65519.9, 65520.0, -70000.0, 2.98e-8, 5.960464477539063e-08,
                             0.333251953125, 0.3332519531250001, 1e-30, -0.0};
    for (double v : probes) {
        uint16_t o = 0;
        oracle_quantize(&v, 1, &o);
        CHECK(fasted::quantize_half(v) == o);
    }
}

static void check_data_layer(const char* csvPath) {
    // seeded generator: the block-parallel builder equals the sequential one and the checker's stream
    const int n = 300, d = 4000;  // above the 2^20-value threshold of the parallel path
    fasted::PointTable par = fasted::build_exponential_table(n, d, 40.0, 10.0, 64, 256, 4);
    fasted::PointTable seq = fasted::build_exponential_table(n, d, 40.0, 10.0, 64, 256, 1);
    CHECK(par.bits == seq.bits && par.n == n && par.d == d && par.nPad == 512 && par.dPad == 4032);
    CHECK(par.name == seq.name);
    std::vector<double> vals((size_t)n * d);
    oracle_exponential_points(n, d, 40.0, 10.0, vals.data());
    std::vector<uint16_t> q(vals.size());
    oracle_quantize(vals.data(), vals.size(), q.data());
    bool same = true;
    for (int i = 0; i < n && same; ++i)
        same = std::memcmp(&par.bits[(size_t)i * par.dPad], &q[(size_t)i * d], (size_t)d * 2) == 0;
    CHECK(same);
    // padding is zeros
    unsigned long long padding = 0;
    for (int i = 0; i < par.nPad; ++i)
        for (int k = (i < n ? d : 0); k < par.dPad; ++k) padding += par.bits[(size_t)i * par.dPad + k];
    CHECK(padding == 0);

    // CSV reader: threaded and sequential parse agree; error paths throw
    if (csvPath) {
        fasted::PointTable a = fasted::load_csv_table(csvPath, ',', 64, 256, 1);
        fasted::PointTable b = fasted::load_csv_table(csvPath, ',', 64, 256, 7);
        CHECK(a.bits == b.bits && a.n == b.n && a.d == b.d && a.n > 0);
    }
    const std::string tmp = "/tmp/fasted_host_check_ragged.csv";
    {
        std::ofstream f(tmp);
        f << "1,2,3\n4,5\n";
    }
    bool threw = false;
    try {
        (void)fasted::load_csv_table(tmp, ',', 64, 256, 2);
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw);
    {
        std::ofstream f(tmp);
    }
    threw = false;
    try {
        (void)fasted::load_csv_table(tmp, ',', 64, 256);
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw);
    std::remove(tmp.c_str());
    threw = false;
    try {
        (void)fasted::load_csv_table("/nonexistent/points.csv", ',', 64, 256);
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw);
}

static void check_tile_order() {
    // every tile of the grid exactly once, for the 256x256 kernel's 8 x 4 sub-rectangles and for other cuts
    const struct {
        long long nq, nc;
        int tm, tn, sr, sc;
        bool upper;
    } cases[] = {{1, 1, 256, 256, 8, 4, false},       {4097, 4097, 256, 256, 8, 4, false}, {9000, 3000, 256, 256, 8, 4, false},
                 {10000, 10000, 256, 256, 8, 4, true}, {70000, 70000, 256, 256, 8, 4, true}, {10000, 10000, 256, 256, 4, 8, true},
                 {5000, 7000, 256, 128, 4, 16, false}, {6000, 6000, 128, 128, 8, 16, false}, {20000, 20000, 256, 256, 16, 2, true}};
    for (const auto& c : cases) {
        const fasted::TileOrder o = fasted::make_tile_order(c.nq, c.nc, c.tm, c.tn, c.sr, c.sc, c.upper);
        std::set<std::pair<unsigned, unsigned>> seen;
        unsigned long long real = 0;
        for (unsigned q = 0; q < (unsigned)fasted::kQueues; ++q)
            for (unsigned long long t = 0; t < o.perQueue; ++t) {
                unsigned tr, tc;
                fasted::tile_order_decode(o, c.sr, c.sc, q, t, &tr, &tc);
                if (tr >= o.tileRows || tc >= o.tileCols) continue;
                CHECK(seen.insert({tr, tc}).second);
                ++real;
            }
        CHECK((o.upperOnly != 0) == c.upper);
        if (!o.upperOnly) {
            CHECK(real == (unsigned long long)o.tileRows * o.tileCols);
        } else {
            // the squares on and above the diagonal: every tile with tc >= tr is there
            for (unsigned tr = 0; tr < o.tileRows; ++tr)
                for (unsigned tc = tr; tc < o.tileCols; ++tc) CHECK(seen.count({tr, tc}) == 1);
        }
    }
    // LDS swizzles: the 16 lanes of every ds_read_b128 phase touch all 64 banks once
    const int groups[2][16] = {{0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27},
                               {4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31}};
    for (int upper = 0; upper < 2; ++upper)
        for (const auto& g : groups) {
            for (int ks = 0; ks < 2; ++ks) {  // 128-byte rows, chunk 4*ks + l/16
                std::set<int> banks;
                for (int l : g) {
                    const int lane = l + 32 * upper, row = lane % 16, chunk = 4 * ks + lane / 16;
                    const int byte = row * 128 + ((chunk ^ fasted::lds_swizzle128(row)) << 4);
                    for (int b = 0; b < 4; ++b) banks.insert((byte / 4 + b) % 64);
                }
                CHECK(banks.size() == 64);
            }
            std::set<int> banks;  // 64-byte rows, chunk l/16
            for (int l : g) {
                const int lane = l + 32 * upper, row = lane % 16, chunk = lane / 16;
                const int byte = row * 64 + ((chunk ^ fasted::lds_swizzle64(row)) << 4);
                for (int b = 0; b < 4; ++b) banks.insert((byte / 4 + b) % 64);
            }
            CHECK(banks.size() == 64);
        }
}

static void check_checker() {
    const int n = 257, d = 70;
    std::vector<double> vals((size_t)n * d);
    oracle_exponential_points(n, d, 40.0, 1.0, vals.data());
    std::vector<uint16_t> pts(vals.size());
    oracle_quantize(vals.data(), vals.size(), pts.data());
    std::vector<float> rz(n), rn(n);
    std::vector<double> exact(n);
    oracle_sum_squared_rz(pts.data(), n, d, rz.data());
    oracle_sum_squared_rn(pts.data(), n, d, rn.data());
    oracle_sum_squared_f64(pts.data(), n, d, exact.data());
    for (int i = 0; i < n; ++i) {
        CHECK(rz[i] <= exact[i] * (1 + 1e-7) && std::fabs(rn[i] - exact[i]) <= d * 6e-8 * exact[i]);
    }
    const double eps = 0.15;
    const unsigned long long cap = (unsigned long long)n * n;
    std::vector<int> q64(cap), c64(cap), q32(cap), c32(cap);
    const unsigned long long f64 = oracle_self_join_f64(pts.data(), n, d, eps, q64.data(), c64.data(), cap);
    const unsigned long long f32 = oracle_self_join_f32(pts.data(), n, d, eps, rz.data(), q32.data(), c32.data(), cap);
    CHECK(f64 >= (unsigned long long)n && f64 <= cap && f32 <= cap);
    // a buffer that is too small: the count is still exact, nothing is written past the capacity
    std::vector<int> smallQ(11, -7), smallC(11, -7);
    CHECK(oracle_self_join_f64(pts.data(), n, d, eps, smallQ.data(), smallC.data(), 10) == f64);
    CHECK(smallQ[10] == -7 && smallC[10] == -7);
    std::vector<double> dist(f64);
    oracle_pair_distances_f64(pts.data(), d, q64.data(), c64.data(), f64, dist.data());
    for (unsigned long long i = 0; i < f64; ++i) CHECK(dist[i] <= eps * (1 + 1e-12));
    unsigned long long stats[5];
    std::vector<int> oq(f64 + f32), oc(f64 + f32), os(f64 + f32);
    oracle_pair_stats(q32.data(), c32.data(), f32, q64.data(), c64.data(), f64, stats, oq.data(), oc.data(), os.data(),
                      oq.size());
    CHECK(stats[0] + stats[2] == f32 && stats[0] + stats[1] == f64);
    // the reference rasterizer visits every tile once
    std::set<std::pair<int, int>> seen;
    int r, c;
    for (unsigned long long i = 0; oracle_raster_coord(i, 16, 24, 8, 96, 96, &r, &c); ++i) CHECK(seen.insert({r, c}).second);
    CHECK(seen.size() == 16 * 24);
    unsigned long long found = 0, stored = 0;
    CHECK(oracle_pairs_get_space(&found, &stored, 3, 2) == 0 && oracle_pairs_get_space(&found, &stored, 3, 2) == -1);
    CHECK(found == 4 && stored == 2);
}

int main(int argc, char** argv) {
    check_quantisation();
    check_data_layer(argc > 1 ? argv[1] : nullptr);
    check_tile_order();
    check_checker();
    if (g_failures) {
        std::fprintf(stderr, "host_check: %d checks failed\n", g_failures);
        return 1;
    }
    std::printf("host_check: all checks held\n");
    return 0;
}
