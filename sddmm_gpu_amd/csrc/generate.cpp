// Synthetic sparse matrices of the five benchmark shapes, generated on the host: what the command-line
// tool's --gen reads instead of a file.  The reference ships no generator (its inputs are downloaded
// Matrix Market files, HiPC18/run.sh:3-6); these stand in for them where there is no network.  Every
// row draws from a generator seeded by (seed, row), so the matrix does not depend on the thread count.
#include <cmath>
#include <cstring>
#include <numeric>
#include "internal.hpp"

using namespace sddmm;

namespace {

struct Rng {  // splitmix64 seeding a xorshift128+
    uint64_t a, b;
    static uint64_t mix(uint64_t &z) {
        z += 0x9e3779b97f4a7c15ull;
        uint64_t x = z;
        x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
        x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
        return x ^ (x >> 31);
    }
    Rng(uint64_t seed, uint64_t stream) {
        uint64_t z = seed * 0x2545f4914f6cdd1dull + stream;
        a = mix(z); b = mix(z);
        if (!(a | b)) b = 1;
    }
    uint64_t next() {
        uint64_t x = a; const uint64_t y = b;
        a = y;
        x ^= x << 23;
        b = x ^ y ^ (x >> 17) ^ (y >> 26);
        return b + y;
    }
    double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }  // [0, 1)
    uint64_t below(uint64_t n) { return (uint64_t)(uniform() * (double)n); }
    double normal() {
        const double u = 1.0 - uniform(), v = uniform();
        return std::sqrt(-2.0 * std::log(u)) * std::cos(6.283185307179586 * v);
    }
};

struct Rows {  // rows under construction: per row a sorted list of distinct columns
    int64_t n_rows = 0, n_cols = 0;
    std::vector<std::vector<int32_t>> cols;
};

int finish(Rows &R, const std::function<float(Rng &)> &value, uint64_t seed, sddmm_coo **out)
{
    int64_t nnz = 0;
    for (const auto &c : R.cols) nnz += (int64_t)c.size();
    if (nnz >= INT32_MAX) return fail(SDDMM_ERR_RANGE, "sddmm_coo_generate: %lld nonzeros do not fit 32-bit offsets", (long long)nnz);
    auto *S = new sddmm_coo;
    S->n_rows = R.n_rows; S->n_cols = R.n_cols; S->nnz = nnz; S->sorted = 1;
    S->rows.resize((size_t)nnz); S->cols.resize((size_t)nnz); S->vals.resize((size_t)nnz);
    std::vector<int64_t> start((size_t)R.n_rows + 1, 0);
    for (int64_t r = 0; r < R.n_rows; ++r) start[(size_t)r + 1] = start[(size_t)r] + (int64_t)R.cols[(size_t)r].size();
    parallel_ranges(R.n_rows, 1024, [&](int64_t b, int64_t e, int) {
        for (int64_t r = b; r < e; ++r) {
            Rng g(seed ^ 0x5bd1e995u, (uint64_t)r);
            int64_t p = start[(size_t)r];
            for (int32_t c : R.cols[(size_t)r]) {
                S->rows[(size_t)p] = (int32_t)r; S->cols[(size_t)p] = c; S->vals[(size_t)p] = value(g);
                ++p;
            }
            std::vector<int32_t>().swap(R.cols[(size_t)r]);
        }
    });
    *out = S;
    return SDDMM_OK;
}

// about deg[r] distinct columns per row, drawn by popularity (weights w): rows that want a small share
// of the columns draw until they have enough distinct ones, the others take the deg largest of the keys
// u^(1/w) (weighted sampling without replacement)
void rows_by_popularity(Rows &R, const std::vector<double> &deg, const std::vector<double> &w, uint64_t seed)
{
    const int64_t n_cols = R.n_cols;
    std::vector<double> cdf((size_t)n_cols);
    std::partial_sum(w.begin(), w.end(), cdf.begin());
    const double total = cdf.back();
    parallel_dynamic(R.n_rows, 64, [&](int64_t b, int64_t e, int) {
        std::vector<uint8_t> seen((size_t)n_cols, 0);
        std::vector<std::pair<double, int32_t>> keys;
        for (int64_t r = b; r < e; ++r) {
            Rng g(seed, (uint64_t)r);
            const int64_t want = std::max<int64_t>(1, std::min<int64_t>(n_cols, (int64_t)std::llround(deg[(size_t)r])));
            auto &c = R.cols[(size_t)r];
            c.reserve((size_t)want);
            if (want * 8 <= n_cols) {
                int64_t tries = 0;
                while ((int64_t)c.size() < want && tries < 64 * want + 64) {
                    ++tries;
                    const double u = g.uniform() * total;
                    const int32_t col = (int32_t)std::min<int64_t>(n_cols - 1, std::upper_bound(cdf.begin(), cdf.end(), u) - cdf.begin());
                    if (!seen[(size_t)col]) { seen[(size_t)col] = 1; c.push_back(col); }
                }
                for (int32_t col : c) seen[(size_t)col] = 0;
            } else {
                keys.resize((size_t)n_cols);
                for (int64_t j = 0; j < n_cols; ++j) keys[(size_t)j] = {std::log(1.0 - g.uniform()) / w[(size_t)j], (int32_t)j};  // log u / w: larger is better
                std::nth_element(keys.begin(), keys.begin() + (want - 1), keys.end(), [](auto &x, auto &y) { return x.first > y.first; });
                for (int64_t j = 0; j < want; ++j) c.push_back(keys[(size_t)j].second);
            }
            std::sort(c.begin(), c.end());
        }
    });
}

std::vector<double> zipf_weights(int64_t n, double s, uint64_t seed)
{
    std::vector<double> w((size_t)n);
    for (int64_t j = 0; j < n; ++j) w[(size_t)j] = std::pow((double)(j + 1), -s);
    Rng g(seed ^ 0xc0115eedull, 0);  // popular columns anywhere, not in front
    for (int64_t j = n - 1; j > 0; --j) std::swap(w[(size_t)j], w[(size_t)g.below((uint64_t)j + 1)]);
    return w;
}

}  // namespace

extern "C" int sddmm_coo_generate(int32_t config, double scale, uint64_t seed, sddmm_coo **out)
{
    if (!out) return fail(SDDMM_ERR_ARG, "sddmm_coo_generate: NULL output");
    *out = nullptr;
    if (!(scale > 0.0) || scale > 1.0) return fail(SDDMM_ERR_ARG, "sddmm_coo_generate: scale must be in (0, 1]");
    try {
        Rows R;
        if (config == 1) {  // uniform: 1 % of the cells of a square matrix, values in (0, 1]
            const int64_t n = std::max<int64_t>(8, (int64_t)(4096 * scale));
            R.n_rows = R.n_cols = n; R.cols.resize((size_t)n);
            const int64_t per_row = std::max<int64_t>(1, (int64_t)std::llround(0.01 * (double)n));
            parallel_ranges(n, 256, [&](int64_t b, int64_t e, int) {
                for (int64_t r = b; r < e; ++r) {
                    Rng g(seed, (uint64_t)r);
                    auto &c = R.cols[(size_t)r];
                    // (a binomial row length around 1 % of the columns)
                    int64_t k = 0;
                    for (int64_t j = 0; j < 4 * per_row; ++j) k += g.uniform() < 0.25;
                    for (int64_t j = 0; j < k; ++j) c.push_back((int32_t)g.below((uint64_t)n));
                    std::sort(c.begin(), c.end());
                    c.erase(std::unique(c.begin(), c.end()), c.end());
                }
            });
            return finish(R, [](Rng &g) { return (float)(1.0 - g.uniform()); }, seed, out);
        }
        if (config == 2 || config == 3) {
            std::vector<double> deg;
            double zipf;
            if (config == 2) {  // bag of words: lognormal document lengths, Zipf(1.1) word frequencies, geometric counts
                R.n_rows = std::max<int64_t>(4, (int64_t)(1500 * scale)); R.n_cols = std::max<int64_t>(16, (int64_t)(12419 * scale));
                const double mean = std::max(2.0, 497.5 * scale), sigma = 0.8, mu = std::log(mean) - sigma * sigma / 2;
                deg.resize((size_t)R.n_rows);
                Rng g(seed ^ 0xd06ull, 1);
                for (auto &d : deg) d = std::min(std::max(std::exp(g.normal() * sigma + mu), 1.0), 0.9 * (double)R.n_cols);
                zipf = 1.1;
            } else {  // recommender: user degrees from a truncated power law, item popularity Zipf(0.9), ratings 1..5
                R.n_rows = std::max<int64_t>(4, (int64_t)(480189 * scale)); R.n_cols = std::max<int64_t>(32, (int64_t)(17770 * std::sqrt(scale)));
                const double M = (double)std::min<int64_t>(std::max<int64_t>(4, (int64_t)(17000 * std::sqrt(scale))), (int64_t)(0.95 * (double)R.n_cols));
                const double beta = 1.42, ex = 1.0 - beta;
                deg.resize((size_t)R.n_rows);
                Rng g(seed ^ 0xd07ull, 1);
                for (auto &d : deg) d = std::min(std::max(std::pow(1.0 - g.uniform() * (1.0 - std::pow(M, ex)), 1.0 / ex), 1.0), M);
                zipf = 0.9;
            }
            R.cols.resize((size_t)R.n_rows);
            rows_by_popularity(R, deg, zipf_weights(R.n_cols, zipf, seed), seed);
            if (config == 2)
                return finish(R, [](Rng &g) { return (float)(std::floor(std::log(1.0 - g.uniform()) / std::log(0.6)) + 1.0); }, seed, out);
            return finish(R, [](Rng &g) { return (float)(1 + g.below(5)); }, seed, out);
        }
        if (config == 4) {  // R-MAT (0.57, 0.19, 0.19, 0.05), duplicates removed, values 1
            const int sc = scale < 1.0 ? std::max(4, 22 + (int)std::lround(std::log2(scale))) : 22;
            const int64_t n = (int64_t)1 << sc, n_edges = std::max<int64_t>(16, (int64_t)(200e6 * scale));
            std::vector<uint64_t> keys((size_t)n_edges);
            constexpr int64_t kBlock = 4096;  // edges per generator, so that the result does not depend on where the threads' ranges begin
            parallel_ranges((n_edges + kBlock - 1) / kBlock, 16, [&](int64_t b, int64_t e, int) {
                for (int64_t blk = b; blk < e; ++blk) {
                    Rng g(seed, (uint64_t)blk);
                    for (int64_t i = blk * kBlock; i < std::min(n_edges, (blk + 1) * kBlock); ++i) {
                        uint64_t row = 0, col = 0;
                        for (int l = 0; l < sc; ++l) {
                            const double u = g.uniform();
                            row = row * 2 + (u >= 0.76);
                            col = col * 2 + ((u >= 0.57 && u < 0.76) || u >= 0.95);
                        }
                        keys[(size_t)i] = row << 32 | col;
                    }
                }
            });
            std::sort(keys.begin(), keys.end());
            keys.erase(std::unique(keys.begin(), keys.end()), keys.end());
            R.n_rows = R.n_cols = n; R.cols.resize((size_t)n);
            for (uint64_t k : keys) R.cols[(size_t)(k >> 32)].push_back((int32_t)(k & 0xffffffffu));
            std::vector<uint64_t>().swap(keys);
            return finish(R, [](Rng &) { return 1.0f; }, seed, out);
        }
        if (config == 5) {  // banded: 64 columns per row, uniform inside +-2048 of the diagonal
            const int64_t n = std::max<int64_t>(64, (int64_t)((double)((int64_t)1 << 20) * scale));
            const int64_t per_row = n >= 4096 ? 64 : 8, half = std::min<int64_t>(2048, n / 2);
            R.n_rows = R.n_cols = n; R.cols.resize((size_t)n);
            parallel_ranges(n, 1024, [&](int64_t b, int64_t e, int) {
                for (int64_t r = b; r < e; ++r) {
                    Rng g(seed, (uint64_t)r);
                    auto &c = R.cols[(size_t)r];
                    for (int64_t j = 0; j < per_row; ++j) {
                        const int64_t col = r - half + (int64_t)g.below((uint64_t)(2 * half + 1));
                        c.push_back((int32_t)std::min<int64_t>(std::max<int64_t>(col, 0), n - 1));  // (clipped at the edges)
                    }
                    std::sort(c.begin(), c.end());
                    c.erase(std::unique(c.begin(), c.end()), c.end());
                }
            });
            return finish(R, [](Rng &g) { return (float)(1.0 - g.uniform()); }, seed, out);
        }
        return fail(SDDMM_ERR_ARG, "sddmm_coo_generate: config must be 1..5");
    } catch (const std::bad_alloc &) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_coo_generate: out of host memory");
    }
}
