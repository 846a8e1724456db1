// Synthetic CSR workloads (host only, no GPU code): the five benchmark
// configurations and the seeded generators the reference's C++ tests use.
//
// Benchmark configurations draw every row from its own counter-based random
// stream (seed, row), so the result does not depend on the number of threads
// and a row can be regenerated on its own (first pass: lengths, second pass:
// contents).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

namespace {

// ---- small counter-based generator (splitmix64 seeding + xoshiro256**) -----
struct Rng {
    uint64_t s[4];
    static uint64_t splitmix(uint64_t& x)
    {
        uint64_t z = (x += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
    Rng(uint64_t seed, uint64_t stream)
    {
        uint64_t x = seed * 0xd1342543de82ef95ull + stream * 0x2545f4914f6cdd1dull + 0x1234567ull;
        for (auto& w : s) w = splitmix(x);
    }
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    uint64_t next()
    {
        const uint64_t r = rotl(s[1] * 5, 7) * 9, t = s[1] << 17;
        s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3]; s[2] ^= t; s[3] = rotl(s[3], 45);
        return r;
    }
    double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }       // [0,1)
    double uniform_open() { return ((double)(next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); } // (0,1)
    uint64_t below(uint64_t n) { return (uint64_t)(((unsigned __int128)next() * n) >> 64); }  // [0,n)
    double normal()
    {
        const double u = uniform_open(), v = uniform();
        return std::sqrt(-2.0 * std::log(u)) * std::cos(6.283185307179586 * v);
    }
};

struct Scratch {
    std::vector<uint64_t> bitmap; // one bit per column, always left cleared
    std::vector<int> cols;
};

// `d` distinct columns, uniform over [lo, hi), ascending.
void sample_distinct(Rng& rng, int lo, int hi, int d, Scratch& sc, std::vector<int>& out)
{
    const int n = hi - lo;
    d = std::max(0, std::min(d, n));
    out.clear();
    if (d == 0) return;
    if ((size_t)(n + 63) / 64 > sc.bitmap.size()) sc.bitmap.assign((size_t)(n + 63) / 64, 0);
    const bool complement = d > n / 2;
    const int draw = complement ? n - d : d;
    std::vector<int>& picked = sc.cols;
    picked.clear();
    while ((int)picked.size() < draw) {
        const int c = (int)rng.below((uint64_t)n);
        uint64_t& w = sc.bitmap[c >> 6];
        const uint64_t bit = 1ull << (c & 63);
        if (!(w & bit)) { w |= bit; picked.push_back(c); }
    }
    if (complement) {
        for (int c = 0; c < n; ++c)
            if (!(sc.bitmap[c >> 6] >> (c & 63) & 1)) out.push_back(lo + c);
    } else {
        out.assign(picked.begin(), picked.end());
        std::sort(out.begin(), out.end());
        for (int& c : out) c += lo;
    }
    for (int c : picked) sc.bitmap[c >> 6] = 0;
}

// Zipf(alpha) on {1..kmax} by rejection (Devroye, Non-Uniform Random Variate
// Generation, X.6), truncated by rejecting draws above kmax.
int zipf(Rng& rng, double alpha, int kmax)
{
    const double am1 = alpha - 1.0, b = std::pow(2.0, am1);
    for (;;) {
        const double u = rng.uniform_open(), v = rng.uniform();
        const double xf = std::floor(std::pow(u, -1.0 / am1));
        if (!(xf >= 1.0) || xf > (double)kmax) continue;
        const double t = std::pow(1.0 + 1.0 / xf, am1);
        if (v * xf * (t - 1.0) / (b - 1.0) <= t / b) return (int)xf;
    }
}

enum Config { kUniform = 1, kLogNormal = 2, kBanded = 3, kPowerLaw = 4, kAttention = 5 };

// Generates row `r`; cols ascending.  vals may be null (length pass).
void gen_row(int config, int M, int ncols, double p0, double p1, uint64_t seed, int r, Scratch& sc,
             std::vector<int>& cols, std::vector<float>* vals)
{
    Rng rng(seed, (uint64_t)r);
    cols.clear();
    float fill = 0.f;
    bool random_vals = true;
    switch (config) {
    case kUniform: { // every (r, c) kept with probability p0 (geometric skipping)
        const double lg = std::log1p(-p0);
        for (double c = std::floor(std::log(rng.uniform_open()) / lg); c < ncols;
             c += 1.0 + std::floor(std::log(rng.uniform_open()) / lg))
            cols.push_back((int)c);
        break;
    }
    case kLogNormal: { // length = min(floor(LogNormal(mean p0, sigma p1)), 20000)
        const double mu = std::log(p0) - 0.5 * p1 * p1;
        const double len = std::floor(std::exp(mu + p1 * rng.normal()));
        sample_distinct(rng, 0, ncols, (int)std::min(len, 20000.0), sc, cols);
        break;
    }
    case kBanded: { // p0 nonzeros inside a band of width p1 around the diagonal
        const int half = (int)p1 / 2;
        sample_distinct(rng, std::max(0, r - half), std::min(ncols, r + half), (int)p0, sc, cols);
        break;
    }
    case kPowerLaw: { // degree = scale * (Zipf(alpha = p0) - 1) + U{1..scale}, in [1, 200000]; value 1/degree
        // A plain Zipf(2.1) on [1, 2e5] averages 4.9 nonzeros per row; stretching it by
        // `scale` keeps the exponent of the tail and the minimum degree of 1 while
        // reaching the intended density (scale 6 -> about 24 per row).
        const int kmax = 200000, scale = std::max(1, (int)p1);
        const int z = zipf(rng, p0, (kmax + scale - 1) / scale);
        const int deg = std::min(kmax, scale * (z - 1) + 1 + (int)rng.below((uint64_t)scale));
        sample_distinct(rng, 0, ncols, deg, sc, cols);
        fill = cols.empty() ? 0.f : 1.0f / (float)cols.size();
        random_vals = false;
        break;
    }
    case kAttention: { // sliding window of width p0 plus p1 random global columns, value 1
        const int half = (int)p0 / 2, lo = std::max(0, r - half), hi = std::min(ncols, r + half);
        std::vector<int> extra;
        sample_distinct(rng, 0, ncols, (int)p1, sc, extra);
        for (int c = lo; c < hi; ++c) cols.push_back(c);
        for (int c : extra)
            if (c < lo || c >= hi) cols.push_back(c);
        std::sort(cols.begin(), cols.end());
        fill = 1.0f;
        random_vals = false;
        break;
    }
    default: break;
    }
    (void)M;
    if (vals) {
        vals->resize(cols.size());
        for (auto& v : *vals) v = random_vals ? (float)(2.0 * rng.uniform() - 1.0) : fill;
    }
}

} // namespace

extern "C" {

// Pass 1: lens[r] = number of nonzeros of row r.
void rode_wl_row_lengths(int config, int M, int ncols, double p0, double p1, uint64_t seed, int* lens)
{
#pragma omp parallel
    {
        Scratch sc;
        std::vector<int> cols;
#pragma omp for schedule(dynamic, 256)
        for (int r = 0; r < M; ++r) {
            gen_row(config, M, ncols, p0, p1, seed, r, sc, cols, nullptr);
            lens[r] = (int)cols.size();
        }
    }
}

// Pass 2: fills cols/vals at row_ptr (the prefix sum of pass 1's lengths).
void rode_wl_fill(int config, int M, int ncols, double p0, double p1, uint64_t seed, const int* row_ptr, int* cols_out,
                  float* vals_out)
{
#pragma omp parallel
    {
        Scratch sc;
        std::vector<int> cols;
        std::vector<float> vals;
#pragma omp for schedule(dynamic, 256)
        for (int r = 0; r < M; ++r) {
            gen_row(config, M, ncols, p0, p1, seed, r, sc, cols, &vals);
            if (cols.empty()) continue; // (an empty row has nothing to copy, and its vectors may have no storage)
            std::memcpy(cols_out + row_ptr[r], cols.data(), cols.size() * sizeof(int));
            std::memcpy(vals_out + row_ptr[r], vals.data(), vals.size() * sizeof(float));
        }
    }
}

// ---- the reference's C++ test generators ------------------------------------
// Same random-call sequence as RoDe_SDDMM/main.cu:181-234 (poisson == 0: row
// length uniform in [1, 2*nnz_per_row]) and RoDe_SDDMM/test.cu:121-169
// (poisson == 1: Poisson(nnz_per_row), at least 1), both capped at n: one
// std::mt19937(seed) drives length, a full std::shuffle of 0..n-1 and the
// U(-1,1) values; every row is then padded to a multiple of pad_to with
// (last column, 0.0f).  With libstdc++ this reproduces their matrices.
struct RefCsr {
    std::vector<int> row_offsets, cols;
    std::vector<float> vals;
};

void* rode_wl_ref_csr_create(int m, int n, int nnz_per_row, int poisson, int pad_to, unsigned seed)
{
    auto* out = new RefCsr;
    std::mt19937 gen(seed);
    std::uniform_real_distribution<float> val_dist(-1.0f, 1.0f);
    std::uniform_int_distribution<int> uni_len(1, nnz_per_row * 2);
    std::poisson_distribution<int> poi_len(nnz_per_row);
    out->row_offsets.push_back(0);
    std::vector<int> perm(n);
    for (int i = 0; i < m; ++i) {
        const int want = poisson ? std::max(1, std::min(poi_len(gen), n)) : std::min(uni_len(gen), n);
        std::iota(perm.begin(), perm.end(), 0);
        std::shuffle(perm.begin(), perm.end(), gen);
        std::vector<int> row(perm.begin(), perm.begin() + want);
        std::sort(row.begin(), row.end());
        for (int c : row) {
            out->cols.push_back(c);
            out->vals.push_back(val_dist(gen));
        }
        if (pad_to > 1) {
            const int rem = want % pad_to;
            for (int j = 0; rem > 0 && j < pad_to - rem; ++j) {
                out->cols.push_back(row.back());
                out->vals.push_back(0.0f);
            }
        }
        out->row_offsets.push_back((int)out->cols.size());
    }
    return out;
}

int rode_wl_ref_csr_nnz(void* h) { return (int)static_cast<RefCsr*>(h)->cols.size(); }

void rode_wl_ref_csr_copy(void* h, int* row_offsets, int* cols, float* vals)
{
    auto* c = static_cast<RefCsr*>(h);
    std::memcpy(row_offsets, c->row_offsets.data(), c->row_offsets.size() * sizeof(int));
    std::memcpy(cols, c->cols.data(), c->cols.size() * sizeof(int));
    std::memcpy(vals, c->vals.data(), c->vals.size() * sizeof(float));
}

void rode_wl_ref_csr_free(void* h) { delete static_cast<RefCsr*>(h); }

// RoDe_SDDMM/main.cu:239-251: std::mt19937(seed), U(-1,1), row-major.
void rode_wl_ref_dense(long long count, unsigned seed, float* out)
{
    std::mt19937 gen(seed);
    std::uniform_real_distribution<float> dist(-1.0f, 1.0f);
    for (long long i = 0; i < count; ++i) out[i] = dist(gen);
}

} // extern "C"
