// Matrix Market (coordinate) text -> CSR, on the host.  The step in front of the RoDe
// path for matrices that come as files (SuiteSparse): the reference's own loader
// (matrix_utils.h / SPC::SparseMatrix, used at Preprocess_opt/_preprocess.cu:2,406-413) is
// missing from its tree; this covers the same ground.  Real / integer / pattern fields,
// general / symmetric / skew-symmetric storage; the result has ascending columns in every
// row, duplicates summed, int32 indices and float32 values.
//
// The text is parsed in parallel: the buffer is cut into one piece per thread at line
// ends, every thread turns its lines into (row, column, value) triples, a counting sort by
// row and a sort by column inside every row order them.
#include <algorithm>
#include <cctype>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <new>
#include <string>
#include <vector>

#include <omp.h>

namespace {

struct Triple {
    int32_t row, col;
    double val;
};

struct Matrix {
    int m = 0, n = 0;
    std::vector<int32_t> row_ptr, col;
    std::vector<float> val;
};

void fail(char* err, int errlen, const std::string& msg)
{
    if (err && errlen > 0) {
        std::strncpy(err, msg.c_str(), errlen - 1);
        err[errlen - 1] = 0;
    }
}

const char* skip_blank(const char* p, const char* end)
{
    while (p < end && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
    return p;
}

const char* line_end(const char* p, const char* end)
{
    if (p >= end) return end; // (an empty text has no address to search from)
    const void* nl = std::memchr(p, '\n', end - p);
    return nl ? static_cast<const char*>(nl) : end;
}

// Non-negative decimal integer; false if there is none at p.
bool parse_index(const char*& p, const char* end, long long& out)
{
    p = skip_blank(p, end);
    if (p >= end || *p < '0' || *p > '9') return false;
    long long v = 0;
    while (p < end && *p >= '0' && *p <= '9') {
        v = v * 10 + (*p - '0');
        if (v > (1ll << 40)) return false;
        ++p;
    }
    out = v;
    return true;
}

bool parse_value(const char*& p, const char* end, double& out)
{
    p = skip_blank(p, end);
    if (p >= end || *p == '\n') return false;
    size_t len = 0;
    while (p + len < end && !std::isspace(static_cast<unsigned char>(p[len]))) ++len;
    // strtod wants a terminated string and the text has none: the token is copied (to the
    // stack, unless it is longer than any sensible number)
    char buf[64];
    std::string big;
    const char* token = buf;
    if (len < sizeof(buf)) {
        std::memcpy(buf, p, len);
        buf[len] = 0;
    } else {
        big.assign(p, len);
        token = big.c_str();
    }
    char* stop = nullptr;
    out = std::strtod(token, &stop);
    if (stop != token + len) return false; // (not a number, or a number followed by something else)
    p += len;
    return true;
}

std::string lower(std::string s)
{
    for (char& c : s) c = static_cast<char>(std::tolower(static_cast<unsigned char>(c)));
    return s;
}

} // namespace

extern "C" {

// Parses the text of a Matrix Market file.  Returns a handle (rode_mtx_free it) and the
// shape and nonzero count of the CSR matrix, or NULL with a message in err.
static void* parse_text(const char* data, size_t len, int* m_out, int* n_out, long long* nnz_out, char* err, int errlen)
{
    const char* p = data;
    const char* end = data + len;
    // banner
    const char* le = line_end(p, end);
    std::string banner(p, le);
    char w[5][64] = {{0}};
    if (std::sscanf(banner.c_str(), "%63s %63s %63s %63s %63s", w[0], w[1], w[2], w[3], w[4]) != 5 ||
        std::string(w[0]) != "%%MatrixMarket" || lower(w[1]) != "matrix") {
        fail(err, errlen, "not a Matrix Market matrix file");
        return nullptr;
    }
    const std::string layout = lower(w[2]), field = lower(w[3]), symmetry = lower(w[4]);
    if (layout != "coordinate") {
        fail(err, errlen, "only the coordinate (sparse) layout is supported, got " + layout);
        return nullptr;
    }
    if (field != "real" && field != "integer" && field != "pattern" && field != "double") {
        fail(err, errlen, "unsupported field " + field);
        return nullptr;
    }
    if (symmetry != "general" && symmetry != "symmetric" && symmetry != "skew-symmetric") {
        fail(err, errlen, "unsupported symmetry " + symmetry);
        return nullptr;
    }
    const bool pattern = field == "pattern";
    p = le < end ? le + 1 : end;
    // comments and blank lines, then the size line
    long long m = 0, n = 0, entries = 0;
    for (;;) {
        if (p >= end) {
            fail(err, errlen, "no size line");
            return nullptr;
        }
        le = line_end(p, end);
        const char* q = skip_blank(p, le);
        if (q < le && *q != '%') {
            if (!parse_index(q, le, m) || !parse_index(q, le, n) || !parse_index(q, le, entries)) {
                fail(err, errlen, "malformed size line");
                return nullptr;
            }
            p = le < end ? le + 1 : end;
            break;
        }
        p = le < end ? le + 1 : end;
    }
    if (m > INT32_MAX || n > INT32_MAX || entries > (1ll << 40)) {
        fail(err, errlen, "matrix too large for 32-bit indices");
        return nullptr;
    }
    // the mirrored entry (c, r) of a symmetric file must be a valid position as well
    if (symmetry != "general" && m != n) {
        fail(err, errlen, "a " + symmetry + " matrix must be square, got " + std::to_string(m) + " x " + std::to_string(n));
        return nullptr;
    }

    // entry lines, one piece of the text per thread
    const int threads = std::max(1, std::min(omp_get_max_threads(), (int)((end - p) / (1 << 16)) + 1));
    std::vector<const char*> cut(threads + 1, end);
    cut[0] = p;
    for (int t = 1; t < threads; ++t) {
        const char* c = p + (end - p) / threads * t;
        c = line_end(c, end);
        cut[t] = c < end ? c + 1 : end;
    }
    std::vector<std::vector<Triple>> parts(threads);
    std::vector<int> bad(threads, 0);
#pragma omp parallel for num_threads(threads) schedule(static, 1)
    for (int t = 0; t < threads; ++t) {
        const char* q = cut[t];
        const char* stop = cut[t + 1];
        std::vector<Triple>& out = parts[t];
        out.reserve((stop - q) / 12 + 16);
        while (q < stop) {
            const char* e = line_end(q, stop);
            const char* s = skip_blank(q, e);
            if (s < e && *s != '%') {
                long long r, c;
                double v = 1.0;
                if (!parse_index(s, e, r) || !parse_index(s, e, c) || (!pattern && !parse_value(s, e, v)) || r < 1 ||
                    r > m || c < 1 || c > n) {
                    bad[t] = 1;
                    break;
                }
                out.push_back(Triple{(int32_t)(r - 1), (int32_t)(c - 1), v});
            }
            q = e < stop ? e + 1 : stop;
        }
    }
    long long found = 0;
    for (int t = 0; t < threads; ++t) {
        if (bad[t]) {
            fail(err, errlen, "malformed entry line or index out of range");
            return nullptr;
        }
        found += (long long)parts[t].size();
    }
    if (found != entries) {
        fail(err, errlen, "header promises " + std::to_string(entries) + " entries, file has " + std::to_string(found));
        return nullptr;
    }

    // counting sort by row (the mirrored half of a symmetric file is added here)
    const double sign = symmetry == "skew-symmetric" ? -1.0 : 1.0;
    const bool mirror = symmetry != "general";
    std::vector<long long> start((size_t)m + 1, 0);
    for (const auto& part : parts)
        for (const Triple& t : part) {
            ++start[t.row + 1];
            if (mirror && t.row != t.col) ++start[t.col + 1];
        }
    for (long long r = 0; r < m; ++r) start[r + 1] += start[r];
    const long long total = start[m];
    std::vector<std::pair<int32_t, double>> sorted((size_t)total);
    {
        std::vector<long long> at(start.begin(), start.end() - 1);
        for (const auto& part : parts)
            for (const Triple& t : part) {
                sorted[at[t.row]++] = {t.col, t.val};
                if (mirror && t.row != t.col) sorted[at[t.col]++] = {t.row, sign * t.val};
            }
    }
    parts.clear();
    parts.shrink_to_fit();

    // columns ascending inside every row (stable, so that duplicates are summed in file order)
    std::vector<long long> kept((size_t)m + 1, 0);
#pragma omp parallel for schedule(dynamic, 1024)
    for (long long r = 0; r < m; ++r) {
        auto first = sorted.begin() + start[r], last = sorted.begin() + start[r + 1];
        std::stable_sort(first, last, [](const auto& a, const auto& b) { return a.first < b.first; });
        long long out = start[r];
        for (long long i = start[r]; i < start[r + 1]; ++i) {
            if (out > start[r] && sorted[out - 1].first == sorted[i].first)
                sorted[out - 1].second += sorted[i].second;
            else
                sorted[out++] = sorted[i];
        }
        kept[r + 1] = out - start[r];
    }
    for (long long r = 0; r < m; ++r) kept[r + 1] += kept[r];
    if (kept[m] > INT32_MAX) {
        fail(err, errlen, "more than 2^31 - 1 nonzeros");
        return nullptr;
    }
    Matrix* mat = new Matrix;
    mat->m = (int)m;
    mat->n = (int)n;
    mat->row_ptr.resize((size_t)m + 1);
    mat->col.resize((size_t)kept[m]);
    mat->val.resize((size_t)kept[m]);
    for (long long r = 0; r <= m; ++r) mat->row_ptr[r] = (int32_t)kept[r];
#pragma omp parallel for schedule(static)
    for (long long r = 0; r < m; ++r)
        for (long long i = 0; i < kept[r + 1] - kept[r]; ++i) {
            mat->col[kept[r] + i] = sorted[start[r] + i].first;
            mat->val[kept[r] + i] = (float)sorted[start[r] + i].second;
        }
    *m_out = mat->m;
    *n_out = mat->n;
    *nnz_out = kept[m];
    return mat;
}

// No exception leaves the library: a size line that asks for more memory than there is
// (std::bad_alloc from the tables sized by it) is reported like any other bad file.
void* rode_mtx_parse(const char* data, size_t len, int* m_out, int* n_out, long long* nnz_out, char* err, int errlen)
{
    try {
        return parse_text(data, len, m_out, n_out, nnz_out, err, errlen);
    } catch (const std::bad_alloc&) {
        fail(err, errlen, "out of memory: the size line describes a matrix that does not fit");
    } catch (const std::exception& e) {
        fail(err, errlen, std::string("parser error: ") + e.what());
    }
    return nullptr;
}

void rode_mtx_copy(void* handle, int* row_ptr, int* col, float* val)
{
    const Matrix* mat = static_cast<const Matrix*>(handle);
    std::memcpy(row_ptr, mat->row_ptr.data(), mat->row_ptr.size() * sizeof(int32_t));
    if (!mat->col.empty()) {
        std::memcpy(col, mat->col.data(), mat->col.size() * sizeof(int32_t));
        std::memcpy(val, mat->val.data(), mat->val.size() * sizeof(float));
    }
}

void rode_mtx_free(void* handle) { delete static_cast<Matrix*>(handle); }

} // extern "C"
