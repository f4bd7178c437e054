// Matrix Market coordinate reader / writer and a raw binary side-file format.
// The text reader memory-maps the file and parses it with all host threads:
// the reference's reader is a serial iostream loop (HiPC18/src/sddmm.cu:257-283)
// that takes minutes at 1e8 nonzeros.
#include "internal.hpp"
#include <charconv>
#include <cctype>
#include <cstdio>
#include <cstring>
#include <fcntl.h>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

using namespace sddmm;

namespace {

struct Mapped {
    const char *p = nullptr;
    size_t n = 0;
    int fd = -1;
    ~Mapped()
    {
        if (p && n) munmap((void *)p, n);
        if (fd >= 0) close(fd);
    }
};

inline const char *skip_ws(const char *s, const char *e)
{
    while (s < e && (*s == ' ' || *s == '\t' || *s == '\r')) ++s;
    return s;
}
inline const char *line_end(const char *s, const char *e)
{
    const char *q = (const char *)memchr(s, '\n', (size_t)(e - s));
    return q ? q : e;
}
inline bool blank_or_comment(const char *s, const char *le)
{
    s = skip_ws(s, le);
    return s == le || *s == '%';
}
inline bool parse_i64(const char *&s, const char *e, int64_t &v)
{
    s = skip_ws(s, e);
    if (s < e && *s == '+') ++s;
    auto r = std::from_chars(s, e, v);
    if (r.ec != std::errc()) return false;
    s = r.ptr;
    return true;
}
inline bool parse_f32(const char *&s, const char *e, float &v)
{
    s = skip_ws(s, e);
    if (s < e && *s == '+') ++s;
    double d;
    auto r = std::from_chars(s, e, d);
    if (r.ec != std::errc()) return false;
    s = r.ptr;
    v = (float)d;
    return true;
}

struct BinHeader {
    char magic[8];  // "SDDMMBIN"
    int64_t n_rows, n_cols, nnz;
    int32_t sorted, reserved;
};

}  // namespace

extern "C" int sddmm_read_mtx(const char *path, sddmm_coo **out)
{
    if (!path || !out) return fail(SDDMM_ERR_ARG, "sddmm_read_mtx: NULL argument");
    *out = nullptr;
    Mapped m;
    m.fd = open(path, O_RDONLY);
    if (m.fd < 0) return fail(SDDMM_ERR_IO, "sddmm_read_mtx: cannot open '%s'", path);
    struct stat st;
    if (fstat(m.fd, &st) != 0) return fail(SDDMM_ERR_IO, "sddmm_read_mtx: cannot stat '%s'", path);
    m.n = (size_t)st.st_size;
    if (m.n == 0) return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: '%s' is empty", path);
    m.p = (const char *)mmap(nullptr, m.n, PROT_READ, MAP_PRIVATE, m.fd, 0);
    if (m.p == MAP_FAILED) {
        m.p = nullptr;
        return fail(SDDMM_ERR_IO, "sddmm_read_mtx: cannot map '%s'", path);
    }
    const char *s = m.p, *e = m.p + m.n;

    bool pattern = false, symmetric = false;
    if (m.n >= 2 && s[0] == '%' && s[1] == '%') {  // banner
        const char *le = line_end(s, e);
        std::string b(s, le);
        for (auto &c : b) c = (char)tolower((unsigned char)c);
        if (b.find("matrixmarket") == std::string::npos || b.find("matrix") == std::string::npos)
            return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: unrecognised banner in '%s'", path);
        if (b.find("coordinate") == std::string::npos)
            return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: only the coordinate format is supported ('%s')", path);
        if (b.find("complex") != std::string::npos)
            return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: complex matrices are not supported ('%s')", path);
        pattern = b.find("pattern") != std::string::npos;
        symmetric = b.find("symmetric") != std::string::npos;  // also skew-/hermitian are rejected below
        if (b.find("skew") != std::string::npos || b.find("hermitian") != std::string::npos)
            return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: skew-symmetric / hermitian not supported ('%s')", path);
        s = le < e ? le + 1 : e;
    }
    // comments, then the size line
    int64_t n_rows = 0, n_cols = 0, nnz = 0;
    for (;;) {
        if (s >= e) return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: no size line in '%s'", path);
        const char *le = line_end(s, e);
        if (blank_or_comment(s, le)) {
            s = le < e ? le + 1 : e;
            continue;
        }
        const char *q = s;
        if (!parse_i64(q, le, n_rows) || !parse_i64(q, le, n_cols) || !parse_i64(q, le, nnz))
            return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: bad size line in '%s'", path);
        s = le < e ? le + 1 : e;
        break;
    }
    if (n_rows < 0 || n_cols < 0 || nnz < 0) return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: negative size in '%s'", path);
    if (n_rows >= INT32_MAX || n_cols >= INT32_MAX || nnz * (symmetric ? 2 : 1) >= INT32_MAX)
        return fail(SDDMM_ERR_RANGE, "sddmm_read_mtx: sizes beyond int32 offsets in '%s'", path);

    sddmm_coo *S = new (std::nothrow) sddmm_coo;
    if (!S) return fail(SDDMM_ERR_NOMEM, "sddmm_read_mtx: out of memory");
    try {
        S->n_rows = n_rows; S->n_cols = n_cols; S->nnz = nnz;
        S->rows.resize((size_t)nnz); S->cols.resize((size_t)nnz); S->vals.resize((size_t)nnz);
    } catch (const std::exception &) {
        delete S;
        return fail(SDDMM_ERR_NOMEM, "sddmm_read_mtx: out of memory for %lld nonzeros", (long long)nnz);
    }

    // chunk the body at line boundaries; pass 1 counts entry lines, pass 2 parses
    const char *body = s;
    const int64_t body_len = e - body;
    int nt = (int)std::max<int64_t>(1, std::min<int64_t>(hw_threads(), body_len / (1 << 20) + 1));
    std::vector<const char *> cb((size_t)nt + 1);
    cb[0] = body; cb[nt] = e;
    for (int t = 1; t < nt; ++t) {
        const char *q = body + body_len * t / nt;
        q = line_end(q, e);
        cb[t] = q < e ? q + 1 : e;
    }
    for (int t = 1; t <= nt; ++t) if (cb[t] < cb[t - 1]) cb[t] = cb[t - 1];
    std::vector<int64_t> cnt((size_t)nt + 1, 0);
    auto over_chunks = [&](const std::function<void(int)> &f) {  // f(chunk) on one thread per chunk
        try {
            parallel_ranges(nt, 1, [&](int64_t b, int64_t e2, int) { for (int64_t t = b; t < e2; ++t) f((int)t); });
            return true;
        } catch (const std::exception &) {
            return false;
        }
    };
    if (!over_chunks([&](int t) {
            int64_t c = 0;
            for (const char *q = cb[t]; q < cb[t + 1];) {
                const char *le = line_end(q, cb[t + 1]);
                if (!blank_or_comment(q, le)) ++c;
                q = le + 1;
            }
            cnt[t + 1] = c;
        })) {
        delete S;
        return fail(SDDMM_ERR_NOMEM, "sddmm_read_mtx: out of memory");
    }
    for (int t = 0; t < nt; ++t) cnt[t + 1] += cnt[t];
    if (cnt[nt] < nnz) {
        delete S;
        return fail(SDDMM_ERR_FORMAT, "sddmm_read_mtx: '%s' declares %lld entries but holds %lld", path,
                    (long long)nnz, (long long)cnt[nt]);
    }
    std::vector<int> err((size_t)nt, 0);
    std::vector<int64_t> err_line((size_t)nt, 0);
    if (!over_chunks([&](int t) {
                int64_t i = cnt[t];
                for (const char *q = cb[t]; q < cb[t + 1] && i < nnz;) {
                    const char *le = line_end(q, cb[t + 1]);
                    if (!blank_or_comment(q, le)) {
                        int64_t r, c;
                        float v = 1.0f;
                        const char *z = q;
                        bool ok = parse_i64(z, le, r) && parse_i64(z, le, c) && (pattern || parse_f32(z, le, v));
                        if (!ok) { err[t] = SDDMM_ERR_FORMAT; err_line[t] = i; return; }
                        if (r < 1 || r > n_rows || c < 1 || c > n_cols) { err[t] = SDDMM_ERR_RANGE; err_line[t] = i; return; }
                        S->rows[i] = (int32_t)(r - 1);
                        S->cols[i] = (int32_t)(c - 1);
                        S->vals[i] = v;
                        ++i;
                    }
                    q = le + 1;
                }
        })) {
        delete S;
        return fail(SDDMM_ERR_NOMEM, "sddmm_read_mtx: out of memory");
    }
    for (int t = 0; t < nt; ++t)
        if (err[t]) {
            int code = err[t];
            long long at = (long long)err_line[t];
            delete S;
            return fail(code, code == SDDMM_ERR_RANGE ? "sddmm_read_mtx: entry %lld of '%s' lies outside the matrix"
                                                      : "sddmm_read_mtx: cannot parse entry %lld of '%s'", at, path);
        }
    if (symmetric) {  // mirror the off-diagonal entries
        int64_t extra = 0;
        for (int64_t i = 0; i < nnz; ++i) extra += S->rows[i] != S->cols[i];
        try {
            S->rows.reserve((size_t)(nnz + extra)); S->cols.reserve((size_t)(nnz + extra)); S->vals.reserve((size_t)(nnz + extra));
        } catch (const std::exception &) {
            delete S;
            return fail(SDDMM_ERR_NOMEM, "sddmm_read_mtx: out of memory");
        }
        for (int64_t i = 0; i < nnz; ++i)
            if (S->rows[i] != S->cols[i]) {
                S->rows.push_back(S->cols[i]); S->cols.push_back(S->rows[i]); S->vals.push_back(S->vals[i]);
            }
        S->nnz = nnz + extra;
    }
    try {
        S->sorted = check_sorted(*S) ? 1 : 0;
    } catch (const std::exception &) {
        delete S;
        return fail(SDDMM_ERR_NOMEM, "out of memory while checking the order of '%s'", path);
    }
    *out = S;
    return SDDMM_OK;
}

extern "C" int sddmm_write_mtx(const sddmm_coo *S, const char *path)
{
    if (!S || !path) return fail(SDDMM_ERR_ARG, "sddmm_write_mtx: NULL argument");
    FILE *f = fopen(path, "w");
    if (!f) return fail(SDDMM_ERR_IO, "sddmm_write_mtx: cannot open '%s'", path);
    std::vector<char> buf(1 << 22);
    setvbuf(f, buf.data(), _IOFBF, buf.size());
    fprintf(f, "%%%%MatrixMarket matrix coordinate real general\n%lld %lld %lld\n", (long long)S->n_rows,
            (long long)S->n_cols, (long long)S->nnz);
    for (int64_t i = 0; i < S->nnz; ++i) fprintf(f, "%d %d %.9g\n", S->rows[i] + 1, S->cols[i] + 1, (double)S->vals[i]);
    bool bad = ferror(f) != 0;
    bad |= fclose(f) != 0;
    return bad ? fail(SDDMM_ERR_IO, "sddmm_write_mtx: write to '%s' failed", path) : SDDMM_OK;
}

extern "C" int sddmm_write_bin(const sddmm_coo *S, const char *path)
{
    if (!S || !path) return fail(SDDMM_ERR_ARG, "sddmm_write_bin: NULL argument");
    FILE *f = fopen(path, "wb");
    if (!f) return fail(SDDMM_ERR_IO, "sddmm_write_bin: cannot open '%s'", path);
    BinHeader h;
    memcpy(h.magic, "SDDMMBIN", 8);
    h.n_rows = S->n_rows; h.n_cols = S->n_cols; h.nnz = S->nnz; h.sorted = S->sorted; h.reserved = 0;
    size_t n = (size_t)S->nnz;
    bool ok = fwrite(&h, sizeof h, 1, f) == 1 && (n == 0 || (fwrite(S->rows.data(), 4, n, f) == n &&
              fwrite(S->cols.data(), 4, n, f) == n && fwrite(S->vals.data(), 4, n, f) == n));
    ok &= fclose(f) == 0;
    return ok ? SDDMM_OK : fail(SDDMM_ERR_IO, "sddmm_write_bin: write to '%s' failed", path);
}

extern "C" int sddmm_read_bin(const char *path, sddmm_coo **out)
{
    if (!path || !out) return fail(SDDMM_ERR_ARG, "sddmm_read_bin: NULL argument");
    *out = nullptr;
    FILE *f = fopen(path, "rb");
    if (!f) return fail(SDDMM_ERR_IO, "sddmm_read_bin: cannot open '%s'", path);
    BinHeader h;
    if (fread(&h, sizeof h, 1, f) != 1 || memcmp(h.magic, "SDDMMBIN", 8) != 0 || h.nnz < 0 || h.n_rows < 0 ||
        h.n_cols < 0 || h.nnz >= INT32_MAX || h.n_rows >= INT32_MAX || h.n_cols >= INT32_MAX) {
        fclose(f);
        return fail(SDDMM_ERR_FORMAT, "sddmm_read_bin: '%s' is not an SDDMM binary matrix", path);
    }
    sddmm_coo *S = new (std::nothrow) sddmm_coo;
    if (!S) { fclose(f); return fail(SDDMM_ERR_NOMEM, "sddmm_read_bin: out of memory"); }
    size_t n = (size_t)h.nnz;
    try {
        S->rows.resize(n); S->cols.resize(n); S->vals.resize(n);
    } catch (const std::exception &) {
        delete S; fclose(f);
        return fail(SDDMM_ERR_NOMEM, "sddmm_read_bin: out of memory");
    }
    bool ok = n == 0 || (fread(S->rows.data(), 4, n, f) == n && fread(S->cols.data(), 4, n, f) == n &&
                         fread(S->vals.data(), 4, n, f) == n);
    fclose(f);
    if (!ok) { delete S; return fail(SDDMM_ERR_FORMAT, "sddmm_read_bin: '%s' is truncated", path); }
    S->n_rows = h.n_rows; S->n_cols = h.n_cols; S->nnz = h.nnz;
    for (size_t i = 0; i < n; ++i)
        if (S->rows[i] < 0 || S->rows[i] >= h.n_rows || S->cols[i] < 0 || S->cols[i] >= h.n_cols) {
            delete S;
            return fail(SDDMM_ERR_RANGE, "sddmm_read_bin: entry %zu of '%s' lies outside the matrix", i, path);
        }
    try {
        S->sorted = check_sorted(*S) ? 1 : 0;
    } catch (const std::exception &) {
        delete S;
        return fail(SDDMM_ERR_NOMEM, "out of memory while checking the order of '%s'", path);
    }
    *out = S;
    return SDDMM_OK;
}
