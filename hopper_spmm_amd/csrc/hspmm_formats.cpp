// Host-side format functions of the C ABI (include/hspmm.h): MatrixMarket
// loading and the CSR -> condensed-tile conversions.  They produce the same arrays
// as the reference's load_matrix (reference src/utils/load.h:152-322),
// CSR2BTCFNOBITMAP (src/utils/convert.h:146-225), CSR2BTCF (convert.h:22-139) and
// BTCF2GBTCF (convert.h:232-276), built differently: whole-file parsing with
// strtoul/strtof, a counting sort by row, and two-pass, multi-threaded window
// conversions without hash maps or growing vectors.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../include/hspmm.h"
#include "host_parallel.hpp"

namespace hspmm_host {

// Stores the text hspmm_last_error() returns on this thread (defined beside it).
void set_error(const std::string &msg);

// IEEE binary32 -> binary16, round to nearest even (what __float2half does on
// the host, reference src/utils/load.h:226).
static uint16_t float_to_half_bits(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7FFFFFFFu;
    if (x > 0x7F800000u) return uint16_t(sign | 0x7E00u | ((x >> 13) & 0x1FFu));   // NaN (quiet)
    if (x >= 0x477FF000u) return uint16_t(sign | 0x7C00u);                         // overflow -> inf
    if (x >= 0x38800000u) {                                                        // normal half
        const uint32_t mant = x & 0x1FFFu;                                         // 13 dropped bits
        uint32_t h = (x - 0x38000000u) >> 13;                                      // rebias 127 -> 15
        if (mant > 0x1000u || (mant == 0x1000u && (h & 1u))) ++h;
        return uint16_t(sign | h);
    }
    if (x < 0x33000001u) return uint16_t(sign);                                    // underflow -> 0
    // subnormal half: value = m * 2^(e-150) with 24-bit m; unit of the result is 2^-24
    const int e = int(x >> 23);
    const uint32_t m = (x & 0x7FFFFFu) | 0x800000u;
    const int shift = 126 - e;                                                     // 14..24
    uint32_t h = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1u))) ++h;
    return uint16_t(sign | h);
}

// IEEE binary32 -> bfloat16, round to nearest even (the implicit float ->
// __nv_bfloat16 conversion of the reference's bf16 build, src/utils/load.h:224).
static uint16_t float_to_bf16_bits(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return uint16_t((x >> 16) | 0x0040u);    // NaN stays NaN (quiet)
    return uint16_t((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}

// ---------------------------------------------------------------------------
// Text parsing.  A data line counts when sscanf(line, "%u %u %f") == 3
// (reference src/utils/load.h:219); the functions below give the same values
// for the text between `p` and `end` without copying the line.
// ---------------------------------------------------------------------------
static inline bool is_space(char ch)
{
    return ch == ' ' || ch == '\t' || ch == '\n' || ch == '\v' || ch == '\f' || ch == '\r';
}

// %u: white space, an optional sign, decimal digits.  Values beyond 64 bits
// saturate as strtoul does; the result is then cut to 32 bits.
static inline bool parse_u32(const char *&p, const char *end, uint32_t &out)
{
    while (p < end && is_space(*p)) ++p;
    bool neg = false;
    if (p < end && (*p == '+' || *p == '-')) { neg = *p == '-'; ++p; }
    if (p >= end || *p < '0' || *p > '9') return false;
    uint64_t v = 0;
    bool over = false;
    while (p < end && *p >= '0' && *p <= '9') {
        const uint64_t d = uint64_t(*p - '0');
        if (v > (UINT64_MAX - d) / 10u) over = true; else v = v * 10u + d;
        ++p;
    }
    if (over) v = UINT64_MAX;
    else if (neg) v = 0u - v;
    out = uint32_t(v);
    return true;
}

// strtof on a copy: every form that the quick path below leaves alone (inf, nan,
// hexadecimal, more than 19 digits, exponents beyond +-22, results near the ends
// of the float range).
static bool parse_float_slow(const char *start, const char *end, float &out)
{
    char buf[1024];
    size_t n = size_t(end - start);
    if (n > sizeof buf - 1) n = sizeof buf - 1;
    std::memcpy(buf, start, n);
    buf[n] = 0;
    char *stop;
    const float f = std::strtof(buf, &stop);
    if (stop == buf) return false;
    out = f;
    return true;
}

// %f.  Quick path: a decimal significand m < 2^53 and a power of ten up to
// 10^22 are both exact doubles, so m * 10^e (or m / 10^-e) is the correctly
// rounded double of the decimal value.  Rounding that double to float gives the
// correctly rounded float unless the double sits exactly half way between two
// floats (then the digits that were rounded away decide, and strtof is asked).
static bool parse_float(const char *p, const char *end, float &out)
{
    static const double p10[23] = {1e0, 1e1, 1e2, 1e3, 1e4, 1e5, 1e6, 1e7, 1e8, 1e9, 1e10, 1e11,
                                   1e12, 1e13, 1e14, 1e15, 1e16, 1e17, 1e18, 1e19, 1e20, 1e21, 1e22};
    while (p < end && is_space(*p)) ++p;
    const char *start = p;
    bool neg = false;
    if (p < end && (*p == '+' || *p == '-')) { neg = *p == '-'; ++p; }
    if (p + 1 < end && p[0] == '0' && (p[1] == 'x' || p[1] == 'X')) return parse_float_slow(start, end, out);
    uint64_t m = 0;
    int e10 = 0, ndig = 0;
    bool any = false;
    while (p < end && *p >= '0' && *p <= '9') {
        any = true;
        if (m || *p != '0') { if (++ndig > 19) return parse_float_slow(start, end, out); m = m * 10u + uint64_t(*p - '0'); }
        ++p;
    }
    if (p < end && *p == '.') {
        ++p;
        while (p < end && *p >= '0' && *p <= '9') {
            any = true;
            if (m || *p != '0') { if (++ndig > 19) return parse_float_slow(start, end, out); m = m * 10u + uint64_t(*p - '0'); }
            --e10;
            ++p;
        }
    }
    if (!any) return parse_float_slow(start, end, out);          // inf, nan, or nothing
    if (p < end && (*p == 'e' || *p == 'E')) {
        const char *q = p + 1;
        bool eneg = false;
        if (q < end && (*q == '+' || *q == '-')) { eneg = *q == '-'; ++q; }
        if (q < end && *q >= '0' && *q <= '9') {
            int ev = 0;
            while (q < end && *q >= '0' && *q <= '9') { if (ev < 100000) ev = ev * 10 + (*q - '0'); ++q; }
            e10 += eneg ? -ev : ev;
        }
    }
    if (m == 0) { out = neg ? -0.0f : 0.0f; return true; }
    if (m >= (uint64_t(1) << 53) || e10 < -22 || e10 > 22) return parse_float_slow(start, end, out);
    double d = double(m);
    d = e10 < 0 ? d / p10[-e10] : d * p10[e10];
    if (!(d > 1e-30 && d < 1e30)) return parse_float_slow(start, end, out);
    uint64_t bits;
    std::memcpy(&bits, &d, 8);
    if ((bits & 0x1FFFFFFFull) == 0x10000000ull) return parse_float_slow(start, end, out);
    out = float(neg ? -d : d);
    return true;
}

struct Triples {
    uint32_t rows = 0, cols = 0, declared = 0;
    std::vector<uint32_t> r, c;
    std::vector<float> v;
};

// The whole file, read-only, through mmap (or read() where mapping fails).
struct FileText {
    const char *data = nullptr;
    size_t size = 0;
    bool mapped = false;
    std::string owned;
    ~FileText() { if (mapped) munmap(const_cast<char *>(data), size); }
    bool open(const char *path)
    {
        const int fd = ::open(path, O_RDONLY);
        if (fd < 0) return false;
        struct stat st;
        if (fstat(fd, &st) == 0 && S_ISREG(st.st_mode) && st.st_size > 0) {
            void *m = mmap(nullptr, size_t(st.st_size), PROT_READ, MAP_PRIVATE, fd, 0);
            if (m != MAP_FAILED) { data = static_cast<const char *>(m); size = size_t(st.st_size); mapped = true; }
        }
        if (!mapped) {
            char buf[1 << 16];
            ssize_t n;
            while ((n = ::read(fd, buf, sizeof buf)) > 0) owned.append(buf, size_t(n));
            data = owned.data(); size = owned.size();
        }
        ::close(fd);
        return true;
    }
};

// The reference reads with fgets into a 1024-byte buffer (src/utils/load.h:155,
// 183, 215): a "line" is a piece of at most 1023 characters that ends after a
// newline, and sscanf stops at a NUL byte.  [pos, return value) is the next piece.
static inline size_t piece_end(const char *txt, size_t pos, size_t size)
{
    const size_t limit = std::min(size, pos + 1023);
    const void *nl = std::memchr(txt + pos, '\n', limit - pos);
    return nl ? size_t(static_cast<const char *>(nl) - txt) + 1 : limit;
}

static inline bool parse_piece(const char *b, const char *e, uint32_t &r, uint32_t &c, float &v)
{
    if (const void *nul = std::memchr(b, 0, size_t(e - b))) e = static_cast<const char *>(nul);
    const char *p = b;
    return parse_u32(p, e, r) && parse_u32(p, e, c) && parse_float(p, e, v);
}

// Header and size line on one thread, then the data lines in blocks that start
// after a newline (every such position starts a piece), one block per worker.
static int read_triples(const char *path, Triples &t, std::string &err)
{
    FileText f;
    if (!f.open(path)) { err = std::string("cannot open file ") + path; return HSPMM_ERR_IO; }
    const char *txt = f.data;
    const size_t size = f.size;
    size_t pos = 0, line_b = 0, line_e = 0;
    bool have = false;
    while (pos < size) {                                                // load.h:183-187
        line_b = pos; line_e = piece_end(txt, pos, size); pos = line_e;
        have = true;
        if (txt[line_b] != '%') break;
    }
    unsigned rows = 0, cols = 0, nnz = 0;
    {
        std::string line(have ? txt + line_b : "", have ? line_e - line_b : 0);
        if (!have || std::sscanf(line.c_str(), "%u %u %u", &rows, &cols, &nnz) != 3) {   // load.h:190
            err = std::string("cannot parse the size line of ") + path;
            return HSPMM_ERR_IO;
        }
    }
    t.rows = rows; t.cols = cols; t.declared = nnz;
    const size_t body = pos;
    const unsigned nw = worker_count(size - body, size_t(1) << 20);
    std::vector<size_t> cut(nw + 1, size);
    cut[0] = body;
    for (unsigned i = 1; i < nw; ++i) {
        size_t want = body + (size - body) / nw * i;
        if (want < cut[i - 1]) want = cut[i - 1];
        const void *nl = want < size ? std::memchr(txt + want, '\n', size - want) : nullptr;
        cut[i] = nl ? size_t(static_cast<const char *>(nl) - txt) + 1 : size;
    }
    std::vector<Triples> part(nw);
    auto work = [&](unsigned wi) {
        Triples &o = part[wi];
        const size_t b = cut[wi], e = cut[wi + 1];
        const size_t guess = (e - b) / 12 + 16;
        o.r.reserve(guess); o.c.reserve(guess); o.v.reserve(guess);
        for (size_t p = b; p < e;) {
            const size_t pe = piece_end(txt, p, e);
            uint32_t r, c; float v;
            if (parse_piece(txt + p, txt + pe, r, c, v)) {
                o.r.push_back(r - 1u); o.c.push_back(c - 1u); o.v.push_back(v);   // load.h:221-222
            }
            p = pe;
        }
    };
    if (nw <= 1) work(0);
    else {
        std::vector<std::thread> th;
        for (unsigned i = 0; i < nw; ++i) th.emplace_back(work, i);
        for (auto &x : th) x.join();
    }
    // the reference stops reading once the declared number of entries is there (load.h:215)
    size_t total = 0;
    for (const Triples &o : part) total += o.r.size();
    if (total > nnz) total = nnz;
    t.r.resize(total); t.c.resize(total); t.v.resize(total);
    size_t at = 0;
    for (const Triples &o : part) {
        const size_t n = std::min(o.r.size(), total - at);
        std::memcpy(t.r.data() + at, o.r.data(), n * 4);
        std::memcpy(t.c.data() + at, o.c.data(), n * 4);
        std::memcpy(t.v.data() + at, o.v.data(), n * 4);
        at += n;
        if (at == total) break;
    }
    return HSPMM_OK;
}

}  // namespace hspmm_host

using namespace hspmm_host;

extern "C" {

int hspmm_mtx_load(const char *path, int dtype, hspmm_csr *out)
{
    if (!path || !out) { set_error("null argument"); return HSPMM_ERR_INVALID; }
    std::memset(out, 0, sizeof *out);
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16) { set_error("unknown dtype"); return HSPMM_ERR_INVALID; }
    Triples t;
    std::string err;
    int rc = read_triples(path, t, err);
    if (rc) { set_error(err); return rc; }
    const size_t nnz = t.r.size();
    if (nnz != t.declared)                                              // load.h:234-238
        std::fprintf(stderr, "warning: %s declares %u entries, %zu were read\n", path, t.declared, nnz);
    for (size_t i = 0; i < nnz; ++i)
        if (t.r[i] >= t.rows || t.c[i] >= t.cols) {
            set_error("entry " + std::to_string(i) + " of " + path + " lies outside the declared shape");
            return HSPMM_ERR_IO;
        }
    const size_t es = dtype == HSPMM_TF32 ? 4 : 2;
    uint32_t *row_ptr = static_cast<uint32_t *>(std::calloc(size_t(t.rows) + 1, 4));
    uint32_t *col_idx = static_cast<uint32_t *>(std::malloc((nnz ? nnz : 1) * 4));
    void *values = std::malloc((nnz ? nnz : 1) * es);
    if (!row_ptr || !col_idx || !values) {
        std::free(row_ptr); std::free(col_idx); std::free(values);
        set_error("out of host memory");
        return HSPMM_ERR_ALLOC;
    }
    // counting sort by row (stable), then a stable sort by column inside each row:
    // the (row, column) order of load.h:137-145, with file order kept for equal keys
    for (size_t i = 0; i < nnz; ++i) row_ptr[t.r[i] + 1]++;
    for (uint32_t r = 0; r < t.rows; ++r) row_ptr[r + 1] += row_ptr[r];
    std::vector<uint32_t> order(nnz), cursor(row_ptr, row_ptr + t.rows);
    for (size_t i = 0; i < nnz; ++i) order[cursor[t.r[i]]++] = uint32_t(i);
    parallel_chunks(t.rows, 4096, [&](size_t rb, size_t re) {
        for (size_t r = rb; r < re; ++r)
            std::stable_sort(order.begin() + row_ptr[r], order.begin() + row_ptr[r + 1],
                             [&](uint32_t a, uint32_t b) { return t.c[a] < t.c[b]; });
    });
    parallel_blocks(nnz, size_t(1) << 16, [&](size_t ib, size_t ie) {
        for (size_t i = ib; i < ie; ++i) {
            const uint32_t s = order[i];
            col_idx[i] = t.c[s];
            if (dtype == HSPMM_FP16) static_cast<uint16_t *>(values)[i] = float_to_half_bits(t.v[s]);
            else if (dtype == HSPMM_BF16) static_cast<uint16_t *>(values)[i] = float_to_bf16_bits(t.v[s]);
            else static_cast<float *>(values)[i] = t.v[s];
        }
    });
    out->rows = t.rows; out->cols = t.cols; out->nnzs = uint32_t(nnz);
    out->row_ptr = row_ptr; out->col_idx = col_idx; out->values = values;
    return HSPMM_OK;
}

void hspmm_csr_free(hspmm_csr *m)
{
    if (!m) return;
    std::free(m->row_ptr); std::free(m->col_idx); std::free(m->values);
    std::memset(m, 0, sizeof *m);
}

}  // extern "C"

namespace hspmm_host {

// Distinct sorted column ids of rows [r0, r1) into `uniq`; returns their number.
static uint32_t window_columns(const uint32_t *row_ptr, const uint32_t *col_idx, uint32_t r0, uint32_t r1,
                               std::vector<uint32_t> &uniq)
{
    const uint32_t b = row_ptr[r0], e = row_ptr[r1];
    uniq.assign(col_idx + b, col_idx + e);
    std::sort(uniq.begin(), uniq.end());
    uniq.erase(std::unique(uniq.begin(), uniq.end()), uniq.end());
    return uint32_t(uniq.size());
}

// Windows a worker takes at a time: what holds about 64 K stored entries (a matrix of few wide
// windows, like block-clustered weights, still spreads over the cores).
static size_t windows_per_worker(size_t nwin, size_t nnz)
{
    if (nnz == 0 || nwin == 0) return 2048;
    const size_t per_window = (nnz + nwin - 1) / nwin;
    return std::max<size_t>(1, std::min<size_t>(2048, (size_t(1) << 16) / std::max<size_t>(1, per_window)));
}

// tiles[w] = number of tiles of window w (0 for a window without entries).
static void count_tiles(uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx, uint32_t cw,
                        std::vector<uint32_t> &tiles)
{
    const size_t nwin = (size_t(rows) + HSPMM_ROW_WINDOW - 1) / HSPMM_ROW_WINDOW;
    tiles.assign(nwin, 0u);
    parallel_chunks(nwin, windows_per_worker(nwin, row_ptr[rows]), [&](size_t wb, size_t we) {
        std::vector<uint32_t> uniq;
        for (size_t w = wb; w < we; ++w) {
            const uint32_t r0 = uint32_t(w * HSPMM_ROW_WINDOW);
            const uint32_t r1 = std::min<uint64_t>(uint64_t(r0) + HSPMM_ROW_WINDOW, rows);
            if (row_ptr[r1] == row_ptr[r0]) continue;                       // convert.h:162
            const uint32_t u = window_columns(row_ptr, col_idx, r0, r1, uniq);
            tiles[w] = (u + cw - 1) / cw;                                   // convert.h:178-185
        }
    });
}

}  // namespace hspmm_host

extern "C" {

// Tile width for an element type: the default (16 for the 16-bit types, 8 for fp32 storage) or, for fp32
// storage, the 4 of the reference's -DMMA_M16N8K4 build (src/common.h:28-35).  0 on a bad request.
static uint32_t tile_width(int dtype, uint32_t col_window)
{
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16) { set_error("unknown dtype"); return 0; }
    const uint32_t dflt = dtype == HSPMM_TF32 ? 8u : 16u;
    if (col_window == 0 || col_window == dflt) return dflt;
    if (dtype == HSPMM_TF32 && col_window == 4u) return 4u;
    set_error("col_window: the element type's default (16 / 8), or 4 for HSPMM_TF32");
    return 0;
}

int hspmm_btcf_sizes_cw(int dtype, uint32_t col_window, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                        uint32_t *eff_row_windows, uint32_t *total_tiles)
{
    const uint32_t cw = tile_width(dtype, col_window);
    if (!cw) return HSPMM_ERR_INVALID;
    if (!row_ptr || !eff_row_windows || !total_tiles || (!col_idx && row_ptr[rows])) {
        set_error("null argument");
        return HSPMM_ERR_INVALID;
    }
    std::vector<uint32_t> tiles;
    count_tiles(rows, row_ptr, col_idx, cw, tiles);
    uint64_t W = 0, T = 0;
    for (uint32_t t : tiles) { W += t != 0; T += t; }
    if (T > 0xFFFFFFFFull) { set_error("tile count exceeds 32 bits"); return HSPMM_ERR_UNSUPPORTED; }
    *eff_row_windows = uint32_t(W);
    *total_tiles = uint32_t(T);
    return HSPMM_OK;
}

int hspmm_btcf_sizes(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                     uint32_t *eff_row_windows, uint32_t *total_tiles)
{
    return hspmm_btcf_sizes_cw(dtype, 0, rows, row_ptr, col_idx, eff_row_windows, total_tiles);
}

int hspmm_btcf_fill(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                    const void *values, int transpose, uint32_t *rowOffset, uint32_t *tcA2B, void *data,
                    uint32_t *rowIdx)
{
    return hspmm_btcf_fill_cw(dtype, 0, rows, row_ptr, col_idx, values, transpose, rowOffset, tcA2B, data, rowIdx);
}

int hspmm_btcf_fill_cw(int dtype, uint32_t col_window, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                       const void *values, int transpose, uint32_t *rowOffset, uint32_t *tcA2B, void *data,
                       uint32_t *rowIdx)
{
    const uint32_t cw = tile_width(dtype, col_window);
    if (!cw) return HSPMM_ERR_INVALID;
    if (!row_ptr || !rowOffset) { set_error("null argument"); return HSPMM_ERR_INVALID; }
    const size_t es = dtype == HSPMM_TF32 ? 4 : 2;
    const size_t tile_elems = size_t(HSPMM_ROW_WINDOW) * cw;
    std::vector<uint32_t> tiles;
    count_tiles(rows, row_ptr, col_idx, cw, tiles);
    const size_t nwin = tiles.size();
    // exclusive scans: effective-window index and first tile of every window
    std::vector<uint32_t> eff_index(nwin + 1, 0u), first_tile(nwin + 1, 0u);
    for (size_t w = 0; w < nwin; ++w) {
        eff_index[w + 1] = eff_index[w] + (tiles[w] != 0);
        first_tile[w + 1] = first_tile[w] + tiles[w];
    }
    rowOffset[0] = 0;                                                        // convert.h:152
    if (first_tile[nwin] && (!tcA2B || !data || !rowIdx || !col_idx || !values)) {
        set_error("null argument");
        return HSPMM_ERR_INVALID;
    }
    parallel_chunks(nwin, windows_per_worker(nwin, row_ptr[rows]), [&](size_t wb, size_t we) {
        std::vector<uint32_t> uniq;
        for (size_t w = wb; w < we; ++w) {
            if (!tiles[w]) continue;
            const uint32_t r0 = uint32_t(w * HSPMM_ROW_WINDOW);
            const uint32_t r1 = std::min<uint64_t>(uint64_t(r0) + HSPMM_ROW_WINDOW, rows);
            const uint32_t u = window_columns(row_ptr, col_idx, r0, r1, uniq);
            const uint32_t ew = eff_index[w], ft = first_tile[w], nt = tiles[w];
            rowOffset[ew + 1] = ft + nt;                                     // convert.h:186
            rowIdx[ew] = r0;                                                 // convert.h:187
            uint32_t *ids = tcA2B + size_t(ft) * cw;
            for (uint32_t i = 0; i < nt * cw; ++i) ids[i] = i < u ? uniq[i] : HSPMM_IDX_MAX;   // convert.h:178-184
            unsigned char *win = static_cast<unsigned char *>(data) + size_t(ft) * tile_elems * es;
            std::memset(win, 0, size_t(nt) * tile_elems * es);               // convert.h:191-193
            for (uint32_t r = r0; r < r1; ++r)
                for (uint32_t id = row_ptr[r]; id < row_ptr[r + 1]; ++id) {  // stored order: a later duplicate wins
                    const uint32_t rank = uint32_t(std::lower_bound(uniq.begin(), uniq.end(), col_idx[id]) - uniq.begin());
                    const uint32_t tc = rank / cw, lc = rank % cw, lr = r % HSPMM_ROW_WINDOW;
                    const size_t off = transpose ? size_t(lc) * HSPMM_ROW_WINDOW + lr       // convert.h:209
                                                 : size_t(lr) * cw + lc;                    // convert.h:212
                    std::memcpy(win + (size_t(tc) * tile_elems + off) * es,
                                static_cast<const unsigned char *>(values) + size_t(id) * es, es);
                }
        }
    });
    return HSPMM_OK;
}

}  // extern "C"

// ---------------------------------------------------------------------------
// Bitmap-compressed tiles (reference CSR2BTCF, src/utils/convert.h:22-139)
// ---------------------------------------------------------------------------
extern "C" {

int hspmm_bitmap_sizes(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                       uint32_t *eff_row_windows, uint32_t *total_tiles, uint32_t *stored)
{
    const int rc = hspmm_btcf_sizes(dtype, rows, row_ptr, col_idx, eff_row_windows, total_tiles);
    if (rc) return rc;
    if (stored) *stored = row_ptr[rows];      // every CSR entry is stored (convert.h:114-119)
    return HSPMM_OK;
}

int hspmm_bitmap_fill(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                      const void *values, int transpose, int bit_layout,
                      uint32_t *rowOffset, uint32_t *nnzOffset, uint32_t *tcA2B, uint64_t *tcBit,
                      void *data, uint32_t *rowIdx)
{
    using namespace hspmm_host;
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16) { set_error("unknown dtype"); return HSPMM_ERR_INVALID; }
    if (bit_layout != HSPMM_BITS_PER_TILE && bit_layout != HSPMM_BITS_AS_REFERENCE) {
        set_error("unknown bit layout");
        return HSPMM_ERR_INVALID;
    }
    if (!row_ptr || !rowOffset || !nnzOffset) { set_error("null argument"); return HSPMM_ERR_INVALID; }
    const uint32_t cw = dtype == HSPMM_TF32 ? 8u : 16u;
    const uint32_t wpt = HSPMM_BITMAP_WORDS(dtype);
    const size_t es = dtype == HSPMM_TF32 ? 4 : 2;
    std::vector<uint32_t> tiles;
    count_tiles(rows, row_ptr, col_idx, cw, tiles);
    const size_t nwin = tiles.size();
    std::vector<uint32_t> eff_index(nwin + 1, 0u), first_tile(nwin + 1, 0u);
    for (size_t w = 0; w < nwin; ++w) {
        eff_index[w + 1] = eff_index[w] + (tiles[w] != 0);
        first_tile[w + 1] = first_tile[w] + tiles[w];
    }
    const uint32_t T = first_tile[nwin];
    rowOffset[0] = 0;                                                        // convert.h:29
    nnzOffset[0] = 0;                                                        // convert.h:136
    if (T && (!tcA2B || !tcBit || !data || !rowIdx || !col_idx || !values)) {
        set_error("null argument");
        return HSPMM_ERR_INVALID;
    }
    if (T) std::memset(tcBit, 0, size_t(T) * wpt * 8);                       // convert.h:67
    // The reference's word index for 8 x 16 tiles lets neighbouring tiles, and so
    // neighbouring windows, share a word: that layout is filled by one thread.
    const bool shared_words = bit_layout == HSPMM_BITS_AS_REFERENCE && wpt == 2;
    auto convert_windows = [&](size_t wb, size_t we) {
        std::vector<uint32_t> uniq, start, cursor;
        for (size_t w = wb; w < we; ++w) {
            if (!tiles[w]) continue;
            const uint32_t r0 = uint32_t(w * HSPMM_ROW_WINDOW);
            const uint32_t r1 = std::min<uint64_t>(uint64_t(r0) + HSPMM_ROW_WINDOW, rows);
            const uint32_t u = window_columns(row_ptr, col_idx, r0, r1, uniq);
            const uint32_t ew = eff_index[w], ft = first_tile[w], nt = tiles[w];
            rowOffset[ew + 1] = ft + nt;                                     // convert.h:58
            rowIdx[ew] = r0;                                                 // convert.h:68
            uint32_t *ids = tcA2B + size_t(ft) * cw;
            for (uint32_t i = 0; i < nt * cw; ++i) ids[i] = i < u ? uniq[i] : HSPMM_IDX_MAX;   // convert.h:50-56
            // Stored entries are grouped by tile, and inside a tile by (row, position in
            // the row) - or by (tile column, row) with `transpose` (convert.h:114-133).  Count
            // per sub-bucket, scan, place.  All entries of earlier windows come first, so
            // the window's part of `data` starts at row_ptr[r0].
            const uint32_t sub = transpose ? cw : 1u;
            start.assign(size_t(nt) * sub + 1, 0u);
            for (uint32_t id = row_ptr[r0]; id < row_ptr[r1]; ++id) {
                const uint32_t rank = uint32_t(std::lower_bound(uniq.begin(), uniq.end(), col_idx[id]) - uniq.begin());
                ++start[size_t(rank / cw) * sub + (transpose ? rank % cw : 0u) + 1];
            }
            for (size_t i = 0; i < size_t(nt) * sub; ++i) start[i + 1] += start[i];
            for (uint32_t t = 0; t < nt; ++t)
                nnzOffset[ft + t + 1] = row_ptr[r0] + start[size_t(t + 1) * sub];             // convert.h:84,135-137
            cursor.assign(start.begin(), start.end() - 1);
            for (uint32_t r = r0; r < r1; ++r)
                for (uint32_t id = row_ptr[r]; id < row_ptr[r + 1]; ++id) {
                    const uint32_t rank = uint32_t(std::lower_bound(uniq.begin(), uniq.end(), col_idx[id]) - uniq.begin());
                    const uint32_t tc = rank / cw, lc = rank % cw, lr = r % HSPMM_ROW_WINDOW;
                    const uint32_t bit = transpose ? lc * HSPMM_ROW_WINDOW + lr              // convert.h:90
                                                   : lr * cw + lc;                           // convert.h:93
                    const size_t word = shared_words ? size_t(ft + tc) + bit / 64u           // convert.h:97-101
                                                     : size_t(ft + tc) * wpt + bit / 64u;
                    tcBit[word] |= uint64_t(1) << (bit % 64u);
                    const uint32_t pos = row_ptr[r0] + cursor[size_t(tc) * sub + (transpose ? lc : 0u)]++;
                    std::memcpy(static_cast<unsigned char *>(data) + size_t(pos) * es,
                                static_cast<const unsigned char *>(values) + size_t(id) * es, es);
                }
        }
    };
    if (shared_words) convert_windows(0, nwin);
    else parallel_chunks(nwin, windows_per_worker(nwin, row_ptr[rows]), convert_windows);
    return HSPMM_OK;
}

int hspmm_bitmap_expand(int dtype, uint32_t total_tiles, const uint32_t *nnzOffset, const uint64_t *tcBit,
                        const void *data, void *dense_tiles)
{
    using namespace hspmm_host;
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16) { set_error("unknown dtype"); return HSPMM_ERR_INVALID; }
    if (total_tiles && (!nnzOffset || !tcBit || !dense_tiles)) { set_error("null argument"); return HSPMM_ERR_INVALID; }
    const uint32_t cw = dtype == HSPMM_TF32 ? 8u : 16u;
    const uint32_t wpt = HSPMM_BITMAP_WORDS(dtype);
    const size_t es = dtype == HSPMM_TF32 ? 4 : 2;
    const size_t tile_bytes = size_t(HSPMM_ROW_WINDOW) * cw * es;
    if (total_tiles && nnzOffset[0] != 0) { set_error("nnzOffset must start at 0"); return HSPMM_ERR_INVALID; }
    if (total_tiles && nnzOffset[total_tiles] && !data) { set_error("null argument"); return HSPMM_ERR_INVALID; }
    // every worker records the first inconsistent tile of its block
    const unsigned nw = worker_count(total_tiles, 1u << 14);
    std::vector<uint32_t> bad_per_block(nw, HSPMM_IDX_MAX);
    uint32_t first_bad = HSPMM_IDX_MAX;
    auto work = [&](unsigned wi) {
        const size_t b = size_t(total_tiles) * wi / nw, e = size_t(total_tiles) * (wi + 1) / nw;
        for (size_t t = b; t < e; ++t) {
            unsigned char *tile = static_cast<unsigned char *>(dense_tiles) + t * tile_bytes;
            std::memset(tile, 0, tile_bytes);
            if (nnzOffset[t + 1] < nnzOffset[t]) { if (bad_per_block[wi] == HSPMM_IDX_MAX) bad_per_block[wi] = uint32_t(t); continue; }
            uint32_t count = 0;
            for (uint32_t k = 0; k < wpt; ++k) count += uint32_t(__builtin_popcountll(tcBit[t * wpt + k]));
            if (count != nnzOffset[t + 1] - nnzOffset[t]) { if (bad_per_block[wi] == HSPMM_IDX_MAX) bad_per_block[wi] = uint32_t(t); continue; }
            size_t src = nnzOffset[t];
            for (uint32_t k = 0; k < wpt; ++k) {
                uint64_t bits = tcBit[t * wpt + k];
                while (bits) {
                    const uint32_t bit = uint32_t(__builtin_ctzll(bits)) + 64u * k;
                    bits &= bits - 1;
                    std::memcpy(tile + size_t(bit) * es, static_cast<const unsigned char *>(data) + src * es, es);
                    ++src;
                }
            }
        }
    };
    if (nw <= 1) work(0);
    else {
        std::vector<std::thread> th;
        for (unsigned i = 0; i < nw; ++i) th.emplace_back(work, i);
        for (auto &t : th) t.join();
    }
    for (uint32_t b : bad_per_block) if (b < first_bad) first_bad = b;
    if (first_bad != HSPMM_IDX_MAX) {
        set_error("tile " + std::to_string(first_bad) + ": the number of set bits differs from its nnzOffset span");
        return HSPMM_ERR_INVALID;
    }
    return HSPMM_OK;
}

// ---------------------------------------------------------------------------
// Grouped format (reference BTCF2GBTCF, src/utils/convert.h:232-276)
// ---------------------------------------------------------------------------
int hspmm_group_sizes(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t min_len,
                      uint32_t *tgl, uint32_t *total_groups)
{
    using namespace hspmm_host;
    if (eff_row_windows && !rowOffset) { set_error("null argument"); return HSPMM_ERR_INVALID; }
    if (min_len == 0) { set_error("min_len must be positive"); return HSPMM_ERR_INVALID; }
    for (uint32_t w = 0; w < eff_row_windows; ++w)
        if (rowOffset[w + 1] <= rowOffset[w]) { set_error("rowOffset must increase strictly"); return HSPMM_ERR_INVALID; }
    // mean tiles per window: the reference adds the counts up as doubles and truncates
    // the quotient (convert.h:239,243); the sum is exact in a double (< 2^53).
    uint32_t mean = 0;
    if (eff_row_windows)
        mean = uint32_t(double(rowOffset[eff_row_windows] - rowOffset[0]) / double(eff_row_windows));
    const uint32_t len = std::max(mean, min_len);                            // convert.h:243
    uint64_t groups = 0;
    for (uint32_t w = 0; w < eff_row_windows; ++w) {
        const uint32_t n = rowOffset[w + 1] - rowOffset[w];
        groups += (uint64_t(n) + len - 1) / len;                             // convert.h:249
    }
    if (groups > 0xFFFFFFFEull) { set_error("group count exceeds 32 bits"); return HSPMM_ERR_UNSUPPORTED; }
    if (tgl) *tgl = len;
    if (total_groups) *total_groups = uint32_t(groups);
    return HSPMM_OK;
}

int hspmm_group_fill(uint32_t eff_row_windows, const uint32_t *rowOffset, const uint32_t *rowIdx,
                     uint32_t tgl, uint32_t *groupOffset, uint32_t *groupRowIdx, uint8_t *atomic)
{
    using namespace hspmm_host;
    if (!groupOffset || (eff_row_windows && (!rowOffset || !rowIdx || !groupRowIdx || !atomic))) {
        set_error("null argument");
        return HSPMM_ERR_INVALID;
    }
    if (tgl == 0) { set_error("tgl must be positive"); return HSPMM_ERR_INVALID; }
    size_t g = 0;
    for (uint32_t w = 0; w < eff_row_windows; ++w) {
        const uint32_t n = rowOffset[w + 1] - rowOffset[w];
        const uint32_t group_num = uint32_t((uint64_t(n) + tgl - 1) / tgl);                   // convert.h:249
        const uint32_t stride = group_num ? uint32_t((uint64_t(n) + group_num - 1) / group_num) : 0u;
        for (uint32_t j = 0; j < group_num; ++j, ++g) {
            groupOffset[g] = rowOffset[w] + stride * j;                      // convert.h:251-252
            groupRowIdx[g] = rowIdx[w];                                      // convert.h:253
            atomic[g] = group_num == 1 ? 0 : 1;                              // convert.h:254-257
        }
    }
    groupOffset[g] = eff_row_windows ? rowOffset[eff_row_windows] : 0u;      // convert.h:261
    return HSPMM_OK;
}

}  // extern "C"
