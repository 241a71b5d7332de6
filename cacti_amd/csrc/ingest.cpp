// Weight ingest: a directory of safetensors files -> the parameter cells of a model.
//
//   TensorsDir::open / _reopen / get   src/util/safetensor.rs:45-160   (file discovery, name table, mmap slices)
//   CellMatcher::match_                src/util/cell.rs:63-112         (rule -> tensor name)
//   Llama::match_pickle_dir            src/librarium/llama.rs:284-302  (the rules of the model)
//   resume_put                         src/spine.rs:1714-1745          (types must agree exactly)
//   set_lossy_cast                     src/op.rs:1112-1135             (bf16 / f32 source -> f16 cell)
//
// The header parser of the reference lives in a sibling crate that is not part of its tree
// (cell_split 0.1.0-devel, TensorsDict::from_reader); it is restated here from the published
// safetensors layout: u64 little-endian header length N, N bytes of JSON mapping each tensor
// name to {"dtype", "shape", "data_offsets": [begin, end]} (offsets relative to byte 8 + N) plus an
// optional "__metadata__" object of strings.
#include <fcntl.h>
#include <glob.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <map>
#include <string>
#include <vector>

#include "../../include/cacti_hip_runtime.h"
#include "common.h"
#include "ingest_internal.h"
#include "runtime.h"

using namespace cacti;

namespace {

// ---- the little JSON the header needs: objects, arrays, strings, non-negative integers ----
struct Json {
    const char *p, *end;
    std::string err;

    void ws()
    {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) p++;
    }
    bool lit(char c)
    {
        ws();
        if (p < end && *p == c) {
            p++;
            return true;
        }
        return false;
    }
    bool fail(const char *what)
    {
        if (err.empty()) err = what;
        return false;
    }
    bool string(std::string &out)
    {
        ws();
        if (p >= end || *p != '"') return fail("expected a string");
        p++;
        out.clear();
        while (p < end && *p != '"') {
            if (*p == '\\') {
                if (++p >= end) return fail("unterminated escape");
                switch (*p) {
                    case 'n': out += '\n'; break;
                    case 't': out += '\t'; break;
                    case 'r': out += '\r'; break;
                    case 'b': out += '\b'; break;
                    case 'f': out += '\f'; break;
                    case 'u': {
                        if (end - p < 5) return fail("short \\u escape");
                        unsigned v = 0;
                        for (int i = 1; i <= 4; i++) {
                            const char c = p[i];
                            v = v * 16 + (c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : 99);
                            if (v > 0xffff) return fail("bad \\u escape");
                        }
                        // tensor names are ASCII in practice; encode the code point as UTF-8
                        if (v < 0x80) out += (char)v;
                        else if (v < 0x800) {
                            out += (char)(0xc0 | (v >> 6));
                            out += (char)(0x80 | (v & 0x3f));
                        } else {
                            out += (char)(0xe0 | (v >> 12));
                            out += (char)(0x80 | ((v >> 6) & 0x3f));
                            out += (char)(0x80 | (v & 0x3f));
                        }
                        p += 4;
                        break;
                    }
                    default: out += *p;         // \" \\ \/
                }
                p++;
            } else {
                out += *p++;
            }
        }
        if (p >= end) return fail("unterminated string");
        p++;
        return true;
    }
    bool uint(uint64_t &out)
    {
        ws();
        if (p >= end || *p < '0' || *p > '9') return fail("expected a non-negative integer");
        out = 0;
        while (p < end && *p >= '0' && *p <= '9') {
            if (out > (UINT64_MAX - 9) / 10) return fail("integer overflow");
            out = out * 10 + (uint64_t)(*p++ - '0');
        }
        return true;
    }
    bool uint_array(std::vector<uint64_t> &out)
    {
        out.clear();
        if (!lit('[')) return fail("expected an array");
        if (lit(']')) return true;
        do {
            uint64_t v;
            if (!uint(v)) return false;
            out.push_back(v);
        } while (lit(','));
        return lit(']') || fail("unterminated array");
    }
    // any value, skipped (the "__metadata__" object and unknown fields)
    bool skip(int depth = 0)
    {
        if (depth > 32) return fail("nesting too deep");
        ws();
        if (p >= end) return fail("unexpected end");
        if (*p == '"') {
            std::string s;
            return string(s);
        }
        if (*p == '{' || *p == '[') {
            const char close = *p == '{' ? '}' : ']';
            const bool obj = *p == '{';
            p++;
            if (lit(close)) return true;
            do {
                if (obj) {
                    std::string k;
                    if (!string(k) || !lit(':')) return fail("bad object");
                }
                if (!skip(depth + 1)) return false;
            } while (lit(','));
            return lit(close) || fail("unterminated container");
        }
        while (p < end && *p != ',' && *p != '}' && *p != ']' && *p != ' ' && *p != '\n' && *p != '\t' && *p != '\r') p++;
        return true;
    }
};

}  // namespace

namespace {

// one file: map it, parse its header, add its tensors (TensorsDir::_reopen, src/util/safetensor.rs:88-113)
int add_file(cacti_tensors_dir *d, const std::string &path)
{
    MappedFile mf;
    const int rc = ingest_map_file(path, 8, "tensors_dir", &mf);
    if (rc) return rc;
    const int file_idx = (int)d->files.size();
    d->files.push_back(mf);
    const unsigned char *b = static_cast<const unsigned char *>(mf.base);
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; i--) hlen = (hlen << 8) | b[i];
    CACTI_REQUIRE(hlen <= mf.size - 8, CACTI_E_FORMAT, "tensors_dir: %s: header length %llu exceeds the file",
                  path.c_str(), (unsigned long long)hlen);
    const uint64_t buf_start = 8 + hlen;
    Json js{reinterpret_cast<const char *>(b + 8), reinterpret_cast<const char *>(b + 8 + hlen), ""};
    bool ok = js.lit('{');
    if (ok && !js.lit('}')) {
        do {
            std::string name;
            if (!(ok = js.string(name) && js.lit(':'))) break;
            if (name == "__metadata__") {
                if (!(ok = js.skip())) break;
                continue;
            }
            TensorEntry e;
            e.file = file_idx;
            bool have_dtype = false, have_shape = false, have_off = false;
            if (!(ok = js.lit('{'))) break;
            if (!js.lit('}')) {
                do {
                    std::string field;
                    if (!(ok = js.string(field) && js.lit(':'))) break;
                    std::vector<uint64_t> arr;
                    if (field == "dtype") {
                        ok = js.string(e.dtype);
                        have_dtype = true;
                    } else if (field == "shape") {
                        ok = js.uint_array(arr);
                        for (uint64_t v : arr) e.shape.push_back((int64_t)v);
                        have_shape = true;
                    } else if (field == "data_offsets") {
                        ok = js.uint_array(arr) && arr.size() == 2;
                        if (ok) {
                            e.off = buf_start + arr[0];
                            e.eoff = buf_start + arr[1];
                        }
                        have_off = true;
                    } else {
                        ok = js.skip();
                    }
                } while (ok && js.lit(','));
                ok = ok && js.lit('}');
            }
            if (!ok) break;
            CACTI_REQUIRE(have_dtype && have_shape && have_off, CACTI_E_FORMAT,
                          "tensors_dir: %s: tensor %s lacks dtype, shape or data_offsets", path.c_str(), name.c_str());
            uint64_t elems = 1;
            for (int64_t v : e.shape) elems *= (uint64_t)v;
            const size_t esz = ingest_dtype_bytes(e.dtype);
            CACTI_REQUIRE(esz != 0, CACTI_E_FORMAT, "tensors_dir: %s: tensor %s has unknown dtype %s", path.c_str(),
                          name.c_str(), e.dtype.c_str());
            // packed_span_bytes == size, src/util/safetensor.rs:127-132
            CACTI_REQUIRE(e.off <= e.eoff && e.eoff <= mf.size && e.eoff - e.off == elems * esz, CACTI_E_FORMAT,
                          "tensors_dir: %s: tensor %s: byte range [%llu, %llu) does not fit its type or the file",
                          path.c_str(), name.c_str(), (unsigned long long)e.off, (unsigned long long)e.eoff);
            // TensorsDirErr::DuplicateName
            CACTI_REQUIRE(d->tensors.find(name) == d->tensors.end(), CACTI_E_FORMAT,
                          "tensors_dir: duplicate tensor name %s (in %s)", name.c_str(), path.c_str());
            d->serial_key.push_back(name);
            d->tensors.emplace(name, std::move(e));
        } while (js.lit(','));
        ok = ok && js.lit('}');
    }
    CACTI_REQUIRE(ok, CACTI_E_FORMAT, "tensors_dir: %s: malformed header (%s)", path.c_str(),
                  js.err.empty() ? "syntax" : js.err.c_str());
    return 0;
}

// ---- CellMatcher -----------------------------------------------------------------------------
struct Pat {
    bool is_int;
    std::string s;                                       // decimal text for an integer
};

// a rule is written "a/b/c"; a component "#12" is Pat::Int(12), anything else Pat::Str
std::vector<Pat> parse_rule(const char *rule)
{
    std::vector<Pat> out;
    const char *p = rule;
    while (true) {
        const char *q = strchr(p, '/');
        std::string tok = q ? std::string(p, q) : std::string(p);
        if (!tok.empty() && tok[0] == '#') out.push_back({true, tok.substr(1)});
        else out.push_back({false, tok});
        if (!q) break;
        p = q + 1;
    }
    return out;
}

// does `key` consume the whole pattern?  Tokens of the key (split at '.') are scanned once, left to
// right; the current pattern element advances when the token equals it (integers and strings) or
// contains it (strings); src/util/cell.rs:73-98
bool key_matches(const std::string &key, const std::vector<Pat> &pat)
{
    size_t idx = 0, start = 0;
    while (true) {
        const size_t dot = key.find('.', start);
        const std::string tok = key.substr(start, dot == std::string::npos ? std::string::npos : dot - start);
        const Pat &pt = pat[idx];
        if (pt.is_int ? tok == pt.s : (tok == pt.s || tok.find(pt.s) != std::string::npos)) idx++;
        if (idx == pat.size()) return true;
        if (dot == std::string::npos) return false;
        start = dot + 1;
    }
}

}  // namespace

CACTI_API int cacti_tensors_dir_open(const char *path, cacti_tensors_dir **out)
{
    CACTI_REQUIRE(path && out, CACTI_E_INVALID, "tensors_dir_open: null argument");
    *out = nullptr;
    std::vector<std::string> files;
    struct stat st;
    CACTI_REQUIRE(stat(path, &st) == 0, CACTI_E_IO, "tensors_dir_open: %s does not exist", path);
    if (S_ISREG(st.st_mode)) {
        files.push_back(path);
    } else {
        // model.safetensors, else the sorted shards model-*-of-*.safetensors (src/util/safetensor.rs:66-87)
        const std::string one = std::string(path) + "/model.safetensors";
        if (stat(one.c_str(), &st) == 0) {
            files.push_back(one);
        } else {
            glob_t g;
            memset(&g, 0, sizeof(g));
            const std::string patt = std::string(path) + "/model-*-of-*.safetensors";
            if (glob(patt.c_str(), 0, nullptr, &g) == 0)
                for (size_t i = 0; i < g.gl_pathc; i++) files.push_back(g.gl_pathv[i]);
            globfree(&g);
            std::sort(files.begin(), files.end());
            CACTI_REQUIRE(!files.empty(), CACTI_E_IO,
                          "tensors_dir_open: %s holds neither model.safetensors nor model-*-of-*.safetensors", path);
        }
    }
    cacti_tensors_dir *d = new cacti_tensors_dir();
    d->path = path;
    for (const std::string &f : files) {
        const int rc = add_file(d, f);
        if (rc) {
            delete d;
            return rc;
        }
    }
    for (auto &kv : d->tensors) d->sorted.push_back(&kv.first);
    *out = d;
    return 0;
}

CACTI_API int cacti_tensors_dir_close(cacti_tensors_dir *dir)
{
    delete dir;
    return 0;
}

CACTI_API int cacti_tensors_dir_count(cacti_tensors_dir *dir) { return dir ? (int)dir->sorted.size() : 0; }

CACTI_API int cacti_tensors_dir_entry(cacti_tensors_dir *dir, int i, char *name, size_t name_cap, char *dtype,
                                      size_t dtype_cap, int *ndim, int64_t *shape8, const void **data,
                                      uint64_t *bytes)
{
    CACTI_REQUIRE(dir && i >= 0 && (size_t)i < dir->sorted.size(), CACTI_E_INVALID, "tensors_dir_entry: index out of range");
    const std::string &key = *dir->sorted[(size_t)i];
    const TensorEntry &e = dir->tensors.at(key);
    CACTI_REQUIRE(e.shape.size() <= 8, CACTI_E_NOTIMPL, "tensors_dir_entry: %s has more than 8 dimensions", key.c_str());
    // a name or dtype that does not fit is an error, not a silently shortened string
    CACTI_REQUIRE(!name || name_cap > key.size(), CACTI_E_INVALID, "tensors_dir_entry: name of %zu bytes needs a larger buffer",
                  key.size());
    CACTI_REQUIRE(!dtype || dtype_cap > e.dtype.size(), CACTI_E_INVALID, "tensors_dir_entry: dtype buffer too small");
    if (name) snprintf(name, name_cap, "%s", key.c_str());
    if (dtype) snprintf(dtype, dtype_cap, "%s", e.dtype.c_str());
    if (ndim) *ndim = (int)e.shape.size();
    if (shape8)
        for (size_t k = 0; k < e.shape.size(); k++) shape8[k] = e.shape[k];
    if (data) *data = static_cast<const char *>(dir->files[(size_t)e.file].base) + e.off;
    if (bytes) *bytes = e.eoff - e.off;
    return 0;
}

CACTI_API int cacti_cell_matcher_match(const char *const *keys, int nkeys, const char *const *rules, int nrules,
                                       int *match)
{
    CACTI_REQUIRE(nkeys >= 0 && nrules >= 0 && (nkeys == 0 || keys) && (nrules == 0 || (rules && match)),
                  CACTI_E_INVALID, "cell_matcher_match: null argument");
    // the key set is ordered (BTreeSet<SmolStr>: byte-wise); a matched key leaves the set
    std::vector<std::pair<std::string, int>> set;
    for (int i = 0; i < nkeys; i++) {
        CACTI_REQUIRE(keys[i], CACTI_E_INVALID, "cell_matcher_match: null key");
        set.emplace_back(keys[i], i);
    }
    std::sort(set.begin(), set.end());
    set.erase(std::unique(set.begin(), set.end(), [](const auto &a, const auto &b) { return a.first == b.first; }),
              set.end());
    for (int r = 0; r < nrules; r++) {
        CACTI_REQUIRE(rules[r] && rules[r][0], CACTI_E_INVALID, "cell_matcher_match: empty rule");
        const std::vector<Pat> pat = parse_rule(rules[r]);
        match[r] = -1;
        for (size_t k = 0; k < set.size(); k++)
            if (key_matches(set[k].first, pat)) {
                match[r] = set[k].second;
                set.erase(set.begin() + (long)k);
                break;
            }
    }
    return 0;
}

// ---- model ------------------------------------------------------------------------------------
namespace cacti {
int llama_load_tensors(cacti_llama *m, cacti_tensors_dir *dir, int *n_matched);
}

CACTI_API int cacti_llama_load_tensors_dir(cacti_llama *model, cacti_tensors_dir *dir, int *n_matched)
{
    CACTI_REQUIRE(model && dir, CACTI_E_INVALID, "llama_load_tensors_dir: null argument");
    return cacti::llama_load_tensors(model, dir, n_matched);
}

// the pieces llama.cpp needs of a directory
namespace cacti {

size_t ingest_dtype_bytes(const std::string &d)
{
    if (d == "F64" || d == "I64" || d == "U64") return 8;
    if (d == "F32" || d == "I32" || d == "U32") return 4;
    if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") return 2;
    if (d == "I8" || d == "U8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
    return 0;
}

int ingest_map_file(const std::string &path, size_t min_size, const char *who, MappedFile *mf)
{
    mf->path = path;
    mf->fd = open(path.c_str(), O_RDONLY);
    CACTI_REQUIRE(mf->fd >= 0, CACTI_E_IO, "%s: cannot open %s", who, path.c_str());
    struct stat st;
    if (fstat(mf->fd, &st) != 0 || (size_t)st.st_size < min_size) {
        close(mf->fd);
        mf->fd = -1;
        set_error("%s: %s is shorter than the %zu bytes its format needs", who, path.c_str(), min_size);
        return CACTI_E_FORMAT;
    }
    mf->size = (size_t)st.st_size;
    mf->base = mmap(nullptr, mf->size, PROT_READ, MAP_PRIVATE, mf->fd, 0);
    if (mf->base == MAP_FAILED) {
        close(mf->fd);
        mf->fd = -1;
        mf->base = nullptr;
        set_error("%s: cannot map %s", who, path.c_str());
        return CACTI_E_IO;
    }
    return 0;
}

int tensors_dir_keys(cacti_tensors_dir *dir, std::vector<const char *> *keys)
{
    keys->clear();
    for (const std::string *s : dir->sorted) keys->push_back(s->c_str());
    return 0;
}

int tensors_dir_lookup(cacti_tensors_dir *dir, int i, const char **dtype, const std::vector<int64_t> **shape,
                       int *fd, uint64_t *off, size_t *bytes)
{
    const TensorEntry &e = dir->tensors.at(*dir->sorted[(size_t)i]);
    *dtype = e.dtype.c_str();
    *shape = &e.shape;
    *fd = dir->files[(size_t)e.file].fd;
    *off = e.off;
    *bytes = (size_t)(e.eoff - e.off);
    return 0;
}

}  // namespace cacti
