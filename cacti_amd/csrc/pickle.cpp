// Weight ingest from torch checkpoints: pytorch_model.bin / pytorch_model-*-of-*.bin -> the same
// table of named, memory-mapped tensors the safetensors reader fills.
//
//   PickleDir::open / open_with_prefix / _reopen   src/util/safepickle.rs:52-119   (file discovery, name table)
//   PickleDir::get                                 src/util/safepickle.rs:125-195  (type, packed-stride check,
//                                                                                  byte range, 64-byte alignment)
//   Dtype::try_from(TorchDtype)                    src/cell/mod.rs:1553-1574       (accepted storage types)
//
// The archive and pickle parser of the reference is a third-party crate outside its tree
// (repugnant_pickle, RepugnantTorchFile::new / tensors()); it is restated here from the published
// formats.  A torch checkpoint is a ZIP archive of stored (uncompressed) records: "<root>/data.pkl"
// holds a pickle of the state dictionary and "<root>/data/<key>" the bytes of storage <key>, each
// padded to a 64-byte file offset.  The pickle is *scanned*, never executed: opcodes build a tree of
// plain values in which a global is only its (module, name) pair and a REDUCE only records its
// callable and arguments.  A tensor is the node
//   REDUCE(torch._utils._rebuild_tensor_v2,
//          (PERSID(("storage", torch.<T>Storage, key, location, numel)), offset, size, stride, ...))
// optionally wrapped in torch._utils._rebuild_parameter(tensor, requires_grad, hooks).
#include <fcntl.h>
#include <glob.h>
#include <string.h>
#include <sys/stat.h>

#include <algorithm>
#include <deque>
#include <memory>
#include <unordered_map>

#include "../../include/cacti_hip_runtime.h"
#include "common.h"
#include "ingest_internal.h"

using namespace cacti;

namespace {

// ---- ZIP: the central directory, with the ZIP64 records archives above 4 GiB carry ----------------
struct ZipRecord {
    uint64_t data_off = 0, size = 0;
    uint16_t method = 0;
};

inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
inline uint32_t rd32(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
inline uint64_t rd64(const uint8_t *p) { return (uint64_t)rd32(p) | ((uint64_t)rd32(p + 4) << 32); }

int zip_records(const MappedFile &mf, std::map<std::string, ZipRecord> *out)
{
    const uint8_t *b = static_cast<const uint8_t *>(mf.base);
    const uint64_t n = mf.size;
    const char *path = mf.path.c_str();
    // end-of-central-directory record: 22 bytes + a comment of at most 65535, found from the back
    uint64_t eocd = UINT64_MAX;
    for (uint64_t back = 22; back <= std::min<uint64_t>(n, 22 + 65535); back++) {
        const uint64_t pos = n - back;
        if (rd32(b + pos) == 0x06054b50u && (uint64_t)rd16(b + pos + 20) == back - 22) {
            eocd = pos;
            break;
        }
    }
    CACTI_REQUIRE(eocd != UINT64_MAX, CACTI_E_FORMAT, "pickle_dir: %s is not a ZIP archive (legacy torch files are not read)", path);
    uint64_t count = rd16(b + eocd + 10), cd_size = rd32(b + eocd + 12), cd_off = rd32(b + eocd + 16);
    if (count == 0xffffu || cd_size == 0xffffffffu || cd_off == 0xffffffffu) {
        // ZIP64: a 20-byte locator right before the record names the 64-bit record
        CACTI_REQUIRE(eocd >= 20 && rd32(b + eocd - 20) == 0x07064b50u, CACTI_E_FORMAT,
                      "pickle_dir: %s: ZIP64 locator missing", path);
        const uint64_t z = rd64(b + eocd - 20 + 8);
        CACTI_REQUIRE(n >= 56 && z <= n - 56 && rd32(b + z) == 0x06064b50u, CACTI_E_FORMAT, "pickle_dir: %s: ZIP64 record missing", path);
        count = rd64(b + z + 32);
        cd_size = rd64(b + z + 40);
        cd_off = rd64(b + z + 48);
    }
    CACTI_REQUIRE(cd_off <= n && cd_size <= n - cd_off, CACTI_E_FORMAT, "pickle_dir: %s: central directory outside the file", path);
    uint64_t p = cd_off;
    const uint64_t cd_end = cd_off + cd_size;
    for (uint64_t i = 0; i < count; i++) {
        CACTI_REQUIRE(p + 46 <= cd_end && rd32(b + p) == 0x02014b50u, CACTI_E_FORMAT,
                      "pickle_dir: %s: malformed central directory entry %llu", path, (unsigned long long)i);
        ZipRecord r;
        r.method = rd16(b + p + 10);
        uint64_t csize = rd32(b + p + 20), usize = rd32(b + p + 24), lho = rd32(b + p + 42);
        const uint32_t nlen = rd16(b + p + 28), elen = rd16(b + p + 30), clen = rd16(b + p + 32);
        CACTI_REQUIRE(p + 46 + nlen + elen + clen <= cd_end, CACTI_E_FORMAT, "pickle_dir: %s: central directory entry overruns", path);
        const std::string name(reinterpret_cast<const char *>(b + p + 46), nlen);
        // the ZIP64 extra field (id 1) holds, in this order, the fields that are saturated above
        for (uint64_t e = p + 46 + nlen, e_end = e + elen; e + 4 <= e_end;) {
            const uint16_t id = rd16(b + e), len = rd16(b + e + 2);
            CACTI_REQUIRE(e + 4 + len <= e_end, CACTI_E_FORMAT, "pickle_dir: %s: extra field overruns (%s)", path, name.c_str());
            if (id == 1) {
                uint64_t q = e + 4;
                const uint64_t q_end = q + len;
                for (uint64_t *f : {&usize, &csize, &lho})
                    if (*f == 0xffffffffu) {
                        CACTI_REQUIRE(q + 8 <= q_end, CACTI_E_FORMAT, "pickle_dir: %s: short ZIP64 field (%s)", path, name.c_str());
                        *f = rd64(b + q);
                        q += 8;
                    }
            }
            e += 4 + (uint64_t)len;
        }
        CACTI_REQUIRE(lho <= n && n - lho >= 30 && rd32(b + lho) == 0x04034b50u, CACTI_E_FORMAT,
                      "pickle_dir: %s: local header of %s outside the file", path, name.c_str());
        r.data_off = lho + 30 + rd16(b + lho + 26) + rd16(b + lho + 28);
        r.size = usize;
        CACTI_REQUIRE(r.data_off <= n && csize <= n - r.data_off, CACTI_E_FORMAT, "pickle_dir: %s: record %s outside the file", path,
                      name.c_str());
        CACTI_REQUIRE(r.method != 0 || csize == usize, CACTI_E_FORMAT, "pickle_dir: %s: stored record %s has two sizes", path, name.c_str());
        (*out)[name] = r;
        p += 46 + nlen + elen + clen;
    }
    return 0;
}

// ---- pickle: a graph of plain values --------------------------------------------------------------
// The values belong to the unpickler that made them (one flat list, freed in a loop) and refer to each
// other by plain pointers: a pickle can make a value its own descendant through the memo, or hang a
// chain of any length below a value after that value was attached elsewhere, and neither may turn into
// a leak or into a teardown that recurses once per level.  Nothing here walks the graph deeper than the
// fixed shape of a tensor entry.
struct PV;
using P = PV *;
struct PV {
    enum Kind { NONE, BOOL, INT, FLOAT, STR, BYTES, TUPLE, LIST, DICT, SET, GLOBAL, REDUCE, PERSID } kind = NONE;
    int64_t i = 0;
    int depth = 1;                     // nesting below this value when its children were attached (a sanity bound only)
    std::string s, s2;                 // STR / BYTES text; GLOBAL module, name
    std::vector<P> items;              // TUPLE, LIST, SET; DICT and REDUCE: key, value, key, value ...
    P callable = nullptr, args = nullptr, state = nullptr;     // REDUCE (+ BUILD state); PERSID: args = the id
};

struct Unpickler {
    static constexpr int kMaxDepth = 256;
    static constexpr size_t kMaxValues = (size_t)1 << 22;       // values made + references held in containers
    const uint8_t *p, *end;
    std::vector<P> stack;
    std::vector<size_t> marks;
    std::unordered_map<uint64_t, P> memo;
    std::string err;
    std::deque<PV> values;             // every value made; addresses stay put as it grows
    size_t held = 0;                   // references stored in containers so far

    P mk(PV::Kind k)
    {
        values.emplace_back();
        values.back().kind = k;
        return &values.back();
    }

    bool fail(const char *what)
    {
        if (err.empty()) err = what;
        return false;
    }
    // records how deep `v` nests once `kids` hang below it
    bool nest(PV &v, const std::vector<P> &kids)
    {
        for (const P &k : kids)
            if (k) v.depth = std::max(v.depth, k->depth + 1);
        return v.depth <= kMaxDepth || fail("values nest too deep");
    }
    bool need(uint64_t k) { return (uint64_t)(end - p) >= k || fail("pickle ends inside an opcode"); }
    bool pop(P *v)
    {
        if (stack.empty() || (!marks.empty() && stack.size() <= marks.back())) return fail("stack underflow");
        *v = stack.back();
        stack.pop_back();
        return true;
    }
    bool pop_mark(std::vector<P> *items)
    {
        if (marks.empty()) return fail("no mark on the stack");
        const size_t m = marks.back();
        marks.pop_back();
        items->assign(stack.begin() + (long)m, stack.end());
        stack.resize(m);
        return true;
    }
    bool line(std::string *s)
    {
        const uint8_t *q = static_cast<const uint8_t *>(memchr(p, '\n', (size_t)(end - p)));
        if (!q) return fail("unterminated line argument");
        s->assign(reinterpret_cast<const char *>(p), (size_t)(q - p));
        p = q + 1;
        return true;
    }
    bool text(PV::Kind k, uint64_t len)
    {
        if (!need(len)) return false;
        P v = mk(k);
        v->s.assign(reinterpret_cast<const char *>(p), (size_t)len);
        p += len;
        stack.push_back(v);
        return true;
    }
    bool integer(int64_t x)
    {
        P v = mk(PV::INT);
        v->i = x;
        stack.push_back(v);
        return true;
    }
    bool long_bytes(uint64_t len)
    {
        if (!need(len)) return false;
        if (len > 8) return fail("integer wider than 64 bits");
        uint64_t x = 0;
        for (uint64_t k = 0; k < len; k++) x |= (uint64_t)p[k] << (8 * k);
        if (len && len < 8 && (p[len - 1] & 0x80)) x |= ~0ull << (8 * len);
        p += len;
        return integer((int64_t)x);
    }
    // container on top of the stack receives key/value pairs (dictionaries and the objects a REDUCE made)
    bool set_items(const std::vector<P> &kv)
    {
        if (kv.size() % 2) return fail("odd number of items for a dictionary");
        if (stack.empty()) return fail("stack underflow");
        PV &d = *stack.back();
        if (d.kind != PV::DICT && d.kind != PV::REDUCE) return fail("items set on a value that is no dictionary");
        held += kv.size();
        d.items.insert(d.items.end(), kv.begin(), kv.end());
        return nest(d, kv);
    }
    bool append_items(const std::vector<P> &it)
    {
        if (stack.empty()) return fail("stack underflow");
        PV &d = *stack.back();
        if (d.kind != PV::LIST && d.kind != PV::SET && d.kind != PV::REDUCE) return fail("append to a value that is no list");
        held += it.size();
        if (d.kind != PV::REDUCE) d.items.insert(d.items.end(), it.begin(), it.end());
        return d.kind == PV::REDUCE || nest(d, it);
    }

    bool run(P *result)
    {
        while (true) {
            if (!need(1)) return false;
            if (stack.size() > (1u << 24)) return fail("stack too deep");
            if (values.size() + held > kMaxValues) return fail("too many values");
            const uint8_t op = *p++;
            P a, b2, c;
            std::vector<P> items;
            switch (op) {
                case 0x80: if (!need(1)) return false; p += 1; break;                                   // PROTO
                case 0x95: if (!need(8)) return false; p += 8; break;                                   // FRAME
                case '.': return pop(result);                                                           // STOP
                case '(': marks.push_back(stack.size()); break;                                         // MARK
                case '0': if (!pop(&a)) return false; break;                                            // POP
                case '1': if (!pop_mark(&items)) return false; break;                                   // POP_MARK
                case '2': if (stack.empty()) return fail("stack underflow"); stack.push_back(stack.back()); break;  // DUP
                case 'N': stack.push_back(mk(PV::NONE)); break;
                case 0x88: case 0x89: a = mk(PV::BOOL); a->i = op == 0x88; stack.push_back(a); break;
                case 'K': if (!need(1)) return false; integer(p[0]); p += 1; break;                     // BININT1
                case 'M': if (!need(2)) return false; integer(rd16(p)); p += 2; break;                  // BININT2
                case 'J': if (!need(4)) return false; integer((int32_t)rd32(p)); p += 4; break;         // BININT
                case 0x8a: { if (!need(1)) return false; const uint64_t l = *p++; if (!long_bytes(l)) return false; break; }       // LONG1
                case 0x8b: { if (!need(4)) return false; const uint64_t l = rd32(p); p += 4; if (!long_bytes(l)) return false; break; }  // LONG4
                case 'G': if (!need(8)) return false; p += 8; stack.push_back(mk(PV::FLOAT)); break;    // BINFLOAT (value unused)
                case 'X': { if (!need(4)) return false; const uint64_t l = rd32(p); p += 4; if (!text(PV::STR, l)) return false; break; }   // BINUNICODE
                case 0x8c: { if (!need(1)) return false; const uint64_t l = *p++; if (!text(PV::STR, l)) return false; break; }            // SHORT_BINUNICODE
                case 0x8d: { if (!need(8)) return false; const uint64_t l = rd64(p); p += 8; if (!text(PV::STR, l)) return false; break; }  // BINUNICODE8
                case 'T': { if (!need(4)) return false; const uint64_t l = rd32(p); p += 4; if (!text(PV::STR, l)) return false; break; }   // BINSTRING
                case 'U': { if (!need(1)) return false; const uint64_t l = *p++; if (!text(PV::STR, l)) return false; break; }             // SHORT_BINSTRING
                case 'B': { if (!need(4)) return false; const uint64_t l = rd32(p); p += 4; if (!text(PV::BYTES, l)) return false; break; } // BINBYTES
                case 'C': { if (!need(1)) return false; const uint64_t l = *p++; if (!text(PV::BYTES, l)) return false; break; }           // SHORT_BINBYTES
                case 0x8e: { if (!need(8)) return false; const uint64_t l = rd64(p); p += 8; if (!text(PV::BYTES, l)) return false; break; } // BINBYTES8
                case '}': stack.push_back(mk(PV::DICT)); break;
                case ']': stack.push_back(mk(PV::LIST)); break;
                case ')': stack.push_back(mk(PV::TUPLE)); break;
                case 0x8f: stack.push_back(mk(PV::SET)); break;                                         // EMPTY_SET
                case 't': case 'l': case 0x91:                                                          // TUPLE, LIST, FROZENSET
                    if (!pop_mark(&items)) return false;
                    a = mk(op == 't' ? PV::TUPLE : op == 'l' ? PV::LIST : PV::SET);
                    held += items.size();
                    a->items = std::move(items);
                    if (!nest(*a, a->items)) return false;
                    stack.push_back(a);
                    break;
                case 'd':                                                                               // DICT
                    if (!pop_mark(&items)) return false;
                    stack.push_back(mk(PV::DICT));
                    if (!set_items(items)) return false;
                    break;
                case 0x85: case 0x86: case 0x87: {                                                      // TUPLE1..3
                    const size_t k = (size_t)(op - 0x84);
                    if (stack.size() < k || (!marks.empty() && stack.size() - k < marks.back())) return fail("stack underflow");
                    a = mk(PV::TUPLE);
                    a->items.assign(stack.end() - (long)k, stack.end());
                    if (!nest(*a, a->items)) return false;
                    stack.resize(stack.size() - k);
                    stack.push_back(a);
                    break;
                }
                case 'q': if (!need(1) || stack.empty()) return fail("bad BINPUT"); memo[*p++] = stack.back(); break;
                case 'r': if (!need(4) || stack.empty()) return fail("bad LONG_BINPUT"); memo[rd32(p)] = stack.back(); p += 4; break;
                case 0x94: if (stack.empty()) return fail("bad MEMOIZE"); { const uint64_t k = memo.size(); memo[k] = stack.back(); } break;
                case 'h': case 'j': {                                                                   // BINGET, LONG_BINGET
                    const uint64_t w = op == 'h' ? 1 : 4;
                    if (!need(w)) return false;
                    const uint64_t k = op == 'h' ? p[0] : rd32(p);
                    p += w;
                    auto it = memo.find(k);
                    if (it == memo.end()) return fail("memo key not set");
                    stack.push_back(it->second);
                    break;
                }
                case 'c':                                                                               // GLOBAL
                    a = mk(PV::GLOBAL);
                    if (!line(&a->s) || !line(&a->s2)) return false;
                    stack.push_back(a);
                    break;
                case 0x93:                                                                              // STACK_GLOBAL
                    if (!pop(&b2) || !pop(&a)) return false;
                    if (a->kind != PV::STR || b2->kind != PV::STR) return fail("STACK_GLOBAL of non-strings");
                    c = mk(PV::GLOBAL);
                    c->s = a->s;
                    c->s2 = b2->s;
                    stack.push_back(c);
                    break;
                case 'R': case 0x81:                                                                    // REDUCE, NEWOBJ
                    if (!pop(&b2) || !pop(&a)) return false;
                    c = mk(PV::REDUCE);
                    c->callable = a;
                    c->args = b2;
                    if (!nest(*c, {a, b2})) return false;
                    stack.push_back(c);
                    break;
                case 0x92:                                                                              // NEWOBJ_EX
                    if (!pop(&c) || !pop(&b2) || !pop(&a)) return false;
                    c = mk(PV::REDUCE);
                    c->callable = a;
                    c->args = b2;
                    if (!nest(*c, {a, b2})) return false;
                    stack.push_back(c);
                    break;
                case 'b':                                                                               // BUILD
                    if (!pop(&a)) return false;
                    if (stack.empty()) return fail("stack underflow");
                    stack.back()->state = a;
                    if (!nest(*stack.back(), {a})) return false;
                    break;
                case 'Q':                                                                               // BINPERSID
                    if (!pop(&a)) return false;
                    c = mk(PV::PERSID);
                    c->args = a;
                    if (!nest(*c, {a})) return false;
                    stack.push_back(c);
                    break;
                case 's':                                                                               // SETITEM
                    if (!pop(&b2) || !pop(&a)) return false;
                    if (!set_items({a, b2})) return false;
                    break;
                case 'u': if (!pop_mark(&items) || !set_items(items)) return false; break;              // SETITEMS
                case 'a': if (!pop(&a) || !append_items({a})) return false; break;                      // APPEND
                case 'e': case 0x90: if (!pop_mark(&items) || !append_items(items)) return false; break;  // APPENDS, ADDITEMS
                default: {
                    char msg[48];
                    snprintf(msg, sizeof(msg), "opcode 0x%02x is not read", op);
                    return fail(msg);
                }
            }
        }
    }
};

bool is_global(const P &v, const char *module, const char *name)
{
    return v && v->kind == PV::GLOBAL && v->s == module && v->s2 == name;
}

// torch.<T>Storage -> the dtype spelling of the tensor table; the set of src/cell/mod.rs:1553-1574
const char *storage_dtype(const std::string &name)
{
    static const struct { const char *storage, *dtype; } kTab[] = {
        {"DoubleStorage", "F64"}, {"FloatStorage", "F32"}, {"HalfStorage", "F16"}, {"BFloat16Storage", "BF16"},
        {"LongStorage", "I64"},   {"IntStorage", "I32"},   {"ShortStorage", "I16"}, {"CharStorage", "I8"},
        {"ByteStorage", "U8"},    {"UInt64Storage", "U64"}, {"UInt32Storage", "U32"}, {"UInt16Storage", "U16"},
    };
    for (const auto &t : kTab)
        if (name == t.storage) return t.dtype;
    return nullptr;
}

bool int_tuple(const P &v, std::vector<int64_t> *out)
{
    if (!v || v->kind != PV::TUPLE) return false;
    out->clear();
    for (const P &x : v->items) {
        if (x->kind != PV::INT) return false;
        out->push_back(x->i);
    }
    return true;
}

// one file: map it, scan its pickle, add its tensors (PickleDir::_reopen + ::get)
int add_pickle_file(cacti_tensors_dir *d, const std::string &path)
{
    MappedFile mf;
    const int rc = ingest_map_file(path, 22, "pickle_dir", &mf);
    if (rc) return rc;
    const int file_idx = (int)d->files.size();
    d->files.push_back(mf);
    std::map<std::string, ZipRecord> recs;
    const int zrc = zip_records(mf, &recs);
    if (zrc) return zrc;
    std::string root;
    const ZipRecord *pkl = nullptr;
    for (const auto &kv : recs) {
        const std::string &nm = kv.first;
        if (nm == "data.pkl" || (nm.size() > 9 && nm.compare(nm.size() - 9, 9, "/data.pkl") == 0)) {
            CACTI_REQUIRE(!pkl, CACTI_E_FORMAT, "pickle_dir: %s holds more than one data.pkl", path.c_str());
            pkl = &kv.second;
            root = nm.substr(0, nm.size() - 8);
        }
    }
    CACTI_REQUIRE(pkl, CACTI_E_FORMAT, "pickle_dir: %s holds no data.pkl record", path.c_str());
    CACTI_REQUIRE(pkl->method == 0, CACTI_E_FORMAT, "pickle_dir: %s: data.pkl is compressed", path.c_str());
    auto bo = recs.find(root + "byteorder");
    if (bo != recs.end()) {
        CACTI_REQUIRE(bo->second.method == 0 && bo->second.size <= 16, CACTI_E_FORMAT,
                      "pickle_dir: %s: the byteorder record is compressed or longer than a byte order's name", path.c_str());
        const std::string order(static_cast<const char *>(mf.base) + bo->second.data_off, (size_t)bo->second.size);
        CACTI_REQUIRE(order == "little", CACTI_E_NOTIMPL, "pickle_dir: %s: byte order %s is not read", path.c_str(), order.c_str());
    }
    const uint8_t *b = static_cast<const uint8_t *>(mf.base);
    Unpickler up;
    up.p = b + pkl->data_off;
    up.end = up.p + pkl->size;
    P top = nullptr;
    CACTI_REQUIRE(up.run(&top), CACTI_E_FORMAT, "pickle_dir: %s: data.pkl: %s", path.c_str(), up.err.c_str());
    // the state dictionary: a dict, or collections.OrderedDict() filled by SETITEMS
    CACTI_REQUIRE(top->kind == PV::DICT || (top->kind == PV::REDUCE && is_global(top->callable, "collections", "OrderedDict")),
                  CACTI_E_FORMAT, "pickle_dir: %s: the pickled value is no dictionary", path.c_str());
    for (size_t k = 0; k + 1 < top->items.size(); k += 2) {
        const P &key = top->items[k];
        P val = top->items[k + 1];
        if (key->kind != PV::STR) continue;
        if (val->kind == PV::REDUCE && is_global(val->callable, "torch._utils", "_rebuild_parameter") && val->args &&
            val->args->kind == PV::TUPLE && !val->args->items.empty())
            val = val->args->items[0];
        if (!(val->kind == PV::REDUCE && is_global(val->callable, "torch._utils", "_rebuild_tensor_v2"))) continue;
        const std::string &name = key->s;
        const char *nm = name.c_str();
        const P &args = val->args;
        CACTI_REQUIRE(args && args->kind == PV::TUPLE && args->items.size() >= 4, CACTI_E_FORMAT,
                      "pickle_dir: %s: tensor %s: short argument tuple", path.c_str(), nm);
        const P &pid = args->items[0];
        CACTI_REQUIRE(pid->kind == PV::PERSID && pid->args && pid->args->kind == PV::TUPLE && pid->args->items.size() >= 5 &&
                          pid->args->items[0]->kind == PV::STR && pid->args->items[0]->s == "storage" &&
                          pid->args->items[1]->kind == PV::GLOBAL && pid->args->items[2]->kind == PV::STR &&
                          pid->args->items[4]->kind == PV::INT,
                      CACTI_E_FORMAT, "pickle_dir: %s: tensor %s: unexpected storage reference", path.c_str(), nm);
        const std::string &st_name = pid->args->items[1]->s2;
        const char *dt = pid->args->items[1]->s == "torch" ? storage_dtype(st_name) : nullptr;
        // "unknown tensor dtype", src/util/safepickle.rs:130-136
        CACTI_REQUIRE(dt, CACTI_E_NOTIMPL, "pickle_dir: %s: tensor %s: unknown tensor dtype %s", path.c_str(), nm, st_name.c_str());
        const uint64_t esz = ingest_dtype_bytes(dt);
        TensorEntry e;
        e.dtype = dt;
        e.file = file_idx;
        std::vector<int64_t> stride;
        CACTI_REQUIRE(args->items[1]->kind == PV::INT && args->items[1]->i >= 0 && int_tuple(args->items[2], &e.shape) &&
                          int_tuple(args->items[3], &stride) && stride.size() == e.shape.size(),
                      CACTI_E_FORMAT, "pickle_dir: %s: tensor %s: unexpected offset, size or stride", path.c_str(), nm);
        // only packed (row-major contiguous) tensors, src/util/safepickle.rs:141-151
        uint64_t elems = 1;
        for (size_t a = e.shape.size(); a-- > 0;) {
            CACTI_REQUIRE(e.shape[a] >= 0, CACTI_E_FORMAT, "pickle_dir: %s: tensor %s: negative dimension", path.c_str(), nm);
            CACTI_REQUIRE((uint64_t)stride[a] == elems, CACTI_E_NOTIMPL,
                          "pickle_dir: %s: loading strided (non-packed) tensors is not supported: %s", path.c_str(), nm);
            CACTI_REQUIRE(!__builtin_mul_overflow(elems, (uint64_t)e.shape[a], &elems), CACTI_E_FORMAT,
                          "pickle_dir: %s: tensor %s: element count exceeds 64 bits", path.c_str(), nm);
        }
        auto rec = recs.find(root + "data/" + pid->args->items[2]->s);
        CACTI_REQUIRE(rec != recs.end(), CACTI_E_FORMAT, "pickle_dir: %s: tensor %s: storage record %s missing", path.c_str(), nm,
                      pid->args->items[2]->s.c_str());
        CACTI_REQUIRE(rec->second.method == 0, CACTI_E_FORMAT, "pickle_dir: %s: tensor %s: storage is compressed", path.c_str(), nm);
        // byte range: the tensor starts `start` elements into its storage and must fit what is left of it
        // (span <= rem_size, offset + rem_size == storage end: src/util/safepickle.rs:152-166)
        CACTI_REQUIRE(pid->args->items[4]->i >= 0, CACTI_E_FORMAT, "pickle_dir: %s: tensor %s: negative storage size", path.c_str(), nm);
        const uint64_t start = (uint64_t)args->items[1]->i, numel = (uint64_t)pid->args->items[4]->i;
        // (no product that could wrap: numel is first held to what the record can hold)
        CACTI_REQUIRE(esz > 0 && numel <= rec->second.size / esz && numel * esz == rec->second.size, CACTI_E_FORMAT,
                      "pickle_dir: %s: tensor %s: storage of %llu elements does not fill its %llu-byte record", path.c_str(), nm,
                      (unsigned long long)numel, (unsigned long long)rec->second.size);
        CACTI_REQUIRE(start <= numel && elems <= numel - start, CACTI_E_FORMAT,
                      "pickle_dir: %s: tensor %s does not fit its storage", path.c_str(), nm);
        e.off = rec->second.data_off + start * esz;
        e.eoff = e.off + elems * esz;
        CACTI_REQUIRE(e.off <= e.eoff && e.eoff <= rec->second.data_off + rec->second.size &&
                          rec->second.data_off + rec->second.size <= mf.size,
                      CACTI_E_FORMAT, "pickle_dir: %s: tensor %s: byte range outside its record", path.c_str(), nm);
        // the reference insists on 64-byte alignment of the first byte (src/util/safepickle.rs:167-177)
        CACTI_REQUIRE(e.off % 64 == 0, CACTI_E_FORMAT, "pickle_dir: %s: tensor %s starts at byte %llu, not 64-byte aligned",
                      path.c_str(), nm, (unsigned long long)e.off);
        // PickleDirErr::DuplicateName
        CACTI_REQUIRE(d->tensors.find(name) == d->tensors.end(), CACTI_E_FORMAT, "pickle_dir: duplicate tensor name %s (in %s)", nm,
                      path.c_str());
        d->serial_key.push_back(name);
        d->tensors.emplace(name, std::move(e));
    }
    return 0;
}

}  // namespace

CACTI_API int cacti_pickle_dir_open(const char *path, const char *prefix, cacti_tensors_dir **out)
{
    CACTI_REQUIRE(path && out, CACTI_E_INVALID, "pickle_dir_open: null argument");
    *out = nullptr;
    const std::string pre = prefix && prefix[0] ? prefix : "pytorch_model";
    std::vector<std::string> files;
    struct stat st;
    CACTI_REQUIRE(stat(path, &st) == 0, CACTI_E_IO, "pickle_dir_open: %s does not exist", path);
    if (S_ISREG(st.st_mode)) {
        files.push_back(path);
    } else {
        // <prefix>.bin, else the sorted shards <prefix>-*-of-*.bin (src/util/safepickle.rs:77-99)
        const std::string one = std::string(path) + "/" + pre + ".bin";
        if (stat(one.c_str(), &st) == 0) {
            files.push_back(one);
        } else {
            glob_t g;
            memset(&g, 0, sizeof(g));
            const std::string patt = std::string(path) + "/" + pre + "-*-of-*.bin";
            if (glob(patt.c_str(), 0, nullptr, &g) == 0)
                for (size_t i = 0; i < g.gl_pathc; i++) files.push_back(g.gl_pathv[i]);
            globfree(&g);
            std::sort(files.begin(), files.end());
            CACTI_REQUIRE(!files.empty(), CACTI_E_IO, "pickle_dir_open: %s holds neither %s.bin nor %s-*-of-*.bin", path, pre.c_str(),
                          pre.c_str());
        }
    }
    cacti_tensors_dir *d = new cacti_tensors_dir();
    d->path = path;
    for (const std::string &f : files) {
        const int rc = add_pickle_file(d, f);
        if (rc) {
            delete d;
            return rc;
        }
    }
    for (auto &kv : d->tensors) d->sorted.push_back(&kv.first);
    *out = d;
    return 0;
}
