// Configuration read from the environment, and the two driver-level handles the reference's FFI
// crate exposes beside streams and events: the device's primary context and the null stream.
//
//   cacti_parse_byte_size     src/algo/str/parse_size.rs:262-400 (default configuration)
//   cacti_vmem_soft_limit     NvGpuMemPool::new, src/pctx/nvgpu.rs:1434-1463
//   CACTI_VMEM_SOFT_LIMIT,
//   CACTI_NVGPU_MEM_ALLOC     cacti_cfg_env/src/lib.rs:107-112, src/pctx/nvgpu.rs:995-1002
//   primary context           cacti_gpu_cu_ffi/src/lib.rs:158-199
//   null stream               cacti_gpu_cu_ffi/src/lib.rs:511-515
#include <hip/hip_runtime.h>
#include <stdlib.h>
#include <string.h>

#include <string>

#include "../../include/cacti_hip_runtime.h"
#include "common.h"

namespace {

// 10^k for the prefix letters; 2^(10 k) after an 'i'
bool prefix_factor(char c, bool binary, uint64_t *f)
{
    static const char kLetters[] = "kmgtpe";
    const char *at = c ? strchr(kLetters, c | 0x20) : nullptr;
    if (!at) return false;
    const int k = (int)(at - kLetters) + 1;
    uint64_t v = 1;
    for (int i = 0; i < k; i++) v *= binary ? 1024u : 1000u;
    *f = v;
    return true;
}

}  // namespace

// status: 0, or CACTI_E_INVALID with the reason in the error text (empty, invalid digit, overflow)
CACTI_API int cacti_parse_byte_size(const char *text, uint64_t *bytes)
{
    CACTI_REQUIRE(text && bytes, CACTI_E_INVALID, "parse_byte_size: null argument");
    size_t n = strlen(text);
    // from the back: an optional B, an optional i (then the prefix is a power of 1024), an optional prefix
    uint64_t unit = 1;
    if (n && (text[n - 1] | 0x20) == 'b') n--;
    bool binary = false;
    if (n && (text[n - 1] | 0x20) == 'i') {
        binary = true;
        n--;
    }
    if (n && prefix_factor(text[n - 1], binary, &unit)) n--;
    // the number: digits [. digits] [e [+-] digits]; blanks and underscores anywhere.  The mantissa
    // keeps the digits that fit 64 bits (the first one dropped rounds it) and the rest only move the
    // decimal point.
    uint64_t mant = 0;
    int64_t point = 0, expo = 0;                  // value = mant * 10^(point + expo)
    enum { EMPTY, INT, INT_FULL, FRAC, FRAC_FULL, EXP_POS, EXP_NEG } st = EMPTY;
    for (size_t i = 0; i < n; i++) {
        const char c = text[i];
        if (c == '_' || c == ' ') continue;
        const bool digit = c >= '0' && c <= '9';
        const uint64_t d = (uint64_t)(c - '0');
        if (digit && (st == EMPTY || st == INT || st == FRAC)) {
            if (mant <= (UINT64_MAX - d) / 10) {
                mant = mant * 10 + d;
                if (st == FRAC) point--;
                else st = INT;
            } else {
                if (d >= 5) mant++;
                if (st == FRAC) st = FRAC_FULL;
                else { st = INT_FULL; point++; }
            }
        } else if (digit && st == INT_FULL) {
            point++;
        } else if (digit && st == FRAC_FULL) {
        } else if (digit && st == EXP_POS) {
            CACTI_REQUIRE(expo <= (INT32_MAX - (int64_t)d) / 10, CACTI_E_INVALID, "parse_byte_size: %s: number too large", text);
            expo = expo * 10 + (int64_t)d;
        } else if (digit && st == EXP_NEG) {
            if (expo >= (INT32_MIN + (int64_t)d) / 10) expo = expo * 10 - (int64_t)d;
        } else if ((c | 0x20) == 'e' && (st == INT || st == FRAC || st == INT_FULL || st == FRAC_FULL)) {
            st = EXP_POS;
        } else if (c == '+' && st == EXP_POS) {
        } else if (c == '-' && st == EXP_POS) {
            st = EXP_NEG;
        } else if (c == '.' && st == INT) {
            st = FRAC;
        } else if (c == '.' && st == INT_FULL) {
            st = FRAC_FULL;
        } else {
            CACTI_REQUIRE(false, CACTI_E_INVALID, "parse_byte_size: %s: invalid digit", text);
        }
    }
    CACTI_REQUIRE(st != EMPTY, CACTI_E_INVALID, "parse_byte_size: %s: no number", text);
    const int64_t e = expo + point;
    if (e >= 0) {
        uint64_t scale = unit;
        for (int64_t i = 0; i < e; i++)
            CACTI_REQUIRE(!__builtin_mul_overflow(scale, (uint64_t)10, &scale), CACTI_E_INVALID,
                          "parse_byte_size: %s: number too large", text);
        CACTI_REQUIRE(!__builtin_mul_overflow(mant, scale, bytes), CACTI_E_INVALID, "parse_byte_size: %s: number too large", text);
    } else if (e >= -38) {
        unsigned __int128 p = 1;
        for (int64_t i = 0; i < -e; i++) p *= 10;
        const unsigned __int128 r = ((unsigned __int128)mant * unit + p / 2) / p;      // to nearest, halves up
        CACTI_REQUIRE(r <= UINT64_MAX, CACTI_E_INVALID, "parse_byte_size: %s: number too large", text);
        *bytes = (uint64_t)r;
    } else {
        *bytes = 0;
    }
    return 0;
}

// The size of the device reserve.  text = NULL or "": the default, 90.01 % of the device rounded up,
// then down to 64 KiB.  A text that reads as a decimal number is a fraction of the device, held to
// [0, 1] and to what is available less 32 MiB; otherwise a byte size; a text that is neither leaves
// the default.  (A plain integer reads as a decimal number: "8589934592" is the fraction 1, "8GiB"
// is eight gibibytes -- the reference's rule.)
CACTI_API int cacti_vmem_soft_limit(const char *text, size_t avail, size_t total, size_t *reserve)
{
    CACTI_REQUIRE(reserve, CACTI_E_INVALID, "vmem_soft_limit: null out pointer");
    size_t r = (size_t)(((unsigned __int128)total * 9001 + 9999) / 10000);
    if (text && text[0]) {
        uint64_t b = 0;
        const bool is_size = cacti_parse_byte_size(text, &b) == 0;
        char *end = nullptr;
        const double f = strtod(text, &end);
        // (what a decimal floating-point literal is: no blanks in front, no hexadecimal form)
        const bool is_frac = end != text && *end == 0 && !strchr(" \t\n\v\f\r", text[0]) && !strpbrk(text, "xX");
        if (is_frac) {
            double v = (double)total * (f > 1 ? 1 : f > 0 ? f : 0);               // not-a-number counts as 0
            const double room = (double)avail - 32.0 * 1024.0 * 1024.0;
            if (v > room) v = room;
            r = v > 0 ? (size_t)v : 0;
        } else if (is_size) {
            r = (size_t)b;
        }
    }
    *reserve = (r >> 16) << 16;
    return 0;
}

// 1 = page-locked host memory for spilled cells, 0 = malloc: "pagelocked" in CACTI_NVGPU_MEM_ALLOC
// (the reference's name; CACTI_GPU_MEM_ALLOC is read first), anything else or unset = malloc.
CACTI_API int cacti_env_host_pagelocked(void)
{
    const char *e = getenv("CACTI_GPU_MEM_ALLOC");
    if (!e) e = getenv("CACTI_NVGPU_MEM_ALLOC");
    return e && strcmp(e, "pagelocked") == 0;
}

// The primary-context calls below are the ones the reference's CudaPrimaryCtx binds (cacti_gpu_cu_ffi/src/lib.rs:
// 158-199); HIP marks them deprecated and keeps them working, and they are wanted here under exactly these names.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wdeprecated-declarations"
CACTI_API int cacti_hip_primary_ctx_retain(int dev, void **pctx)
{
    CACTI_REQUIRE(pctx, CACTI_E_INVALID, "primary_ctx_retain: null out pointer");
    hipCtx_t c = nullptr;
    CACTI_HIP(hipDevicePrimaryCtxRetain(&c, dev));
    *pctx = c;
    return 0;
}
CACTI_API int cacti_hip_primary_ctx_release(int dev)
{
    CACTI_HIP(hipDevicePrimaryCtxRelease(dev));
    return 0;
}
CACTI_API int cacti_hip_primary_ctx_set_flags(int dev, unsigned flags)
{
    CACTI_HIP(hipDevicePrimaryCtxSetFlags(dev, flags));
    return 0;
}
CACTI_API int cacti_hip_primary_ctx_reset(int dev)
{
    using namespace cacti;
    CACTI_REQUIRE(live_contexts(dev) == 0, CACTI_E_STATE,
                  "primary_ctx_reset: %d device context(s) of this library are alive on device %d; destroy "
                  "them first (a reset frees their pool, streams and events)", live_contexts(dev), dev);
    CACTI_HIP(hipDevicePrimaryCtxReset(dev));
    module_epoch_advance();        // function attributes and symbol addresses are looked up again
    return 0;
}

// The null stream: the handle every entry point accepts for "the device's default stream".
#pragma clang diagnostic pop

CACTI_API void *cacti_hip_stream_null(void) { return nullptr; }
