#include "code_object.h"

#include <cstring>
#include <string_view>

#include <dlfcn.h>

namespace xsched::hip::codeobj
{

namespace
{

// ---- bounded little-endian reads ---------------------------------------------------------

struct Span
{
    const uint8_t *p = nullptr;
    size_t n = 0;

    bool Has(size_t off, size_t len) const { return off <= n && len <= n - off; }
    template <typename T> bool Get(size_t off, T *v) const
    {
        if (!Has(off, sizeof(T))) return false;
        memcpy(v, p + off, sizeof(T)); // x86-64 and the code object are both little-endian
        return true;
    }
    Span Sub(size_t off, size_t len) const { return Has(off, len) ? Span { p + off, len } : Span {}; }
};

constexpr size_t kUnbounded = ~(size_t)0 >> 1;

// ---- MessagePack -------------------------------------------------------------------------

// The subset of the format the metadata uses is all of it except extension types, which
// are skipped like any other value. Every read checks the remaining length; `ok` turns
// false for good at the first violation.
class MsgReader
{
public:
    explicit MsgReader(Span s): cur_(s.p), end_(s.p + s.n) {}
    bool ok = true;

    bool MapHeader(uint32_t *n) { return Container(0x80, 0x8F, 0xDE, n); }
    bool ArrayHeader(uint32_t *n) { return Container(0x90, 0x9F, 0xDC, n); }

    bool Str(std::string_view *s)
    {
        uint8_t t;
        if (!Peek(&t)) return false;
        size_t len;
        if (t >= 0xA0 && t <= 0xBF) { ++cur_; len = t & 0x1F; }
        else if (t == 0xD9) { ++cur_; uint8_t v; if (!Raw(&v)) return false; len = v; }
        else if (t == 0xDA) { ++cur_; uint16_t v; if (!Big(&v)) return false; len = v; }
        else if (t == 0xDB) { ++cur_; uint32_t v; if (!Big(&v)) return false; len = v; }
        else return false; // not a string: nothing consumed
        if (!Room(len)) return false;
        *s = std::string_view((const char *)cur_, len);
        cur_ += len;
        return true;
    }

    bool UInt(uint64_t *v)
    {
        uint8_t t;
        if (!Peek(&t)) return false;
        if (t <= 0x7F) { ++cur_; *v = t; return true; }
        if (t == 0xCC || t == 0xD0) { ++cur_; uint8_t x; if (!Raw(&x)) return false; *v = x; return t == 0xCC || x < 0x80; }
        if (t == 0xCD || t == 0xD1) { ++cur_; uint16_t x; if (!Big(&x)) return false; *v = x; return t == 0xCD || x < 0x8000; }
        if (t == 0xCE || t == 0xD2) { ++cur_; uint32_t x; if (!Big(&x)) return false; *v = x; return t == 0xCE || x < 0x80000000u; }
        if (t == 0xCF || t == 0xD3) { ++cur_; uint64_t x; if (!Big(&x)) return false; *v = x; return t == 0xCF || x < (1ull << 63); }
        return false; // negative or not an integer: nothing consumed
    }

    /// Steps over one value of any type.
    bool Skip(int depth = 0)
    {
        if (depth > 32) return Fail();
        uint8_t t;
        if (!Peek(&t)) return false;
        uint32_t n;
        if ((t >= 0x80 && t <= 0x8F) || t == 0xDE || t == 0xDF) {
            if (!MapHeader(&n)) return false;
            for (uint32_t i = 0; i < n; ++i) if (!Skip(depth + 1) || !Skip(depth + 1)) return false;
            return true;
        }
        if ((t >= 0x90 && t <= 0x9F) || t == 0xDC || t == 0xDD) {
            if (!ArrayHeader(&n)) return false;
            for (uint32_t i = 0; i < n; ++i) if (!Skip(depth + 1)) return false;
            return true;
        }
        if ((t >= 0xA0 && t <= 0xBF) || (t >= 0xD9 && t <= 0xDB)) { std::string_view s; return Str(&s); }
        ++cur_;
        if (t <= 0x7F || t >= 0xE0 || t == 0xC0 || t == 0xC2 || t == 0xC3) return true;
        switch (t) {
        case 0xCC: case 0xD0: return Advance(1);
        case 0xCD: case 0xD1: return Advance(2);
        case 0xCE: case 0xD2: case 0xCA: return Advance(4);
        case 0xCF: case 0xD3: case 0xCB: return Advance(8);
        case 0xC4: { uint8_t v; return Raw(&v) && Advance(v); }              // bin 8
        case 0xC5: { uint16_t v; return Big(&v) && Advance(v); }             // bin 16
        case 0xC6: { uint32_t v; return Big(&v) && Advance(v); }             // bin 32
        case 0xC7: { uint8_t v; return Raw(&v) && Advance((size_t)v + 1); }  // ext 8: type byte + data
        case 0xC8: { uint16_t v; return Big(&v) && Advance((size_t)v + 1); } // ext 16
        case 0xC9: { uint32_t v; return Big(&v) && Advance((size_t)v + 1); } // ext 32
        case 0xD4: return Advance(2);                                        // fixext 1
        case 0xD5: return Advance(3);
        case 0xD6: return Advance(5);
        case 0xD7: return Advance(9);
        case 0xD8: return Advance(17);
        default: return Fail();                                              // 0xC1 is never used
        }
    }

private:
    bool Fail() { ok = false; return false; }
    bool Room(size_t len) { return (size_t)(end_ - cur_) >= len ? true : Fail(); }
    bool Peek(uint8_t *t) { if (!ok || !Room(1)) return false; *t = *cur_; return true; }
    bool Advance(size_t len) { if (!Room(len)) return false; cur_ += len; return true; }
    bool Raw(uint8_t *v) { if (!Room(1)) return false; *v = *cur_++; return true; }
    template <typename T> bool Big(T *v)
    {
        if (!Room(sizeof(T))) return false;
        T x = 0;
        for (size_t i = 0; i < sizeof(T); ++i) x = (T)((x << 8) | cur_[i]);
        cur_ += sizeof(T);
        *v = x;
        return true;
    }
    // fix form [lo, hi]; 16-bit form at `wide`, 32-bit form at `wide + 1`
    bool Container(uint8_t lo, uint8_t hi, uint8_t wide, uint32_t *n)
    {
        uint8_t t;
        if (!Peek(&t)) return false;
        if (t >= lo && t <= hi) { ++cur_; *n = t & 0x0F; return true; }
        if (t == wide) { ++cur_; uint16_t v; if (!Big(&v)) return false; *n = v; return true; }
        if (t == (uint8_t)(wide + 1)) { ++cur_; uint32_t v; if (!Big(&v)) return false; *n = v; return true; }
        return false; // another type: nothing consumed
    }

    const uint8_t *cur_;
    const uint8_t *end_;
};

bool ReadArg(MsgReader &r, KernelArg *arg, bool *hidden)
{
    uint32_t fields;
    if (!r.MapHeader(&fields)) return false;
    bool have_offset = false, have_size = false;
    *hidden = false;
    for (uint32_t f = 0; f < fields; ++f) {
        std::string_view key;
        if (!r.Str(&key)) { if (!r.Skip() || !r.Skip()) return false; continue; }
        uint64_t v;
        std::string_view kind;
        if (key == ".offset") { if (!r.UInt(&v)) return false; arg->offset = (uint32_t)v; have_offset = true; }
        else if (key == ".size") { if (!r.UInt(&v)) return false; arg->size = (uint32_t)v; have_size = true; }
        else if (key == ".value_kind") { if (!r.Str(&kind)) return false; *hidden = kind.substr(0, 7) == "hidden_"; }
        else if (!r.Skip()) return false;
    }
    return have_offset && have_size;
}

bool ReadKernel(MsgReader &r, KernelLayout *k)
{
    uint32_t fields;
    if (!r.MapHeader(&fields)) return false;
    for (uint32_t f = 0; f < fields; ++f) {
        std::string_view key;
        if (!r.Str(&key)) { if (!r.Skip() || !r.Skip()) return false; continue; }
        if (key == ".name") {
            std::string_view name;
            if (!r.Str(&name)) return false;
            k->name = std::string(name);
        } else if (key == ".kernarg_segment_size") {
            uint64_t v;
            if (!r.UInt(&v)) return false;
            k->kernarg_bytes = (uint32_t)v;
        } else if (key == ".args") {
            uint32_t n;
            if (!r.ArrayHeader(&n)) return false;
            for (uint32_t i = 0; i < n; ++i) {
                KernelArg arg;
                bool hidden;
                if (!ReadArg(r, &arg, &hidden)) return false;
                if (!hidden) k->args.push_back(arg);
            }
        } else if (!r.Skip()) {
            return false;
        }
    }
    return !k->name.empty();
}

ParseStatus ReadMetadata(Span note, std::vector<KernelLayout> *out)
{
    MsgReader r(note);
    uint32_t fields;
    if (!r.MapHeader(&fields)) return ParseStatus::kMalformed;
    for (uint32_t f = 0; f < fields; ++f) {
        std::string_view key;
        if (!r.Str(&key)) { if (!r.Skip() || !r.Skip()) return ParseStatus::kMalformed; continue; }
        if (key != "amdhsa.kernels") { if (!r.Skip()) return ParseStatus::kMalformed; continue; }
        uint32_t n;
        if (!r.ArrayHeader(&n)) return ParseStatus::kMalformed;
        for (uint32_t i = 0; i < n; ++i) {
            KernelLayout k;
            if (!ReadKernel(r, &k)) return ParseStatus::kMalformed;
            out->push_back(std::move(k));
        }
    }
    return r.ok ? ParseStatus::kOk : ParseStatus::kMalformed;
}

// ---- ELF ---------------------------------------------------------------------------------

constexpr uint32_t kPtNote = 4;
constexpr uint32_t kNtAmdgpuMetadata = 32;

ParseStatus ReadElf(Span elf, std::vector<KernelLayout> *out)
{
    uint8_t klass = 0, data = 0;
    if (!elf.Get(4, &klass) || !elf.Get(5, &data)) return ParseStatus::kMalformed;
    if (klass != 2 || data != 1) return ParseStatus::kNotCodeObject; // 64-bit little-endian only
    uint64_t phoff;
    uint16_t phentsize, phnum;
    if (!elf.Get(0x20, &phoff) || !elf.Get(0x36, &phentsize) || !elf.Get(0x38, &phnum)) return ParseStatus::kMalformed;
    if (phentsize < 56) return phnum == 0 ? ParseStatus::kNoMetadata : ParseStatus::kMalformed;
    for (uint16_t i = 0; i < phnum; ++i) {
        const size_t ph = phoff + (size_t)i * phentsize;
        uint32_t type;
        uint64_t offset, filesz;
        if (!elf.Get(ph, &type) || !elf.Get(ph + 8, &offset) || !elf.Get(ph + 32, &filesz)) return ParseStatus::kMalformed;
        if (type != kPtNote) continue;
        if (!elf.Has(offset, filesz)) return ParseStatus::kMalformed;
        const Span notes = elf.Sub(offset, filesz);
        size_t at = 0;
        while (at + 12 <= notes.n) {
            uint32_t namesz = 0, descsz = 0, ntype = 0;
            notes.Get(at, &namesz); notes.Get(at + 4, &descsz); notes.Get(at + 8, &ntype);
            const size_t name_at = at + 12;
            const size_t desc_at = name_at + (((size_t)namesz + 3) & ~(size_t)3);
            if (!notes.Has(name_at, namesz) || !notes.Has(desc_at, descsz)) return ParseStatus::kMalformed;
            const bool amdgpu = namesz >= 6 && memcmp(notes.p + name_at, "AMDGPU", 6) == 0 &&
                                (namesz == 6 || notes.p[name_at + 6] == 0);
            if (amdgpu && ntype == kNtAmdgpuMetadata) return ReadMetadata(notes.Sub(desc_at, descsz), out);
            at = desc_at + (((size_t)descsz + 3) & ~(size_t)3);
        }
    }
    return ParseStatus::kNoMetadata;
}

// ---- clang offload bundle ------------------------------------------------------------------

constexpr char kBundleMagic[] = "__CLANG_OFFLOAD_BUNDLE__"; // 24 characters
constexpr char kCompressedMagic[] = "CCOB";

ParseStatus ReadBundle(Span image, const char *arch, std::vector<KernelLayout> *out)
{
    uint64_t entries;
    if (!image.Get(24, &entries)) return ParseStatus::kMalformed;
    if (entries > 4096) return ParseStatus::kMalformed;
    size_t at = 32;
    Span chosen, fallback;
    for (uint64_t i = 0; i < entries; ++i) {
        uint64_t offset, size, triple_len;
        if (!image.Get(at, &offset) || !image.Get(at + 8, &size) || !image.Get(at + 16, &triple_len)) return ParseStatus::kMalformed;
        if (!image.Has(at + 24, triple_len)) return ParseStatus::kMalformed;
        const std::string_view triple((const char *)image.p + at + 24, triple_len);
        at += 24 + triple_len;
        if (triple.find("amdgcn") == std::string_view::npos || size == 0) continue;
        if (!image.Has(offset, size)) return ParseStatus::kMalformed;
        if (fallback.p == nullptr) fallback = image.Sub(offset, size);
        if (chosen.p == nullptr && arch != nullptr && *arch != 0 && triple.find(arch) != std::string_view::npos) {
            chosen = image.Sub(offset, size);
        }
    }
    if (chosen.p == nullptr) chosen = fallback;
    if (chosen.p == nullptr) return ParseStatus::kNoDeviceImage;
    if (chosen.n < 4 || memcmp(chosen.p, "\177ELF", 4) != 0) return ParseStatus::kNotCodeObject;
    return ReadElf(chosen, out);
}

// ---- compressed offload bundle ----------------------------------------------------------------

// Header written by clang's offload bundler in front of the compressed bytes of a whole
// bundle (clang/lib/Driver/OffloadBundler.cpp, CompressedOffloadBundle):
//   "CCOB", u16 version, u16 method (0 zlib, 1 zstd), then
//   version 1:                u32 uncompressed size, u64 hash            (20 bytes)
//   version 2: u32 file size, u32 uncompressed size, u64 hash            (24 bytes)
//   version 3: u64 file size, u64 uncompressed size, u64 hash            (32 bytes)
// The decompressors are taken from the system's libzstd / libz at run time; a machine without
// them reads such images as "compressed", which callers handle.
typedef size_t (*ZstdDecompressFn)(void *dst, size_t dst_cap, const void *src, size_t src_size);
typedef unsigned (*ZstdIsErrorFn)(size_t code);
typedef int (*ZlibUncompressFn)(unsigned char *dst, unsigned long *dst_len, const unsigned char *src, unsigned long src_len);

bool Decompress(uint16_t method, Span in, std::vector<uint8_t> *out)
{
    if (method == 1) {
        static void *lib = dlopen("libzstd.so.1", RTLD_NOW | RTLD_LOCAL);
        static auto decompress = lib ? (ZstdDecompressFn)dlsym(lib, "ZSTD_decompress") : nullptr;
        static auto is_error = lib ? (ZstdIsErrorFn)dlsym(lib, "ZSTD_isError") : nullptr;
        if (decompress == nullptr || is_error == nullptr) return false;
        const size_t n = decompress(out->data(), out->size(), in.p, in.n);
        return !is_error(n) && n == out->size();
    }
    if (method == 0) {
        static void *lib = dlopen("libz.so.1", RTLD_NOW | RTLD_LOCAL);
        static auto uncompress = lib ? (ZlibUncompressFn)dlsym(lib, "uncompress") : nullptr;
        if (uncompress == nullptr) return false;
        unsigned long n = out->size();
        return uncompress(out->data(), &n, in.p, in.n) == 0 && n == out->size();
    }
    return false;
}

ParseStatus ReadCompressed(Span image, const char *arch, std::vector<KernelLayout> *out)
{
    uint16_t version, method;
    if (!image.Get(4, &version) || !image.Get(6, &method)) return ParseStatus::kMalformed;
    size_t header, file_size = 0, raw_size;
    if (version == 1) {
        uint32_t raw;
        if (!image.Get(8, &raw)) return ParseStatus::kMalformed;
        header = 20; raw_size = raw;
    } else if (version == 2) {
        uint32_t file, raw;
        if (!image.Get(8, &file) || !image.Get(12, &raw)) return ParseStatus::kMalformed;
        header = 24; file_size = file; raw_size = raw;
    } else if (version == 3) {
        uint64_t file, raw;
        if (!image.Get(8, &file) || !image.Get(16, &raw)) return ParseStatus::kMalformed;
        header = 32; file_size = file; raw_size = raw;
    } else {
        return ParseStatus::kCompressed;
    }
    size_t packed;
    if (file_size != 0) {
        if (file_size < header || !image.Has(0, file_size)) return ParseStatus::kMalformed;
        packed = file_size - header;
    } else {
        if (image.n == kUnbounded) return ParseStatus::kCompressed; // version 1 does not say where it ends
        if (image.n < header) return ParseStatus::kMalformed;
        packed = image.n - header;
    }
    // A damaged header must not make this allocate gigabytes: a bundle unpacks to at most a few
    // hundred MB, and the formats at hand do not pack better than 256 : 1.
    if (raw_size == 0 || raw_size > ((size_t)1 << 30) || raw_size / 256 > packed) return ParseStatus::kMalformed;
    std::vector<uint8_t> raw(raw_size);
    if (!Decompress(method, image.Sub(header, packed), &raw)) return ParseStatus::kCompressed;
    const Span plain { raw.data(), raw.size() };
    if (plain.Has(0, 24) && memcmp(plain.p, kBundleMagic, 24) == 0) return ReadBundle(plain, arch, out);
    return ParseStatus::kNotCodeObject;
}

} // namespace

const char *ToString(ParseStatus status)
{
    switch (status) {
    case ParseStatus::kOk: return "ok";
    case ParseStatus::kNotCodeObject: return "not a code object";
    case ParseStatus::kCompressed: return "compressed offload bundle that could not be unpacked";
    case ParseStatus::kNoDeviceImage: return "bundle without an amdgcn image";
    case ParseStatus::kNoMetadata: return "no AMDGPU metadata note";
    case ParseStatus::kMalformed: return "malformed image";
    }
    return "?";
}

ParseStatus ReadKernelLayouts(const void *image, size_t bytes, const char *arch,
                              std::vector<KernelLayout> *out)
{
    if (image == nullptr || out == nullptr) return ParseStatus::kNotCodeObject;
    const Span all { (const uint8_t *)image, bytes == 0 ? kUnbounded : bytes };
    if (!all.Has(0, 4)) return ParseStatus::kNotCodeObject;
    if (memcmp(all.p, kCompressedMagic, 4) == 0) return ReadCompressed(all, arch, out);
    if (memcmp(all.p, "\177ELF", 4) == 0) return ReadElf(all, out);
    if (all.Has(0, 24) && memcmp(all.p, kBundleMagic, 24) == 0) return ReadBundle(all, arch, out);
    return ParseStatus::kNotCodeObject;
}

} // namespace xsched::hip::codeobj
