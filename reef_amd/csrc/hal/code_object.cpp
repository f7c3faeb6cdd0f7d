#include "hal/code_object.h"

#include <elf.h>

#include <cstdio>
#include <cstring>
#include <vector>

namespace reef {
namespace hal {
namespace {

// ---- MessagePack cursor: just enough to walk the AMDGPU metadata ---------------
struct Mp {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;

    uint64_t be(int n) {
        uint64_t v = 0;
        if (p + n > end) { ok = false; return 0; }
        for (int i = 0; i < n; ++i) v = (v << 8) | *p++;
        return v;
    }
    // Kinds: 0 nil/bool/other scalar, 1 int, 2 str, 3 array, 4 map
    struct Tok { int kind; int64_t ival; const char* s; uint32_t len; };
    Tok next() {
        Tok t{0, 0, nullptr, 0};
        if (p >= end) { ok = false; return t; }
        uint8_t b = *p++;
        if (b <= 0x7f) { t.kind = 1; t.ival = b; }
        else if (b >= 0xe0) { t.kind = 1; t.ival = (int8_t)b; }
        else if ((b & 0xf0) == 0x80) { t.kind = 4; t.len = b & 0x0f; }
        else if ((b & 0xf0) == 0x90) { t.kind = 3; t.len = b & 0x0f; }
        else if ((b & 0xe0) == 0xa0) { t.kind = 2; t.len = b & 0x1f; str(t); }
        else switch (b) {
            case 0xc0: case 0xc2: case 0xc3: break;
            case 0xc4: { uint32_t n = (uint32_t)be(1); skip(n); break; }       // bin8
            case 0xc5: { uint32_t n = (uint32_t)be(2); skip(n); break; }
            case 0xc6: { uint32_t n = (uint32_t)be(4); skip(n); break; }
            case 0xca: skip(4); break;                                         // float32
            case 0xcb: skip(8); break;
            case 0xcc: t.kind = 1; t.ival = (int64_t)be(1); break;
            case 0xcd: t.kind = 1; t.ival = (int64_t)be(2); break;
            case 0xce: t.kind = 1; t.ival = (int64_t)be(4); break;
            case 0xcf: t.kind = 1; t.ival = (int64_t)be(8); break;
            case 0xd0: t.kind = 1; t.ival = (int8_t)be(1); break;
            case 0xd1: t.kind = 1; t.ival = (int16_t)be(2); break;
            case 0xd2: t.kind = 1; t.ival = (int32_t)be(4); break;
            case 0xd3: t.kind = 1; t.ival = (int64_t)be(8); break;
            case 0xd9: t.kind = 2; t.len = (uint32_t)be(1); str(t); break;
            case 0xda: t.kind = 2; t.len = (uint32_t)be(2); str(t); break;
            case 0xdb: t.kind = 2; t.len = (uint32_t)be(4); str(t); break;
            case 0xdc: t.kind = 3; t.len = (uint32_t)be(2); break;
            case 0xdd: t.kind = 3; t.len = (uint32_t)be(4); break;
            case 0xde: t.kind = 4; t.len = (uint32_t)be(2); break;
            case 0xdf: t.kind = 4; t.len = (uint32_t)be(4); break;
            default: ok = false; break;  // ext types do not occur in this metadata
        }
        return t;
    }
    void str(Tok& t) {
        if (p + t.len > end) { ok = false; t.len = 0; return; }
        t.s = (const char*)p;
        p += t.len;
    }
    void skip(uint32_t n) {
        if (p + n > end) { ok = false; return; }
        p += n;
    }
    // Skip one whole value (recursively).
    void skip_value() {
        Tok t = next();
        if (!ok) return;
        if (t.kind == 3) for (uint32_t i = 0; i < t.len && ok; ++i) skip_value();
        else if (t.kind == 4) for (uint32_t i = 0; i < t.len && ok; ++i) { skip_value(); skip_value(); }
    }
};

bool key_is(const Mp::Tok& t, const char* k) {
    return t.kind == 2 && t.len == std::strlen(k) && std::memcmp(t.s, k, t.len) == 0;
}

bool parse_metadata(const uint8_t* b, size_t n, std::map<std::string, KernelMeta>* out) {
    Mp mp{b, b + n};
    Mp::Tok root = mp.next();
    if (!mp.ok || root.kind != 4) return false;
    for (uint32_t i = 0; i < root.len && mp.ok; ++i) {
        Mp::Tok k = mp.next();
        if (!key_is(k, "amdhsa.kernels")) { mp.skip_value(); continue; }
        Mp::Tok arr = mp.next();
        if (arr.kind != 3) return false;
        for (uint32_t j = 0; j < arr.len && mp.ok; ++j) {
            Mp::Tok km = mp.next();
            if (km.kind != 4) return false;
            KernelMeta meta;
            std::string name;
            for (uint32_t f = 0; f < km.len && mp.ok; ++f) {
                Mp::Tok fk = mp.next();
                if (key_is(fk, ".name")) { Mp::Tok v = mp.next(); name.assign(v.s ? v.s : "", v.len); }
                else if (key_is(fk, ".vgpr_count")) meta.vgprs = (int)mp.next().ival;
                else if (key_is(fk, ".agpr_count")) meta.agprs = (int)mp.next().ival;
                else if (key_is(fk, ".sgpr_count")) meta.sgprs = (int)mp.next().ival;
                else if (key_is(fk, ".group_segment_fixed_size")) meta.lds = (int)mp.next().ival;
                else if (key_is(fk, ".private_segment_fixed_size")) meta.scratch = (int)mp.next().ival;
                else if (key_is(fk, ".kernarg_segment_size")) meta.kernarg = (int)mp.next().ival;
                else if (key_is(fk, ".max_flat_workgroup_size")) meta.max_threads = (int)mp.next().ival;
                else mp.skip_value();
            }
            if (!name.empty()) (*out)[name] = meta;
        }
    }
    return mp.ok;
}

bool parse_elf(const uint8_t* b, size_t n, std::map<std::string, KernelMeta>* out, std::string* err) {
    if (n < sizeof(Elf64_Ehdr) || std::memcmp(b, ELFMAG, SELFMAG) != 0 || b[EI_CLASS] != ELFCLASS64) {
        *err = "not an ELF64 code object";
        return false;
    }
    const Elf64_Ehdr* eh = (const Elf64_Ehdr*)b;
    if (eh->e_shoff == 0 || eh->e_shoff + (uint64_t)eh->e_shnum * sizeof(Elf64_Shdr) > n) {
        *err = "bad section table";
        return false;
    }
    const Elf64_Shdr* sh = (const Elf64_Shdr*)(b + eh->e_shoff);
    for (int i = 0; i < eh->e_shnum; ++i) {
        if (sh[i].sh_type != SHT_NOTE) continue;
        if (sh[i].sh_offset + sh[i].sh_size > n) continue;
        const uint8_t* p = b + sh[i].sh_offset;
        const uint8_t* e = p + sh[i].sh_size;
        while (p + sizeof(Elf64_Nhdr) <= e) {
            const Elf64_Nhdr* nh = (const Elf64_Nhdr*)p;
            const uint8_t* name = p + sizeof(Elf64_Nhdr);
            const uint8_t* desc = name + ((nh->n_namesz + 3) & ~3u);
            if (desc + nh->n_descsz > e) break;
            if (nh->n_type == 32 && nh->n_namesz >= 6 && std::memcmp(name, "AMDGPU", 6) == 0) {
                if (parse_metadata(desc, nh->n_descsz, out)) return true;
            }
            p = desc + ((nh->n_descsz + 3) & ~3u);
        }
    }
    *err = "no AMDGPU metadata note";
    return false;
}

}  // namespace

bool read_code_object_metadata(const char* path, std::map<std::string, KernelMeta>* out,
                               std::string* err) {
    std::string dummy;
    if (!err) err = &dummy;
    FILE* fp = std::fopen(path, "rb");
    if (!fp) { *err = std::string("cannot open ") + path; return false; }
    std::fseek(fp, 0, SEEK_END);
    long sz = std::ftell(fp);
    std::fseek(fp, 0, SEEK_SET);
    std::vector<uint8_t> buf(sz > 0 ? (size_t)sz : 0);
    size_t got = buf.empty() ? 0 : std::fread(buf.data(), 1, buf.size(), fp);
    std::fclose(fp);
    if (got != buf.size() || buf.size() < 32) { *err = "short read"; return false; }

    static const char kBundle[] = "__CLANG_OFFLOAD_BUNDLE__";
    if (std::memcmp(buf.data(), kBundle, 24) == 0) {
        uint64_t n;
        std::memcpy(&n, buf.data() + 24, 8);
        size_t off = 32;
        for (uint64_t i = 0; i < n && off + 24 <= buf.size(); ++i) {
            uint64_t o, s, ts;
            std::memcpy(&o, buf.data() + off, 8);
            std::memcpy(&s, buf.data() + off + 8, 8);
            std::memcpy(&ts, buf.data() + off + 16, 8);
            off += 24;
            if (off + ts > buf.size()) break;
            std::string triple((const char*)buf.data() + off, ts);
            off += ts;
            if (triple.find("amdgcn") != std::string::npos && s > 0 && o + s <= buf.size())
                return parse_elf(buf.data() + o, s, out, err);
        }
        *err = "offload bundle holds no amdgcn code object";
        return false;
    }
    return parse_elf(buf.data(), buf.size(), out, err);
}

}  // namespace hal
}  // namespace reef
