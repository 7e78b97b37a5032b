#include "npy.h"

#include <cstdio>
#include <cstring>

namespace cubert {

namespace {

bool find_key(const std::string& h, const char* key, size_t* pos) {
    std::string k1 = std::string("'") + key + "'";
    std::string k2 = std::string("\"") + key + "\"";
    size_t p = h.find(k1);
    if (p == std::string::npos) p = h.find(k2);
    if (p == std::string::npos) return false;
    p = h.find(':', p);
    if (p == std::string::npos) return false;
    *pos = p + 1;
    return true;
}

void skip_ws(const std::string& h, size_t* p) {
    while (*p < h.size() && (h[*p] == ' ' || h[*p] == '\t')) ++*p;
}

}  // namespace

bool npy_parse_header(const std::string& h, std::vector<size_t>* shape, std::string* descr,
                      bool* fortran, std::string* err) {
    size_t p;
    if (!find_key(h, "descr", &p)) { *err = "npy header: no 'descr'"; return false; }
    skip_ws(h, &p);
    if (p >= h.size() || (h[p] != '\'' && h[p] != '"')) {
        *err = "npy header: structured dtypes are not supported";
        return false;
    }
    char q = h[p];
    size_t e = h.find(q, p + 1);
    if (e == std::string::npos) { *err = "npy header: unterminated descr"; return false; }
    *descr = h.substr(p + 1, e - p - 1);

    if (!find_key(h, "fortran_order", &p)) { *err = "npy header: no 'fortran_order'"; return false; }
    skip_ws(h, &p);
    if (h.compare(p, 4, "True") == 0) *fortran = true;
    else if (h.compare(p, 5, "False") == 0) *fortran = false;
    else { *err = "npy header: bad fortran_order"; return false; }

    if (!find_key(h, "shape", &p)) { *err = "npy header: no 'shape'"; return false; }
    skip_ws(h, &p);
    if (p >= h.size() || h[p] != '(') { *err = "npy header: bad shape"; return false; }
    size_t close = h.find(')', p);
    if (close == std::string::npos) { *err = "npy header: bad shape"; return false; }
    shape->clear();
    size_t i = p + 1;
    while (i < close) {
        while (i < close && (h[i] == ' ' || h[i] == ',')) ++i;
        if (i >= close) break;
        if (h[i] < '0' || h[i] > '9') { *err = "npy header: bad shape entry"; return false; }
        size_t v = 0;
        while (i < close && h[i] >= '0' && h[i] <= '9') { v = v * 10 + size_t(h[i] - '0'); ++i; }
        if (i < close && h[i] == 'L') ++i;      // Python 2 long suffix
        shape->push_back(v);
    }
    return true;
}

bool npy_load_f32(const std::string& path, NpyArray* out, std::string* err) {
    FILE* f = std::fopen(path.c_str(), "rb");
    if (!f) { *err = "cannot open " + path; return false; }
    auto fail = [&](const std::string& m) { *err = path + ": " + m; std::fclose(f); return false; };
    unsigned char pre[12];
    if (std::fread(pre, 1, 10, f) != 10) return fail("truncated preamble");
    if (std::memcmp(pre, "\x93NUMPY", 6) != 0) return fail("not an .npy file (bad magic)");
    int major = pre[6];
    size_t hlen;
    if (major == 1) {
        hlen = size_t(pre[8]) | (size_t(pre[9]) << 8);
    } else if (major == 2 || major == 3) {
        if (std::fread(pre + 10, 1, 2, f) != 2) return fail("truncated preamble");
        hlen = size_t(pre[8]) | (size_t(pre[9]) << 8) | (size_t(pre[10]) << 16) | (size_t(pre[11]) << 24);
    } else {
        return fail("unsupported .npy format version " + std::to_string(major));
    }
    if (hlen == 0 || hlen > (1u << 20)) return fail("implausible header length");
    std::string header(hlen, '\0');
    if (std::fread(&header[0], 1, hlen, f) != hlen) return fail("truncated header");
    std::string descr, perr;
    bool fortran = false;
    if (!npy_parse_header(header, &out->shape, &descr, &fortran, &perr)) return fail(perr);
    if (descr != "<f4" && descr != "|f4" && descr != "=f4")
        return fail("dtype '" + descr + "' is not little-endian float32 ('<f4')");
    if (fortran && out->shape.size() > 1) return fail("fortran_order arrays are not supported");
    size_t n = out->numel();
    out->data.resize(n);
    if (n && std::fread(out->data.data(), sizeof(float), n, f) != n) return fail("truncated data");
    if (std::fgetc(f) != EOF) return fail("trailing bytes after the array data");
    std::fclose(f);
    return true;
}

}  // namespace cubert
