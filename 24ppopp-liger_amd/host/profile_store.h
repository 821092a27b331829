// profile_store.h -- kernel-duration dictionaries and their JSON files, plus GEMM decomposition.
//
// Counterpart of the reference's src/utils.h: MainDictToFile / MainFileToDict / SubDictToFile / SubFileToDict
// (:106-215, same JSON schema: an array of {"kernel_name","batch_size","seq_len","duration"} objects where
// "duration" is a number in the main file and an array of factor-1 numbers in the sub file) and
// decompose_callback (:218-260).  The reader is a small hand-written parser (the reference pulls in nlohmann/json).
// A missing file or malformed text yields an empty dictionary and `false` instead of an exception.
#pragma once
#include <cctype>
#include <cstdlib>
#include <fstream>
#include <sstream>

#include "func_wrapper.h"

namespace liger {

// ---- writers ---------------------------------------------------------------------------------------------
inline bool MainDictToFile(const MainDict& data, const std::string& filename) {
    std::ostringstream ss;
    ss << "[";
    bool first = true;
    for (const auto& e : data) {
        if (!first) ss << ",";
        first = false;
        ss << "{\"kernel_name\":" << e.first.kernel_name << ",\"batch_size\":" << e.first.batch_size
           << ",\"seq_len\":" << e.first.seq_len << ",\"duration\":" << e.second << "}";
    }
    ss << "]";
    std::ofstream f(filename);
    if (!f.is_open()) return false;
    f << ss.str();
    return true;
}

inline bool SubDictToFile(const SubDict& data, const std::string& filename) {
    std::ostringstream ss;
    ss << "[";
    bool first = true;
    for (const auto& e : data) {
        if (!first) ss << ",";
        first = false;
        ss << "{\"kernel_name\":" << e.first.kernel_name << ",\"batch_size\":" << e.first.batch_size
           << ",\"seq_len\":" << e.first.seq_len << ",\"duration\": [";
        for (size_t i = 0; i < e.second.size(); ++i) ss << (i ? "," : "") << e.second[i];
        ss << "]}";
    }
    ss << "]";
    std::ofstream f(filename);
    if (!f.is_open()) return false;
    f << ss.str();
    return true;
}

// ---- reader: just enough JSON for the schema above -----------------------------------------------------------
namespace detail {
struct JsonCursor {
    const std::string& s;
    size_t i = 0;
    bool ok = true;
    explicit JsonCursor(const std::string& str) : s(str) {}
    void ws() { while (i < s.size() && isspace((unsigned char)s[i])) ++i; }
    bool eat(char c) { ws(); if (i < s.size() && s[i] == c) { ++i; return true; } return false; }
    bool peek(char c) { ws(); return i < s.size() && s[i] == c; }
    double number() {
        ws();
        const char* b = s.c_str() + i;
        char* e = nullptr;
        double v = strtod(b, &e);
        if (e == b) { ok = false; return 0; }
        i += (size_t)(e - b);
        return v;
    }
    std::string str() {
        ws();
        std::string r;
        if (!eat('"')) { ok = false; return r; }
        while (i < s.size() && s[i] != '"') r += s[i++];
        if (i >= s.size()) ok = false; else ++i;
        return r;
    }
};
// parses one {...} record; `vec` receives an array-valued duration, `scalar` a numeric one
inline bool parse_record(JsonCursor& c, kernel_info& key, double& scalar, std::vector<float>& vec, bool& is_vec) {
    if (!c.eat('{')) return false;
    bool have[4] = {false, false, false, false};
    while (c.ok) {
        std::string k = c.str();
        if (!c.eat(':')) return false;
        if (k == "duration") {
            have[3] = true;
            if (c.peek('[')) {
                is_vec = true;
                c.eat('[');
                if (!c.peek(']')) {
                    do { vec.push_back((float)c.number()); } while (c.ok && c.eat(','));
                }
                if (!c.eat(']')) return false;
            } else {
                is_vec = false;
                scalar = c.number();
            }
        } else {
            int v = (int)c.number();
            if (k == "kernel_name") { key.kernel_name = v; have[0] = true; }
            else if (k == "batch_size") { key.batch_size = v; have[1] = true; }
            else if (k == "seq_len") { key.seq_len = v; have[2] = true; }
        }
        if (c.eat(',')) continue;
        break;
    }
    return c.ok && c.eat('}') && have[0] && have[1] && have[2] && have[3];
}
inline bool slurp(const std::string& filename, std::string& out) {
    std::ifstream f(filename);
    if (!f.is_open()) return false;
    std::stringstream b;
    b << f.rdbuf();
    out = b.str();
    return true;
}
}  // namespace detail

inline bool MainFileToDict(const std::string& filename, MainDict& dict) {
    dict.clear();
    std::string text;
    if (!detail::slurp(filename, text)) return false;
    detail::JsonCursor c(text);
    if (!c.eat('[')) return false;
    if (c.eat(']')) return true;
    do {
        kernel_info key{0, 0, 0};
        double d = 0;
        std::vector<float> v;
        bool is_vec = false;
        if (!detail::parse_record(c, key, d, v, is_vec) || is_vec) { dict.clear(); return false; }
        dict[key] = (float)d;
    } while (c.eat(','));
    if (!c.eat(']')) { dict.clear(); return false; }
    return true;
}
inline MainDict MainFileToDict(const std::string& filename) {
    MainDict d;
    MainFileToDict(filename, d);
    return d;
}

inline bool SubFileToDict(const std::string& filename, SubDict& dict) {
    dict.clear();
    std::string text;
    if (!detail::slurp(filename, text)) return false;
    detail::JsonCursor c(text);
    if (!c.eat('[')) return false;
    if (c.eat(']')) return true;
    do {
        kernel_info key{0, 0, 0};
        double d = 0;
        std::vector<float> v;
        bool is_vec = false;
        if (!detail::parse_record(c, key, d, v, is_vec) || !is_vec) { dict.clear(); return false; }
        dict[key] = v;
    } while (c.eat(','));
    if (!c.eat(']')) { dict.clear(); return false; }
    return true;
}
inline SubDict SubFileToDict(const std::string& filename) {
    SubDict d;
    SubFileToDict(filename, d);
    return d;
}

// ---- GEMM decomposition  (utils.h:218-260) -----------------------------------------------------------------------
// Returns the GEMM that computes units [start, start + n) of `factor` equal units of old_func's output along `axis`.
// The reference scales cuBLAS's m by n/factor without moving any pointer, so all of its pieces recompute the leading
// columns; here the weight / bias / output (or activation / output) pointers are offset so that the pieces of one
// GEMM tile its output exactly.  Unit boundaries are rounded to the epilogue's granularity (whole heads for the
// head-transposing epilogue, whole gate/up groups for the GeGLU epilogue, 8 elements otherwise) so that every piece keeps the vectorised paths.
inline int split_point(int extent, int unit, int factor, int gran) {
    if (unit <= 0) return 0;
    if (unit >= factor) return extent;
    if (extent % gran != 0) gran = 1;
    return (int)(((int64_t)(extent / gran) * unit) / factor) * gran;
}

inline FuncWrap decompose_callback(const FuncWrap& old_func, int factor, int n, float duration = 0.0f, int start = 0,
                                   split_axis axis = SPLIT_OUT_COLS) {
    GemmDesc g = old_func.args_gemm;
    const size_t es = (g.dtype == LG_F16) ? 2 : 4;
    if (g.epilogue == LG_EPI_BIAS_HEADS) axis = SPLIT_OUT_COLS;  // token rows would move the (batch, seq) decode of rows
    if (axis == SPLIT_OUT_COLS) {
        // GeGLU: whole (gate, up) groups of 32 features, which produce 16 output columns
        int gran = (g.epilogue == LG_EPI_BIAS_HEADS) ? g.epi_d : (g.epilogue == LG_EPI_BIAS_GEGLU ? 32 : 8);
        // tiled weights: a piece starts at a whole 16-feature tile (their feature counts are multiples of 16, so it divides)
        while (g.transa == LG_OP_TILED && gran % 16 != 0) gran *= 2;
        const int c0 = split_point(g.m, start, factor, gran), c1 = split_point(g.m, start + n, factor, gran);
        g.A = (const char*)g.A + (g.transa ? (size_t)c0 * g.lda : (size_t)c0) * es;
        if (g.bias) g.bias = (const char*)g.bias + (size_t)c0 * es;
        if (g.epilogue == LG_EPI_BIAS_HEADS) g.C = (char*)g.C + (size_t)(c0 / g.epi_d) * g.ldc * g.epi_d * es;
        else if (g.epilogue == LG_EPI_BIAS_GEGLU) g.C = (char*)g.C + (size_t)(c0 / 2) * es;
        else g.C = (char*)g.C + (size_t)c0 * es;
        g.m = c1 - c0;
    } else {
        const int r0 = split_point(g.n, start, factor, 1), r1 = split_point(g.n, start + n, factor, 1);
        g.B = (const char*)g.B + (size_t)r0 * g.ldb * es;
        g.C = (char*)g.C + (size_t)r0 * g.ldc * es;
        g.n = r1 - r0;
    }
    FuncWrap f(old_func.name, duration, GEMM, [g](const DynamicInitParam& D) { GemmEx(D, g); }, g, old_func.label, old_func.rclass);
    return f;
}

}  // namespace liger
