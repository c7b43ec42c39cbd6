// Importer for the textual form of VPUIP programs (include/nce_vpuip.h): a hand-written scanner for the
// handful of operations and types that matter, conversion of NCEClusterTask to nce_cluster_task_desc_t, and
// in-order execution on one stream.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cctype>
#include <cstring>
#include <map>
#include <memory>
#include <new>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/nce_vpuip.h"
#include "nce_log.h"

namespace {

struct ParseError: std::runtime_error {
    using std::runtime_error::runtime_error;
};

// ---- text helpers -----------------------------------------------------------------------------------

std::string trim(const std::string& s) {
    size_t a = 0, b = s.size();
    while (a < b && isspace((unsigned char)s[a])) ++a;
    while (b > a && isspace((unsigned char)s[b - 1])) --b;
    return s.substr(a, b - a);
}

bool starts_with(const std::string& s, size_t pos, const char* lit) {
    return s.compare(pos, strlen(lit), lit) == 0;
}

// End (exclusive) of the piece of text that starts at pos and runs to the next ',' or closing bracket at depth 0.
// '<' '(' '[' '{' nest; the '>' of "->" is not a bracket; string literals are opaque.
size_t balanced_end(const std::string& s, size_t pos) {
    int depth = 0;
    for (size_t i = pos; i < s.size(); ++i) {
        const char c = s[i];
        if (c == '"') {
            i = s.find('"', i + 1);
            if (i == std::string::npos) throw ParseError("unterminated string literal");
            continue;
        }
        if (c == '-' && i + 1 < s.size() && s[i + 1] == '>') {
            ++i;
            continue;
        }
        if (c == '<' || c == '(' || c == '[' || c == '{') {
            ++depth;
        } else if (c == '>' || c == ')' || c == ']' || c == '}') {
            if (depth == 0) return i;
            --depth;
        } else if (c == ',' && depth == 0) {
            return i;
        }
    }
    return s.size();
}

// Split "a, b<c, d>, e" at top-level commas.
std::vector<std::string> split_top(const std::string& s) {
    std::vector<std::string> out;
    size_t pos = 0;
    while (pos < s.size()) {
        const size_t e = balanced_end(s, pos);
        const std::string piece = trim(s.substr(pos, e - pos));
        if (!piece.empty()) out.push_back(piece);
        if (e >= s.size()) break;
        if (s[e] != ',') throw ParseError("unbalanced brackets in '" + s.substr(0, 60) + "'");
        pos = e + 1;
    }
    return out;
}

// Text between the bracket at `open` and its partner.
std::string inside(const std::string& s, size_t open, size_t* close_out = nullptr) {
    const size_t e = [&] {
        size_t i = open + 1;
        for (;;) {
            i = balanced_end(s, i);
            if (i >= s.size()) throw ParseError("unbalanced brackets");
            if (s[i] != ',') return i;
            ++i;
        }
    }();
    if (close_out) *close_out = e;
    return s.substr(open + 1, e - open - 1);
}

// "{a = 1 : i64, b = [1, 2], flag}" -> map (unit attributes map to "").
std::map<std::string, std::string> parse_dict(const std::string& body) {
    std::map<std::string, std::string> m;
    for (const std::string& item : split_top(body)) {
        size_t eq = std::string::npos;
        int depth = 0;
        for (size_t i = 0; i < item.size(); ++i) {
            const char c = item[i];
            if (c == '<' || c == '(' || c == '[' || c == '{') ++depth;
            else if (c == '>' || c == ')' || c == ']' || c == '}') --depth;
            else if (c == '=' && depth == 0) {
                eq = i;
                break;
            }
        }
        if (eq == std::string::npos) m[trim(item)] = "";
        else m[trim(item.substr(0, eq))] = trim(item.substr(eq + 1));
    }
    return m;
}

int64_t int_of(const std::string& v, const char* what) {  // "5 : i64" or "5"
    const std::string t = trim(v.substr(0, v.find(':')));
    if (t.empty()) throw ParseError(std::string(what) + ": expected an integer, got '" + v + "'");
    char* end = nullptr;
    const long long x = strtoll(t.c_str(), &end, 10);
    if (*end != '\0') throw ParseError(std::string(what) + ": expected an integer, got '" + v + "'");
    return x;
}

std::vector<int64_t> ints_of(const std::string& v, const char* what) {  // "[1, 2, 3]"
    const std::string t = trim(v);
    if (t.size() < 2 || t.front() != '[') throw ParseError(std::string(what) + ": expected an array, got '" + v + "'");
    std::vector<int64_t> out;
    for (const std::string& e : split_top(t.substr(1, t.rfind(']') - 1))) out.push_back(int_of(e, what));
    return out;
}

std::string angle_arg(const std::string& v, const char* what) {  // "#VPU.mpe_mode<CUBOID_16x16>" -> CUBOID_16x16
    const size_t a = v.find('<');
    if (a == std::string::npos) throw ParseError(std::string(what) + ": expected <...>, got '" + v + "'");
    return trim(inside(v, a));
}

// ---- types -------------------------------------------------------------------------------------------

struct TensorType {
    int64_t dims[4] = {1, 1, 1, 1};
    int rank = 0;
    int32_t dtype = -1;
    int32_t elem_bytes = 1;
    int32_t zero_point = 0;
    int perm[4] = {0, 1, 2, 3};  // memory order, outermost first, as logical dimension numbers
    bool has_strides = false;
    int64_t strides_elems[4] = {0, 0, 0, 0};
    int32_t section = -1, index = 0;
    bool plain_memref = false;  // false: distributed / sparse / unknown type
    std::string type_name;      // the type as written when it is no plain memref; else the element type as written
};

struct Aliases {
    std::map<std::string, std::string> hash, bang;  // "#NHWC" -> text, "!qElemType" -> text
};

void parse_order(const std::string& text, const Aliases& al, TensorType* t) {
    std::string v = trim(text);
    if (!v.empty() && v[0] == '#' && v.find('<') == std::string::npos) {
        const auto it = al.hash.find(v);
        if (it != al.hash.end()) v = it->second;
        else {  // well-known names even without an alias line
            static const std::map<std::string, std::string> known = {
                {"#NCHW", "0123"}, {"#NHWC", "0231"}, {"#NWHC", "0321"}, {"#NWCH", "0312"}, {"#NCWH", "0132"}, {"#NHCW", "0213"}};
            const auto k = known.find(v);
            if (k == known.end()) throw ParseError("unknown layout alias " + v);
            for (int i = 0; i < 4; ++i) t->perm[i] = k->second[i] - '0';
            return;
        }
    }
    // affine_map<(d0, d1, d2, d3) -> (d0, d2, d3, d1)>
    const size_t arrow = v.find("->");
    if (arrow == std::string::npos) throw ParseError("cannot read layout '" + v + "'");
    const size_t open = v.find('(', arrow);
    if (open == std::string::npos) throw ParseError("cannot read layout '" + v + "'");
    const std::vector<std::string> res = split_top(inside(v, open));
    if (res.size() > 4) throw ParseError("layouts of rank > 4 are not supported");
    for (size_t i = 0; i < res.size(); ++i) {
        if (res[i].size() < 2 || res[i][0] != 'd') throw ParseError("cannot read layout '" + v + "'");
        t->perm[i] = atoi(res[i].c_str() + 1);
    }
}

void parse_element(const std::string& text, const Aliases& al, TensorType* t) {
    std::string v = trim(text);
    if (!v.empty() && v[0] == '!' && !starts_with(v, 0, "!quant.")) {
        const auto it = al.bang.find(v);
        if (it == al.bang.end()) throw ParseError("unknown type alias " + v);
        v = trim(it->second);
    }
    t->zero_point = 0;
    if (starts_with(v, 0, "!quant.uniform<")) {
        const std::string body = inside(v, v.find('<'));
        // storage[<lo:hi>]:expressed[:axis], scale[:zp] | {s[:zp], ...}
        const std::vector<std::string> parts = split_top(body);
        if (parts.size() != 2) throw ParseError("cannot read quantized type '" + v + "'");
        const std::string storage = parts[0].substr(0, parts[0].find_first_of("<:"));
        if (storage == "u8") t->dtype = NCE_DT_U8;
        else if (storage == "i8") t->dtype = NCE_DT_I8;
        else t->dtype = -1;
        t->elem_bytes = 1;
        auto zp_of = [](const std::string& sz) -> int64_t {
            const size_t c = sz.find(':');
            return c == std::string::npos ? 0 : strtoll(sz.c_str() + c + 1, nullptr, 10);
        };
        const std::string& q = parts[1];
        if (!q.empty() && q[0] == '{') {
            const std::vector<std::string> per = split_top(q.substr(1, q.rfind('}') - 1));
            if (per.empty()) throw ParseError("empty per-axis quantization in '" + v + "'");
            const int64_t zp0 = zp_of(per[0]);
            for (const std::string& e : per)
                if (zp_of(e) != zp0) throw ParseError("per-axis zero points that differ are not supported: '" + v + "'");
            t->zero_point = (int32_t)zp0;
        } else {
            t->zero_point = (int32_t)zp_of(q);
        }
        return;
    }
    if (v == "ui8" || v == "u8") {
        t->dtype = NCE_DT_U8;
        t->elem_bytes = 1;
    } else if (v == "si8" || v == "i8") {
        t->dtype = NCE_DT_I8;
        t->elem_bytes = 1;
    } else if (v == "si32" || v == "i32") {
        t->dtype = NCE_DT_SI32;
        t->elem_bytes = 4;
    } else {
        t->dtype = -1;
        if (v == "f16" || v == "bf16" || v == "si16" || v == "ui16" || v == "i16") t->elem_bytes = 2;
        else if (v == "f32" || v == "ui32") t->elem_bytes = 4;
        else if (v == "f64" || v == "si64" || v == "ui64" || v == "i64") t->elem_bytes = 8;
        else t->elem_bytes = 1;  // i1, 4-bit types ...: not addressable per element here
    }
}

void parse_section(const std::string& text, TensorType* t) {  // "@DDR" or "[@CMX_NN, 0]"
    std::string v = trim(text);
    t->index = 0;
    if (!v.empty() && v[0] == '[') {
        const std::vector<std::string> p = split_top(v.substr(1, v.rfind(']') - 1));
        if (p.empty()) throw ParseError("cannot read memory space '" + v + "'");
        if (p.size() > 1) t->index = (int32_t)int_of(p[1], "memory space index");
        v = p[0];
    }
    if (v == "@CMX_NN") t->section = NCE_VPUIP_SECTION_CMX_NN;
    else if (v == "@DDR") t->section = NCE_VPUIP_SECTION_DDR;
    else t->section = -1;
}

TensorType parse_type(const std::string& text, const Aliases& al) {
    std::string v = trim(text);
    for (int hop = 0; hop < 4 && !v.empty() && v[0] == '!' && !starts_with(v, 0, "!quant."); ++hop) {
        const auto it = al.bang.find(v);
        if (it == al.bang.end()) break;
        v = trim(it->second);
    }
    TensorType t;
    if (!starts_with(v, 0, "memref<")) {  // distributed / sparse buffers: not a plain memref
        t.type_name = v.substr(0, v.find_first_of("< "));
        return t;
    }
    t.plain_memref = true;
    const std::string body = inside(v, 6);
    const std::vector<std::string> parts = split_top(body);
    if (parts.empty()) throw ParseError("empty memref type");
    // shape and element type: "1x32x56x56x!quant.uniform<...>"
    const std::string& se = parts[0];
    size_t pos = 0;
    while (pos < se.size() && isdigit((unsigned char)se[pos])) {
        size_t e = pos;
        while (e < se.size() && isdigit((unsigned char)se[e])) ++e;
        if (e >= se.size() || se[e] != 'x') break;
        if (t.rank >= 4) throw ParseError("memrefs of rank > 4 are not supported: '" + v + "'");
        t.dims[t.rank++] = strtoll(se.c_str() + pos, nullptr, 10);
        pos = e + 1;
    }
    parse_element(se.substr(pos), al, &t);
    t.type_name = trim(se.substr(pos));
    for (int i = 0; i < 4; ++i) t.perm[i] = i;
    for (size_t i = 1; i < parts.size(); ++i) {
        const std::string& p = parts[i];
        if (p[0] == '@' || p[0] == '[') parse_section(p, &t);
        else if (p[0] == '#' || starts_with(p, 0, "affine_map")) parse_order(p, al, &t);
        else if (p[0] == '{') {
            const auto d = parse_dict(p.substr(1, p.rfind('}') - 1));
            if (d.count("order")) parse_order(d.at("order"), al, &t);
            if (d.count("strides")) {
                const std::vector<int64_t> s = ints_of(d.at("strides"), "strides");
                if ((int)s.size() != t.rank) throw ParseError("strides do not match the rank in '" + v + "'");
                t.has_strides = true;
                for (int k = 0; k < t.rank; ++k) t.strides_elems[k] = s[k];
            }
        }
    }
    return t;
}

// ---- program -----------------------------------------------------------------------------------------

struct Buffer {
    nce_vpuip_buffer_t pub{};
    bool plain = false;
    bool dense = false;        // bytes are contiguous: byte_size == number of elements * element size
    std::string type_name;     // see TensorType
};

struct Task {
    nce_cluster_task_desc_t desc{};
    std::vector<nce_dpu_task_t> variants;
    nce_ppe_task_t ppe{};
    bool has_ppe = false;
    int input = -1, weights = -1, table = -1, output = -1;  // buffer indices
    int line = 0;
};

struct Op {
    int kind = 0;
    int task = -1;          // NCE task index
    int src = -1, dst = -1; // DMA buffer indices
    int line = 0;
};

struct Binding {
    uint8_t* base = nullptr;
    int64_t size = 0;
};

}  // namespace

struct nce_vpuip_program_s {
    std::vector<Buffer> buffers;
    std::map<std::string, int> by_name;
    std::vector<Task> tasks;
    std::vector<Op> ops;
    std::map<std::pair<int, int>, Binding> bindings;
    std::string function;
};

namespace {

int line_of(const std::string& s, size_t pos) {
    return 1 + (int)std::count(s.begin(), s.begin() + std::min(pos, s.size()), '\n');
}

// a * b and a + b for non-negative byte counts; a ParseError instead of a wrapped value
int64_t mul_checked(int64_t a, int64_t b) {
    int64_t r;
    if (a < 0 || b < 0 || __builtin_mul_overflow(a, b, &r)) throw ParseError("tensor extent overflows 63 bits");
    return r;
}
int64_t add_checked(int64_t a, int64_t b) {
    int64_t r;
    if (a < 0 || b < 0 || __builtin_add_overflow(a, b, &r)) throw ParseError("tensor extent overflows 63 bits");
    return r;
}

void finish_buffer(const TensorType& t, Buffer* b) {
    b->plain = t.plain_memref;
    b->type_name = t.type_name;
    b->pub.dtype = t.dtype;
    b->pub.elem_bytes = t.elem_bytes;
    b->pub.zero_point = t.zero_point;
    for (int i = 0; i < 4; ++i) b->pub.dims[i] = 1;
    // ranks below 4 are right-aligned into N, C, H, W
    const int shift = 4 - t.rank;
    for (int i = 0; i < t.rank; ++i) b->pub.dims[i + shift] = t.dims[i];
    int64_t strides[4] = {0, 0, 0, 0};
    if (t.has_strides) {
        for (int i = 0; i < t.rank; ++i) strides[i + shift] = mul_checked(t.strides_elems[i], t.elem_bytes);
    } else {
        int64_t s = t.elem_bytes;
        for (int i = t.rank - 1; i >= 0; --i) {
            const int d = t.perm[i];
            if (d < 0 || d >= t.rank) throw ParseError("layout names a dimension outside the rank");
            strides[d + shift] = s;
            s = mul_checked(s, t.dims[d]);
        }
    }
    int64_t span = t.elem_bytes;
    for (int i = 0; i < 4; ++i) {
        if (strides[i] == 0) strides[i] = span;  // padding dimensions of extent 1
        b->pub.strides_bytes[i] = strides[i];
    }
    span = t.elem_bytes;
    int64_t elems = 1;
    for (int i = 0; i < 4; ++i) {
        if (b->pub.dims[i] <= 0) throw ParseError("tensor with an empty dimension");
        span = add_checked(span, mul_checked(b->pub.dims[i] - 1, b->pub.strides_bytes[i]));
        elems = mul_checked(elems, b->pub.dims[i]);
    }
    b->pub.byte_size = span;
    b->dense = span == mul_checked(elems, t.elem_bytes);
}

int add_buffer(nce_vpuip_program_s* p, const std::string& name, const TensorType& t, int32_t section, int32_t index, int64_t offset) {
    Buffer b;
    finish_buffer(t, &b);
    const size_t n = std::min(sizeof(b.pub.name) - 1, name.size());
    memcpy(b.pub.name, name.data(), n);
    b.pub.section = section;
    b.pub.index = index;
    b.pub.byte_offset = offset;
    add_checked(offset, b.pub.byte_size);  // (the end of the buffer inside its section must be representable)
    p->buffers.push_back(b);
    p->by_name[name] = (int)p->buffers.size() - 1;
    return (int)p->buffers.size() - 1;
}

// "%3 = " before position pos (same statement)
std::string result_name_before(const std::string& s, size_t pos) {
    size_t i = pos;
    while (i > 0 && isspace((unsigned char)s[i - 1])) --i;
    if (i == 0 || s[i - 1] != '=') return "";
    --i;
    while (i > 0 && isspace((unsigned char)s[i - 1])) --i;
    size_t e = i;
    while (i > 0 && (isalnum((unsigned char)s[i - 1]) || s[i - 1] == '_' || s[i - 1] == '%' || s[i - 1] == ':' || s[i - 1] == '.')) --i;
    std::string name = s.substr(i, e - i);
    const size_t colon = name.find(':');  // "%3:2 = ..."
    if (colon != std::string::npos) name = name.substr(0, colon);
    return name;
}

void set_tensor(nce_tensor_t* t, const Buffer& b) {
    t->data = nullptr;
    t->dtype = b.pub.dtype;
    t->zero_point = b.pub.zero_point;
    for (int i = 0; i < 4; ++i) {
        t->dims[i] = b.pub.dims[i];
        t->strides_bytes[i] = b.pub.strides_bytes[i];
    }
}

int32_t mpe_mode_of(const std::string& name) {
    static const char* names[] = {"VECTOR", "MATRIX", "VECTOR_FP16", "CUBOID_16x16", "CUBOID_8x16", "CUBOID_4x16", "NOP"};
    for (int i = 0; i < 7; ++i)
        if (name == names[i]) return i;
    throw ParseError("unknown mpe_mode " + name);
}

int32_t task_type_of(const std::string& name) {
    if (name == "CONV") return NCE_TASK_CONV;
    if (name == "DWCONV") return NCE_TASK_DWCONV;
    if (name == "MAXPOOL") return NCE_TASK_MAXPOOL;
    if (name == "AVEPOOL") return NCE_TASK_AVEPOOL;
    if (name == "ELTWISE") return NCE_TASK_ELTWISE;
    throw ParseError("NCE task type " + name + " is not supported (CONV, DWCONV, MAXPOOL, AVEPOOL, ELTWISE are)");
}

int32_t ppe_mode_of(const std::string& name) {  // VPU::PPEMode, tblgen/.../VPU/attributes.td:263-303
    static const std::map<std::string, int32_t> modes = {{"STORE", 0}, {"LOAD", 1}, {"CLEAR", 2}, {"NOOP", 3}, {"HALT", 4},
        {"ADD", 5}, {"SUB", 6}, {"MULT", 7}, {"MAXIMUM", 8}, {"MINIMUM", 9}, {"AND", 10}, {"OR", 11}, {"XOR", 12},
        {"LRELU", 13}, {"LRELUX", 14}, {"LPRELU", 15}, {"CEIL", 16}, {"FLOOR", 17}, {"POW", 18}, {"EXP", 19}, {"SIGMOID", 20},
        {"TANH", 21}, {"SQRT", 22}, {"RSQRT", 23}, {"FLEXARB", 24}, {"NOT", 25}, {"ABS", 26}, {"NEG", 27}};
    const auto it = modes.find(name);
    if (it == modes.end()) throw ParseError("unknown PPE mode " + name);
    return it->second;
}

void parse_padding(const std::string& v, int32_t* l, int32_t* r, int32_t* t, int32_t* b) {
    const auto d = parse_dict(angle_arg(v, "padding"));
    auto get = [&](const char* k) {
        const auto it = d.find(k);
        if (it == d.end()) throw ParseError(std::string("padding without '") + k + "'");
        return (int32_t)int_of(it->second, k);
    };
    *l = get("left");
    *r = get("right");
    *t = get("top");
    *b = get("bottom");
}

size_t skip_ws(const std::string& s, size_t pos) {
    while (pos < s.size() && isspace((unsigned char)s[pos])) ++pos;
    return pos;
}

int operand_buffer(nce_vpuip_program_s* p, const std::string& ssa, const char* role, int line) {
    const auto it = p->by_name.find(ssa);
    if (it == p->by_name.end())
        throw ParseError("line " + std::to_string(line) + ": " + role + " operand " + ssa + " is not a declared buffer or function argument");
    return it->second;
}

// Parses one NCEClusterTask starting right after the op name; returns the position after its PPE region.
size_t parse_nce_task(nce_vpuip_program_s* p, const std::string& s, size_t pos, const Aliases& al) {
    (void)al;
    Task task;
    task.line = line_of(s, pos);
    const std::string where = "line " + std::to_string(task.line) + ": ";
    pos = skip_ws(s, pos);
    if (pos >= s.size() || s[pos] != '{') throw ParseError(where + "expected the attribute dictionary of NCEClusterTask");
    size_t close;
    const auto attrs = parse_dict(inside(s, pos, &close));
    pos = close + 1;
    nce_cluster_task_desc_t& d = task.desc;
    if (!attrs.count("task_type")) throw ParseError(where + "NCEClusterTask without task_type");
    d.task_type = task_type_of(angle_arg(attrs.at("task_type"), "task_type"));
    if (attrs.count("kernel_size")) {
        const auto k = ints_of(attrs.at("kernel_size"), "kernel_size");
        if (k.size() != 2) throw ParseError(where + "kernel_size must have two entries");
        d.kernel_size[0] = (int32_t)k[0];
        d.kernel_size[1] = (int32_t)k[1];
    }
    if (attrs.count("kernel_strides")) {
        const auto k = ints_of(attrs.at("kernel_strides"), "kernel_strides");
        if (k.size() != 2) throw ParseError(where + "kernel_strides must have two entries");
        d.kernel_strides[0] = (int32_t)k[0];
        d.kernel_strides[1] = (int32_t)k[1];
    }
    if (attrs.count("kernel_padding"))
        parse_padding(attrs.at("kernel_padding"), &d.kernel_pad_left, &d.kernel_pad_right, &d.kernel_pad_top, &d.kernel_pad_bottom);
    static const std::pair<const char*, uint32_t> flag_names[] = {
        {"is_continued", NCE_FLAG_IS_CONTINUED}, {"is_segmented", NCE_FLAG_IS_SEGMENTED},
        {"input_channels_compression", NCE_FLAG_INPUT_CHANNELS_COMPRESSION}, {"is_superdense", NCE_FLAG_IS_SUPERDENSE},
        {"is_inplace", NCE_FLAG_IS_INPLACE}, {"is_permute_quantize", NCE_FLAG_IS_PERMUTE_QUANTIZE},
        {"is_small_kernel_optimized", NCE_FLAG_IS_SMALL_KERNEL_OPTIMIZED}};
    for (const auto& f : flag_names)
        if (attrs.count(f.first)) d.flags |= f.second;

    // operands: name(%ssa : type) ... until "->"
    for (;;) {
        pos = skip_ws(s, pos);
        if (starts_with(s, pos, "->")) break;
        size_t e = pos;
        while (e < s.size() && (isalnum((unsigned char)s[e]) || s[e] == '_')) ++e;
        if (e == pos || e >= s.size() || s[e] != '(') throw ParseError(where + "cannot read the operand list of NCEClusterTask");
        const std::string role = s.substr(pos, e - pos);
        size_t rp;
        const std::string body = inside(s, e, &rp);
        pos = rp + 1;
        const std::string ssa = trim(body.substr(0, body.find(':')));
        if (role == "input") task.input = operand_buffer(p, ssa, "input", task.line);
        else if (role == "weights") task.weights = operand_buffer(p, ssa, "weights", task.line);
        else if (role == "weight_table") task.table = operand_buffer(p, ssa, "weight_table", task.line);
        else if (role == "outputs") task.output = operand_buffer(p, ssa, "outputs", task.line);
        else if (role == "parent_input" || role == "parent_output" || role == "activation_window" || role == "instruction_list_table" ||
                 role == "profiling_data") {
            // views of the same memory / 30XX lookup tables / profiling: nothing to execute
        } else {
            throw ParseError(where + "operand '" + role + "' (sparsity / storage elements) is not supported");
        }
    }
    if (task.input < 0 || task.output < 0) throw ParseError(where + "NCEClusterTask needs input(...) and outputs(...)");
    // skip the result type(s) up to "variants"
    const size_t var = s.find("variants", pos);
    if (var == std::string::npos) throw ParseError(where + "NCEClusterTask without a variants region");
    pos = s.find('{', var);
    if (pos == std::string::npos) throw ParseError(where + "NCEClusterTask without a variants region");
    size_t vclose;
    const std::string vbody = inside(s, pos, &vclose);
    for (size_t q = 0;;) {
        q = vbody.find("DPUTask", q);
        if (q == std::string::npos) break;
        const size_t ob = vbody.find('{', q);
        if (ob == std::string::npos) throw ParseError(where + "DPUTask without attributes");
        size_t cb;
        const auto va = parse_dict(inside(vbody, ob, &cb));
        q = cb + 1;
        nce_dpu_task_t v{};
        if (!va.count("outStart") || !va.count("outEnd")) throw ParseError(where + "DPUTask needs outStart and outEnd");
        const auto st = ints_of(va.at("outStart"), "outStart"), en = ints_of(va.at("outEnd"), "outEnd");
        if (st.size() != 3 || en.size() != 3) throw ParseError(where + "outStart / outEnd must have three entries");
        for (int i = 0; i < 3; ++i) {
            v.out_start[i] = (int32_t)st[i];
            v.out_end[i] = (int32_t)en[i];
        }
        if (va.count("pad")) parse_padding(va.at("pad"), &v.pad_left, &v.pad_right, &v.pad_top, &v.pad_bottom);
        v.mpe_mode = va.count("mpe_mode") ? mpe_mode_of(angle_arg(va.at("mpe_mode"), "mpe_mode")) : NCE_MPE_CUBOID_16x16;
        if (va.count("cluster_id")) v.cluster_id = (int32_t)int_of(va.at("cluster_id"), "cluster_id");
        task.variants.push_back(v);
    }
    pos = vclose + 1;
    // PPE : { PPETask <MODE> {...} }
    pos = skip_ws(s, pos);
    if (starts_with(s, pos, "PPE")) {
        pos = s.find('{', pos);
        if (pos == std::string::npos) throw ParseError(where + "PPE region without a body");
        size_t pclose;
        const std::string pbody = inside(s, pos, &pclose);
        const size_t pt = pbody.find("PPETask");
        if (pt != std::string::npos) {
            size_t q = skip_ws(pbody, pt + 7);
            std::string mode;
            if (q < pbody.size() && pbody[q] == '<') {
                size_t mc;
                mode = trim(inside(pbody, q, &mc));
                q = mc + 1;
            } else if (q < pbody.size() && pbody[q] == '"') {
                const size_t mc = pbody.find('"', q + 1);
                mode = pbody.substr(q + 1, mc - q - 1);
                q = mc + 1;
            } else {
                throw ParseError(where + "PPETask without a mode");
            }
            nce_ppe_task_t& pp = task.ppe;
            pp.mode = ppe_mode_of(mode);
            pp.clamp_low = INT32_MIN;
            pp.clamp_high = INT32_MAX;
            pp.lrelu_mult = 1;
            pp.round_mode = NCE_ROUND_HALF_UP;
            pp.clamp_domain = NCE_CLAMP_POST_ZP;
            q = skip_ws(pbody, q);
            if (q < pbody.size() && pbody[q] == '{') {
                const auto pa = parse_dict(inside(pbody, q));
                auto clamp32 = [](int64_t v) { return (int32_t)std::max<int64_t>(INT32_MIN, std::min<int64_t>(INT32_MAX, v)); };
                if (pa.count("clamp_low")) pp.clamp_low = clamp32(int_of(pa.at("clamp_low"), "clamp_low"));
                if (pa.count("clamp_high")) pp.clamp_high = clamp32(int_of(pa.at("clamp_high"), "clamp_high"));
                if (pa.count("lrelu_mult")) pp.lrelu_mult = (int32_t)int_of(pa.at("lrelu_mult"), "lrelu_mult");
                if (pa.count("lrelu_shift")) pp.lrelu_shift = (int32_t)int_of(pa.at("lrelu_shift"), "lrelu_shift");
                auto first = [&](const char* k, int32_t* out) {
                    const auto v = ints_of(pa.at(k), k);
                    if (v.size() != 1) throw ParseError(where + k + " must have exactly one entry");
                    *out = (int32_t)v[0];
                };
                if (pa.count("quant_mult") && pa.count("quant_shift")) {
                    pp.has_quant = 1;
                    first("quant_mult", &pp.quant_mult);
                    first("quant_shift", &pp.quant_shift);
                }
                if (pa.count("quant_post_shift")) pp.quant_post_shift = (int32_t)int_of(pa.at("quant_post_shift"), "quant_post_shift");
                if (pa.count("in1_quant_mult") && pa.count("in2_quant_mult")) {
                    pp.has_in_mult = 1;
                    first("in1_quant_mult", &pp.in1_quant_mult);
                    first("in2_quant_mult", &pp.in2_quant_mult);
                }
            }
            task.has_ppe = true;
        }
        pos = pclose + 1;
    }
    set_tensor(&d.input, p->buffers[task.input]);
    set_tensor(&d.output, p->buffers[task.output]);
    if (task.weights >= 0) set_tensor(&d.weights, p->buffers[task.weights]);
    if (task.table >= 0) set_tensor(&d.weight_table, p->buffers[task.table]);
    for (const int b : {task.input, task.output, task.weights, task.table}) {
        if (b < 0) continue;
        const Buffer& buf = p->buffers[b];
        if (!buf.plain)
            throw ParseError(where + "operand " + buf.pub.name + " has type " + (buf.type_name.empty() ? "(unknown)" : buf.type_name) +
                             ": only plain memrefs are supported (no distributed or sparse buffers)");
        if (buf.pub.dtype < 0)
            throw ParseError(where + "operand " + buf.pub.name + " has element type " + buf.type_name + ": only u8 / i8 tensors and si32 tables are executable here");
    }
    Op op;
    op.kind = NCE_VPUIP_OP_NCE_TASK;
    op.task = (int)p->tasks.size();
    op.line = task.line;
    p->tasks.push_back(std::move(task));
    p->ops.push_back(op);
    return pos;
}

size_t parse_dma(nce_vpuip_program_s* p, const std::string& s, size_t pos) {
    Op op;
    op.kind = NCE_VPUIP_OP_DMA;
    op.line = line_of(s, pos);
    const size_t in = s.find("inputs(", pos), out = s.find("outputs(", pos);
    if (in == std::string::npos || out == std::string::npos) throw ParseError("line " + std::to_string(op.line) + ": NNDMA without inputs(...) / outputs(...)");
    size_t c1, c2;
    const std::string a = inside(s, in + 6, &c1), b = inside(s, out + 7, &c2);
    const auto src = p->by_name.find(trim(a.substr(0, a.find(':')))), dst = p->by_name.find(trim(b.substr(0, b.find(':'))));
    op.src = src == p->by_name.end() ? -1 : src->second;  // e.g. a constant: reported when the program is run
    op.dst = dst == p->by_name.end() ? -1 : dst->second;
    p->ops.push_back(op);
    return c2 + 1;
}

void parse_program(const std::string& raw, nce_vpuip_program_s* p) {
    // whole-line comments (lit RUN / CHECK lines) carry no program text
    std::string s;
    {
        size_t pos = 0;
        while (pos < raw.size()) {
            size_t eol = raw.find('\n', pos);
            if (eol == std::string::npos) eol = raw.size();
            const size_t q = skip_ws(raw, pos);
            if (!(q + 1 < eol && raw[q] == '/' && raw[q + 1] == '/')) s.append(raw, pos, eol - pos);
            s += '\n';  // keep line numbers
            pos = eol + 1;
        }
    }
    Aliases al;
    {   // "#NAME = ..." and "!NAME = ..." at the start of a line; values may span lines
        size_t pos = 0;
        while (pos < s.size()) {
            size_t eol = s.find('\n', pos);
            if (eol == std::string::npos) eol = s.size();
            if ((s[pos] == '#' || s[pos] == '!') && pos < eol) {
                const size_t eq = s.find('=', pos);
                if (eq != std::string::npos && eq < eol) {
                    const std::string name = trim(s.substr(pos, eq - pos));
                    size_t stop = s.find('\n', eq);
                    if (stop == std::string::npos) stop = s.size();
                    // take whole lines until the brackets balance
                    std::string value = s.substr(eq + 1, stop - eq - 1);
                    auto depth_of = [](const std::string& t) {
                        int d = 0;
                        for (size_t i = 0; i < t.size(); ++i) {
                            if (t[i] == '-' && i + 1 < t.size() && t[i + 1] == '>') { ++i; continue; }
                            if (t[i] == '<' || t[i] == '(' || t[i] == '[' || t[i] == '{') ++d;
                            else if (t[i] == '>' || t[i] == ')' || t[i] == ']' || t[i] == '}') --d;
                        }
                        return d;
                    };
                    while (depth_of(value) > 0 && stop < s.size()) {
                        size_t next = s.find('\n', stop + 1);
                        if (next == std::string::npos) next = s.size();
                        value += s.substr(stop, next - stop);
                        stop = next;
                    }
                    (name[0] == '#' ? al.hash : al.bang)[name] = trim(value);
                    eol = stop;
                }
            }
            pos = eol + 1;
        }
    }
    // function arguments
    const size_t fn = s.find("func.func");
    if (fn == std::string::npos) throw ParseError("no func.func in the program");
    const size_t at = s.find('@', fn);
    const size_t lp = s.find('(', fn);
    if (at == std::string::npos || lp == std::string::npos || at > lp) throw ParseError("cannot read the function signature");
    p->function = trim(s.substr(at + 1, lp - at - 1));
    size_t rp;
    const std::string args = inside(s, lp, &rp);
    int argno = 0;
    for (const std::string& a : split_top(args)) {
        const size_t colon = a.find(':');
        if (colon == std::string::npos) throw ParseError("cannot read function argument '" + a + "'");
        const TensorType t = parse_type(a.substr(colon + 1), al);
        add_buffer(p, trim(a.substr(0, colon)), t, NCE_VPUIP_SECTION_ARGUMENT, argno++, 0);
    }
    // The body of THIS function: from the first '{' outside the signature's types to its matching '}'. SSA names and
    // operations of later functions of the module (lit files hold several) are not part of the program.
    size_t body_open = std::string::npos;
    {
        int depth = 0;
        for (size_t i = rp + 1; i < s.size(); ++i) {
            const char c = s[i];
            if (c == '-' && i + 1 < s.size() && s[i + 1] == '>') { ++i; continue; }
            if (c == '{' && depth == 0) { body_open = i; break; }
            if (c == '<' || c == '(' || c == '[' || c == '{') ++depth;
            else if (c == '>' || c == ')' || c == ']' || c == '}') --depth;
        }
    }
    if (body_open == std::string::npos) throw ParseError("function @" + p->function + " has no body");
    const size_t body_close = balanced_end(s, body_open + 1);
    // body: the three operation kinds, in text order
    size_t pos = body_open;
    for (;;) {
        const size_t db = s.find("VPURT.DeclareBuffer", pos), nt = s.find("VPUIP.NCEClusterTask", pos), dm = s.find("VPUIP.NNDMA", pos);
        const size_t next = std::min(db, std::min(nt, dm));
        if (next == std::string::npos || next >= body_close) break;
        if (next == db) {
            const int line = line_of(s, db);
            const std::string name = result_name_before(s, db);
            size_t q = skip_ws(s, db + strlen("VPURT.DeclareBuffer"));
            if (q >= s.size() || (s[q] != '<' && s[q] != '"')) throw ParseError("line " + std::to_string(line) + ": DeclareBuffer without a section");
            std::string section;
            if (s[q] == '<') {
                size_t c;
                section = trim(inside(s, q, &c));
                q = c + 1;
            } else {
                const size_t c = s.find('"', q + 1);
                section = s.substr(q + 1, c - q - 1);
                q = c + 1;
            }
            q = skip_ws(s, q);
            int32_t index = 0;
            if (q < s.size() && s[q] == '[') {
                size_t c;
                const std::vector<std::string> idx = split_top(inside(s, q, &c));
                if (!idx.empty()) index = (int32_t)int_of(idx[0], "section index");
                q = skip_ws(s, c + 1);
            }
            if (q >= s.size() || s[q] != '<') throw ParseError("line " + std::to_string(line) + ": DeclareBuffer without a byte offset");
            size_t c;
            const int64_t offset = int_of(inside(s, q, &c), "byte offset");
            q = skip_ws(s, c + 1);
            if (!starts_with(s, q, "->")) throw ParseError("line " + std::to_string(line) + ": DeclareBuffer without a result type");
            q = skip_ws(s, q + 2);
            // a type ends where the line ends
            size_t eol = s.find('\n', q);
            if (eol == std::string::npos) eol = s.size();
            const TensorType t = parse_type(s.substr(q, eol - q), al);
            int32_t sec;
            if (section == "CMX_NN") sec = NCE_VPUIP_SECTION_CMX_NN;
            else if (section == "DDR") sec = NCE_VPUIP_SECTION_DDR;
            else if (section == "NetworkInput") sec = NCE_VPUIP_SECTION_NETWORK_INPUT;
            else if (section == "NetworkOutput") sec = NCE_VPUIP_SECTION_NETWORK_OUTPUT;
            else throw ParseError("line " + std::to_string(line) + ": section <" + section + "> is not supported");
            if (name.empty()) throw ParseError("line " + std::to_string(line) + ": DeclareBuffer without a result name");
            add_buffer(p, name, t, sec, index, offset);
            pos = eol;
        } else if (next == nt) {
            pos = parse_nce_task(p, s, nt + strlen("VPUIP.NCEClusterTask"), al);
        } else {
            pos = parse_dma(p, s, dm + strlen("VPUIP.NNDMA"));
        }
    }
}

uint8_t* address_of(const nce_vpuip_program_s* p, const Buffer& b, std::string* why) {
    const auto it = p->bindings.find({b.pub.section, b.pub.index});
    if (it == p->bindings.end() || it->second.base == nullptr) {
        *why = std::string("buffer ") + b.pub.name + ": section " + std::to_string(b.pub.section) + " index " + std::to_string(b.pub.index) + " is not bound";
        return nullptr;
    }
    if (b.pub.byte_offset < 0 || b.pub.byte_offset + b.pub.byte_size > it->second.size) {
        *why = std::string("buffer ") + b.pub.name + " (offset " + std::to_string(b.pub.byte_offset) + ", " + std::to_string(b.pub.byte_size) +
               " bytes) does not fit the " + std::to_string(it->second.size) + " bytes bound to its section";
        return nullptr;
    }
    return it->second.base + b.pub.byte_offset;
}

nce_result_t resolve_task(nce_vpuip_program_s* p, int i, nce_cluster_task_desc_t* out, nce_log_handle_t log) {
    Task& t = p->tasks[i];
    *out = t.desc;
    std::string why;
    const struct {
        int buf;
        nce_tensor_t* dst;
    } ops[] = {{t.input, &out->input}, {t.weights, &out->weights}, {t.table, &out->weight_table}, {t.output, &out->output}};
    for (const auto& o : ops) {
        if (o.buf < 0) continue;
        o.dst->data = address_of(p, p->buffers[o.buf], &why);
        if (o.dst->data == nullptr) {
            if (log) log->add(1, "vpuip: task %d (line %d): %s", i, t.line, why.c_str());
            return NCE_RESULT_ERROR_INVALID_ARGUMENT;
        }
    }
    out->variants = t.variants.empty() ? nullptr : t.variants.data();
    out->num_variants = (uint32_t)t.variants.size();
    out->ppe = t.has_ppe ? &t.ppe : nullptr;
    return NCE_RESULT_SUCCESS;
}

}  // namespace

extern "C" {

nce_result_t nceVpuipParse(const char* mlir_text, nce_vpuip_program_handle_t* program, nce_log_handle_t log) {
    if (program == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    *program = nullptr;
    if (mlir_text == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    try {
        std::unique_ptr<nce_vpuip_program_s> p(new nce_vpuip_program_s());
        parse_program(mlir_text, p.get());
        *program = p.release();
        return NCE_RESULT_SUCCESS;
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (const std::exception& e) {
        if (log) log->add(1, "vpuip: %s", e.what());
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    }
}

nce_result_t nceVpuipDestroy(nce_vpuip_program_handle_t program) {
    if (program == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    delete program;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceVpuipGetInfo(nce_vpuip_program_handle_t program, nce_vpuip_info_t* info) {
    if (program == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (info == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    memset(info, 0, sizeof(*info));
    info->num_buffers = (int32_t)program->buffers.size();
    info->num_ops = (int32_t)program->ops.size();
    info->num_tasks = (int32_t)program->tasks.size();
    info->num_dmas = info->num_ops - info->num_tasks;
    const size_t n = std::min(sizeof(info->function) - 1, program->function.size());
    memcpy(info->function, program->function.data(), n);
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceVpuipGetBuffer(nce_vpuip_program_handle_t program, int32_t i, nce_vpuip_buffer_t* buffer) {
    if (program == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (buffer == nullptr || i < 0 || i >= (int32_t)program->buffers.size()) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *buffer = program->buffers[i].pub;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceVpuipGetOp(nce_vpuip_program_handle_t program, int32_t i, int32_t* kind, int32_t* task_index) {
    if (program == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (kind == nullptr || task_index == nullptr || i < 0 || i >= (int32_t)program->ops.size()) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *kind = program->ops[i].kind;
    *task_index = program->ops[i].task;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceVpuipBind(nce_vpuip_program_handle_t program, int32_t section, int32_t index, void* base, int64_t size_bytes) {
    if (program == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (base == nullptr || size_bytes <= 0) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    program->bindings[{section, index}] = Binding{static_cast<uint8_t*>(base), size_bytes};
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceVpuipGetTask(nce_vpuip_program_handle_t program, int32_t task_index, nce_cluster_task_desc_t* desc, nce_log_handle_t log) {
    if (program == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (desc == nullptr || task_index < 0 || task_index >= (int32_t)program->tasks.size()) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    return resolve_task(program, task_index, desc, log);
}

nce_result_t nceVpuipEnqueue(nce_vpuip_program_handle_t program, nce_executor_handle_t executor, void* hip_stream) {
    if (program == nullptr || executor == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    // the executor's log is not reachable from here; errors of the tasks themselves land in it through Enqueue
    try {
        for (const Op& op : program->ops) {
            if (op.kind == NCE_VPUIP_OP_NCE_TASK) {
                nce_cluster_task_desc_t d;
                nce_result_t r = resolve_task(program, op.task, &d, nullptr);
                if (r != NCE_RESULT_SUCCESS) return r;
                r = nceClusterTaskEnqueue(executor, &d, hip_stream);  // (sets the executor's device)
                if (r != NCE_RESULT_SUCCESS) return r;
            } else {
                if (op.src < 0 || op.dst < 0) return NCE_RESULT_ERROR_UNSUPPORTED;  // e.g. a copy out of a constant
                const Buffer& a = program->buffers[op.src];
                const Buffer& b = program->buffers[op.dst];
                // One flat copy: both sides dense (a strided view would also overwrite the bytes between its rows) and of
                // the same shape and order; layout-changing and strided DMAs are not implemented.
                if (!a.dense || !b.dense || a.pub.byte_size != b.pub.byte_size || a.pub.elem_bytes != b.pub.elem_bytes ||
                    memcmp(a.pub.dims, b.pub.dims, sizeof(a.pub.dims)) != 0 || memcmp(a.pub.strides_bytes, b.pub.strides_bytes, sizeof(a.pub.strides_bytes)) != 0)
                    return NCE_RESULT_ERROR_UNSUPPORTED;
                std::string why;
                uint8_t* src = address_of(program, a, &why);
                uint8_t* dst = address_of(program, b, &why);
                if (src == nullptr || dst == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
                // (the copy goes to the device the stream belongs to; a task before it has made the executor's device current)
                if (hipMemcpyAsync(dst, src, (size_t)a.pub.byte_size, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(hip_stream)) != hipSuccess)
                    return NCE_RESULT_ERROR_UNKNOWN;
            }
        }
        return NCE_RESULT_SUCCESS;
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (...) {
        return NCE_RESULT_ERROR_UNKNOWN;
    }
}

}  // extern "C"
