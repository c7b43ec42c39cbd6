// Front end for the reference's single-operation test descriptors (include/nce_hwtest.h): a small JSON
// reader, the descriptor parser with the reference's keys and error messages, and the five task builders.
#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <new>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/nce_hwtest.h"
#include "../../include/nce_params.h"
#include "nce_log.h"

namespace {

// ---- JSON ------------------------------------------------------------------------------------------
// Just what the descriptors use: objects, arrays, strings (with escapes), numbers, booleans, null.

struct JValue;
using JObject = std::map<std::string, JValue>;
using JArray = std::vector<JValue>;

struct JValue {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool b = false;
    double num = 0.0;
    bool integral = false;  // written without fraction / exponent and exactly representable
    int64_t inum = 0;
    std::string str;
    std::shared_ptr<JArray> arr;
    std::shared_ptr<JObject> obj;

    // Accessors with the semantics of llvm::json::Object::get*: absent or wrong type -> nullptr / false.
    const JValue* get(const char* key) const {
        if (kind != Object) return nullptr;
        const auto it = obj->find(key);
        return it == obj->end() ? nullptr : &it->second;
    }
    const JObject* getObject(const char* key) const {
        const JValue* v = get(key);
        return v && v->kind == Object ? v->obj.get() : nullptr;
    }
    const JValue* getObjectValue(const char* key) const {
        const JValue* v = get(key);
        return v && v->kind == Object ? v : nullptr;
    }
    const JArray* getArray(const char* key) const {
        const JValue* v = get(key);
        return v && v->kind == Array ? v->arr.get() : nullptr;
    }
    bool getString(const char* key, std::string* out) const {
        const JValue* v = get(key);
        if (!v || v->kind != String) return false;
        *out = v->str;
        return true;
    }
    bool asInteger(int64_t* out) const {  // a number with an integral value (llvm::json::Value::getAsInteger)
        if (kind != Number) return false;
        if (integral) {
            *out = inum;
            return true;
        }
        double ip;
        if (std::modf(num, &ip) == 0.0 && std::fabs(num) < 9.2e18) {
            *out = (int64_t)num;
            return true;
        }
        return false;
    }
    bool getInteger(const char* key, int64_t* out) const {
        const JValue* v = get(key);
        return v && v->asInteger(out);
    }
    bool getNumber(const char* key, double* out) const {
        const JValue* v = get(key);
        if (!v || v->kind != Number) return false;
        *out = v->num;
        return true;
    }
    bool getBoolean(const char* key, bool* out) const {
        const JValue* v = get(key);
        if (!v || v->kind != Bool) return false;
        *out = v->b;
        return true;
    }
};

class JParser {
public:
    explicit JParser(const std::string& text): s_(text) {
    }
    JValue parse() {
        JValue v = value();
        ws();
        if (p_ != s_.size()) fail("text after the end of the document");
        return v;
    }

private:
    const std::string& s_;
    size_t p_ = 0;

    [[noreturn]] void fail(const char* what) {
        throw std::runtime_error("HWTEST JSON parsing failed: " + std::string(what) + " at offset " + std::to_string(p_));
    }
    void ws() {
        while (p_ < s_.size() && (s_[p_] == ' ' || s_[p_] == '\t' || s_[p_] == '\n' || s_[p_] == '\r')) ++p_;
    }
    bool eat(const char* lit) {
        const size_t n = strlen(lit);
        if (s_.compare(p_, n, lit) == 0) {
            p_ += n;
            return true;
        }
        return false;
    }
    // Nesting is bounded: value() recurses per level, and a descriptor of thousands of '[' must end as a parse error,
    // not as a stack overflow that no catch block can turn into a result code.
    static constexpr int kMaxDepth = 64;
    int depth_ = 0;
    struct DepthGuard {
        int& d;
        explicit DepthGuard(int& depth) : d(depth) { ++d; }
        ~DepthGuard() { --d; }
    };
    JValue value() {
        const DepthGuard guard(depth_);
        if (depth_ > kMaxDepth) fail("nesting deeper than 64 levels");
        ws();
        if (p_ >= s_.size()) fail("unexpected end of text");
        JValue v;
        const char c = s_[p_];
        if (c == '{') {
            ++p_;
            v.kind = JValue::Object;
            v.obj = std::make_shared<JObject>();
            ws();
            if (p_ < s_.size() && s_[p_] == '}') {
                ++p_;
                return v;
            }
            for (;;) {
                ws();
                if (p_ >= s_.size() || s_[p_] != '"') fail("expected a member name");
                std::string key = string();
                ws();
                if (p_ >= s_.size() || s_[p_] != ':') fail("expected ':'");
                ++p_;
                (*v.obj)[key] = value();
                ws();
                if (p_ < s_.size() && s_[p_] == ',') {
                    ++p_;
                    continue;
                }
                if (p_ < s_.size() && s_[p_] == '}') {
                    ++p_;
                    return v;
                }
                fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            ++p_;
            v.kind = JValue::Array;
            v.arr = std::make_shared<JArray>();
            ws();
            if (p_ < s_.size() && s_[p_] == ']') {
                ++p_;
                return v;
            }
            for (;;) {
                v.arr->push_back(value());
                ws();
                if (p_ < s_.size() && s_[p_] == ',') {
                    ++p_;
                    continue;
                }
                if (p_ < s_.size() && s_[p_] == ']') {
                    ++p_;
                    return v;
                }
                fail("expected ',' or ']'");
            }
        }
        if (c == '"') {
            v.kind = JValue::String;
            v.str = string();
            return v;
        }
        if (eat("true")) {
            v.kind = JValue::Bool;
            v.b = true;
            return v;
        }
        if (eat("false")) {
            v.kind = JValue::Bool;
            return v;
        }
        if (eat("null")) return v;
        if (c == '-' || (c >= '0' && c <= '9')) {
            const size_t start = p_;
            if (s_[p_] == '-') ++p_;
            while (p_ < s_.size() && isdigit((unsigned char)s_[p_])) ++p_;
            bool integral = true;
            if (p_ < s_.size() && s_[p_] == '.') {
                integral = false;
                ++p_;
                while (p_ < s_.size() && isdigit((unsigned char)s_[p_])) ++p_;
            }
            if (p_ < s_.size() && (s_[p_] == 'e' || s_[p_] == 'E')) {
                integral = false;
                ++p_;
                if (p_ < s_.size() && (s_[p_] == '+' || s_[p_] == '-')) ++p_;
                while (p_ < s_.size() && isdigit((unsigned char)s_[p_])) ++p_;
            }
            const std::string tok = s_.substr(start, p_ - start);
            if (tok.empty() || tok == "-") fail("malformed number");
            v.kind = JValue::Number;
            v.num = strtod(tok.c_str(), nullptr);
            if (integral && tok.size() <= 18) {
                v.integral = true;
                v.inum = strtoll(tok.c_str(), nullptr, 10);
            }
            return v;
        }
        fail("unexpected character");
    }
    std::string string() {
        std::string out;
        ++p_;  // opening quote
        while (p_ < s_.size() && s_[p_] != '"') {
            char c = s_[p_++];
            if (c == '\\') {
                if (p_ >= s_.size()) fail("unterminated escape");
                const char e = s_[p_++];
                switch (e) {
                case 'n': c = '\n'; break;
                case 't': c = '\t'; break;
                case 'r': c = '\r'; break;
                case 'b': c = '\b'; break;
                case 'f': c = '\f'; break;
                case 'u': {
                    if (p_ + 4 > s_.size()) fail("short \\u escape");
                    const unsigned code = (unsigned)strtoul(s_.substr(p_, 4).c_str(), nullptr, 16);
                    p_ += 4;
                    c = code < 0x80 ? (char)code : '?';  // descriptors are ASCII
                    break;
                }
                default: c = e;  // \" \\ \/
                }
            }
            out += c;
        }
        if (p_ >= s_.size()) fail("unterminated string");
        ++p_;
        return out;
    }
};

// Drop lines that consist of a '//' comment (test_case_json_parser.cpp:22-36).
std::string strip_comment_lines(const std::string& text) {
    std::string out;
    size_t pos = 0;
    while (pos <= text.size()) {
        size_t eol = text.find('\n', pos);
        if (eol == std::string::npos) eol = text.size();
        size_t q = pos;
        while (q < eol && text[q] == ' ') ++q;
        const bool comment = q + 1 < eol && text[q] == '/' && text[q + 1] == '/';
        if (!comment) out.append(text, pos, eol - pos);
        if (eol < text.size()) out += '\n';
        pos = eol + 1;
    }
    return out;
}

bool iequal(const std::string& a, const char* b) {  // the reference compares names case-insensitively (:54-62)
    if (a.size() != strlen(b)) return false;
    for (size_t i = 0; i < a.size(); ++i)
        if (tolower((unsigned char)a[i]) != tolower((unsigned char)b[i])) return false;
    return true;
}

void copy_str(char* dst, size_t cap, const std::string& s) {
    const size_t n = std::min(cap - 1, s.size());
    memcpy(dst, s.data(), n);
    dst[n] = '\0';
}

struct Layer {
    nce_hwtest_layer_t pub{};
    std::vector<double> scales;
};

}  // namespace

// Case types that expand to several NCE tasks (include/nce_hwtest.h, nce_hwtest_program_t).
enum ProgramKind { PROGRAM_SINGLE = 0, PROGRAM_DOUBLE_CONV, PROGRAM_RACE_DPU, PROGRAM_DIFFERENT_CLUSTERS, PROGRAM_MULTI_CLUSTERS };

struct nce_hwtest_case_s {
    nce_hwtest_case_t pub{};
    Layer in, wt, out;
    bool has_conv = false, has_pool = false, has_ew = false;
    int program = PROGRAM_SINGLE;
    Layer wt2;                          // DoubleZMajorConvolution: second entry of "weight"
    std::vector<Layer> outs;            // every entry of "output" (MultiClustersDPU: one per cluster)
    int64_t iteration_count = 1;        // RaceConditionDPU
    int64_t num_clusters = 1;           // RaceConditionDPU
    std::vector<int64_t> clusters;      // DifferentClustersDPU: output_cluster; MultiClustersDPU: task_clusters
    int split_dim = 0;                  // MultiClustersDPU: 1 = SOK (channels), 2 = SOH (rows)
    bool broadcast = false;             // MultiClustersDPU
};

namespace {

[[noreturn]] void bad(const char* msg) {
    throw std::runtime_error(msg);
}

int32_t dtype_of(const std::string& name) {  // to_dtype, :64-90; only the 8-bit integer types run here
    if (iequal(name, "uint8")) return NCE_DT_U8;
    if (iequal(name, "int8")) return NCE_DT_I8;
    if (iequal(name, "int32")) return NCE_DT_SI32;
    return -1;
}

// loadQuantizationParams, :386-407
void load_quant(const JValue& obj, const char* who, Layer* l) {
    const JValue* qp = obj.getObjectValue("quantization");
    if (!qp) return;
    l->pub.has_quant = 1;
    const JArray* scales = qp->getArray("scale");
    if (!scales) bad("loadQuantizationParams: cannot find scale config param");
    for (const JValue& e : *scales)
        if (e.kind == JValue::Number) l->scales.push_back(e.num);
    int64_t zp;
    double lo, hi;
    if (!qp->getInteger("zeropoint", &zp) || !qp->getNumber("low_range", &lo) || !qp->getNumber("high_range", &hi))
        throw std::runtime_error(std::string(who) + ": quantization needs zeropoint, low_range and high_range");
    l->pub.zero_point = zp;
    l->pub.low_range = (int64_t)lo;
    l->pub.high_range = (int64_t)hi;
    l->pub.num_scales = (int32_t)std::min<size_t>(l->scales.size(), NCE_HWTEST_MAX_SCALES);
    l->pub.scale0 = l->scales.empty() ? 0.0 : l->scales[0];
}

// loadInputLayer / loadWeightLayer / loadOutputLayer, :464-585: arrays of objects; the first entry is the operand.
size_t layer_count(const JValue& root, const char* key) {
    const JArray* arr = root.getArray(key);
    return arr ? arr->size() : 0;
}

void load_layer(const JValue& root, const char* key, const char* missing_shape, Layer* l, size_t index = 0) {
    const JArray* arr = root.getArray(key);
    if (!arr || arr->size() <= index) return;
    const JValue& obj = (*arr)[index];
    if (obj.kind != JValue::Object) throw std::runtime_error(std::string(key) + ": entries must be objects");
    const JArray* shape = obj.getArray("shape");
    if (!shape) bad(missing_shape);
    if (shape->size() > 4) throw std::runtime_error(std::string(key) + ": shape has more than 4 dimensions");
    for (size_t i = 0; i < shape->size(); ++i) {
        int64_t v;
        if (!(*shape)[i].asInteger(&v)) throw std::runtime_error(std::string(key) + ": shape entries must be integers");
        l->pub.shape[i] = v;
    }
    load_quant(obj, key, l);
    std::string dt;
    if (!obj.getString("dtype", &dt)) throw std::runtime_error(std::string(key) + ": missing dtype");
    l->pub.present = 1;
    l->pub.dtype = dtype_of(dt);
    copy_str(l->pub.dtype_name, sizeof(l->pub.dtype_name), dt);
    std::string path;
    if (obj.getString("file_path", &path)) copy_str(l->pub.file_path, sizeof(l->pub.file_path), path);
}

void load_int_list(const JArray& arr, int32_t* dst, size_t cap, const char* who) {
    if (arr.size() > cap) throw std::runtime_error(std::string(who) + ": too many entries");
    for (size_t i = 0; i < arr.size(); ++i) {
        int64_t v;
        if (arr[i].asInteger(&v)) dst[i] = (int32_t)v;
    }
}

// loadConvLayer, :640-701
void load_conv(const JValue& root, nce_hwtest_case_s* c) {
    const JValue* op = root.getObjectValue("conv_op");
    if (!op) bad("loadConvLayer: missing conv_op config");
    const JArray* strides = op->getArray("stride");
    if (!strides) bad("loadConvLayer: missing strides");
    load_int_list(*strides, c->pub.stride, 2, "conv_op.stride");
    const JArray* pads = op->getArray("pad");
    if (!pads) bad("loadConvLayer: missing pads");
    load_int_list(*pads, c->pub.pad, 4, "conv_op.pad");
    int64_t v;
    if (!op->getInteger("group", &v)) bad("loadConvLayer: missing group");
    c->pub.group = (int32_t)v;
    if (!op->getInteger("dilation", &v)) bad("loadConvLayer: missing dilation");
    c->pub.dilation = (int32_t)v;
    bool b;
    c->pub.compress = op->getBoolean("compress", &b) && b;
    c->pub.act_sparsity = op->getBoolean("act_sparsity", &b) && b;
    std::string mpe;
    if (op->getString("mpe_mode", &mpe)) {
        if (mpe == "CUBOID_8x16") c->pub.mpe_mode = NCE_MPE_CUBOID_8x16;
        else if (mpe == "CUBOID_4x16") c->pub.mpe_mode = NCE_MPE_CUBOID_4x16;
    }
    c->has_conv = true;
}

// loadPoolLayer, :703-742
void load_pool(const JValue& root, nce_hwtest_case_s* c) {
    const JValue* op = root.getObjectValue("pool_op");
    if (!op) bad("loadPoolLayer: missing pool_op config");
    const JArray* ks = op->getArray("kernel_shape");
    if (!ks) bad("loadPoolLayer: missing kernel_shape");
    load_int_list(*ks, c->pub.kernel, 2, "pool_op.kernel_shape");
    const JArray* strides = op->getArray("stride");
    if (!strides) bad("loadPoolLayer: missing stride");
    load_int_list(*strides, c->pub.stride, 2, "pool_op.stride");
    if (const JArray* pads = op->getArray("pad")) load_int_list(*pads, c->pub.pad, 4, "pool_op.pad");
    c->has_pool = true;
}

// loadEltwiseLayer, :609-638
void load_eltwise(const JValue& root, nce_hwtest_case_s* c) {
    const JValue* op = root.getObjectValue("ew_op");
    if (!op) bad("loadEltwiseLayer: missing ew_op config");
    std::string mode;
    if (!op->getString("mode", &mode) || (mode != "ADD" && mode != "SUB" && mode != "MULT"))
        bad("loadEltwiseLayer: failed to get valid operation type");
    copy_str(c->pub.ew_mode, sizeof(c->pub.ew_mode), mode);
    c->has_ew = true;
}

// loadActivationLayer + to_activation_type, :744-790, :164-197
void load_activation(const JValue& root, nce_hwtest_case_s* c) {
    const JValue* act = root.getObjectValue("activation");
    if (!act) return;
    const JValue* name = act->get("name");
    // (older descriptors write "name": null for no activation; accepted as None)
    if (!name || (name->kind != JValue::String && name->kind != JValue::Null)) bad("loadActivationLayer: activation name must be a string");
    const std::string n = name->kind == JValue::String ? name->str : std::string();
    if (n.empty() || iequal(n, "None")) c->pub.activation = NCE_HWTEST_ACT_NONE;
    else if (iequal(n, "LeakyReLU") || iequal(n, "PReLU")) c->pub.activation = NCE_HWTEST_ACT_LEAKY_RELU;
    else if (iequal(n, "ReLU")) c->pub.activation = NCE_HWTEST_ACT_RELU;
    else if (iequal(n, "ReLUX")) c->pub.activation = NCE_HWTEST_ACT_RELUX;
    else c->pub.activation = NCE_HWTEST_ACT_OTHER;
    act->getNumber("alpha", &c->pub.alpha);
    act->getNumber("max", &c->pub.maximum);
}

void load_output_order(const JValue& root, nce_hwtest_case_s* c) {  // to_odu_permutation, :118-135
    std::string order;
    if (!root.getString("output_order", &order)) bad("output_order: missing");
    static const char* known[] = {"NHWC", "NWHC", "NWCH", "NCWH", "NHCW", "NCHW"};
    bool ok = false;
    for (const char* k : known) ok |= iequal(order, k);
    if (!ok) throw std::runtime_error("ODUPermutation value not supported: " + order);
    for (char& ch : order) ch = (char)tolower((unsigned char)ch);
    copy_str(c->pub.output_order, sizeof(c->pub.output_order), order);
}

// TestCaseJsonDescriptor::parse, :847-1026, for the case types that map to an NCE task; the others are
// recognised (task_type = -1) but none of their private sections is read.
void parse_case(const std::string& text, nce_hwtest_case_s* c) {
    const std::string filtered = strip_comment_lines(text);
    bool blank = true;
    for (char ch : filtered) blank &= isspace((unsigned char)ch) != 0;
    if (blank) bad("Expected non-empty filtered JSON");
    JParser parser(filtered);
    const JValue root = parser.parse();
    if (root.kind != JValue::Object) bad("Expected to get JSON as an object");

    std::string arch;
    if (!root.getString("architecture", &arch)) bad("Failed to get architecture");
    if (arch == "VPUX30XX") c->pub.arch = NCE_ARCH_VPUX30XX;
    else if (arch == "VPUX37XX") c->pub.arch = NCE_ARCH_VPUX37XX;
    else bad("Failed to parse architecture");
    std::string backend;
    if (!root.getString("compiler_backend", &backend)) bad("Failed to get compiler_backend");
    if (!iequal(backend, "Flatbuffer") && !iequal(backend, "ELF")) bad("Failed to parse compiler_backend");
    std::string case_type;
    if (!root.getString("case_type", &case_type)) bad("Failed to get case type");
    copy_str(c->pub.case_type, sizeof(c->pub.case_type), case_type);

    c->pub.mpe_mode = NCE_MPE_CUBOID_16x16;
    copy_str(c->pub.output_order, sizeof(c->pub.output_order), "nhwc");
    load_layer(root, "input", "loadInputLayer: missing shape", &c->in);
    load_layer(root, "output", "loadOutputLayer: missing shape", &c->out);
    load_activation(root, c);

    c->pub.task_type = -1;
    if (iequal(case_type, "ZMajorConvolution")) {
        c->pub.task_type = NCE_TASK_CONV;
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt);
        load_conv(root, c);
        load_output_order(root, c);
    } else if (iequal(case_type, "DepthWiseConv")) {
        c->pub.task_type = NCE_TASK_DWCONV;
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt);
        load_conv(root, c);
    } else if (iequal(case_type, "EltwiseDense")) {
        c->pub.task_type = NCE_TASK_ELTWISE;
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt);
        load_eltwise(root, c);
    } else if (iequal(case_type, "DoubleZMajorConvolution")) {
        // two chained convolutions (buildDoubleConvTest.cpp:55-492); parse: test_case_json_parser.cpp:887-908
        c->pub.task_type = NCE_TASK_CONV;
        c->program = PROGRAM_DOUBLE_CONV;
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt);
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt2, 1);
        if (!c->wt2.pub.present) bad("DoubleZMajorConvolution: the weight list needs two entries");
        load_conv(root, c);
        load_output_order(root, c);
    } else if (iequal(case_type, "RaceConditionDPU")) {
        // the same convolution on num_clusters clusters, iteration_count times each; every cluster's output must hold the
        // same bytes (buildRaceConditionDPUTest.cpp:41-243); parse: :909-915, loadIterationCount / loadNumClusters :783-794
        c->pub.task_type = NCE_TASK_CONV;
        c->program = PROGRAM_RACE_DPU;
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt);
        load_conv(root, c);
        if (!root.getInteger("iteration_count", &c->iteration_count) || c->iteration_count < 1) bad("RaceConditionDPU: iteration_count must be a positive integer");
        if (!root.getInteger("num_clusters", &c->num_clusters) || c->num_clusters < 1) bad("RaceConditionDPU: num_clusters must be a positive integer");
    } else if (iequal(case_type, "DifferentClustersDPU")) {
        // one convolution whose operands sit in the CMX of different clusters and whose output goes to every cluster of
        // output_cluster (buildDIfferentClustersDPUTest.cpp:25-260); parse: loadDPUTaskParams, :417-434
        c->pub.task_type = NCE_TASK_CONV;
        c->program = PROGRAM_DIFFERENT_CLUSTERS;
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt);
        load_conv(root, c);
        const JValue* tp = root.getObjectValue("DPUTaskParams");
        const JArray* oc = tp ? tp->getArray("output_cluster") : nullptr;
        if (!oc) bad("loadDPUTaskParams: cannot find output_cluster config param");
        for (const JValue& e : *oc) {
            int64_t v;
            if (e.asInteger(&v)) c->clusters.push_back(v);
        }
        int64_t v;
        if (!tp->getInteger("input_cluster", &v) || !tp->getInteger("weights_cluster", &v) || !tp->getInteger("weights_table_cluster", &v))
            bad("loadDPUTaskParams: input_cluster, weights_cluster and weights_table_cluster are required");
        if (c->clusters.empty()) bad("loadDPUTaskParams: output_cluster is empty");
    } else if (iequal(case_type, "MultiClustersDPU")) {
        // one convolution split over clusters along the rows (SOH) or the output channels (SOK)
        // (buildMultiClustersDPUTest.cpp:289-626); parse: loadMultiClusterDPUParams, :436-459
        c->pub.task_type = NCE_TASK_CONV;
        c->program = PROGRAM_MULTI_CLUSTERS;
        load_layer(root, "weight", "loadWeightLayer: missing shape", &c->wt);
        load_conv(root, c);
        load_output_order(root, c);
        const JValue* tp = root.getObjectValue("DPUTaskParams");
        const JArray* tc = tp ? tp->getArray("task_clusters") : nullptr;
        if (!tc) bad("loadMultiClusterDPUParams: cannot find task_clusters config param");
        for (const JValue& e : *tc) {
            int64_t v;
            if (e.asInteger(&v)) c->clusters.push_back(v);
        }
        std::string seg;
        if (!tp->getString("segmentation", &seg) || (seg != "SOK" && seg != "SOH")) bad("loadMultiClusterDPUParams: failed to get valid segmentation type");
        c->split_dim = seg == "SOK" ? 1 : 2;  // (SegmentationType's value is the dimension split: C = 1, H = 2)
        bool b = false;
        if (!tp->getBoolean("broadcast", &b)) bad("loadMultiClusterDPUParams: broadcast is required");
        c->broadcast = b;
        if (c->clusters.empty()) bad("loadMultiClusterDPUParams: task_clusters is empty");
        for (size_t i = 0; i < layer_count(root, "output"); ++i) {
            Layer l;
            load_layer(root, "output", "loadOutputLayer: missing shape", &l, i);
            c->outs.push_back(l);
        }
        if (c->outs.size() != c->clusters.size()) bad("MultiClustersDPU: one output entry per task cluster is required");
    } else if (iequal(case_type, "MaxPool")) {
        c->pub.task_type = NCE_TASK_MAXPOOL;
        load_pool(root, c);
    } else if (iequal(case_type, "AvgPool")) {
        c->pub.task_type = NCE_TASK_AVEPOOL;
        load_pool(root, c);
    } else {
        static const char* other[] = {"DMA", "DMAcompressAct", "SparseZMajorConvolution",
                                      "EltwiseMultDW", "EltwiseSparse",
                                      "ActShave", "ReadAfterWriteDPUDMA", "ReadAfterWriteDMADPU", "ReadAfterWriteACTDMA",
                                      "ReadAfterWriteDMAACT", "ReadAfterWriteDPUACT", "ReadAfterWriteACTDPU",
                                      "RaceConditionDMA", "RaceConditionDPUDMA",
                                      "RaceConditionDPUDMAACT", "RaceConditionDPUACT", "RaceCondition",
                                      "StorageElementTableDPU", "DualChannelDMA", "GenerateScaleTable"};
        bool known = false;
        for (const char* k : other) known |= iequal(case_type, k);
        if (!known) throw std::runtime_error("Unsupported case type: " + case_type);
    }
    if (c->has_conv && c->wt.pub.present) {
        c->pub.kernel[0] = (int32_t)c->wt.pub.shape[2];
        c->pub.kernel[1] = (int32_t)c->wt.pub.shape[3];
    }
    c->pub.input = c->in.pub;
    c->pub.weight = c->wt.pub;
    c->pub.output = c->out.pub;
}

// ---- builders --------------------------------------------------------------------------------------

struct Unsupported: std::runtime_error {
    using std::runtime_error::runtime_error;
};

void dense_nhwc(nce_tensor_t* t, int32_t dtype, int64_t n, int64_t ch, int64_t h, int64_t w, int64_t zp) {
    t->data = nullptr;
    t->dtype = dtype;
    t->zero_point = (int32_t)zp;
    t->dims[0] = n;
    t->dims[1] = ch;
    t->dims[2] = h;
    t->dims[3] = w;
    t->strides_bytes[1] = 1;
    t->strides_bytes[3] = ch;
    t->strides_bytes[2] = ch * w;
    t->strides_bytes[0] = ch * w * h;
}

void need_quant8(const Layer& l, const char* who) {
    if (!l.pub.present) throw Unsupported(std::string(who) + ": missing");
    if (l.pub.dtype != NCE_DT_U8 && l.pub.dtype != NCE_DT_I8)
        throw Unsupported(std::string(who) + ": dtype '" + l.pub.dtype_name + "' is not an 8-bit integer type");
    if (!l.pub.has_quant || l.scales.empty()) throw Unsupported(std::string(who) + ": quantization parameters are required");
}

int32_t storage_min(int32_t dtype) {
    return dtype == NCE_DT_I8 ? -128 : 0;
}
int32_t storage_max(int32_t dtype) {
    return dtype == NCE_DT_I8 ? 127 : 255;
}

// Word [2] and [3] of every row, scales broadcast per channel as getMultShiftFunc does
// (src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:252-264): rescale = (w * in) / out; bias 0.
void fill_table(int32_t arch, int64_t oc, int64_t ptr_step, const std::vector<double>& w, const std::vector<double>& in,
                const std::vector<double>& out, int32_t* table) {
    auto at = [&](const std::vector<double>& v, int64_t i) {
        if (v.size() == 1) return v[0];
        if ((int64_t)v.size() != oc) throw std::runtime_error("per-channel scale count does not match the output channels");
        return v[(size_t)i];
    };
    for (int64_t c = 0; c < oc; ++c) {
        const double rescale = (at(w, c) * at(in, c)) / at(out, c);
        int32_t mult = 0, shift = 0, post = 0;
        if (nceQuantApproximate(arch, rescale, &mult, &shift, &post) != NCE_RESULT_SUCCESS || post != 0)
            throw Unsupported("scale " + std::to_string(rescale) + " has no 16-bit multiplier / 6-bit shift form");
        uint32_t word2 = ((uint32_t)shift << 8) | ((uint32_t)mult << 16);
        if (arch == NCE_ARCH_VPUX30XX) word2 |= 1u | (1u << 14);
        int32_t* row = table + 4 * c;
        row[0] = (int32_t)(c * ptr_step);
        row[1] = 0xFFFFFF;  // SPARSITY_PTR_WHEN_NO_SPARSITY
        memcpy(&row[2], &word2, 4);
        row[3] = 0;
    }
}

void default_ppe(nce_ppe_task_t* ppe) {
    memset(ppe, 0, sizeof(*ppe));
    ppe->mode = NCE_PPE_NOOP;
    ppe->clamp_low = INT32_MIN;
    ppe->clamp_high = INT32_MAX;
    ppe->lrelu_mult = 1;
    ppe->lrelu_shift = 0;
    ppe->round_mode = NCE_ROUND_HALF_UP;
    ppe->clamp_domain = NCE_CLAMP_POST_ZP;
}

void build(const nce_hwtest_case_s& c, nce_cluster_task_desc_t* d, nce_dpu_task_t* var, nce_ppe_task_t* ppe, int32_t* table,
           int32_t cap_rows, int32_t* rows) {
    const nce_hwtest_case_t& p = c.pub;
    if (p.task_type < 0) throw Unsupported(std::string("case type '") + p.case_type + "' is not an NCE task this executor runs");
    need_quant8(c.in, "input");
    need_quant8(c.out, "output");
    if (c.in.scales.size() != 1) throw Unsupported("input: per-channel activation scales are not supported");
    const int64_t N = p.input.shape[0], IC = p.input.shape[1], IH = p.input.shape[2], IW = p.input.shape[3];
    const int64_t OC = p.output.shape[1], OH = p.output.shape[2], OW = p.output.shape[3];
    if (p.output.shape[0] != N) throw std::runtime_error("output batch differs from input batch");

    memset(d, 0, sizeof(*d));
    memset(var, 0, sizeof(*var));
    default_ppe(ppe);
    *rows = 0;
    d->task_type = p.task_type;
    dense_nhwc(&d->input, p.input.dtype, N, IC, IH, IW, p.input.zero_point);
    dense_nhwc(&d->output, p.output.dtype, N, OC, OH, OW, p.output.zero_point);
    {   // ODU permutation: the output is dense in the order "output_order" names, outermost first
        // (oduPermutationToLayout, hwtest_utils.cpp; getODUPermutationType, nce_cluster_task.cpp:764-780)
        int64_t stride = 1;
        for (int i = 3; i >= 1; --i) {
            const char dim = p.output_order[i];
            const int idx = dim == 'c' ? 1 : dim == 'h' ? 2 : 3;
            d->output.strides_bytes[idx] = stride;
            stride *= d->output.dims[idx];
        }
        d->output.strides_bytes[0] = stride;
    }
    d->weights.dtype = NCE_DT_U8;
    d->weight_table.dtype = NCE_DT_SI32;
    // JSON pads are [top, left, bottom, right] (hwtest_utils.hpp:24-35, convertNBPadtoNCETaskPad hwtest_utils.cpp:218-227)
    d->kernel_pad_top = p.pad[0];
    d->kernel_pad_left = p.pad[1];
    d->kernel_pad_bottom = p.pad[2];
    d->kernel_pad_right = p.pad[3];
    d->kernel_size[0] = p.kernel[0];
    d->kernel_size[1] = p.kernel[1];
    d->kernel_strides[0] = p.stride[0];
    d->kernel_strides[1] = p.stride[1];
    // one variant over the whole output (buildZMConvTest.cpp:360-371)
    var->out_end[0] = (int32_t)OW - 1;
    var->out_end[1] = (int32_t)OH - 1;
    var->out_end[2] = (int32_t)OC - 1;
    var->pad_left = d->kernel_pad_left;
    var->pad_right = d->kernel_pad_right;
    var->pad_top = d->kernel_pad_top;
    var->pad_bottom = d->kernel_pad_bottom;
    d->variants = var;
    d->num_variants = 1;
    d->ppe = ppe;

    const int32_t out_dt = p.output.dtype;
    const int64_t zp_out = p.output.zero_point;
    auto table_tensor = [&](int64_t n_rows) {
        if (table == nullptr || cap_rows < n_rows) throw std::runtime_error("weights table buffer is too small");
        nce_tensor_t& t = d->weight_table;
        t.dtype = NCE_DT_SI32;
        t.dims[0] = n_rows;
        t.dims[1] = 1;
        t.dims[2] = 1;
        t.dims[3] = 4;
        t.strides_bytes[0] = 16;
        t.strides_bytes[1] = 16;
        t.strides_bytes[2] = 16;
        t.strides_bytes[3] = 4;
        *rows = (int32_t)n_rows;
    };
    // dw / pool / eltwise builders clamp in the zero-point-free domain (buildDWConv.cpp:259-270,
    // buildMaxPoolTest.cpp:294-304, buildAvgPoolTest.cpp:171-190, buildEltwiseTest.cpp:151-174)
    auto clamp_pre_zp = [&]() {
        ppe->clamp_low = (int32_t)(storage_min(out_dt) - zp_out);
        ppe->clamp_high = (int32_t)(storage_max(out_dt) - zp_out);
        ppe->clamp_domain = NCE_CLAMP_PRE_ZP;
    };
    const std::vector<double> one{1.0};

    switch (p.task_type) {
    case NCE_TASK_CONV: {
        need_quant8(c.wt, "weight");
        if (p.group != 1) throw Unsupported("conv_op.group must be 1 for a ZMajorConvolution");
        if (p.dilation != 1) throw Unsupported("conv_op.dilation must be 1");
        if (p.compress || p.act_sparsity) throw Unsupported("compressed / sparse convolutions are not implemented");
        const int64_t KY = p.weight.shape[2], KX = p.weight.shape[3];
        if (p.weight.shape[0] != OC || p.weight.shape[1] != IC) throw std::runtime_error("weight shape does not match input / output channels");
        // Input channels that are no multiple of 16: the builder pads the input buffer and the weights' IC dimension to
        // the alignment (paddedInputCMXShape / paddedWeightsCMXShape, buildZMConvTest.cpp:111-136). The descriptor
        // describes those padded buffers; the caller fills the padding channels of the weights with the weights' zero
        // point (so that they contribute nothing) and may leave any bytes in the padding channels of the input.
        const int64_t ICP = (IC + 15) / 16 * 16;
        if (ICP != IC) {
            dense_nhwc(&d->input, p.input.dtype, N, ICP, IH, IW, p.input.zero_point);
        }
        d->weights.dtype = p.weight.dtype;
        d->weights.zero_point = (int32_t)p.weight.zero_point;
        d->weights.dims[0] = OC;
        d->weights.dims[1] = ICP;
        d->weights.dims[2] = KY;
        d->weights.dims[3] = KX;
        d->weights.strides_bytes[1] = 1;              // OYXI: IC innermost
        d->weights.strides_bytes[3] = ICP;            // KX
        d->weights.strides_bytes[2] = ICP * KX;       // KY
        d->weights.strides_bytes[0] = ICP * KX * KY;  // OC
        table_tensor(OC);
        fill_table(p.arch, OC, ICP * KX * KY, c.wt.scales, c.in.scales, c.out.scales, table);
        var->mpe_mode = p.mpe_mode;
        // storage-domain clamp, activation maximum, PReLU slope (buildZMConvTest.cpp:375-404)
        ppe->clamp_low = storage_min(out_dt);
        ppe->clamp_high = storage_max(out_dt);
        if (p.activation != NCE_HWTEST_ACT_NONE) {
            if (p.maximum != 0) ppe->clamp_high = (int32_t)p.maximum;
            if (p.activation == NCE_HWTEST_ACT_LEAKY_RELU) ppe->mode = NCE_PPE_LPRELU;
            else if (p.activation == NCE_HWTEST_ACT_RELUX) ppe->mode = NCE_PPE_LRELUX;
            else throw Unsupported("Encountered unsupported activation type");  // getPPEMode, buildZMConvTest.cpp:33-44
            int32_t m = 1, s = 0;
            if (ncePReLUApproximate(p.arch, p.alpha, &m, &s) != NCE_RESULT_SUCCESS) throw Unsupported("activation alpha has no PReLU approximation");
            ppe->lrelu_mult = m;
            ppe->lrelu_shift = s;
        }
        break;
    }
    case NCE_TASK_DWCONV: {
        need_quant8(c.wt, "weight");
        if (p.dilation != 1) throw Unsupported("conv_op.dilation must be 1");
        const int64_t KY = p.weight.shape[2], KX = p.weight.shape[3];
        if (p.weight.shape[0] != OC || OC != IC || p.weight.shape[1] != 1) throw std::runtime_error("depthwise weights must be [C, 1, KY, KX] with C = input = output channels");
        if (p.activation != NCE_HWTEST_ACT_NONE) throw Unsupported("the depthwise builder takes no activation");
        const int64_t row = 16 * ((KY * KX + 15) / 16);  // one padded row of taps per channel (buildDWConv.cpp:31-48)
        d->weights.dtype = p.weight.dtype;
        d->weights.zero_point = (int32_t)p.weight.zero_point;
        d->weights.dims[0] = OC;
        d->weights.dims[1] = row;
        d->weights.dims[2] = 1;
        d->weights.dims[3] = 1;
        d->weights.strides_bytes[1] = 1;
        d->weights.strides_bytes[2] = row;
        d->weights.strides_bytes[3] = row;
        d->weights.strides_bytes[0] = row;
        table_tensor(OC);
        fill_table(p.arch, OC, row, c.wt.scales, c.in.scales, c.out.scales, table);
        var->mpe_mode = NCE_MPE_CUBOID_8x16;
        clamp_pre_zp();
        break;
    }
    case NCE_TASK_MAXPOOL:
    case NCE_TASK_AVEPOOL: {
        if (OC != IC) throw std::runtime_error("pool output channels differ from input channels");
        if (p.activation != NCE_HWTEST_ACT_NONE) throw Unsupported("the pool builders take no activation");
        var->mpe_mode = NCE_MPE_CUBOID_16x16;
        clamp_pre_zp();
        const bool per_channel = c.out.scales.size() > 1;
        if (p.task_type == NCE_TASK_AVEPOOL) {
            const double area = (double)p.kernel[0] * (double)p.kernel[1];
            if (per_channel) {  // table with weight scale 1 / area (buildAvgPoolTest.cpp:53-66,116-148)
                table_tensor(OC);
                fill_table(p.arch, OC, 0, std::vector<double>{1.0 / area}, c.in.scales, c.out.scales, table);
            } else {  // calculateQuantScaleVectorForAvgPool, ppe_utils.cpp:72-106
                const double scale = c.in.scales[0] / c.out.scales[0] / area;
                int32_t m = 0, s = 0, post = 0;
                if (nceQuantApproximate(p.arch, scale, &m, &s, &post) != NCE_RESULT_SUCCESS || post != 0) throw Unsupported("average pool scale has no fixed-point form");
                ppe->has_quant = 1;
                ppe->quant_mult = m;
                ppe->quant_shift = s;
            }
        } else if (per_channel) {  // buildMaxPoolTest.cpp:222-240
            table_tensor(OC);
            fill_table(p.arch, OC, 0, one, c.in.scales, c.out.scales, table);
        }
        break;
    }
    case NCE_TASK_ELTWISE: {
        need_quant8(c.wt, "weight");
        if (strcmp(p.ew_mode, "ADD") != 0) throw Unsupported(std::string("ew_op.mode '") + p.ew_mode + "': only ADD maps to an NCE eltwise task here");
        if (p.activation != NCE_HWTEST_ACT_NONE) throw Unsupported("the eltwise builder takes no activation");
        for (int i = 0; i < 4; ++i)
            if (p.weight.shape[i] != p.input.shape[i] || p.output.shape[i] != p.input.shape[i]) throw std::runtime_error("eltwise operands and output must have the same shape");
        if (p.weight.dtype != p.input.dtype) throw Unsupported("eltwise operands must share the storage type");
        dense_nhwc(&d->weights, p.weight.dtype, N, IC, IH, IW, p.weight.zero_point);
        d->kernel_size[0] = d->kernel_size[1] = 0;
        d->kernel_strides[0] = d->kernel_strides[1] = 0;
        var->mpe_mode = NCE_MPE_CUBOID_8x16;
        ppe->mode = NCE_PPE_ADD;
        clamp_pre_zp();
        if (c.out.scales.size() > 1) {  // buildEltwiseTest.cpp:100-125
            table_tensor(OC);
            fill_table(p.arch, OC, 0, one, c.in.scales, c.out.scales, table);
        } else {  // calculateQuantScaleVectorForEltwise, ppe_utils.cpp:18-70: first operand's scale only
            const double scale = c.in.scales[0] / c.out.scales[0];
            int32_t m = 0, s = 0, post = 0;
            if (nceQuantApproximate(p.arch, scale, &m, &s, &post) != NCE_RESULT_SUCCESS || post != 0) throw Unsupported("eltwise scale has no fixed-point form");
            ppe->has_quant = 1;
            ppe->quant_mult = m;
            ppe->quant_shift = s;
        }
        break;
    }
    default: throw Unsupported("unknown task type");
    }
}


// ---- case types that expand to several tasks ---------------------------------------------------------

int64_t conv_out(int64_t in, int64_t k, int64_t pad_a, int64_t pad_b, int64_t stride) {
    return (in - k + pad_a + pad_b) / stride + 1;
}

// Rows (SOH) or channels (SOK) each cluster computes. Without broadcast the case lists one output per cluster and the
// sizes are theirs (buildMultiClustersDPUTest.cpp:306-321); with broadcast every entry has the whole shape and the split
// is the even one of the distributed output type: ceil(size / clusters) per cluster, channels in multiples of 16
// (DistributedAttrs, :36-93) - the last cluster takes what is left.
std::vector<int64_t> cluster_sizes(const nce_hwtest_case_s& c, int64_t parent) {
    const size_t n = c.clusters.size();
    std::vector<int64_t> sizes(n, 0);
    if (!c.broadcast) {
        for (size_t i = 0; i < n; ++i) sizes[i] = c.outs[i].pub.shape[c.split_dim];
        return sizes;
    }
    int64_t per = (parent + (int64_t)n - 1) / (int64_t)n;
    if (c.split_dim == 1) per = (per + 15) / 16 * 16;
    int64_t left = parent;
    for (size_t i = 0; i < n; ++i) {
        sizes[i] = std::max<int64_t>(0, std::min(per, left));
        left -= sizes[i];
    }
    return sizes;
}

void parent_output_shape(const nce_hwtest_case_s& c, int64_t (&shape)[4]) {
    for (int i = 0; i < 4; ++i) shape[i] = c.pub.output.shape[i];
    if (c.program == PROGRAM_MULTI_CLUSTERS && !c.broadcast)
        for (size_t k = 1; k < c.outs.size(); ++k) shape[c.split_dim] += c.outs[k].pub.shape[c.split_dim];
}

void program_of(const nce_hwtest_case_s& c, nce_hwtest_program_t* g) {
    memset(g, 0, sizeof(*g));
    const nce_hwtest_case_t& p = c.pub;
    g->num_tasks = 1;
    g->num_outputs = 1;
    for (int i = 0; i < 4; ++i) g->output_shape[0][i] = p.output.shape[i];
    auto outputs = [&](size_t n) {
        if (n > NCE_HWTEST_MAX_OUTPUTS) throw Unsupported("more clusters than this front end describes (" + std::to_string(NCE_HWTEST_MAX_OUTPUTS) + ")");
        g->num_outputs = (int32_t)n;
        for (size_t k = 0; k < n; ++k)
            for (int i = 0; i < 4; ++i) g->output_shape[k][i] = p.output.shape[i];
    };
    switch (c.program) {
    case PROGRAM_DOUBLE_CONV:
        g->num_tasks = 2;
        g->num_intermediates = 1;
        g->intermediate_shape[0] = p.input.shape[0];
        g->intermediate_shape[1] = p.weight.shape[0];
        g->intermediate_shape[2] = conv_out(p.input.shape[2], p.weight.shape[2], p.pad[0], p.pad[2], std::max(1, p.stride[0]));
        g->intermediate_shape[3] = conv_out(p.input.shape[3], p.weight.shape[3], p.pad[1], p.pad[3], std::max(1, p.stride[1]));
        break;
    case PROGRAM_RACE_DPU:
        outputs((size_t)c.num_clusters);
        if (c.iteration_count * c.num_clusters > 1 << 20) throw Unsupported("iteration_count x num_clusters is too large");
        g->num_tasks = (int32_t)(c.iteration_count * c.num_clusters);
        g->outputs_identical = 1;
        break;
    case PROGRAM_DIFFERENT_CLUSTERS:
        outputs(c.clusters.size());
        g->num_tasks = g->num_outputs;
        g->outputs_identical = 1;
        break;
    case PROGRAM_MULTI_CLUSTERS: {
        const size_t n = c.clusters.size();
        outputs(n);
        if (c.broadcast) {  // every cluster's buffer receives every slice
            g->num_tasks = (int32_t)(n * n);
            g->outputs_identical = 1;
        } else {
            g->num_tasks = (int32_t)n;
            for (size_t k = 0; k < n; ++k)
                for (int i = 0; i < 4; ++i) g->output_shape[k][i] = c.outs[k].pub.shape[i];
        }
        break;
    }
    default: break;
    }
}

// Task `index` of a case. Single-task cases: index 0 is nceHwtestBuildTask's task.
void build_at(const nce_hwtest_case_s& c, int32_t index, nce_cluster_task_desc_t* d, nce_dpu_task_t* var, nce_ppe_task_t* ppe,
              int32_t* table, int32_t cap_rows, int32_t* rows, nce_hwtest_binding_t* bind) {
    nce_hwtest_program_t g;
    program_of(c, &g);
    if (index < 0 || index >= g.num_tasks) throw std::runtime_error("task index out of range");
    memset(bind, 0, sizeof(*bind));
    bind->input_tensor = -1;
    if (c.program == PROGRAM_SINGLE) {
        build(c, d, var, ppe, table, cap_rows, rows);
        return;
    }
    // These builders add no PPE task and take no activation (only buildZMConvTest.cpp does): NOOP, storage-range clamp.
    if (c.pub.activation != NCE_HWTEST_ACT_NONE) throw Unsupported(std::string("case type '") + c.pub.case_type + "' takes no activation");
    nce_hwtest_case_s one = c;  // the convolution this task is, as a single-task case
    one.program = PROGRAM_SINGLE;
    switch (c.program) {
    case PROGRAM_DOUBLE_CONV: {
        // Both convolutions share kernel size (taken from the first weights), strides and paddings, and both weights tables
        // are computed from the case's input, first-weights and output types (buildDoubleConvTest.cpp:329-360,
        // hwtest.cpp:114: weightTypes.front()); the tensor between them has the output's type and is dense NHWC.
        if (c.wt2.pub.shape[2] != c.wt.pub.shape[2] || c.wt2.pub.shape[3] != c.wt.pub.shape[3])
            throw Unsupported("DoubleZMajorConvolution: both weights must have the kernel size of the first");
        if (index == 0) {
            for (int i = 0; i < 4; ++i) one.pub.output.shape[i] = one.out.pub.shape[i] = g.intermediate_shape[i];
            copy_str(one.pub.output_order, sizeof(one.pub.output_order), "nhwc");
            bind->output_tensor = -1;
        } else {
            if (c.wt2.pub.shape[1] != g.intermediate_shape[1]) throw std::runtime_error("second weights' input channels differ from the first weights' output channels");
            one.in.pub.dtype = c.out.pub.dtype;
            one.in.pub.zero_point = c.out.pub.zero_point;
            copy_str(one.in.pub.dtype_name, sizeof(one.in.pub.dtype_name), c.out.pub.dtype_name);
            for (int i = 0; i < 4; ++i) one.in.pub.shape[i] = g.intermediate_shape[i];
            one.pub.input = one.in.pub;
            for (int i = 0; i < 4; ++i) one.wt.pub.shape[i] = c.wt2.pub.shape[i];  // (type and scales stay the first weights')
            one.pub.weight = one.wt.pub;
            bind->input_tensor = 0;
            bind->weight_layer = 1;
        }
        build(one, d, var, ppe, table, cap_rows, rows);
        break;
    }
    case PROGRAM_RACE_DPU:
        // iteration i runs the task once per cluster (buildRaceConditionDPUTest.cpp:135-215)
        build(one, d, var, ppe, table, cap_rows, rows);
        bind->output_tensor = index % (int32_t)c.num_clusters;
        var->cluster_id = bind->output_tensor;
        break;
    case PROGRAM_DIFFERENT_CLUSTERS:
        build(one, d, var, ppe, table, cap_rows, rows);
        bind->output_tensor = index;
        var->cluster_id = (int32_t)c.clusters[(size_t)index];
        break;
    case PROGRAM_MULTI_CLUSTERS: {
        // Cluster `slice` computes its rows or channels of the parent output (:543-581; paddings per cluster as
        // getMulticlusteringPaddings, hwtest_utils.cpp:527-597). With broadcast every cluster's output tensor is the whole
        // parent: the task is the whole convolution with ONE workload, the slice's box. Without broadcast the cluster's own
        // tensor holds just the slice, and the task is the convolution that produces it on its own: the slice's weights
        // and table rows (channels), or the input rows the slice reads with the paddings that remain (rows); the binding
        // says where in the case's weights / input that view starts.
        const int32_t n = (int32_t)c.clusters.size();
        const int32_t slice = c.broadcast ? index % n : index;
        int64_t parent[4];
        parent_output_shape(c, parent);
        const std::vector<int64_t> sizes = cluster_sizes(c, parent[c.split_dim]);
        int64_t start = 0;
        for (int32_t k = 0; k < slice; ++k) start += sizes[(size_t)k];
        const int64_t size = sizes[(size_t)slice];
        if (size <= 0 || start + size > parent[c.split_dim]) throw std::runtime_error("MultiClustersDPU: cluster slices do not fit the output");
        // effective paddings and input rows of output rows [start, start + size)
        const int64_t sy = std::max(1, c.pub.stride[0]), IH = c.pub.input.shape[2], KY = c.pub.weight.shape[2];
        const int64_t first = start * sy - c.pub.pad[0], last = (start + size - 1) * sy - c.pub.pad[0] + KY - 1;
        const int64_t pad_top = std::max<int64_t>(0, -first), pad_bottom = std::max<int64_t>(0, last - (IH - 1));
        for (int i = 0; i < 4; ++i) one.pub.output.shape[i] = one.out.pub.shape[i] = parent[i];
        if (c.broadcast) {
            build(one, d, var, ppe, table, cap_rows, rows);
            const int box = c.split_dim == 1 ? 2 : 1;  // out_start / out_end are (x, y, z)
            var->out_start[box] = (int32_t)start;
            var->out_end[box] = (int32_t)(start + size - 1);
            if (c.split_dim == 2) {
                var->pad_top = (int32_t)pad_top;
                var->pad_bottom = (int32_t)pad_bottom;
            }
            bind->output_tensor = index / n;
        } else {
            one.pub.output.shape[c.split_dim] = one.out.pub.shape[c.split_dim] = size;
            if (c.split_dim == 1) {
                one.pub.weight.shape[0] = one.wt.pub.shape[0] = size;
                auto cut = [&](std::vector<double>* v) {
                    if (v->size() > 1) {
                        if ((int64_t)v->size() != parent[1]) throw std::runtime_error("per-channel scale count does not match the output channels");
                        *v = std::vector<double>(v->begin() + start, v->begin() + start + size);
                    }
                };
                cut(&one.wt.scales);
                cut(&one.out.scales);
                build(one, d, var, ppe, table, cap_rows, rows);
                bind->weights_offset_bytes = start * d->weights.strides_bytes[0];
            } else {
                const int64_t r0 = std::max<int64_t>(0, first), r1 = std::min(IH - 1, last);
                if (r1 < r0) throw std::runtime_error("MultiClustersDPU: a cluster's rows read no input row");
                one.pub.input.shape[2] = one.in.pub.shape[2] = r1 - r0 + 1;
                one.pub.pad[0] = (int32_t)pad_top;
                one.pub.pad[2] = (int32_t)pad_bottom;
                build(one, d, var, ppe, table, cap_rows, rows);
                const int64_t row_bytes = d->input.strides_bytes[2];
                d->input.strides_bytes[0] = IH * row_bytes;  // a view of the case's input
                bind->input_offset_bytes = r0 * row_bytes;
            }
            bind->output_tensor = slice;
        }
        var->cluster_id = (int32_t)c.clusters[(size_t)slice];
        break;
    }
    default: throw Unsupported("unknown program kind");
    }
}

void log_error(nce_log_handle_t log, const char* what) {
    if (log != nullptr) log->add(1, "hwtest: %s", what);
}

}  // namespace

extern "C" {

nce_result_t nceHwtestParse(const char* json_text, nce_hwtest_case_handle_t* out_case, nce_log_handle_t log) {
    if (out_case == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    *out_case = nullptr;
    if (json_text == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    try {
        std::unique_ptr<nce_hwtest_case_s> c(new nce_hwtest_case_s());
        parse_case(json_text, c.get());
        *out_case = c.release();
        return NCE_RESULT_SUCCESS;
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (const std::exception& e) {
        log_error(log, e.what());
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    }
}

nce_result_t nceHwtestDestroy(nce_hwtest_case_handle_t hw_case) {
    if (hw_case == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    delete hw_case;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceHwtestGetCase(nce_hwtest_case_handle_t hw_case, nce_hwtest_case_t* out) {
    if (hw_case == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (out == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    *out = hw_case->pub;
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceHwtestGetScales(nce_hwtest_case_handle_t hw_case, int32_t which, double* scales, int32_t capacity) {
    if (hw_case == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (scales == nullptr || capacity < 0 || which < 0 || which > 2) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    const Layer& l = which == 0 ? hw_case->in : which == 1 ? hw_case->wt : hw_case->out;
    const size_t n = std::min<size_t>((size_t)capacity, l.scales.size());
    for (size_t i = 0; i < n; ++i) scales[i] = l.scales[i];
    return NCE_RESULT_SUCCESS;
}

nce_result_t nceHwtestBuildTask(nce_hwtest_case_handle_t hw_case, nce_cluster_task_desc_t* desc, nce_dpu_task_t* variant,
                                nce_ppe_task_t* ppe, int32_t* table, int32_t table_capacity_rows, int32_t* table_rows,
                                nce_log_handle_t log) {
    if (hw_case == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (desc == nullptr || variant == nullptr || ppe == nullptr || table_rows == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    try {
        nce_hwtest_binding_t binding;
        build_at(*hw_case, 0, desc, variant, ppe, table, table_capacity_rows, table_rows, &binding);
        return NCE_RESULT_SUCCESS;
    } catch (const Unsupported& e) {
        log_error(log, e.what());
        return NCE_RESULT_ERROR_UNSUPPORTED;
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (const std::exception& e) {
        log_error(log, e.what());
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    }
}

nce_result_t nceHwtestGetProgram(nce_hwtest_case_handle_t hw_case, nce_hwtest_program_t* out, nce_log_handle_t log) {
    if (hw_case == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (out == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    try {
        program_of(*hw_case, out);
        return NCE_RESULT_SUCCESS;
    } catch (const Unsupported& e) {
        log_error(log, e.what());
        return NCE_RESULT_ERROR_UNSUPPORTED;
    } catch (const std::exception& e) {
        log_error(log, e.what());
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    }
}

nce_result_t nceHwtestBuildTaskAt(nce_hwtest_case_handle_t hw_case, int32_t index, nce_cluster_task_desc_t* desc, nce_dpu_task_t* variant,
                                  nce_ppe_task_t* ppe, int32_t* table, int32_t table_capacity_rows, int32_t* table_rows,
                                  nce_hwtest_binding_t* binding, nce_log_handle_t log) {
    if (hw_case == nullptr) return NCE_RESULT_ERROR_INVALID_NULL_HANDLE;
    if (desc == nullptr || variant == nullptr || ppe == nullptr || table_rows == nullptr || binding == nullptr) return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    try {
        build_at(*hw_case, index, desc, variant, ppe, table, table_capacity_rows, table_rows, binding);
        return NCE_RESULT_SUCCESS;
    } catch (const Unsupported& e) {
        log_error(log, e.what());
        return NCE_RESULT_ERROR_UNSUPPORTED;
    } catch (const std::bad_alloc&) {
        return NCE_RESULT_ERROR_OUT_OF_MEMORY;
    } catch (const std::exception& e) {
        log_error(log, e.what());
        return NCE_RESULT_ERROR_INVALID_ARGUMENT;
    }
}

}  // extern "C"
