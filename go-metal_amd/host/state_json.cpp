// JSON form of optimizer.OptimizerState, field for field what Go's encoding/json writes for
// the struct tags at optimizer/interface.go:47-51 and checkpoints/checkpoint.go:81-86:
//   {"type": "...", "parameters": {...}, "state_data": [{"name", "shape", "data", "state_type"}]}
// Parsing turns every JSON number into a float64 ParamValue, as Go's decoder does for
// map[string]interface{}; float32 data is printed with 9 significant digits, which
// round-trips every binary32 value exactly.
#include "optimizer.hpp"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace gometal {
namespace optimizer {

static void appendEscaped(std::string &out, const std::string &s)
{
    out.push_back('"');
    for (unsigned char c : s) {
        switch (c) {
        case '"': out += "\\\""; break;
        case '\\': out += "\\\\"; break;
        case '\n': out += "\\n"; break;
        case '\r': out += "\\r"; break;
        case '\t': out += "\\t"; break;
        default:
            if (c < 0x20) {
                char buf[8];
                std::snprintf(buf, sizeof buf, "\\u%04x", c);
                out += buf;
            } else {
                out.push_back((char)c);
            }
        }
    }
    out.push_back('"');
}

// JSON has no inf / NaN: encoding/json's Marshal fails with an UnsupportedValueError
// ("json: unsupported value: NaN"), and so does this encoder; `bad` receives Go's spelling of
// the first such value.
static void appendFloat(std::string &out, double v, int digits, std::string &bad)
{
    if (!std::isfinite(v)) {
        if (bad.empty()) bad = std::isnan(v) ? "NaN" : (v > 0 ? "+Inf" : "-Inf");
        out += "null";
        return;
    }
    char buf[40];
    std::snprintf(buf, sizeof buf, "%.*g", digits, v);
    out += buf;
}

std::pair<std::string, Error> OptimizerState::ToJSON() const
{
    std::string out, bad;
    out.reserve(256 + StateData.size() * 64);
    out += "{\"type\":";
    appendEscaped(out, Type);
    out += ",\"parameters\":{";
    bool first = true;
    for (const auto &kv : Parameters) {          // std::map iterates in key order, like encoding/json
        if (!first) out.push_back(',');
        first = false;
        appendEscaped(out, kv.first);
        out.push_back(':');
        if (const double *d = std::get_if<double>(&kv.second)) appendFloat(out, *d, 17, bad);
        else if (const float *f = std::get_if<float>(&kv.second)) appendFloat(out, *f, 9, bad);
        else if (const bool *b = std::get_if<bool>(&kv.second)) out += *b ? "true" : "false";
        else if (const uint64_t *u = std::get_if<uint64_t>(&kv.second)) out += std::to_string(*u);
        else appendEscaped(out, std::get<std::string>(kv.second));
    }
    out += "},\"state_data\":[";
    for (size_t t = 0; t < StateData.size(); t++) {
        const auto &tensor = StateData[t];
        if (t) out.push_back(',');
        out += "{\"name\":";
        appendEscaped(out, tensor.Name);
        out += ",\"shape\":[";
        for (size_t i = 0; i < tensor.Shape.size(); i++) {
            if (i) out.push_back(',');
            out += std::to_string(tensor.Shape[i]);
        }
        out += "],\"data\":[";
        for (size_t i = 0; i < tensor.Data.size(); i++) {
            if (i) out.push_back(',');
            appendFloat(out, tensor.Data[i], 9, bad);
        }
        out += "],\"state_type\":";
        appendEscaped(out, tensor.StateType);
        out.push_back('}');
    }
    out += "]}";
    if (!bad.empty()) return {std::string(), Errorf("json: unsupported value: %s", bad.c_str())};
    return {std::move(out), ""};
}

namespace {

struct Parser {
    const char *p;
    const char *end;
    Error err;

    void ws()
    {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) p++;
    }
    bool fail(const char *what)
    {
        if (err.empty()) err = Errorf("invalid optimizer state JSON: %s", what);
        return false;
    }
    bool expect(char c)
    {
        ws();
        if (p < end && *p == c) {
            p++;
            return true;
        }
        return fail("unexpected character");
    }
    bool peek(char c)
    {
        ws();
        return p < end && *p == c;
    }
    bool string(std::string &out)
    {
        ws();
        if (p >= end || *p != '"') return fail("expected a string");
        p++;
        out.clear();
        while (p < end && *p != '"') {
            if (*p == '\\') {
                if (++p >= end) return fail("bad escape");
                switch (*p) {
                case 'n': out.push_back('\n'); break;
                case 't': out.push_back('\t'); break;
                case 'r': out.push_back('\r'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'u': {
                    if (end - p < 5) return fail("bad \\u escape");
                    char hex[5] = {p[1], p[2], p[3], p[4], 0};
                    unsigned long cp = std::strtoul(hex, nullptr, 16);
                    if (cp < 0x80) out.push_back((char)cp);
                    else out.push_back('?');          // names here are ASCII
                    p += 4;
                    break;
                }
                default: out.push_back(*p);
                }
                p++;
            } else {
                out.push_back(*p++);
            }
        }
        if (p >= end) return fail("unterminated string");
        p++;
        return true;
    }
    // A JSON number, by the JSON grammar only: -? (0 | [1-9][0-9]*) (. [0-9]+)? ([eE] [+-]? [0-9]+)?
    // (strtod alone would also take "nan", "inf", hex floats and a leading '+').  A value beyond the
    // float64 range is an error, as in encoding/json ("cannot unmarshal number 1e400").
    bool number(double &out)
    {
        ws();
        const char *q = p;
        if (q < end && *q == '-') q++;
        if (q >= end || *q < '0' || *q > '9') return fail("expected a number");
        if (*q == '0') q++;
        else while (q < end && *q >= '0' && *q <= '9') q++;
        if (q < end && *q == '.') {
            q++;
            if (q >= end || *q < '0' || *q > '9') return fail("expected a digit after the decimal point");
            while (q < end && *q >= '0' && *q <= '9') q++;
        }
        if (q < end && (*q == 'e' || *q == 'E')) {
            q++;
            if (q < end && (*q == '+' || *q == '-')) q++;
            if (q >= end || *q < '0' || *q > '9') return fail("expected a digit in the exponent");
            while (q < end && *q >= '0' && *q <= '9') q++;
        }
        const std::string token(p, q);           // strtod needs a terminated string of exactly this token
        out = std::strtod(token.c_str(), nullptr);
        if (!std::isfinite(out)) return fail("number out of range");
        p = q;
        return true;
    }
    // An element of a []float32 / []int: a JSON null leaves the element at zero, as encoding/json
    // does ("the JSON null value has no effect" on a non-pointer value).
    bool elementIsNull()
    {
        ws();
        return literal("null");
    }
    bool literal(const char *word)
    {
        const size_t n = std::strlen(word);
        if ((size_t)(end - p) >= n && std::strncmp(p, word, n) == 0) {
            p += n;
            return true;
        }
        return false;
    }
    // skips any value (unknown keys)
    bool skip()
    {
        ws();
        if (p >= end) return fail("truncated");
        if (*p == '"') {
            std::string s;
            return string(s);
        }
        if (*p == '{' || *p == '[') {
            const char open = *p, close = (*p == '{') ? '}' : ']';
            p++;
            if (peek(close)) {
                p++;
                return true;
            }
            for (;;) {
                if (open == '{') {
                    std::string k;
                    if (!string(k) || !expect(':')) return false;
                }
                if (!skip()) return false;
                if (peek(',')) {
                    p++;
                    continue;
                }
                return expect(close);
            }
        }
        if (literal("true") || literal("false") || literal("null")) return true;
        double d;
        return number(d);
    }
};

}  // namespace

std::pair<std::string, Error> OptimizerState::ToCheckpointJSON() const
{
    // field order of checkpoints.Checkpoint (checkpoint.go:38-52); a nil model spec and weight
    // list encode as null, the zero TrainingState as zeros
    std::string out = "{\"model_spec\":null,\"weights\":null,\"training_state\":{\"epoch\":0,\"step\":0,"
                      "\"learning_rate\":0,\"best_loss\":0,\"best_accuracy\":0,\"total_steps\":0},"
                      "\"optimizer_state\":";
    auto [body, err] = ToJSON();
    if (!err.empty()) return {std::string(), err};
    out += body;
    out += ",\"metadata\":{\"version\":\"1.0.0\",\"framework\":\"go-metal\","
           "\"created_at\":\"0001-01-01T00:00:00Z\"}}";
    return {std::move(out), ""};
}

std::pair<OptimizerState, Error> OptimizerState::FromCheckpointJSON(const std::string &text)
{
    Parser ps{text.data(), text.data() + text.size(), ""};
    if (!ps.expect('{')) return {OptimizerState{}, ps.err};
    if (!ps.peek('}')) {
        for (;;) {
            std::string key;
            if (!ps.string(key) || !ps.expect(':')) return {OptimizerState{}, ps.err};
            ps.ws();
            if (key == "optimizer_state") {
                if (ps.literal("null")) break;
                const char *begin = ps.p;
                if (!ps.skip()) return {OptimizerState{}, ps.err};
                return FromJSON(std::string(begin, ps.p));
            }
            if (!ps.skip()) return {OptimizerState{}, ps.err};
            if (ps.peek(',')) {
                ps.p++;
                continue;
            }
            break;
        }
    }
    return {OptimizerState{}, Errorf("checkpoint has no optimizer state")};
}

std::pair<OptimizerState, Error> OptimizerState::FromJSON(const std::string &text)
{
    OptimizerState st;
    Parser ps{text.data(), text.data() + text.size(), ""};
    if (!ps.expect('{')) return {st, ps.err};
    if (!ps.peek('}')) {
        for (;;) {
            std::string key;
            if (!ps.string(key) || !ps.expect(':')) return {st, ps.err};
            if (key == "type") {
                if (!ps.string(st.Type)) return {st, ps.err};
            } else if (key == "parameters") {
                if (!ps.expect('{')) return {st, ps.err};
                if (!ps.peek('}')) {
                    for (;;) {
                        std::string name;
                        if (!ps.string(name) || !ps.expect(':')) return {st, ps.err};
                        ps.ws();
                        if (ps.peek('"')) {
                            std::string s;
                            if (!ps.string(s)) return {st, ps.err};
                            st.Parameters[name] = s;
                        } else if (ps.literal("true")) {
                            st.Parameters[name] = true;
                        } else if (ps.literal("false")) {
                            st.Parameters[name] = false;
                        } else if (ps.peek('{') || ps.peek('[')) {
                            if (!ps.skip()) return {st, ps.err};
                        } else if (ps.literal("null")) {
                            // a nil interface value: every typed lookup falls back to its default
                        } else {
                            double d;
                            if (!ps.number(d)) return {st, ps.err};
                            st.Parameters[name] = d;
                        }
                        if (ps.peek(',')) {
                            ps.p++;
                            continue;
                        }
                        break;
                    }
                }
                if (!ps.expect('}')) return {st, ps.err};
            } else if (key == "state_data") {
                st.StateData.clear();          // a repeated key replaces the slice, as encoding/json does
                ps.ws();
                if (ps.literal("null")) {
                    // Go writes a nil slice as null
                } else {
                    if (!ps.expect('[')) return {st, ps.err};
                    if (!ps.peek(']')) {
                        for (;;) {
                            checkpoints::OptimizerTensor t;
                            if (!ps.expect('{')) return {st, ps.err};
                            if (!ps.peek('}')) {
                                for (;;) {
                                    std::string f;
                                    if (!ps.string(f) || !ps.expect(':')) return {st, ps.err};
                                    if (f == "name") {
                                        if (!ps.string(t.Name)) return {st, ps.err};
                                    } else if (f == "state_type") {
                                        if (!ps.string(t.StateType)) return {st, ps.err};
                                    } else if (f == "shape" || f == "data") {
                                        ps.ws();
                                        if (ps.literal("null")) {
                                        } else {
                                            if (!ps.expect('[')) return {st, ps.err};
                                            if (!ps.peek(']')) {
                                                for (;;) {
                                                    double d = 0;
                                                    if (!ps.elementIsNull() && !ps.number(d)) return {st, ps.err};
                                                    if (f == "shape") {
                                                        // an int field: integral and in range, else
                                                        // "cannot unmarshal number into Go struct field of type int"
                                                        if (d != std::floor(d) || d < -2147483648.0 || d > 2147483647.0) {
                                                            ps.fail("shape entry is not an int");
                                                            return {st, ps.err};
                                                        }
                                                        t.Shape.push_back((int)d);
                                                    } else {
                                                        // a float32 field: a value that rounds to infinity is refused
                                                        if (std::fabs(d) > 3.4028235677973366e38) {
                                                            ps.fail("data entry is out of the float32 range");
                                                            return {st, ps.err};
                                                        }
                                                        t.Data.push_back((float)d);
                                                    }
                                                    if (ps.peek(',')) {
                                                        ps.p++;
                                                        continue;
                                                    }
                                                    break;
                                                }
                                            }
                                            if (!ps.expect(']')) return {st, ps.err};
                                        }
                                    } else if (!ps.skip()) {
                                        return {st, ps.err};
                                    }
                                    if (ps.peek(',')) {
                                        ps.p++;
                                        continue;
                                    }
                                    break;
                                }
                            }
                            if (!ps.expect('}')) return {st, ps.err};
                            st.StateData.push_back(std::move(t));
                            if (ps.peek(',')) {
                                ps.p++;
                                continue;
                            }
                            break;
                        }
                    }
                    if (!ps.expect(']')) return {st, ps.err};
                }
            } else if (!ps.skip()) {
                return {st, ps.err};
            }
            if (ps.peek(',')) {
                ps.p++;
                continue;
            }
            break;
        }
    }
    if (!ps.expect('}')) return {st, ps.err};
    ps.ws();
    if (ps.p != ps.end) {          // encoding/json: "invalid character ... after top-level value"
        ps.fail("data after the top-level value");
        return {st, ps.err};
    }
    return {st, ""};
}

}  // namespace optimizer
}  // namespace gometal
