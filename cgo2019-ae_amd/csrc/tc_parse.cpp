// Expression grammar of the reference generator, restated in C++.
//
// Follows cogent/src/generators/tc_gen_etc.py:4-18 (lines starting with '#'
// are skipped, every other line is an expression) and
// cogent/src/algs/bases/tc_gen_inputs.py:29-108: the characters '[', ']' and
// ';' are deleted, the line is split on whitespace, and the tokens are read by
// POSITION:
//     0 output name      1 output "idx,size,idx,size,..."   2 operator
//     3 "sum(idx,size,...)"   4 "*"   5 left name   6 left "idx,idx,..."
//     7 "*"   8 right name   9 right "idx,idx,..."
// so index lists must not contain blanks ("whitespace-sensitive").  Inputs the
// reference cannot process -- fewer than ten tokens (its list index raises), a
// blank line, an odd idx/size list, a size that is not an integer -- are
// reported as errors here instead of a crash or a silent mis-parse.
#include "tc_ir.hpp"
#include <cctype>
#include <cstdlib>
#include <fstream>
#include <sstream>

namespace cogent {

static std::vector<std::string> split_ws(const std::string& s)
{
    std::vector<std::string> out;
    std::istringstream is(s);
    std::string t;
    while (is >> t) out.push_back(t);
    return out;
}

static std::vector<std::string> split_comma(const std::string& s)
{
    std::vector<std::string> out;
    std::string cur;
    for (char ch : s) {
        if (ch == ',') { out.push_back(cur); cur.clear(); }
        else cur.push_back(ch);
    }
    out.push_back(cur);
    return out;
}

static bool parse_int(const std::string& s, int& v)
{
    if (s.empty()) return false;
    size_t i = 0;
    if (s[0] == '+' || s[0] == '-') i = 1;
    if (i == s.size()) return false;
    for (size_t j = i; j < s.size(); j++) if (!isdigit((unsigned char)s[j])) return false;
    long long x = atoll(s.c_str());
    if (x > 2147483647LL || x < -2147483648LL) return false;
    v = (int)x;
    return true;
}

static bool is_name(const std::string& s)
{
    if (s.empty()) return false;
    for (char ch : s) if (!(isalnum((unsigned char)ch) || ch == '_')) return false;
    return true;
}

static bool parse_pairs(const std::string& list, const char* what, std::vector<std::string>& names,
                        std::vector<int>& sizes, std::string& err)
{
    std::vector<std::string> items = split_comma(list);
    if (items.size() % 2 != 0) {
        // tc_gen_inputs.py:63-64 / :84-85 print "ERROR: ... should have indices and their representative problem sizes"
        err = std::string("the ") + what + " must list every index with its representative problem size (idx,size,idx,size,...)";
        return false;
    }
    for (size_t i = 0; i < items.size(); i += 2) {
        int v = 0;
        if (!is_name(items[i])) { err = std::string("bad index name '") + items[i] + "' in the " + what; return false; }
        if (!parse_int(items[i + 1], v)) { err = std::string("representative size '") + items[i + 1] + "' of index '" + items[i] + "' is not an integer"; return false; }
        if (v <= 0) { err = std::string("representative size of index '") + items[i] + "' must be positive"; return false; }
        names.push_back(items[i]);
        sizes.push_back(v);
    }
    return true;
}

static std::string replace_all(std::string s, const std::string& from, const std::string& to)
{
    size_t pos = 0;
    while ((pos = s.find(from, pos)) != std::string::npos) { s.replace(pos, from.size(), to); pos += to.size(); }
    return s;
}

bool parse_expression_line(const std::string& line, Contraction& c, std::string& err)
{
    c = Contraction();
    c.text = line;
    std::string s;
    for (char ch : line) if (ch != '[' && ch != ']' && ch != ';') s.push_back(ch);
    std::vector<std::string> tok = split_ws(s);
    if (tok.empty()) { err = "empty expression line"; return false; }
    if (tok.size() < 10) { err = "expression needs ten blank-separated fields: out [..] op sum(..) * a [..] * b [..];"; return false; }

    c.out_name = tok[0];
    c.op = tok[2];
    c.a_name = tok[5];
    c.b_name = tok[8];
    if (c.op == "+=") c.sign = 1;
    else if (c.op == "-=") c.sign = -1;
    else { err = "operator must be += or -=, got '" + c.op + "'"; return false; }
    if (!is_name(c.out_name) || !is_name(c.a_name) || !is_name(c.b_name)) { err = "bad tensor name"; return false; }

    std::vector<std::string> out_names, int_names;
    std::vector<int> out_sizes, int_sizes;
    if (!parse_pairs(tok[1], "output tensor", out_names, out_sizes, err)) return false;
    // "sum(" and ")" are deleted wherever they occur (tc_gen_inputs.py:77-78)
    std::string inner = replace_all(replace_all(tok[3], "sum(", ""), ")", "");
    if (tok[3].find("sum(") == std::string::npos) { err = "fourth field must be sum(idx,size,...)"; return false; }
    if (!parse_pairs(inner, "sum()", int_names, int_sizes, err)) return false;

    auto find = [&](const std::string& n) -> int {
        for (int i = 0; i < (int)c.indices.size(); i++) if (c.indices[i].name == n) return i;
        return -1;
    };
    for (size_t i = 0; i < out_names.size(); i++) {
        if (find(out_names[i]) >= 0) { err = "index '" + out_names[i] + "' listed twice"; return false; }
        Index ix; ix.name = out_names[i]; ix.rep_size = out_sizes[i]; ix.internal = false;
        c.out_idx.push_back((int)c.indices.size());
        c.indices.push_back(ix);
    }
    for (size_t i = 0; i < int_names.size(); i++) {
        if (find(int_names[i]) >= 0) { err = "index '" + int_names[i] + "' listed twice"; return false; }
        Index ix; ix.name = int_names[i]; ix.rep_size = int_sizes[i]; ix.internal = true;
        c.int_idx.push_back((int)c.indices.size());
        c.indices.push_back(ix);
    }
    auto operand = [&](const std::string& list, std::vector<int>& ids) -> bool {
        for (const std::string& n : split_comma(list)) {
            int id = find(n);
            if (id < 0) { err = "input index '" + n + "' is neither an output index nor summed"; return false; }
            for (int v : ids) if (v == id) { err = "index '" + n + "' repeated inside one input"; return false; }
            ids.push_back(id);
        }
        return true;
    };
    if (!operand(tok[6], c.a_idx) || !operand(tok[9], c.b_idx)) return false;

    // a contraction: every output index in exactly one input, every summed index in both
    for (int id : c.out_idx) {
        if (c.in_a(id) == c.in_b(id)) { err = "output index '" + c.indices[id].name + "' must appear in exactly one input"; return false; }
    }
    for (int id : c.int_idx) {
        if (!c.in_a(id) || !c.in_b(id)) { err = "summed index '" + c.indices[id].name + "' must appear in both inputs"; return false; }
    }
    if ((int)c.indices.size() > 12) { err = "more than 12 distinct indices"; return false; }
    return true;
}

bool parse_expression_text(const std::string& text, std::vector<Contraction>& out, std::string& err)
{
    std::istringstream is(text);
    std::string line;
    int lineno = 0;
    while (std::getline(is, line)) {
        lineno++;
        if (!line.empty() && line.back() == '\r') line.pop_back();
        if (!line.empty() && line[0] == '#') continue;     // tc_gen_etc.py:11
        Contraction c;
        std::string e;
        if (!parse_expression_line(line, c, e)) {
            err = "line " + std::to_string(lineno) + ": " + e;
            return false;
        }
        out.push_back(c);
    }
    if (out.empty()) { err = "no expression found"; return false; }
    return true;
}

bool parse_expression_file(const std::string& path, std::vector<Contraction>& out, std::string& err)
{
    std::ifstream f(path);
    if (!f) { err = "cannot open '" + path + "'"; return false; }
    std::stringstream ss;
    ss << f.rdbuf();
    return parse_expression_text(ss.str(), out, err);
}

long long contraction_flops(const Contraction& c, const int* sizes)
{
    // cogent/src/codes/kernels/tc_interface.py:289-305: 2 * product of all extents
    long long f = 2;
    for (int i = 0; i < c.n_idx(); i++) f *= sizes[i];
    return f;
}

long long contraction_bytes(const Contraction& c, DType t, const int* sizes)
{
    long long nc = 1, na = 1, nb = 1;
    for (int id : c.out_idx) nc *= sizes[id];
    for (int id : c.a_idx) na *= sizes[id];
    for (int id : c.b_idx) nb *= sizes[id];
    return (long long)(t == DType::F64 ? 8 : 4) * (na + nb + 2 * nc);
}

}  // namespace cogent
