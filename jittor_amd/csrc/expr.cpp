#include "expr.h"
#include "common.h"
#include <cctype>
#include <map>

namespace mjt {

namespace {

struct Token {
    enum Kind { NUM_INT, NUM_FLOAT, IDENT, EXTRA, OP, END } kind;
    std::string text;
    int64_t ival = 0;
};

std::vector<Token> tokenize(const std::string& s) {
    std::vector<Token> out;
    size_t i = 0, n = s.size();
    while (i < n) {
        unsigned char c = s[i];
        if (isspace(c)) {
            i++;
            continue;
        }
        Token t;
        if (c == '@') {
            MJT_CHECK(i + 1 < n && s[i + 1] == 'e', "index expression '" << s << "': '@' must start @eK(...)");
            size_t j = i + 2;
            MJT_CHECK(j < n && isdigit((unsigned char)s[j]), "index expression '" << s << "': missing K in @eK");
            int64_t k = 0;
            while (j < n && isdigit((unsigned char)s[j])) k = k * 10 + (s[j++] - '0');
            t.kind = Token::EXTRA;
            t.ival = k;
            i = j;
        } else if (isdigit(c)) {
            size_t j = i;
            if (c == '0' && j + 1 < n && (s[j + 1] == 'x' || s[j + 1] == 'X')) {
                j += 2;
                int64_t v = 0;
                MJT_CHECK(j < n && isxdigit((unsigned char)s[j]), "bad hex literal in '" << s << "'");
                while (j < n && isxdigit((unsigned char)s[j])) {
                    char h = (char)tolower(s[j++]);
                    v = v * 16 + (isdigit((unsigned char)h) ? h - '0' : h - 'a' + 10);
                }
                t.kind = Token::NUM_INT;
                t.ival = v;
            } else if (c == '0' && j + 1 < n && (s[j + 1] == 'b' || s[j + 1] == 'B')) {
                j += 2;
                int64_t v = 0;
                MJT_CHECK(j < n && (s[j] == '0' || s[j] == '1'), "bad binary literal in '" << s << "'");
                while (j < n && (s[j] == '0' || s[j] == '1')) v = v * 2 + (s[j++] - '0');
                t.kind = Token::NUM_INT;
                t.ival = v;
            } else {
                int64_t v = 0;
                while (j < n && isdigit((unsigned char)s[j])) v = v * 10 + (s[j++] - '0');
                if (j < n && (s[j] == '.' || s[j] == 'e' || s[j] == 'E')) {
                    if (s[j] == '.') {
                        j++;
                        while (j < n && isdigit((unsigned char)s[j])) j++;
                    }
                    if (j < n && (s[j] == 'e' || s[j] == 'E')) {
                        j++;
                        if (j < n && (s[j] == '+' || s[j] == '-')) j++;
                        while (j < n && isdigit((unsigned char)s[j])) j++;
                    }
                    if (j < n && s[j] == 'f') j++;
                    t.kind = Token::NUM_FLOAT;
                    t.text = s.substr(i, j - i);
                } else {
                    t.kind = Token::NUM_INT;
                    t.ival = v;
                }
            }
            i = j;
        } else if (isalpha(c) || c == '_') {
            size_t j = i;
            while (j < n && (isalnum((unsigned char)s[j]) || s[j] == '_')) j++;
            t.kind = Token::IDENT;
            t.text = s.substr(i, j - i);
            i = j;
        } else {
            static const char* two[] = {"<<", ">>", "<=", ">=", "==", "!=", "&&", "||", "//"};
            t.kind = Token::OP;
            bool found = false;
            for (const char* op : two)
                if (i + 1 < n && s[i] == op[0] && s[i + 1] == op[1]) {
                    t.text = op;
                    found = true;
                    break;
                }
            // the reference rejects '//' and recommends int(a/b)
            // (opt/pass/loop_var_analyze_pass.cc:298-309)
            MJT_CHECK(!(found && t.text == "//"),
                      "index expression '" << s << "': '//' is not a C operator, use int(a/b)");
            if (!found) {
                MJT_CHECK(strchr("+-*/%<>&^|!~?:(),", c) != nullptr,
                          "index expression '" << s << "': unexpected character '" << (char)c << "'");
                t.text = std::string(1, (char)c);
            }
            i += t.text.size();
        }
        out.push_back(t);
    }
    Token e;
    e.kind = Token::END;
    out.push_back(e);
    return out;
}

int bin_prec(const std::string& op) {
    static const std::map<std::string, int> p = {
        {"||", 1}, {"&&", 2}, {"|", 3}, {"^", 4}, {"&", 5}, {"==", 6}, {"!=", 6}, {"<", 7}, {"<=", 7},
        {">", 7},  {">=", 7}, {"<<", 8}, {">>", 8}, {"+", 9}, {"-", 9}, {"*", 10}, {"/", 10}, {"%", 10}};
    auto it = p.find(op);
    return it == p.end() ? -1 : it->second;
}

bool is_cast_name(const std::string& s) {
    static const char* names[] = {"int", "int32", "int64", "index_t", "float", "float32", "double", "float64", "bool"};
    for (const char* n : names)
        if (s == n) return true;
    return false;
}

struct Parser {
    const std::string& src;
    std::vector<Token> t;
    size_t p = 0;
    explicit Parser(const std::string& s) : src(s), t(tokenize(s)) {}

    const Token& peek() const { return t[p]; }
    Token take() { return t[p++]; }
    bool peek_op(const char* op) const { return t[p].kind == Token::OP && t[p].text == op; }
    void expect(const char* op) {
        MJT_CHECK(peek_op(op), "index expression '" << src << "': expected '" << op << "'");
        p++;
    }

    std::unique_ptr<Expr> ternary() {
        auto c = binary(1);
        if (peek_op("?")) {
            p++;
            auto a = ternary();
            expect(":");
            auto b = ternary();
            auto e = std::make_unique<Expr>();
            e->kind = Expr::TERNARY;
            e->kids.push_back(std::move(c));
            e->kids.push_back(std::move(a));
            e->kids.push_back(std::move(b));
            return e;
        }
        return c;
    }
    std::unique_ptr<Expr> binary(int minprec) {
        auto lhs = unary();
        for (;;) {
            if (peek().kind != Token::OP) return lhs;
            int pr = bin_prec(peek().text);
            if (pr < 0 || pr < minprec) return lhs;
            std::string op = take().text;
            auto rhs = binary(pr + 1);
            auto e = std::make_unique<Expr>();
            e->kind = Expr::BINARY;
            e->text = op;
            e->kids.push_back(std::move(lhs));
            e->kids.push_back(std::move(rhs));
            lhs = std::move(e);
        }
    }
    std::vector<std::unique_ptr<Expr>> args() {
        std::vector<std::unique_ptr<Expr>> a;
        expect("(");
        if (peek_op(")")) {
            p++;
            return a;
        }
        for (;;) {
            a.push_back(ternary());
            if (peek_op(")")) {
                p++;
                return a;
            }
            expect(",");
        }
    }
    std::unique_ptr<Expr> unary() {
        Token k = take();
        auto e = std::make_unique<Expr>();
        if (k.kind == Token::OP && (k.text == "-" || k.text == "+" || k.text == "!" || k.text == "~")) {
            e->kind = Expr::UNARY;
            e->text = k.text;
            e->kids.push_back(unary());
            return e;
        }
        if (k.kind == Token::OP && k.text == "(") {
            auto inner = ternary();
            expect(")");
            return inner;
        }
        if (k.kind == Token::NUM_INT) {
            e->kind = Expr::CONST_INT;
            e->ival = k.ival;
            return e;
        }
        if (k.kind == Token::NUM_FLOAT) {
            e->kind = Expr::CONST_FLOAT;
            e->text = k.text;
            return e;
        }
        if (k.kind == Token::EXTRA) {
            e->kind = Expr::EXTRA;
            e->extra = (int)k.ival;
            e->kids = args();
            return e;
        }
        if (k.kind == Token::IDENT) {
            if (is_cast_name(k.text) && peek_op("(")) {
                auto a = args();
                MJT_CHECK(a.size() == 1, "index expression '" << src << "': cast takes one argument");
                e->kind = Expr::CAST;
                e->text = k.text;
                e->kids = std::move(a);
                return e;
            }
            e->kind = Expr::VAR;
            e->text = k.text;
            return e;
        }
        MJT_FAIL(MJT_ERR_INVALID, "index expression '" << src << "': unexpected token");
    }
};

// name + decimal suffix, e.g. "xshape3" -> ("xshape", 3)
bool split_name(const std::string& s, std::string* base, int* idx) {
    size_t j = s.size();
    while (j > 0 && isdigit((unsigned char)s[j - 1])) j--;
    if (j == s.size() || j == 0) return false;
    *base = s.substr(0, j);
    *idx = atoi(s.c_str() + j);
    return true;
}

int64_t c_div(int64_t a, int64_t b) { return a / b; }   // C++ integer division truncates toward zero

}  // namespace

std::unique_ptr<Expr> parse_expr(const std::string& s) {
    Parser ps(s);
    auto e = ps.ternary();
    MJT_CHECK(ps.peek().kind == Token::END, "index expression '" << s << "': trailing tokens");
    return e;
}

void validate_expr(const Expr& e, const ExprEnv& env) {
    if (e.kind == Expr::VAR) {
        if (e.text == "XDIM" || e.text == "YDIM") return;
        std::string base;
        int idx = 0;
        bool ok = false;
        if (split_name(e.text, &base, &idx)) {
            if (base == "i") ok = idx < env.n_loop;
            else if (base == "xshape" || base == "xstride") ok = idx < env.xdim;
            else if (base == "yshape" || base == "ystride") ok = idx < env.ydim;
        }
        MJT_CHECK(ok, "index expression: unknown identifier '" << e.text << "'");
    }
    if (e.kind == Expr::EXTRA) {
        MJT_CHECK(e.extra >= 0 && e.extra < (int)env.extra_rank.size(),
                  "index expression: @e" << e.extra << " but only " << env.extra_rank.size() << " extras");
        MJT_CHECK((int)e.kids.size() == env.extra_rank[e.extra],
                  "index expression: @e" << e.extra << " expects " << env.extra_rank[e.extra] << " indexes, got "
                                         << e.kids.size());
    }
    for (auto& k : e.kids) validate_expr(*k, env);
}

std::string emit_c(const Expr& e) {
    switch (e.kind) {
        case Expr::CONST_INT: return std::to_string(e.ival);
        case Expr::CONST_FLOAT: return e.text;
        case Expr::VAR: return e.text;
        case Expr::UNARY: return "(" + e.text + emit_c(*e.kids[0]) + ")";
        case Expr::BINARY: return "(" + emit_c(*e.kids[0]) + e.text + emit_c(*e.kids[1]) + ")";
        case Expr::TERNARY:
            return "(" + emit_c(*e.kids[0]) + "?" + emit_c(*e.kids[1]) + ":" + emit_c(*e.kids[2]) + ")";
        case Expr::CAST: {
            std::string t = e.text;
            if (t == "int32") t = "int";
            if (t == "int64") t = "long long";
            if (t == "float32") t = "float";
            if (t == "float64") t = "double";
            return "((" + t + ")" + emit_c(*e.kids[0]) + ")";
        }
        case Expr::EXTRA: {
            std::string n = "e" + std::to_string(e.extra);
            std::string s = n + "p[";
            for (size_t i = 0; i < e.kids.size(); i++) {
                if (i) s += "+";
                s += "(index_t)(" + emit_c(*e.kids[i]) + ")*" + n + "stride" + std::to_string(i);
            }
            if (e.kids.empty()) s += "0";
            return s + "]";
        }
    }
    return "";
}

bool is_pure(const Expr& e) {
    if (e.kind == Expr::EXTRA) return false;
    for (auto& k : e.kids)
        if (!is_pure(*k)) return false;
    return true;
}

static bool is_const(const Affine& a) {
    for (int i = 0; i < 10; i++)
        if (a.coef[i]) return false;
    return true;
}

bool affine_of(const Expr& e, const std::vector<int64_t>& xshape, const std::vector<int64_t>& yshape, Affine* out) {
    Affine r;
    switch (e.kind) {
        case Expr::CONST_INT: r.c0 = e.ival; break;
        case Expr::CONST_FLOAT: return false;
        case Expr::EXTRA: return false;
        case Expr::CAST: {
            if (e.text == "float" || e.text == "float32" || e.text == "double" || e.text == "float64" || e.text == "bool")
                return false;
            return affine_of(*e.kids[0], xshape, yshape, out);
        }
        case Expr::VAR: {
            if (e.text == "XDIM") { r.c0 = (int64_t)xshape.size(); break; }
            if (e.text == "YDIM") { r.c0 = (int64_t)yshape.size(); break; }
            std::string base;
            int idx = 0;
            if (!split_name(e.text, &base, &idx)) return false;
            if (base == "i") {
                if (idx >= 10) return false;
                r.coef[idx] = 1;
            } else if (base == "xshape" && idx < (int)xshape.size()) {
                r.c0 = xshape[idx];
            } else if (base == "yshape" && idx < (int)yshape.size()) {
                r.c0 = yshape[idx];
            } else if (base == "xstride" && idx < (int)xshape.size()) {
                r.c0 = 1;
                for (size_t d = idx + 1; d < xshape.size(); d++) r.c0 *= xshape[d];
            } else if (base == "ystride" && idx < (int)yshape.size()) {
                r.c0 = 1;
                for (size_t d = idx + 1; d < yshape.size(); d++) r.c0 *= yshape[d];
            } else
                return false;
            break;
        }
        case Expr::UNARY: {
            Affine a;
            if (!affine_of(*e.kids[0], xshape, yshape, &a)) return false;
            if (e.text == "+") r = a;
            else if (e.text == "-") {
                r.c0 = -a.c0;
                for (int i = 0; i < 10; i++) r.coef[i] = -a.coef[i];
            } else if (is_const(a)) {
                r.c0 = e.text == "!" ? !a.c0 : ~a.c0;
            } else
                return false;
            break;
        }
        case Expr::TERNARY: {
            Affine c, a, b;
            if (!affine_of(*e.kids[0], xshape, yshape, &c) || !is_const(c)) return false;
            if (!affine_of(*e.kids[c.c0 ? 1 : 2], xshape, yshape, &a)) return false;
            r = a;
            (void)b;
            break;
        }
        case Expr::BINARY: {
            Affine a, b;
            if (!affine_of(*e.kids[0], xshape, yshape, &a)) return false;
            if (!affine_of(*e.kids[1], xshape, yshape, &b)) return false;
            const std::string& op = e.text;
            if (op == "+" || op == "-") {
                int s = op == "+" ? 1 : -1;
                r.c0 = a.c0 + s * b.c0;
                for (int i = 0; i < 10; i++) r.coef[i] = a.coef[i] + s * b.coef[i];
            } else if (op == "*") {
                if (is_const(a)) {
                    r.c0 = a.c0 * b.c0;
                    for (int i = 0; i < 10; i++) r.coef[i] = a.c0 * b.coef[i];
                } else if (is_const(b)) {
                    r.c0 = a.c0 * b.c0;
                    for (int i = 0; i < 10; i++) r.coef[i] = b.c0 * a.coef[i];
                } else
                    return false;
            } else if (is_const(a) && is_const(b)) {
                int64_t x = a.c0, y = b.c0;
                if ((op == "/" || op == "%") && y == 0) return false;
                if (op == "/") r.c0 = c_div(x, y);
                else if (op == "%") r.c0 = x % y;
                else if (op == "<<") r.c0 = x << y;
                else if (op == ">>") r.c0 = x >> y;
                else if (op == "<") r.c0 = x < y;
                else if (op == "<=") r.c0 = x <= y;
                else if (op == ">") r.c0 = x > y;
                else if (op == ">=") r.c0 = x >= y;
                else if (op == "==") r.c0 = x == y;
                else if (op == "!=") r.c0 = x != y;
                else if (op == "&") r.c0 = x & y;
                else if (op == "|") r.c0 = x | y;
                else if (op == "^") r.c0 = x ^ y;
                else if (op == "&&") r.c0 = x && y;
                else if (op == "||") r.c0 = x || y;
                else return false;
            } else
                return false;
            break;
        }
    }
    *out = r;
    return true;
}

}  // namespace mjt

using namespace mjt;

extern "C" int mjt_expr_affine(const char* expr, const mjt_tensor* x, const mjt_tensor* y, int64_t* c0,
                               int64_t coef[MJT_MAX_DIM]) {
    int result = 0;
    int rc = guarded([&] {
        MJT_CHECK(expr && x && y && c0 && coef, "mjt_expr_affine: null argument");
        auto e = parse_expr(expr);
        ExprEnv env;
        env.n_loop = MJT_MAX_DIM;
        env.xdim = x->ndim;
        env.ydim = y->ndim;
        // extras are not known here: any @eK makes the expression non-affine
        std::vector<int64_t> xs(x->shape, x->shape + x->ndim), ys(y->shape, y->shape + y->ndim);
        Affine a;
        if (is_pure(*e)) {
            validate_expr(*e, env);
            if (affine_of(*e, xs, ys, &a)) {
                *c0 = a.c0;
                for (int i = 0; i < MJT_MAX_DIM; i++) coef[i] = a.coef[i];
                result = 1;
            }
        }
    });
    return rc < 0 ? rc : result;
}
