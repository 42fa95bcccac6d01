// forms.cpp -- see forms.hpp.
#include "forms.hpp"

#include <algorithm>
#include <map>
#include <memory>

#include "hostfield.hpp"
#include "transcript.hpp"

namespace exh {

namespace {

struct Node {
  enum Kind { INT, VAR, OP } kind;
  long long value = 0;
  std::string name;  // variable, or operator
  std::vector<std::unique_ptr<Node>> args;
};

std::string upcase(std::string s) {
  for (char &c : s) c = (char)toupper((unsigned char)c);
  return s;
}

struct Parser {
  const std::string &s;
  size_t pos = 0;
  bool ok = true;
  explicit Parser(const std::string &text) : s(text) {}
  void skip() {
    while (pos < s.size() && isspace((unsigned char)s[pos])) pos++;
  }
  std::unique_ptr<Node> parse() {
    skip();
    if (pos >= s.size()) {
      ok = false;
      return nullptr;
    }
    auto node = std::make_unique<Node>();
    if (s[pos] == '(') {
      pos++;
      node->kind = Node::OP;
      bool first = true;
      for (;;) {
        skip();
        if (pos >= s.size()) {
          ok = false;
          return nullptr;
        }
        if (s[pos] == ')') {
          pos++;
          break;
        }
        if (first) {
          size_t start = pos;
          while (pos < s.size() && !isspace((unsigned char)s[pos]) && s[pos] != '(' && s[pos] != ')') pos++;
          node->name = upcase(s.substr(start, pos - start));
          first = false;
          if (node->name.empty()) {
            ok = false;
            return nullptr;
          }
        } else {
          auto arg = parse();
          if (!ok) return nullptr;
          node->args.push_back(std::move(arg));
        }
      }
      if (first) ok = false;  // ()
      return node;
    }
    if (s[pos] == ')') {
      ok = false;
      return nullptr;
    }
    size_t start = pos;
    while (pos < s.size() && !isspace((unsigned char)s[pos]) && s[pos] != '(' && s[pos] != ')') pos++;
    std::string tok = s.substr(start, pos - start);
    size_t digits = tok[0] == '-' || tok[0] == '+' ? 1 : 0;
    bool is_int = tok.size() > digits;
    for (size_t i = digits; i < tok.size(); i++) is_int = is_int && isdigit((unsigned char)tok[i]);
    if (is_int) {
      node->kind = Node::INT;
      // reduce a decimal of any length mod p, keeping the sign
      long long acc = 0;
      for (size_t i = digits; i < tok.size(); i++) acc = (acc * 10 + (tok[i] - '0')) % (long long)P;
      node->value = tok[0] == '-' ? (P - acc) % P : acc;
    } else {
      node->kind = Node::VAR;
      node->name = upcase(tok);
    }
    return node;
  }
};

typedef std::map<std::vector<std::string>, uint32_t> Poly;

void add_term(Poly &p, const std::vector<std::string> &m, uint32_t c) {
  uint32_t &slot = p[m];
  slot = fadd(slot, c % P);
}

Poly multiply(const Poly &a, const Poly &b) {
  Poly out;
  for (auto &x : a)
    for (auto &y : b) {
      std::vector<std::string> m(x.first);
      m.insert(m.end(), y.first.begin(), y.first.end());
      std::sort(m.begin(), m.end());
      add_term(out, m, fmul(x.second, y.second));
    }
  return out;
}

bool expand_node(const Node &n, Poly *out) {
  out->clear();
  if (n.kind == Node::INT) {
    add_term(*out, {}, (uint32_t)n.value);
    return true;
  }
  if (n.kind == Node::VAR) {
    if (n.name == "NIL") return false;
    add_term(*out, {n.name}, 1);
    return true;
  }
  const std::string &op = n.name;
  if (op == "+") {
    for (auto &a : n.args) {
      Poly p;
      if (!expand_node(*a, &p)) return false;
      for (auto &t : p) add_term(*out, t.first, t.second);
    }
    return true;
  }
  if (op == "-") {
    if (n.args.empty()) return false;
    for (size_t i = 0; i < n.args.size(); i++) {
      Poly p;
      if (!expand_node(*n.args[i], &p)) return false;
      bool negate = n.args.size() == 1 || i > 0;
      for (auto &t : p) add_term(*out, t.first, negate ? fneg(t.second) : t.second);
    }
    return true;
  }
  if (op == "*") {
    Poly acc;
    add_term(acc, {}, 1);
    for (auto &a : n.args) {
      Poly p;
      if (!expand_node(*a, &p)) return false;
      acc = multiply(acc, p);
    }
    *out = acc;
    return true;
  }
  if (op == "EXPT") {
    if (n.args.size() != 2 || n.args[1]->kind != Node::INT) return false;
    // the exponent was reduced mod p by the parser; exponents in statements are tiny
    long long k = n.args[1]->value;
    if (k > 64) return false;
    Poly base, acc;
    if (!expand_node(*n.args[0], &base)) return false;
    add_term(acc, {}, 1);
    for (long long i = 0; i < k; i++) acc = multiply(acc, base);
    *out = acc;
    return true;
  }
  return false;
}

}  // namespace

int expand_form(const std::string &text, std::vector<Term> *out) {
  Parser parser(text);
  auto root = parser.parse();
  parser.skip();
  Poly poly;
  if (!parser.ok || parser.pos != text.size() || !expand_node(*root, &poly)) {
    set_error("invalid-parameter: form: expected an integer, a symbol, or (+|-|* form...) or (expt form k)");
    return E_PARAM;
  }
  out->clear();
  for (auto &t : poly)
    if (t.second) out->push_back(Term{t.first, t.second});
  // graded order: by degree, then by variables (src/forms.lisp:31-36)
  std::stable_sort(out->begin(), out->end(), [](const Term &a, const Term &b) {
    if (a.vars.size() != b.vars.size()) return a.vars.size() < b.vars.size();
    return a.vars < b.vars;
  });
  return OK;
}

int compile_statement(const std::string &text, const std::vector<std::string> &tables,
                      const std::vector<std::string> &constants, Statement *st) {
  st->text = text;
  st->tables.clear();
  st->constants.clear();
  for (auto &t : tables) st->tables.push_back(upcase(t));
  for (auto &c : constants) st->constants.push_back(upcase(c));
  int status = expand_form(text, &st->terms);
  if (status) return status;
  st->degree = 0;
  std::map<std::vector<int>, Group> groups;
  for (const Term &term : st->terms) {
    std::vector<int> tabs, consts;
    for (const std::string &v : term.vars) {
      auto ti = std::find(st->tables.begin(), st->tables.end(), v);
      auto ci = std::find(st->constants.begin(), st->constants.end(), v);
      if (ti != st->tables.end())
        tabs.push_back((int)(ti - st->tables.begin()));
      else if (ci != st->constants.end())
        consts.push_back((int)(ci - st->constants.begin()));
      else {
        set_error("invalid-parameter: free-variables: " + v);
        return E_PARAM;
      }
    }
    std::sort(tabs.begin(), tabs.end());
    st->degree = std::max(st->degree, (int)tabs.size());
    Group &g = groups[tabs];
    g.tabs = tabs;
    g.parts.push_back(Group::Part{term.coeff, consts});
  }
  st->groups.clear();
  for (auto &kv : groups) st->groups.push_back(kv.second);
  // constant group first, then by degree, then by tables: a fixed order for the kernels' accumulators
  std::stable_sort(st->groups.begin(), st->groups.end(), [](const Group &a, const Group &b) {
    if (a.tabs.size() != b.tabs.size()) return a.tabs.size() < b.tabs.size();
    return a.tabs < b.tabs;
  });
  st->planned_points = -1;
  return OK;
}

void Statement::plan(int points) {
  if (planned_points == points) return;
  planned_points = points;
  nacc = 0;
  for (Group &g : groups) {
    g.evalx.clear();
    g.acc_base = nacc;
    int d = (int)g.tabs.size();
    if (d == 0) continue;  // its sum is the sum of the weights: no device work
    if (d >= points) {     // the wire points 0, 2, 3, ..., points
      g.evalx.push_back(0);
      for (int x = 2; x <= points; x++) g.evalx.push_back(x);
    } else {  // degree d: d + 1 cheap points, extrapolated on the host
      for (int x = 0; x <= d; x++) g.evalx.push_back(x);
    }
    nacc += (int)g.evalx.size();
  }
}

void Statement::plan_claim() {
  planned_points = -2;
  nacc = 0;
  for (Group &g : groups) {
    g.evalx.clear();
    g.acc_base = nacc;
    if (g.tabs.empty()) continue;
    g.evalx = {0, 1};
    nacc += 2;
  }
}

std::string Statement::key() const {
  std::string k = "T" + std::to_string(T()) + ":";
  for (const Group &g : groups) {
    if (g.tabs.empty()) continue;
    k += "[";
    for (size_t i = 0; i < g.tabs.size(); i++) k += (i ? "," : "") + std::to_string(g.tabs[i]);
    k += "]@";
    for (size_t i = 0; i < g.evalx.size(); i++) k += (i ? "," : "") + std::to_string(g.evalx[i]);
    k += ";";
  }
  return k;
}

void evaluate_statement(const Statement &st, int D, const uint32_t *tv, const uint32_t *cv, uint32_t *out) {
  hf::E acc = hf::zero(D);
  for (const Group &g : st.groups) {
    hf::E prod = hf::lift(1, D);
    for (int t : g.tabs) prod = hf::mul(prod, hf::from(tv + (size_t)t * D, D));
    hf::E coef = hf::zero(D);
    for (const Group::Part &part : g.parts) {
      hf::E c = hf::lift(part.coeff, D);
      for (int k : part.consts) c = hf::mul(c, hf::from(cv + (size_t)k * D, D));
      coef = hf::add(coef, c);
    }
    acc = hf::add(acc, hf::mul(coef, prod));
  }
  memcpy(out, acc.data(), 4 * D);
}

void group_coefficients(const Statement &st, int D, const uint32_t *cv, uint32_t *out) {
  for (size_t g = 0; g < st.groups.size(); g++) {
    hf::E coef = hf::zero(D);
    for (const Group::Part &part : st.groups[g].parts) {
      hf::E c = hf::lift(part.coeff, D);
      for (int k : part.consts) c = hf::mul(c, hf::from(cv + (size_t)k * D, D));
      coef = hf::add(coef, c);
    }
    memcpy(out + g * D, coef.data(), 4 * D);
  }
}

}  // namespace exh
