// forms.cpp -- see forms.hpp.
#include "forms.hpp"

#include <string.h>

#include <algorithm>
#include <map>
#include <memory>
#include <sstream>

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


// ---- the written shape of a form: a sum of products whose factors are integers, constants, tables
// or linear forms in the tables.  Returns false when the form has another shape.
struct Product {
  uint32_t coeff = 1;
  std::vector<int> consts;
  std::vector<Linear> factors;  // a plain table is the linear form 1 * table + 0
  bool zero = false;
};

struct Shape {
  const std::vector<std::string> *tables, *constants;
  int find(const std::vector<std::string> &names, const std::string &v) const {
    auto it = std::find(names.begin(), names.end(), v);
    return it == names.end() ? -1 : (int)(it - names.begin());
  }
  // a form that expands to integer multiples of tables plus an integer
  bool linear(const Node &n, Linear *out) const {
    Poly p;
    if (!expand_node(n, &p)) return false;
    std::map<int, uint32_t> by_table;
    out->constant = 0;
    for (auto &t : p) {
      if (t.first.size() > 1) return false;
      if (t.first.empty()) {
        out->constant = t.second;
        continue;
      }
      int ti = find(*tables, t.first[0]);
      if (ti < 0) return false;
      if (t.second) by_table[ti] = t.second;
    }
    out->terms.assign(by_table.begin(), by_table.end());
    return true;
  }
  bool factor(const Node &n, Product *out) const {
    if (n.kind == Node::INT) {
      out->coeff = fmul(out->coeff, (uint32_t)n.value);
      return true;
    }
    if (n.kind == Node::VAR) {
      int ci = find(*constants, n.name);
      if (ci >= 0 && find(*tables, n.name) < 0) {
        out->consts.push_back(ci);
        return true;
      }
    }
    if (n.kind == Node::OP && n.name == "*") {
      for (auto &a : n.args)
        if (!factor(*a, out)) return false;
      return true;
    }
    if (n.kind == Node::OP && n.name == "EXPT" && n.args.size() == 2 && n.args[1]->kind == Node::INT &&
        n.args[1]->value <= MAXDEG) {
      for (long long i = 0; i < n.args[1]->value; i++)
        if (!factor(*n.args[0], out)) return false;
      return true;
    }
    Linear lin;
    if (!linear(n, &lin)) return false;
    if (lin.terms.empty()) {  // an integer after all
      out->coeff = fmul(out->coeff, lin.constant);
      return true;
    }
    out->factors.push_back(lin);
    return true;
  }
  bool sum(const Node &n, bool negate, std::vector<Product> *out) const {
    if (n.kind == Node::OP && n.name == "+") {
      for (auto &a : n.args)
        if (!sum(*a, negate, out)) return false;
      return true;
    }
    if (n.kind == Node::OP && n.name == "-" && !n.args.empty()) {
      for (size_t i = 0; i < n.args.size(); i++)
        if (!sum(*n.args[i], negate != (n.args.size() == 1 || i > 0), out)) return false;
      return true;
    }
    Product prod;
    if (!factor(n, &prod)) return false;
    if (negate) prod.coeff = fneg(prod.coeff);
    out->push_back(prod);
    return true;
  }
};

bool is_table(const Linear &l) { return l.terms.size() == 1 && l.terms[0].second == 1 && l.constant == 0; }

void sort_groups(std::vector<Group> *groups) {
  // constant group first, then by degree, then by factors: a fixed order for the kernels' accumulators
  std::stable_sort(groups->begin(), groups->end(), [](const Group &a, const Group &b) {
    if (a.tabs.size() != b.tabs.size()) return a.tabs.size() < b.tabs.size();
    return a.tabs < b.tabs;
  });
}

// the factored groups multiplied out again, as a polynomial in table and constant names
Poly multiply_out(const Statement &st, const std::vector<Group> &groups, const std::vector<Linear> &linear) {
  Poly total;
  for (const Group &g : groups) {
    Poly prod;
    add_term(prod, {}, 1);
    for (int f : g.tabs) {
      Poly lin;
      if (f < st.T())
        add_term(lin, {st.tables[f]}, 1);
      else {
        const Linear &l = linear[f - st.T()];
        for (auto &t : l.terms) add_term(lin, {st.tables[t.first]}, t.second);
        if (l.constant) add_term(lin, {}, l.constant);
      }
      prod = multiply(prod, lin);
    }
    Poly coef;
    for (const Group::Part &part : g.parts) {
      std::vector<std::string> m;
      for (int k : part.consts) m.push_back(st.constants[k]);
      std::sort(m.begin(), m.end());
      add_term(coef, m, part.coeff);
    }
    Poly term = multiply(prod, coef);
    for (auto &t : term) add_term(total, t.first, t.second);
  }
  for (auto it = total.begin(); it != total.end();) it = it->second ? std::next(it) : total.erase(it);
  return total;
}

void factor_statement(const Node &root, Statement *st) {
  st->factored_groups.clear();
  st->factored_linear.clear();
  Shape shape{&st->tables, &st->constants};
  std::vector<Product> products;
  if (!shape.sum(root, false, &products)) return;
  std::map<Linear, int> ids;
  std::map<std::vector<int>, Group> groups;
  for (const Product &prod : products) {
    if (prod.coeff == 0) continue;
    std::vector<int> factors;
    for (const Linear &l : prod.factors) {
      if (is_table(l)) {
        factors.push_back(l.terms[0].first);
        continue;
      }
      auto it = ids.find(l);
      if (it == ids.end()) {
        it = ids.emplace(l, st->T() + (int)st->factored_linear.size()).first;
        st->factored_linear.push_back(l);
      }
      factors.push_back(it->second);
    }
    std::sort(factors.begin(), factors.end());
    Group &g = groups[factors];
    g.tabs = factors;
    std::vector<int> consts(prod.consts);
    std::sort(consts.begin(), consts.end());
    g.parts.push_back(Group::Part{prod.coeff, consts});
  }
  for (auto &kv : groups) st->factored_groups.push_back(kv.second);
  sort_groups(&st->factored_groups);
  // accept the written shape only if it multiplies out to the canonical expansion
  Poly expanded;
  for (const Term &t : st->terms) add_term(expanded, t.vars, t.coeff);
  if (multiply_out(*st, st->factored_groups, st->factored_linear) != expanded) {
    st->factored_groups.clear();
    st->factored_linear.clear();
  }
}

// products per pair and round of a shape planned for POINTS wire points: every evaluation of a group
// costs its degree (degree - 1 for the factors, 1 for the weight)
long plan_groups(std::vector<Group> *groups, int points, int *nacc) {
  long cost = 0;
  *nacc = 0;
  for (Group &g : *groups) {
    g.evalx.clear();
    g.acc_base = *nacc;
    int d = (int)g.tabs.size();
    if (d == 0) continue;  // its sum is the sum of the weights: no device work
    if (points < 0)
      g.evalx = {0, 1};  // the honest claim
    else if (d >= points) {  // the wire points 0, 2, 3, ..., points
      g.evalx.push_back(0);
      for (int x = 2; x <= points; x++) g.evalx.push_back(x);
    } else {  // degree d: d + 1 cheap points, extrapolated on the host
      for (int x = 0; x <= d; x++) g.evalx.push_back(x);
    }
    *nacc += (int)g.evalx.size();
    cost += (long)g.evalx.size() * d;
  }
  return cost;
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
  st->expanded_groups.clear();
  for (auto &kv : groups) st->expanded_groups.push_back(kv.second);
  sort_groups(&st->expanded_groups);
  Parser parser(text);
  auto root = parser.parse();
  factor_statement(*root, st);
  st->groups = st->expanded_groups;
  st->linear.clear();
  st->planned_points = -1;
  return OK;
}

// both shapes are planned; the factored one is taken only when it needs fewer products
static void choose_shape(Statement *st, int points) {
  int nacc_e = 0, nacc_f = 0;
  long cost_e = plan_groups(&st->expanded_groups, points, &nacc_e);
  bool factored = false;
  if (!st->factored_groups.empty() && (int)st->factored_linear.size() <= MAXV &&
      st->T() + (int)st->factored_linear.size() <= MAXT) {
    bool fits = true;
    for (const Linear &l : st->factored_linear) fits = fits && (int)l.terms.size() <= MAXVT;
    long cost_f = plan_groups(&st->factored_groups, points, &nacc_f);
    factored = fits && cost_f < cost_e;
  }
  st->groups = factored ? st->factored_groups : st->expanded_groups;
  st->linear = factored ? st->factored_linear : std::vector<Linear>();
  st->nacc = factored ? nacc_f : nacc_e;
}

void Statement::plan(int points) {
  if (direct) return;  // made for its wire points already
  if (planned_points == points) return;
  planned_points = points;
  choose_shape(this, points);
}

void Statement::plan_claim() {
  planned_points = -2;
  choose_shape(this, -1);
}

std::string Statement::key() const {
  if (direct) return direct_key;
  std::string k = "T" + std::to_string(T()) + ":";
  for (const Linear &l : linear) {
    k += "(";
    for (auto &t : l.terms) k += std::to_string(t.second) + "*" + std::to_string(t.first) + "+";
    k += std::to_string(l.constant) + ")";
  }
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
    for (int f : g.tabs) {
      if (f < st.T()) {
        prod = hf::mul(prod, hf::from(tv + (size_t)f * D, D));
        continue;
      }
      const Linear &l = st.linear[f - st.T()];
      hf::E v = hf::lift(l.constant, D);
      for (auto &t : l.terms) v = hf::add(v, hf::mul(hf::lift(t.second, D), hf::from(tv + (size_t)t.first * D, D)));
      prod = hf::mul(prod, v);
    }
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

bool make_desc(const Statement &st, StmtDesc *out) {
  StmtDesc d;
  memset(&d, 0, sizeof(d));
  d.T = st.T();
  if (st.direct) {  // no groups: the wire points are the accumulators
    if (d.T < 1 || d.T > MAXT || st.nacc > MAXEV || st.groups.size() != 1) return false;
    d.nacc = st.nacc;
    d.nev[0] = st.nacc;
    for (int k = 0; k < st.nacc; k++) d.ev[0][k] = st.groups[0].evalx[(size_t)k];
    d.maxx = st.groups[0].evalx.back();
    *out = d;
    return true;
  }
  d.NV = (int)st.linear.size();
  if (d.T < 1 || d.NV > MAXV || d.T + d.NV > MAXT || st.nacc > MAXACC) return false;
  for (int v = 0; v < d.NV; v++) {
    const Linear &l = st.linear[v];
    if ((int)l.terms.size() > MAXVT) return false;
    d.vn[v] = (int)l.terms.size();
    for (size_t k = 0; k < l.terms.size(); k++) {
      d.vtab[v][k] = l.terms[k].first;
      d.vcoef[v][k] = l.terms[k].second;
      d.vcoefm[v][k] = to_mont(l.terms[k].second);
    }
    d.vconst[v] = l.constant;
  }
  int g = 0, maxx = 0;
  for (const Group &grp : st.groups) {
    if (grp.tabs.empty()) continue;
    if (g >= MAXG || (int)grp.tabs.size() > MAXDEG || (int)grp.evalx.size() > MAXEV || grp.evalx.back() > MAXX)
      return false;
    d.deg[g] = (int)grp.tabs.size();
    for (size_t j = 0; j < grp.tabs.size(); j++) d.tab[g][j] = grp.tabs[j];
    d.nev[g] = (int)grp.evalx.size();
    for (size_t k = 0; k < grp.evalx.size(); k++) {
      d.ev[g][k] = grp.evalx[k];
      if (grp.evalx[k] > maxx) maxx = grp.evalx[k];
    }
    g++;
  }
  d.G = g, d.nacc = st.nacc, d.maxx = maxx;
  *out = d;
  return true;
}

std::string desc_source(const StmtDesc &d, const std::string &name) {
  std::ostringstream o;
  o << "struct " << name << " {\n  static constexpr StmtDesc d = {" << d.T << ", " << d.G << ", " << d.nacc << ", "
        << d.maxx << ",\n    {";
  for (int g = 0; g < MAXG; g++) o << d.deg[g] << (g + 1 < MAXG ? "," : "");
  o << "},\n    {";
  for (int g = 0; g < MAXG; g++) {
    o << "{";
    for (int j = 0; j < MAXDEG; j++) o << d.tab[g][j] << (j + 1 < MAXDEG ? "," : "");
    o << "}" << (g + 1 < MAXG ? "," : "");
  }
  o << "},\n    {";
  for (int g = 0; g < MAXG; g++) o << d.nev[g] << (g + 1 < MAXG ? "," : "");
  o << "},\n    {";
  for (int g = 0; g < MAXG; g++) {
    o << "{";
    for (int k = 0; k < MAXEV; k++) o << d.ev[g][k] << (k + 1 < MAXEV ? "," : "");
    o << "}" << (g + 1 < MAXG ? "," : "");
  }
  o << "},\n    " << d.NV << ", {";
  for (int v = 0; v < MAXV; v++) o << d.vn[v] << (v + 1 < MAXV ? "," : "");
  o << "},\n    {";
  for (int v = 0; v < MAXV; v++) {
    o << "{";
    for (int k = 0; k < MAXVT; k++) o << d.vtab[v][k] << (k + 1 < MAXVT ? "," : "");
    o << "}" << (v + 1 < MAXV ? "," : "");
  }
  for (int which = 0; which < 2; which++) {
    o << "},\n    {";
    for (int v = 0; v < MAXV; v++) {
      o << "{";
      for (int k = 0; k < MAXVT; k++)
        o << (which ? d.vcoefm[v][k] : d.vcoef[v][k]) << "u" << (k + 1 < MAXVT ? "," : "");
      o << "}" << (v + 1 < MAXV ? "," : "");
    }
  }
  o << "},\n    {";
  for (int v = 0; v < MAXV; v++) o << d.vconst[v] << "u" << (v + 1 < MAXV ? "," : "");
  o << "}};\n};\n";
  return o.str();
}

// ---- the direct form
namespace {

// One walk of the written form serves both the code and the constants: it numbers the constant slots in the order
// it meets them, so the values are computed by the same walk with the constants at hand.
struct DirectWalk {
  const Statement &st;
  std::ostringstream code;
  int vars = 0, slots = 0;
  bool failed = false;
  std::map<std::string, std::string> seen;  // a subform's text -> the variable that holds it
  // evaluation of the slots (when const_vals is set)
  int D = 0;
  const uint32_t *const_vals = nullptr;
  std::vector<hf::E> values;

  explicit DirectWalk(const Statement &s) : st(s) {}
  int find(const std::vector<std::string> &names, const std::string &v) const {
    auto it = std::find(names.begin(), names.end(), v);
    return it == names.end() ? -1 : (int)(it - names.begin());
  }
  std::string text(const Node &n) const {
    if (n.kind == Node::INT) return std::to_string(n.value);
    if (n.kind == Node::VAR) return n.name;
    std::string s = "(" + n.name;
    for (auto &a : n.args) s += " " + text(*a);
    return s + ")";
  }
  bool table_free(const Node &n) const {
    if (n.kind == Node::INT) return true;
    if (n.kind == Node::VAR) return find(st.tables, n.name) < 0;
    if (n.name == "EXPT" && n.args.size() == 2 && n.args[1]->kind == Node::INT && n.args[1]->value == 0) return true;
    for (auto &a : n.args)
      if (!table_free(*a)) return false;
    return true;
  }
  bool integer_only(const Node &n) const {  // no named constant: an integer mod p, a base-field scalar
    if (n.kind == Node::INT) return true;
    if (n.kind == Node::VAR) return false;
    for (auto &a : n.args)
      if (!integer_only(*a)) return false;
    return true;
  }
  hf::E value(const Node &n) {  // of a table-free subform, at the constants
    if (n.kind == Node::INT) return hf::lift((uint32_t)n.value, D);
    if (n.kind == Node::VAR) {
      int ci = find(st.constants, n.name);
      if (ci < 0) {
        failed = true;
        return hf::zero(D);
      }
      return hf::from(const_vals + (size_t)ci * D, D);
    }
    if (n.name == "+" || n.name == "-") {
      hf::E acc = hf::zero(D);
      for (size_t i = 0; i < n.args.size(); i++) {
        bool negate = n.name == "-" && (n.args.size() == 1 || i > 0);
        acc = negate ? hf::sub(acc, value(*n.args[i])) : hf::add(acc, value(*n.args[i]));
      }
      return acc;
    }
    if (n.name == "*") {
      hf::E acc = hf::lift(1, D);
      for (auto &a : n.args) acc = hf::mul(acc, value(*a));
      return acc;
    }
    if (n.name == "EXPT" && n.args.size() == 2 && n.args[1]->kind == Node::INT) {
      hf::E acc = hf::lift(1, D), base = n.args[1]->value ? value(*n.args[0]) : hf::zero(D);
      for (long long i = 0; i < n.args[1]->value; i++) acc = hf::mul(acc, base);
      return acc;
    }
    failed = true;
    return hf::zero(D);
  }
  // a constant slot for the sum (signs) or the product of table-free subforms
  std::map<std::string, int> slot_of;        // a slot's text -> its number (a constant met again is the same slot)
  std::map<int, std::string> slot_variable;  // slots already loaded into a variable
  int slot(const std::vector<std::pair<const Node *, bool>> &items, bool product) {
    std::string key = product ? "*" : "+";
    for (auto &it : items) key += (it.second ? " -" : " +") + text(*it.first);
    auto hit = slot_of.find(key);
    if (hit != slot_of.end()) return hit->second;
    slot_of[key] = slots;
    if (const_vals) {
      hf::E acc = product ? hf::lift(1, D) : hf::zero(D);
      for (auto &it : items) {
        hf::E v = value(*it.first);
        acc = product ? hf::mul(acc, v) : (it.second ? hf::sub(acc, v) : hf::add(acc, v));
      }
      values.push_back(acc);
    }
    return slots++;
  }
  std::string fresh() { return "v" + std::to_string(vars++); }
  std::string load_slot(int k) {
    auto hit = slot_variable.find(k);
    if (hit != slot_variable.end()) return hit->second;
    std::string v = fresh();
    code << "    const Ext<D> " << v << " = load_ext<D>(kc + " << k << " * D);\n";
    slot_variable[k] = v;
    return v;
  }
  // the variable holding the subform's value (Montgomery form)
  std::string gen(const Node &n) {
    if (table_free(n)) return load_slot(slot({{&n, false}}, false));
    if (n.kind == Node::VAR) return "t[" + std::to_string(find(st.tables, n.name)) + "]";
    const std::string key = text(n);
    auto hit = seen.find(key);
    if (hit != seen.end()) return hit->second;
    std::string out;
    if (n.name == "+" || n.name == "-") {
      std::vector<std::pair<const Node *, bool>> consts;
      for (size_t i = 0; i < n.args.size(); i++) {
        const bool negate = n.name == "-" && (n.args.size() == 1 || i > 0);
        if (table_free(*n.args[i])) {
          consts.push_back({n.args[i].get(), negate});
          continue;
        }
        const std::string a = gen(*n.args[i]);
        const std::string v = fresh();
        if (out.empty())
          code << "    const Ext<D> " << v << " = " << (negate ? "ext_sub<D>(ext_zero<D>(), " + a + ")" : a) << ";\n";
        else
          code << "    const Ext<D> " << v << " = " << (negate ? "ext_sub<D>(" : "ext_add<D>(") << out << ", " << a << ");\n";
        out = v;
      }
      if (!consts.empty()) {
        const std::string k = load_slot(slot(consts, false)), v = fresh();
        code << "    const Ext<D> " << v << " = ext_add<D>(" << out << ", " << k << ");\n";
        out = v;
      }
    } else if (n.name == "*") {
      std::vector<std::pair<const Node *, bool>> consts;
      bool integers = true;
      for (auto &arg : n.args) {
        if (table_free(*arg)) {
          consts.push_back({arg.get(), false});
          integers = integers && integer_only(*arg);
          continue;
        }
        const std::string a = gen(*arg);
        if (out.empty()) {
          out = a;
          continue;
        }
        const std::string v = fresh();
        code << "    const Ext<D> " << v << " = ext_mul_mont<D>(" << out << ", " << a << ");\n";
        out = v;
      }
      if (!consts.empty()) {
        const int k = slot(consts, true);
        std::string v;
        if (!integers) (void)load_slot(k);  // (its line comes before the product's)
        v = fresh();
        if (integers)  // a base-field scalar: its Montgomery form is the slot's first word
          code << "    const Ext<D> " << v << " = ext_scale_mont<D>(" << out << ", kc[" << k << " * D]);\n";
        else {
          const std::string kv = load_slot(k);
          code << "    const Ext<D> " << v << " = ext_mul_mont<D>(" << out << ", " << kv << ");\n";
        }
        out = v;
      }
    } else if (n.name == "EXPT" && n.args.size() == 2 && n.args[1]->kind == Node::INT && n.args[1]->value >= 1 &&
               n.args[1]->value <= MAXDEG) {
      const std::string a = gen(*n.args[0]);
      out = a;
      for (long long i = 1; i < n.args[1]->value; i++) {
        const std::string v = fresh();
        code << "    const Ext<D> " << v << " = ext_mul_mont<D>(" << out << ", " << a << ");\n";
        out = v;
      }
    } else {
      failed = true;
      return "t[0]";
    }
    seen[key] = out;
    return out;
  }
};

}  // namespace

bool make_direct(const Statement &st, int points, Statement *out) {
  if (st.T() < 1 || st.T() > MAXT || points < 1 || points > MAXEV || points + 1 > MAXX + 1) return false;
  Parser parser(st.text);
  auto root = parser.parse();
  if (!parser.ok || !root) return false;
  DirectWalk walk(st);
  const std::string result = walk.gen(*root);
  if (walk.failed) return false;
  Statement d = st;
  d.direct = true;
  d.direct_code = walk.code.str() + "    return " + result + ";\n";
  d.direct_slots = walk.slots;
  d.expanded_groups.clear(), d.factored_groups.clear(), d.factored_linear.clear(), d.linear.clear();
  Group g;
  g.tabs = {0};  // (not the constant group)
  g.parts.push_back(Group::Part{1u, {}});
  for (int k = 0; k < points; k++) g.evalx.push_back(k == 0 ? 0 : k + 1);
  g.acc_base = 0;
  d.groups = {g};
  d.nacc = points;
  d.planned_points = points;
  d.direct_key = "direct:" + std::to_string(points) + "|";
  for (auto &t : st.tables) d.direct_key += t + ",";
  d.direct_key += "|";
  for (auto &c : st.constants) d.direct_key += c + ",";
  d.direct_key += "|" + walk.text(*root);
  *out = d;
  return true;
}

void direct_slot_values(const Statement &st, int D, const uint32_t *const_vals, uint32_t *out) {
  Parser parser(st.text);
  auto root = parser.parse();
  DirectWalk walk(st);
  walk.D = D, walk.const_vals = const_vals;
  (void)walk.gen(*root);
  for (size_t k = 0; k < walk.values.size(); k++) memcpy(out + k * D, walk.values[k].data(), 4 * (size_t)D);
}

std::string direct_source(const Statement &st, const StmtDesc &d, const std::string &name) {
  // the descriptor's initialiser as desc_source writes it, inside a type that carries the evaluator
  std::string plain = desc_source(d, name);
  const size_t from = plain.find("= {") + 2, to = plain.rfind("};\n};");
  const std::string init = plain.substr(from, to - from + 1);
  std::ostringstream o;
  o << "struct " << name << "Desc : StmtDesc {\n  static constexpr bool direct = true;\n"
    << "  // the statement at the tables' values t (Montgomery form) with the constant slots kc (Montgomery form)\n"
    << "  template <int D>\n  static __device__ __forceinline__ Ext<D> eval(const Ext<D> *t, const uint32_t *kc) {\n"
    << st.direct_code << "  }\n};\n"
    << "struct " << name << " {\n  static constexpr " << name << "Desc d = {" << init << "};\n};\n";
  return o.str();
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
