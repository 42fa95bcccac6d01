// forms.hpp -- statements as data: the s-expression forms of the reference (src/forms.lisp) parsed,
// expanded into the canonical sum of monomials, and compiled into the table-monomial groups the
// round kernels are generated from.
#pragma once
#include <stdint.h>

#include <string>
#include <utility>
#include <vector>

#include "stmtdesc.hpp"

namespace exh {

struct Term {  // coefficient * product of variables (names upper-cased, sorted)
  std::vector<std::string> vars;
  uint32_t coeff;
};

// EXPAND (src/forms.lisp:57-78): like terms merged, zero terms dropped, graded order.
// Returns OK or E_PARAM (malformed form; message in last_error()).
int expand_form(const std::string &text, std::vector<Term> *out);

// One group of a compiled statement: a multiset of tables with the constant-side of every term
// over it, so that  statement = sum_g coefficient_g(constants) * prod_{t in g} table_t.
struct Group {
  // factor indices, sorted; empty: the constant group.  An index below T is a table, T + v is the
  // statement's linear form v
  std::vector<int> tabs;
  struct Part {
    uint32_t coeff;
    std::vector<int> consts;  // constant indices (with repetition)
  };
  std::vector<Part> parts;
  // evaluation points of the group's round polynomial computed on the device (X values); the host
  // extrapolates to the wire points when the group's degree is below the statement's
  std::vector<int> evalx;
  int acc_base = 0;  // index of its first accumulator
};

// A factor that is not a single table: sum of integer multiples of tables plus an integer, as in
// (+ c0 3) or (- c1 c0).  Kept as a factor instead of being multiplied out, a product of such forms
// needs one accumulator per evaluation point instead of one per monomial.
struct Linear {
  std::vector<std::pair<int, uint32_t>> terms;  // (table, coefficient mod p), by table
  uint32_t constant = 0;
  bool operator<(const Linear &o) const { return terms != o.terms ? terms < o.terms : constant < o.constant; }
};

struct Statement {
  std::string text;
  std::vector<std::string> tables, constants;
  std::vector<Term> terms;
  int degree = 0;  // in the tables (src/sumcheck.lisp:33-35)
  int T() const { return (int)tables.size(); }
  int C() const { return (int)constants.size(); }
  // the statement as sum_g coefficient_g * prod(factors of g), in two equivalent shapes: one group per
  // table monomial of the expanded form, and (when the form is a sum of products of linear forms) one
  // group per written product.  plan() points `groups` at the cheaper one.
  std::vector<Group> expanded_groups, factored_groups;
  std::vector<Linear> factored_linear;
  std::vector<Group> groups;   // the planned shape; constant group (if any) included
  std::vector<Linear> linear;  // its linear forms
  int nacc = 0;                // accumulators per round over all groups
  // the device evaluation points are chosen for POINTS = max(header degree, 1) wire points
  void plan(int points);
  // every group at X = 0 and X = 1 only: what the honest claim (HYPERCUBE-SUM) needs
  void plan_claim();
  int planned_points = -1;
  std::string key() const;  // canonical description of the table groups, for kernel lookup
  // A statement in direct form (make_direct): no groups of table monomials; the kernels evaluate the written form
  // itself at every wire point, into one accumulator per point.  `groups` then holds one stand-in group with
  // coefficient 1 whose accumulators are the wire points.
  bool direct = false;
  std::string direct_code;  // the body of the generated evaluator: statements ending in `return v<N>;`
  int direct_slots = 0;     // its constant slots: table-free subforms, evaluated on the host for every proof
  std::string direct_key;
};

// The statement as a kernel evaluates it when it is too wide for the groups' accumulators: the written form as
// straight-line code over the tables' values at a point (every value in Montgomery form), table-free subforms
// collapsed into constant slots, repeated subforms computed once.  POINTS wire points (X = 0, 2, 3, ...).
// False when the form has more than MAXT tables or more than MAXEV wire points.
bool make_direct(const Statement &st, int points, Statement *out);
// the direct statement's constant slots at the constants' values: out[slot * D ..), canonical
void direct_slot_values(const Statement &st, int D, const uint32_t *const_vals, uint32_t *out);
// `struct <name>` for a direct statement: the descriptor with its evaluator
std::string direct_source(const Statement &st, const StmtDesc &d, const std::string &name);

int compile_statement(const std::string &text, const std::vector<std::string> &tables,
                      const std::vector<std::string> &constants, Statement *out);

// the statement over F_p^D at the given table and constant values (exact, host side)
void evaluate_statement(const Statement &st, int D, const uint32_t *table_vals, const uint32_t *const_vals,
                        uint32_t *out);
// the descriptor of the planned statement for the kernels; false when it exceeds their limits
bool make_desc(const Statement &st, StmtDesc *out);
// the descriptor as the text of `struct <name> { static constexpr StmtDesc d = {...}; };`, what a kernel is
// instantiated with, at build time or at run time
std::string desc_source(const StmtDesc &d, const std::string &name);
// the groups' coefficients at the constants: out[g*D .. g*D+D)
void group_coefficients(const Statement &st, int D, const uint32_t *const_vals, uint32_t *out);

}  // namespace exh
