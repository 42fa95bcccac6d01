// stmtdesc.hpp -- the descriptor a round kernel is generated from (or interprets), and its limits.
#pragma once

namespace exh {

constexpr int MAXT = 16;    // tables plus linear forms per statement
constexpr int MAXV = 8;     // linear forms per statement
constexpr int MAXVT = 4;    // tables per linear form
constexpr int MAXG = 16;    // table groups per statement
constexpr int MAXDEG = 6;   // tables per group
constexpr int MAXEV = 6;    // evaluation points per group
constexpr int MAXACC = 36;  // accumulators (group, point) per statement
constexpr int MAXX = 7;     // largest evaluation point
constexpr int BLOCK = 256;  // threads per workgroup

// A statement as the kernels see it: G groups, group g the product of the deg[g] factors tab[g][..],
// evaluated at the nev[g] points ev[g][..]; accumulators are numbered group by group, point by point.
// Factor t < T is table t; factor T + v is the linear form sum_k vcoef[v][k] * table vtab[v][k] + vconst[v]
// (vcoef canonical and, for the kernels' products, in Montgomery form in vcoefm).
struct StmtDesc {
  int T, G, nacc, maxx;
  int deg[MAXG];
  int tab[MAXG][MAXDEG];
  int nev[MAXG];
  int ev[MAXG][MAXEV];
  int NV;
  int vn[MAXV];
  int vtab[MAXV][MAXVT];
  unsigned vcoef[MAXV][MAXVT], vcoefm[MAXV][MAXVT];
  unsigned vconst[MAXV];
};

#if defined(__HIPCC__)
#define EXH_DESC_FN __host__ __device__
#else
#define EXH_DESC_FN
#endif

// ---- the slots of the base-field sweep that serves rounds 0 and 1 (the kernels and their generator agree here)
// the index of X among group g's evaluation points, or -1
template <class Desc>
EXH_DESC_FN constexpr int ev_index(const Desc &d, int g, int x) {
  int at = -1;
  for (int e = 0; e < MAXEV; e++)
    if (e < d.nev[g] && d.ev[g][e] == x) at = e;
  return at;
}
// per group: nev * (deg + 1) slots of round 1, then nev extras unless X = 1 is an evaluation point anyway
template <class Desc>
EXH_DESC_FN constexpr int group_slots(const Desc &d, int g) {
  return d.nev[g] * (d.deg[g] + 1) + (ev_index(d, g, 1) < 0 ? d.nev[g] : 0);
}
template <class Desc>
EXH_DESC_FN constexpr int node_slots(const Desc &d) {
  int n = 0;
  for (int g = 0; g < d.G; g++) n += group_slots(d, g);
  return n;
}

// the launches per round of the base-field sweep for degree D and the slots each takes: the slots are split
// evenly over launches of at most NODES_CAP4 (F_p^4) or NODES_CAP8 (F_p^8) slots, what two wavefronts per SIMD
// have the registers for at two registers a slot and coordinate; no launches when the slot sums do not fit the
// accumulators' buffers
constexpr int NODES_CAP4 = 20, NODES_CAP8 = 8;
template <class Desc>
EXH_DESC_FN constexpr int nodes_slots_per_pass(const Desc &d, int D) {
  int slots = node_slots(d), cap = D == 4 ? NODES_CAP4 : NODES_CAP8, passes = (slots + cap - 1) / cap;
  return (slots + passes - 1) / passes;
}
template <class Desc>
EXH_DESC_FN constexpr int nodes_launches(const Desc &d, int D) {
  int slots = node_slots(d), cap = D == 4 ? NODES_CAP4 : NODES_CAP8;
  return (slots + cap - 1) / cap;
}

}  // namespace exh
