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

}  // namespace exh
