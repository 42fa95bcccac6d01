// stmtdesc.hpp -- the descriptor a round kernel is generated from (or interprets), and its limits.
#pragma once

namespace exh {

constexpr int MAXT = 16;    // tables per statement
constexpr int MAXG = 16;    // table groups per statement
constexpr int MAXDEG = 6;   // tables per group
constexpr int MAXEV = 6;    // evaluation points per group
constexpr int MAXACC = 36;  // accumulators (group, point) per statement
constexpr int MAXX = 7;     // largest evaluation point
constexpr int BLOCK = 256;  // threads per workgroup

// A statement as the kernels see it: G groups, group g the product of the deg[g] tables tab[g][..],
// evaluated at the nev[g] points ev[g][..]; accumulators are numbered group by group, point by point.
struct StmtDesc {
  int T, G, nacc, maxx;
  int deg[MAXG];
  int tab[MAXG][MAXDEG];
  int nev[MAXG];
  int ev[MAXG][MAXEV];
};

}  // namespace exh
