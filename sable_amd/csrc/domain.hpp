// domain.hpp -- the device side of the domain layer (src/domain.lisp:288-331): the leaves of each
// lookup's fraction tree and the sumcheck's tables, from the columns resident in HBM.  The protocol
// around them (DOMAIN-STATEMENT, PROVE-DOMAIN, VERIFY-DOMAIN) is the host's.
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

namespace exh {

enum ColumnKind { COL_FULL = 0, COL_ROW = 1, COL_COL = 2 };

struct DomainColumn {
  std::string name;  // upper-cased
  int kind = COL_FULL, c = 0;
  bool shared = false;
  const uint32_t *ptr = nullptr;  // K 2^n base values for :FULL, K 2^(n-c) for :ROW c, K 2^c for :COL c; no K if shared
  uint64_t entries = 0;
};

// the entries a column of the kind holds, or 0 when (kind, c, shared) is not a column of an n-variable domain
uint64_t column_entries(int kind, int c, bool shared, int n, int K);

// TABLE-VALUES (src/domain.lisp:311-321): the column at the half's points (half < 0: at every point below
// 2^(n-1)), K blocks of 2^(n-1) base values
int domain_table(const DomainColumn &col, int half, int n, int K, uint32_t *out);

// DOMAIN-LEAVES (src/domain.lisp:298-309) of one lookup: p = num (1 when the lookup has none) and
// q = Z - tag - sum_i beta_i v_i at every (block, x), as K 2^n EXTs of degree D each; the forms are over the
// column names
int domain_leaves(int D, int n, int K, const std::vector<DomainColumn> &columns, const std::string &tag,
                  const std::vector<std::string> &values, const char *num, const uint32_t *z, const uint32_t *betas,
                  uint32_t *p, uint32_t *q);

}  // namespace exh
