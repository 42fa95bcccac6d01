// domain.hip -- see domain.hpp.
#include "domain.hpp"

#include <string.h>

#include "context.hpp"
#include "field.hpp"
#include "forms.hpp"

namespace exh {

namespace {

constexpr int DL_MAXCOLS = 16;    // columns a lookup's forms may name
constexpr int DL_MAXFORMS = 10;   // numerator, tag and up to eight values
constexpr int DL_MAXTERMS = 64;   // monomials over all of a lookup's forms
constexpr int DL_MAXVARS = 160;   // column occurrences over all monomials
constexpr int DL_BLOCK = 256;

struct DevColumn {
  const uint32_t *ptr;
  int kind, c, shared;
};

// COLUMN-VALUE (src/domain.lisp:288-296): the column in block b at the in-block index x
__device__ __forceinline__ uint32_t column_value(const DevColumn &col, uint64_t b, uint64_t x, int n) {
  if (col.kind == COL_FULL) return col.ptr[(b << n) + x];
  if (col.kind == COL_ROW) return col.ptr[(col.shared ? 0 : b << (n - col.c)) + (x >> col.c)];
  return col.ptr[(col.shared ? 0 : b << col.c) + (x & (((uint64_t)1 << col.c) - 1))];
}

__global__ __launch_bounds__(DL_BLOCK) void domain_table_kernel(DevColumn col, uint64_t offset, int n, uint64_t n_out,
                                                                uint32_t *out) {
  uint64_t o = (uint64_t)blockIdx.x * DL_BLOCK + threadIdx.x;
  if (o >= n_out) return;
  uint64_t half = (uint64_t)1 << (n - 1);
  out[o] = column_value(col, o >> (n - 1), (o & (half - 1)) + offset, n);
}

// A lookup's forms as sums of monomials over the columns: form f is the terms term_start[f] .. term_start[f+1],
// term t the coefficient coef[t] times the columns vars[var_start[t] .. var_start[t+1]).
struct LeafProgram {
  int n, n_cols, n_values, has_num;
  DevColumn cols[DL_MAXCOLS];
  uint16_t term_start[DL_MAXFORMS + 1];
  uint16_t var_start[DL_MAXTERMS + 1];
  uint32_t coef[DL_MAXTERMS];
  uint8_t vars[DL_MAXVARS];
  uint32_t z[8];
  uint32_t betas[DL_MAXFORMS - 2][8];
};

__device__ __forceinline__ uint32_t form_value(const LeafProgram &pr, int f, uint64_t b, uint64_t x) {
  uint32_t sum = 0;
  for (int t = pr.term_start[f]; t < pr.term_start[f + 1]; t++) {
    uint32_t prod = pr.coef[t];
    for (int v = pr.var_start[t]; v < pr.var_start[t + 1]; v++)
      prod = fmul(prod, column_value(pr.cols[pr.vars[v]], b, x, pr.n));
    sum = fadd(sum, prod);
  }
  return sum;
}

template <int D>
__global__ __launch_bounds__(DL_BLOCK) void domain_leaves_kernel(LeafProgram pr, uint64_t n_out, uint32_t *p,
                                                                 uint32_t *q) {
  uint64_t i = (uint64_t)blockIdx.x * DL_BLOCK + threadIdx.x;
  if (i >= n_out) return;
  uint64_t b = i >> pr.n, x = i & (((uint64_t)1 << pr.n) - 1);
  uint32_t pv[D], qv[D];
#pragma unroll
  for (int j = 0; j < D; j++) pv[j] = 0, qv[j] = pr.z[j];
  pv[0] = pr.has_num ? form_value(pr, 0, b, x) : 1u;
  qv[0] = fsub(qv[0], form_value(pr, 1, b, x));
  for (int k = 0; k < pr.n_values; k++) {
    uint32_t v = form_value(pr, 2 + k, b, x);
#pragma unroll
    for (int j = 0; j < D; j++) qv[j] = fsub(qv[j], fmul(pr.betas[k][j], v));
  }
#pragma unroll
  for (int j = 0; j < D; j += 4) {
    *reinterpret_cast<uint4 *>(p + i * D + j) = make_uint4(pv[j], pv[j + 1], pv[j + 2], pv[j + 3]);
    *reinterpret_cast<uint4 *>(q + i * D + j) = make_uint4(qv[j], qv[j + 1], qv[j + 2], qv[j + 3]);
  }
}

DevColumn dev_column(const DomainColumn &col) { return DevColumn{col.ptr, col.kind, col.c, col.shared ? 1 : 0}; }

int check_column(const DomainColumn &col, int n, int K) {
  uint64_t want = column_entries(col.kind, col.c, col.shared, n, K);
  if (!want || col.entries != want) {
    set_error("invalid-parameter: column " + col.name + ": kind, c or size do not fit the domain");
    return E_PARAM;
  }
  return OK;
}

}  // namespace

uint64_t column_entries(int kind, int c, bool shared, int n, int K) {
  uint64_t blocks = shared ? 1 : (uint64_t)K;
  if (kind == COL_FULL) return shared ? 0 : blocks << n;
  if (c < 0 || c > n) return 0;
  if (kind == COL_ROW) return blocks << (n - c);
  if (kind == COL_COL) return blocks << c;
  return 0;
}

int domain_table(const DomainColumn &col, int half, int n, int K, uint32_t *out) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if (n < 2 || n > 40 || K < 1 || half > 1) {
    set_error("invalid-parameter: domain table arguments");
    return E_PARAM;
  }
  if ((status = check_column(col, n, K))) return status;
  uint64_t n_out = (uint64_t)K << (n - 1);
  uint64_t offset = half > 0 ? (uint64_t)1 << (n - 1) : 0;
  hipLaunchKernelGGL(domain_table_kernel, dim3((uint32_t)((n_out + DL_BLOCK - 1) / DL_BLOCK)), dim3(DL_BLOCK), 0,
                     c.stream, dev_column(col), offset, n, n_out, out);
  EXH_HIP(hipGetLastError());
  return OK;
}

int domain_leaves(int D, int n, int K, const std::vector<DomainColumn> &columns, const std::string &tag,
                  const std::vector<std::string> &values, const char *num, const uint32_t *z, const uint32_t *betas,
                  uint32_t *p, uint32_t *q) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if ((D != 4 && D != 8) || n < 2 || n > 40 || K < 1 || (int)columns.size() > DL_MAXCOLS ||
      (int)values.size() > DL_MAXFORMS - 2) {
    set_error("invalid-parameter: domain leaves: at most 16 columns and 8 values per lookup");
    return E_PARAM;
  }
  LeafProgram pr;
  memset(&pr, 0, sizeof(pr));
  pr.n = n, pr.n_cols = (int)columns.size(), pr.n_values = (int)values.size(), pr.has_num = num != nullptr;
  for (size_t k = 0; k < columns.size(); k++) {
    if ((status = check_column(columns[k], n, K))) return status;
    pr.cols[k] = dev_column(columns[k]);
  }
  std::vector<std::string> texts = {num ? std::string(num) : std::string("1"), tag};
  texts.insert(texts.end(), values.begin(), values.end());
  int terms = 0, vars = 0;
  for (size_t f = 0; f < texts.size(); f++) {
    std::vector<Term> expanded;
    if ((status = expand_form(texts[f], &expanded))) return status;
    pr.term_start[f] = (uint16_t)terms;
    for (const Term &t : expanded) {
      if (terms >= DL_MAXTERMS || vars + (int)t.vars.size() > DL_MAXVARS) {
        set_error("invalid-parameter: domain leaves: the lookup's forms have too many monomials");
        return E_PARAM;
      }
      pr.coef[terms] = t.coeff;
      pr.var_start[terms] = (uint16_t)vars;
      for (const std::string &v : t.vars) {
        int at = -1;
        for (size_t k = 0; k < columns.size(); k++)
          if (columns[k].name == v) at = (int)k;
        if (at < 0) {
          set_error("invalid-parameter: domain leaves: " + v + " is not a column");
          return E_PARAM;
        }
        pr.vars[vars++] = (uint8_t)at;
      }
      terms++;
    }
  }
  for (size_t f = texts.size(); f <= DL_MAXFORMS; f++) pr.term_start[f] = (uint16_t)terms;
  pr.var_start[terms] = (uint16_t)vars;
  memcpy(pr.z, z, 4 * D);
  for (size_t k = 0; k < values.size(); k++) memcpy(pr.betas[k], betas + k * D, 4 * D);
  uint64_t n_out = (uint64_t)K << n;
  dim3 grid((uint32_t)((n_out + DL_BLOCK - 1) / DL_BLOCK));
  if (D == 4)
    hipLaunchKernelGGL(domain_leaves_kernel<4>, grid, dim3(DL_BLOCK), 0, c.stream, pr, n_out, p, q);
  else
    hipLaunchKernelGGL(domain_leaves_kernel<8>, grid, dim3(DL_BLOCK), 0, c.stream, pr, n_out, p, q);
  EXH_HIP(hipGetLastError());
  return OK;
}

}  // namespace exh
