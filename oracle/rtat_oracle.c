/*
 * rtat_oracle.c — CPU restatement of the reference's execution path (see rtat_oracle.h).
 * TEST INFRASTRUCTURE ONLY: linked by tests/, the smoke check and the bench's CPU baseline.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   orc_dgemm / orc_dsyrk / orc_dtrsm   against scipy.linalg.blas (an independent library
 *                                       routine), identity / diagonal special cases, and the
 *                                       reference's own self-check of its TRSM loops against
 *                                       its GEMM loops (tests/matrixop_test.cpp:58-109);
 *   orc_dgeam                           against numpy index permutation, bit for bit;
 *   orc_*_workspace                     against hand-computed element counts per variant;
 *   orc_*_variant                       every variant equals the default variant, the
 *                                       identity the reference's tests assert
 *                                       (tests/executor_test.cpp:23-86, 139-222, 234-287);
 *   orc_dfill                           range / symmetry / structure properties and a few
 *                                       committed vectors.
 */
#define _GNU_SOURCE
#include "rtat_oracle.h"

#include <dlfcn.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------ */
/* optional host CBLAS                                                                   */
/* ------------------------------------------------------------------------------------ */
typedef void (*cblas_dgemm_fn)(int, int, int, int, int, int, double, const double*, int,
                               const double*, int, double, double*, int);
typedef void (*cblas_dsyrk_fn)(int, int, int, int, int, double, const double*, int, double,
                               double*, int);
typedef void (*cblas_dtrsm_fn)(int, int, int, int, int, int, int, double, const double*, int,
                               double*, int);
typedef int (*get_threads_fn)(void);

static void* g_lib = NULL;
static cblas_dgemm_fn g_dgemm = NULL;
static cblas_dsyrk_fn g_dsyrk = NULL;
static cblas_dtrsm_fn g_dtrsm = NULL;
static char g_lib_name[512] = "loops";

static void* sym2(void* lib, const char* a, const char* b) {
  void* s = dlsym(lib, a);
  return s ? s : dlsym(lib, b);
}

int orc_cblas_on(const char* path) {
  static const char* guesses[] = {"libopenblas.so.0", "libopenblas.so", "libmkl_rt.so", NULL};
  orc_cblas_off();
  void* lib = NULL;
  const char* used = NULL;
  if (path != NULL) {
    lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    used = path;
  }
  for (int i = 0; lib == NULL && guesses[i] != NULL; ++i) {
    lib = dlopen(guesses[i], RTLD_NOW | RTLD_LOCAL);
    used = guesses[i];
  }
  if (lib == NULL) return 0;
  g_dgemm = (cblas_dgemm_fn)sym2(lib, "cblas_dgemm", "scipy_cblas_dgemm");
  g_dsyrk = (cblas_dsyrk_fn)sym2(lib, "cblas_dsyrk", "scipy_cblas_dsyrk");
  g_dtrsm = (cblas_dtrsm_fn)sym2(lib, "cblas_dtrsm", "scipy_cblas_dtrsm");
  if (!g_dgemm || !g_dsyrk || !g_dtrsm) {
    dlclose(lib);
    g_dgemm = NULL; g_dsyrk = NULL; g_dtrsm = NULL;
    return 0;
  }
  g_lib = lib;
  strncpy(g_lib_name, used, sizeof(g_lib_name) - 1);
  get_threads_fn nt = (get_threads_fn)sym2(lib, "openblas_get_num_threads",
                                           "scipy_openblas_get_num_threads");
  if (nt == NULL) nt = (get_threads_fn)dlsym(lib, "mkl_get_max_threads");
  int threads = nt ? nt() : 1;
  return threads > 0 ? threads : 1;
}

void orc_cblas_off(void) {
  if (g_lib) dlclose(g_lib);
  g_lib = NULL;
  g_dgemm = NULL; g_dsyrk = NULL; g_dtrsm = NULL;
  strcpy(g_lib_name, "loops");
}

const char* orc_cblas_name(void) { return g_lib_name; }

/* CBLAS enum values: ColMajor 102, NoTrans 111, Trans 112, Upper 121, Lower 122,
 * NonUnit 131, Unit 132, Left 141, Right 142 — the same numbers hipBLAS uses. */

/* ------------------------------------------------------------------------------------ */
/* layer 1                                                                               */
/* ------------------------------------------------------------------------------------ */

/* The call gpuTgemm makes (matrixop.h:24-32).  Loop nest in the order of the reference's
 * own host check (tests/common.h:185-192): per output element, scale by beta, then add the
 * alpha-weighted products one k at a time.  Unlike that check, beta == 0 overwrites C
 * without reading it — the rule of the BLAS routine the reference binds. */
void orc_dgemm(int transa, int transb, int m, int n, int k, double alpha, const double* A,
               int lda, const double* B, int ldb, double beta, double* C, int ldc) {
  if (m <= 0 || n <= 0) return;
  if (g_dgemm && k > 0) {
    g_dgemm(102, transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
    return;
  }
  const int ta = transa == ORC_OP_T, tb = transb == ORC_OP_T;
  for (int j = 0; j < n; ++j) {
    for (int i = 0; i < m; ++i) {
      double acc = 0.0;
      if (alpha != 0.0) {
        for (int l = 0; l < k; ++l) {
          const double a = ta ? A[(size_t)i * lda + l] : A[(size_t)l * lda + i];
          const double b = tb ? B[(size_t)l * ldb + j] : B[(size_t)j * ldb + l];
          acc += a * b;
        }
      }
      double* c = &C[(size_t)j * ldc + i];
      *c = (beta == 0.0) ? alpha * acc : alpha * acc + beta * *c;
    }
  }
}

/* The call gpuTsyrk makes (matrixop.h:56-63): only the uplo triangle of C is written. */
void orc_dsyrk(int uplo, int trans, int n, int k, double alpha, const double* A, int lda,
               double beta, double* C, int ldc) {
  if (n <= 0) return;
  if (g_dsyrk && k > 0) {
    g_dsyrk(102, uplo, trans, n, k, alpha, A, lda, beta, C, ldc);
    return;
  }
  const int t = trans == ORC_OP_T;
  for (int j = 0; j < n; ++j) {
    const int i_lo = (uplo == ORC_LOWER) ? j : 0;
    const int i_hi = (uplo == ORC_LOWER) ? n : j + 1;
    for (int i = i_lo; i < i_hi; ++i) {
      double acc = 0.0;
      if (alpha != 0.0) {
        for (int l = 0; l < k; ++l) {
          const double a = t ? A[(size_t)i * lda + l] : A[(size_t)l * lda + i];
          const double b = t ? A[(size_t)j * lda + l] : A[(size_t)l * lda + j];
          acc += a * b;
        }
      }
      double* c = &C[(size_t)j * ldc + i];
      *c = (beta == 0.0) ? alpha * acc : alpha * acc + beta * *c;
    }
  }
}

/* The call gpuTtrsm makes (matrixop.h:87-95): substitution, one right-hand side at a time,
 * in the order of the reference's host check (tests/common.h:195-267): scale by alpha, then
 * eliminate.  That check ignores unit_diag (its third bool is unnamed); this one honours
 * it, as the BLAS routine does. */
void orc_dtrsm(int side, int uplo, int trans, int diag, int m, int n, double alpha,
               const double* A, int lda, double* B, int ldb) {
  if (m <= 0 || n <= 0) return;
  if (g_dtrsm) {
    g_dtrsm(102, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb);
    return;
  }
  const int left = side == ORC_LEFT, t = trans == ORC_OP_T, unit = diag == ORC_UNIT;
  const int eff_lower = (uplo == ORC_LOWER) != t; /* triangle of op(A) */
  const int na = left ? m : n;
#define OPA(i, j) (t ? A[(size_t)(i) * lda + (j)] : A[(size_t)(j) * lda + (i)])
  if (alpha == 0.0) {
    for (int j = 0; j < n; ++j)
      for (int i = 0; i < m; ++i) B[(size_t)j * ldb + i] = 0.0;
    return;
  }
  if (left) {
    /* op(A) x = alpha b for every column of B */
    for (int c = 0; c < n; ++c) {
      double* x = &B[(size_t)c * ldb];
      for (int i = 0; i < m; ++i) x[i] *= alpha;
      if (eff_lower) {
        for (int q = 0; q < na; ++q) {
          if (!unit) x[q] /= OPA(q, q);
          for (int i = q + 1; i < na; ++i) x[i] -= x[q] * OPA(i, q);
        }
      } else {
        for (int q = na - 1; q >= 0; --q) {
          if (!unit) x[q] /= OPA(q, q);
          for (int i = 0; i < q; ++i) x[i] -= x[q] * OPA(i, q);
        }
      }
    }
  } else {
    /* x op(A) = alpha b for every row of B; column q of X needs the columns that op(A)
     * couples it to: those after q when op(A) is lower, those before when upper. */
    for (int j = 0; j < n; ++j)
      for (int i = 0; i < m; ++i) B[(size_t)j * ldb + i] *= alpha;
    if (eff_lower) {
      for (int q = na - 1; q >= 0; --q) {
        for (int l = q + 1; l < na; ++l) {
          const double a = OPA(l, q);
          for (int i = 0; i < m; ++i) B[(size_t)q * ldb + i] -= B[(size_t)l * ldb + i] * a;
        }
        if (!unit) {
          const double d = OPA(q, q);
          for (int i = 0; i < m; ++i) B[(size_t)q * ldb + i] /= d;
        }
      }
    } else {
      for (int q = 0; q < na; ++q) {
        for (int l = 0; l < q; ++l) {
          const double a = OPA(l, q);
          for (int i = 0; i < m; ++i) B[(size_t)q * ldb + i] -= B[(size_t)l * ldb + i] * a;
        }
        if (!unit) {
          const double d = OPA(q, q);
          for (int i = 0; i < m; ++i) B[(size_t)q * ldb + i] /= d;
        }
      }
    }
  }
#undef OPA
}

/* The call gpuTgeam makes (matrixop.h:118-126): C = alpha op(A) + beta op(B), m x n.  An
 * operand with a zero scalar is not read; alpha == 1 alone is a bit copy; the two-operand
 * sum is rounded once (fma), which equals alpha*a + beta*b whenever one product is exact —
 * every case the reference produces (alpha is 1.0 in each accumulate it builds,
 * gemm.cpp:212-214, syrk.cpp:94-95, trsm.cpp:100-101).  C may alias an untransposed
 * operand of equal ld. */
void orc_dgeam(int transa, int transb, int m, int n, double alpha, const double* A, int lda,
               double beta, const double* B, int ldb, double* C, int ldc) {
  const int ta = transa == ORC_OP_T, tb = transb == ORC_OP_T;
  for (int j = 0; j < n; ++j) {
    for (int i = 0; i < m; ++i) {
      double v;
      if (alpha == 0.0 && beta == 0.0) {
        v = 0.0;
      } else if (beta == 0.0) {
        const double a = ta ? A[(size_t)i * lda + j] : A[(size_t)j * lda + i];
        v = (alpha == 1.0) ? a : alpha * a;
      } else if (alpha == 0.0) {
        const double b = tb ? B[(size_t)i * ldb + j] : B[(size_t)j * ldb + i];
        v = (beta == 1.0) ? b : beta * b;
      } else {
        const double a = ta ? A[(size_t)i * lda + j] : A[(size_t)j * lda + i];
        const double b = tb ? B[(size_t)i * ldb + j] : B[(size_t)j * ldb + i];
        v = fma(beta, b, alpha * a);
      }
      C[(size_t)j * ldc + i] = v;
    }
  }
}

/* ------------------------------------------------------------------------------------ */
/* operand generator                                                                     */
/* ------------------------------------------------------------------------------------ */
static uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

static double unit_uniform(uint64_t seed, uint32_t i, uint32_t j) {
  uint64_t z = mix64(seed * 0x9E3779B97F4A7C15ull + (((uint64_t)j << 32) | (uint64_t)i));
  return (double)(z >> 11) * (1.0 / 9007199254740992.0);
}

void orc_dfill(double* A, int m, int n, int ld, uint64_t seed, int kind) {
  for (int j = 0; j < n; ++j) {
    for (int i = 0; i < ld; ++i) {
      double v;
      if (i >= m) {
        v = NAN;
      } else if (kind == 1) {
        const uint32_t hi = (uint32_t)(i > j ? i : j), lo = (uint32_t)(i > j ? j : i);
        v = 2.0 * unit_uniform(seed, hi, lo) - 1.0;
      } else if (kind == 2) {
        const double u = unit_uniform(seed, (uint32_t)i, (uint32_t)j);
        if (i > j) v = (2.0 * u - 1.0) / (double)m;
        else if (i == j) v = 1.0 + u;
        else v = NAN;
      } else if (kind == 4) {
        const uint32_t hi = (uint32_t)(i > j ? i : j), lo = (uint32_t)(i > j ? j : i);
        const double u = unit_uniform(seed, hi, lo);
        v = (i == j) ? 1.0 + u : (2.0 * u - 1.0) / (double)m;
      } else if (kind == 3) {
        v = 1.0 - unit_uniform(seed, (uint32_t)i, (uint32_t)j);
      } else {
        v = 2.0 * unit_uniform(seed, (uint32_t)i, (uint32_t)j) - 1.0;
      }
      A[(size_t)j * ld + i] = v;
    }
  }
}

/* ------------------------------------------------------------------------------------ */
/* layer 2: the matrix-op tree (matrixop.h:142-617)                                      */
/* ------------------------------------------------------------------------------------ */
typedef struct { size_t m, n, ld; } dims_t;
typedef struct { double* p; dims_t d; } mat_t;
typedef struct { char* p; size_t bytes; } space_t;

enum kind { K_LEAF, K_MOVE, K_ACCUMULATE, K_MULT, K_MULT_ALLOC, K_TRS, K_TRS_ALLOC, K_SYRK,
            K_SYRK_ALLOC };

typedef struct node {
  enum kind kind;
  struct node* op[3];
  int nops;
  int out_operand; /* index of the operand computed straight into out_space, or -1 */
  mat_t leaf;
  double alpha, beta;
  int f0, f1, f2, f3; /* transpose / transa / side_left ..., per kind */
  size_t pad;
} node_t;

static size_t round_up(size_t x, size_t pad) { return ((x + pad - 1) / pad) * pad; }

static dims_t node_dims(const node_t* nd) {
  dims_t d = {0, 0, 0};
  switch (nd->kind) {
    case K_LEAF: return nd->leaf.d;
    case K_MOVE: { /* matrixop.h:321-327 */
      dims_t a = node_dims(nd->op[0]);
      d.m = nd->f0 ? a.n : a.m;
      d.n = nd->f0 ? a.m : a.n;
      d.ld = round_up(d.m, nd->pad);
      return d;
    }
    case K_ACCUMULATE: return node_dims(nd->op[1]); /* :290 */
    case K_MULT: return node_dims(nd->op[2]);       /* :375-378 */
    case K_MULT_ALLOC: {                            /* :415-422 */
      dims_t a = node_dims(nd->op[0]), b = node_dims(nd->op[1]);
      d.m = nd->f0 ? a.n : a.m;
      d.n = nd->f1 ? b.m : b.n;
      d.ld = round_up(d.m, nd->pad);
      return d;
    }
    case K_TRS: return node_dims(nd->op[1]); /* :467-470 */
    case K_TRS_ALLOC: {                      /* :514-518 */
      dims_t b = node_dims(nd->op[1]);
      d.m = b.m; d.n = b.n;
      d.ld = round_up(b.m, nd->pad);
      return d;
    }
    case K_SYRK: return node_dims(nd->op[1]); /* :559-562 */
    case K_SYRK_ALLOC: {                      /* :595-600 */
      dims_t a = node_dims(nd->op[0]);
      d.m = d.n = nd->f1 ? a.n : a.m;
      d.ld = round_up(d.m, nd->pad);
      return d;
    }
  }
  return d;
}

/* Elements the node's own result occupies in out_space (0 when it writes into an operand). */
static size_t node_out_req(const node_t* nd) {
  switch (nd->kind) {
    case K_MOVE: case K_MULT_ALLOC: case K_TRS_ALLOC: case K_SYRK_ALLOC: {
      dims_t d = node_dims(nd);
      return d.ld * d.n;
    }
    default: return 0;
  }
}

/* matrixop.h:172-185: own output, plus the high-water mark over operands of (outputs of the
 * operands so far that are not the output operand) + (scratch of the current operand). */
static size_t node_workspace_req(const node_t* nd) {
  size_t operand_space = 0, extra = 0;
  for (int i = 0; i < nd->nops; ++i) {
    const node_t* c = nd->op[i];
    if (i != nd->out_operand) operand_space += node_out_req(c);
    const size_t c_scratch = node_workspace_req(c) - node_out_req(c);
    if (operand_space + c_scratch > extra) extra = operand_space + c_scratch;
  }
  return node_out_req(nd) + extra;
}

static space_t peel(space_t* s, size_t elems) { /* workspace.h:32-40 */
  space_t out = {s->p, elems * sizeof(double)};
  s->p += out.bytes;
  s->bytes -= out.bytes;
  return out;
}

static mat_t node_execute(const node_t* nd, space_t out_space, space_t scratch);

/* matrixop.h:192-210 */
static void compute_operands(const node_t* nd, space_t out_space, space_t scratch, mat_t* res) {
  for (int i = 0; i < nd->nops; ++i) {
    space_t mine;
    if (i == nd->out_operand) mine = out_space;
    else mine = peel(&scratch, node_out_req(nd->op[i]));
    res[i] = node_execute(nd->op[i], mine, scratch);
  }
}

static mat_t node_execute(const node_t* nd, space_t out_space, space_t scratch) {
  mat_t r[3];
  mat_t out;
  if (nd->kind == K_LEAF) return nd->leaf;
  compute_operands(nd, out_space, scratch, r);
  switch (nd->kind) {
    case K_MOVE: /* :329-343: B(out_space) = alpha op(A), beta = 0 */
      out.p = (double*)out_space.p;
      out.d = node_dims(nd);
      orc_dgeam(nd->f0 ? ORC_OP_T : ORC_OP_N, ORC_OP_N, (int)out.d.m, (int)out.d.n, nd->alpha,
                r[0].p, (int)r[0].d.ld, 0.0, out.p, (int)out.d.ld, out.p, (int)out.d.ld);
      return out;
    case K_ACCUMULATE: /* :292-304: B = alpha op(A) + beta B in place */
      orc_dgeam(nd->f0 ? ORC_OP_T : ORC_OP_N, ORC_OP_N, (int)r[1].d.m, (int)r[1].d.n, nd->alpha,
                r[0].p, (int)r[0].d.ld, nd->beta, r[1].p, (int)r[1].d.ld, r[1].p,
                (int)r[1].d.ld);
      return r[1];
    case K_MULT: { /* :382-393, gpuTgemm :20-22 */
      const int k = (int)(nd->f0 ? r[0].d.m : r[0].d.n);
      orc_dgemm(nd->f0 ? ORC_OP_T : ORC_OP_N, nd->f1 ? ORC_OP_T : ORC_OP_N, (int)r[2].d.m,
                (int)r[2].d.n, k, nd->alpha, r[0].p, (int)r[0].d.ld, r[1].p, (int)r[1].d.ld,
                nd->beta, r[2].p, (int)r[2].d.ld);
      return r[2];
    }
    case K_MULT_ALLOC: { /* :426-438 */
      out.p = (double*)out_space.p;
      out.d = node_dims(nd);
      const int k = (int)(nd->f0 ? r[0].d.m : r[0].d.n);
      orc_dgemm(nd->f0 ? ORC_OP_T : ORC_OP_N, nd->f1 ? ORC_OP_T : ORC_OP_N, (int)out.d.m,
                (int)out.d.n, k, nd->alpha, r[0].p, (int)r[0].d.ld, r[1].p, (int)r[1].d.ld, 0.0,
                out.p, (int)out.d.ld);
      return out;
    }
    case K_TRS:       /* :474-484 */
    case K_TRS_ALLOC: /* :522-532: operand 1 was computed into out_space; solved in place */
      orc_dtrsm(nd->f0 ? ORC_LEFT : ORC_RIGHT, nd->f1 ? ORC_LOWER : ORC_UPPER,
                nd->f2 ? ORC_OP_T : ORC_OP_N, nd->f3 ? ORC_UNIT : ORC_NON_UNIT, (int)r[1].d.m,
                (int)r[1].d.n, nd->alpha, r[0].p, (int)r[0].d.ld, r[1].p, (int)r[1].d.ld);
      return r[1];
    case K_SYRK: { /* :566-576, gpuTsyrk :53-54 */
      const int k = (int)(nd->f1 ? r[0].d.m : r[0].d.n);
      orc_dsyrk(nd->f0 ? ORC_LOWER : ORC_UPPER, nd->f1 ? ORC_OP_T : ORC_OP_N, (int)r[1].d.n, k,
                nd->alpha, r[0].p, (int)r[0].d.ld, nd->beta, r[1].p, (int)r[1].d.ld);
      return r[1];
    }
    case K_SYRK_ALLOC: { /* :604-615: zero the scratch, then syrk with beta = 0 */
      out.p = (double*)out_space.p;
      out.d = node_dims(nd);
      orc_dgeam(ORC_OP_N, ORC_OP_N, (int)out.d.m, (int)out.d.n, 0.0, out.p, (int)out.d.ld, 0.0,
                out.p, (int)out.d.ld, out.p, (int)out.d.ld);
      const int k = (int)(nd->f1 ? r[0].d.m : r[0].d.n);
      orc_dsyrk(nd->f0 ? ORC_LOWER : ORC_UPPER, nd->f1 ? ORC_OP_T : ORC_OP_N, (int)out.d.n, k,
                nd->alpha, r[0].p, (int)r[0].d.ld, 0.0, out.p, (int)out.d.ld);
      return out;
    }
    default: break;
  }
  out.p = NULL;
  out.d.m = out.d.n = out.d.ld = 0;
  return out;
}

/* A fixed pool is enough: no variant builds more than eight nodes. */
typedef struct { node_t n[12]; int used; } pool_t;

static node_t* mk(pool_t* pl, enum kind k) {
  node_t* nd = &pl->n[pl->used++];
  memset(nd, 0, sizeof(*nd));
  nd->kind = k;
  nd->out_operand = -1;
  nd->pad = 1;
  return nd;
}

static node_t* mk_leaf(pool_t* pl, const double* p, size_t m, size_t n, size_t ld) {
  node_t* nd = mk(pl, K_LEAF);
  nd->leaf.p = (double*)p;
  nd->leaf.d.m = m; nd->leaf.d.n = n; nd->leaf.d.ld = ld;
  return nd;
}

static node_t* mk_move(pool_t* pl, node_t* a, double alpha, int transpose, size_t pad) {
  node_t* nd = mk(pl, K_MOVE);
  nd->op[0] = a; nd->nops = 1;
  nd->alpha = alpha; nd->f0 = transpose; nd->pad = pad;
  return nd;
}

static node_t* mk_accumulate(pool_t* pl, node_t* a, node_t* b, double alpha, double beta,
                             int transpose) {
  node_t* nd = mk(pl, K_ACCUMULATE);
  nd->op[0] = a; nd->op[1] = b; nd->nops = 2; nd->out_operand = 1;
  nd->alpha = alpha; nd->beta = beta; nd->f0 = transpose;
  return nd;
}

/* Runs a finished tree the way Executor::internal_execute does (executor.h:46-53). */
static int run_tree(const node_t* root, void* ws, size_t ws_bytes) {
  if (node_workspace_req(root) * sizeof(double) > ws_bytes) return -2;
  space_t none = {NULL, 0};
  space_t scratch = {(char*)ws, ws_bytes};
  node_execute(root, none, scratch);
  return 0;
}

/* ---- GEMM variants (gemm.cpp:75-134 with pads, :183-221 without) ---------------------- */
static node_t* gemm_tree(pool_t* pl, const char* v, int transa, int transb, int m, int n, int k,
                         double alpha, const double* A, int lda, const double* B, int ldb,
                         double beta, double* C, int ldc) {
  const size_t len = strlen(v);
  if (len != 3 && len != 6) return NULL;
  for (int i = 0; i < 3; ++i)
    if (v[i] != 'N' && v[i] != 'T') return NULL;
  for (size_t i = 3; i < len; ++i)
    if (v[i] != 'N' && v[i] != 'P') return NULL;
  const int ta = v[0] == 'T', tb = v[1] == 'T', tc = v[2] == 'T';
  const int pa = len == 6 && v[3] == 'P', pb = len == 6 && v[4] == 'P',
            pc = len == 6 && v[5] == 'P';
  int opa_t = transa == ORC_OP_T, opb_t = transb == ORC_OP_T;
  node_t* a = mk_leaf(pl, A, opa_t ? k : m, opa_t ? m : k, lda);
  node_t* b = mk_leaf(pl, B, opb_t ? n : k, opb_t ? k : n, ldb);
  node_t* c = mk_leaf(pl, C, m, n, ldc);
  if (ta) opa_t = !opa_t;
  if (ta || pa) a = mk_move(pl, a, 1.0, ta, pa ? 32 : 1);
  if (tb) opb_t = !opb_t;
  if (tb || pb) b = mk_move(pl, b, 1.0, tb, pb ? 32 : 1);
  if (tc) {
    /* (alpha op(A) op(B))^T = alpha op(B)^T op(A)^T into scratch, then C = S^T + beta C */
    node_t* s = mk(pl, K_MULT_ALLOC);
    s->op[0] = b; s->op[1] = a; s->nops = 2;
    s->f0 = !opb_t; s->f1 = !opa_t; s->alpha = alpha; s->pad = pc ? 32 : 1;
    return mk_accumulate(pl, s, c, 1.0, beta, 1);
  }
  if (pc) {
    node_t* s = mk(pl, K_MULT_ALLOC);
    s->op[0] = a; s->op[1] = b; s->nops = 2;
    s->f0 = opa_t; s->f1 = opb_t; s->alpha = alpha; s->pad = 32;
    return mk_accumulate(pl, s, c, 1.0, beta, 0);
  }
  node_t* mult = mk(pl, K_MULT);
  mult->op[0] = a; mult->op[1] = b; mult->op[2] = c; mult->nops = 3; mult->out_operand = 2;
  mult->f0 = opa_t; mult->f1 = opb_t; mult->alpha = alpha; mult->beta = beta;
  return mult;
}

long orc_gemm_workspace(const char* variant, int transa, int transb, int m, int n, int k,
                        int lda, int ldb, int ldc) {
  pool_t pl = {.used = 0};
  node_t* t = gemm_tree(&pl, variant, transa, transb, m, n, k, 1.0, NULL, lda, NULL, ldb, 0.0,
                        NULL, ldc);
  return t ? (long)(node_workspace_req(t) * sizeof(double)) : -1;
}

int orc_gemm_variant(const char* variant, int transa, int transb, int m, int n, int k,
                     double alpha, const double* A, int lda, const double* B, int ldb,
                     double beta, double* C, int ldc, void* ws, size_t ws_bytes) {
  pool_t pl = {.used = 0};
  node_t* t = gemm_tree(&pl, variant, transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C,
                        ldc);
  return t ? run_tree(t, ws, ws_bytes) : -1;
}

/* ---- SYRK variants (syrk.cpp:71-104) -------------------------------------------------- */
static node_t* syrk_tree(pool_t* pl, const char* v, int uplo, int trans, int n, int k,
                         double alpha, const double* A, int lda, double beta, double* C,
                         int ldc) {
  if (strlen(v) != 2) return NULL;
  for (int i = 0; i < 2; ++i)
    if (v[i] != 'T' && v[i] != 'F') return NULL;
  int t = trans == ORC_OP_T, lower = uplo == ORC_LOWER;
  node_t* a = mk_leaf(pl, A, t ? k : n, t ? n : k, lda);
  node_t* c = mk_leaf(pl, C, n, n, ldc);
  if (v[0] == 'T') {
    t = !t;
    a = mk_move(pl, a, 1.0, 1, 1);
  }
  if (v[1] == 'T') {
    /* the other triangle of a fresh zeroed scratch, added back transposed */
    lower = !lower;
    node_t* s = mk(pl, K_SYRK_ALLOC);
    s->op[0] = a; s->nops = 1;
    s->f0 = lower; s->f1 = t; s->alpha = alpha;
    return mk_accumulate(pl, s, c, 1.0, beta, 1);
  }
  node_t* s = mk(pl, K_SYRK);
  s->op[0] = a; s->op[1] = c; s->nops = 2; s->out_operand = 1;
  s->f0 = lower; s->f1 = t; s->alpha = alpha; s->beta = beta;
  return s;
}

long orc_syrk_workspace(const char* variant, int uplo, int trans, int n, int k, int lda,
                        int ldc) {
  pool_t pl = {.used = 0};
  node_t* t = syrk_tree(&pl, variant, uplo, trans, n, k, 1.0, NULL, lda, 0.0, NULL, ldc);
  return t ? (long)(node_workspace_req(t) * sizeof(double)) : -1;
}

int orc_syrk_variant(const char* variant, int uplo, int trans, int n, int k, double alpha,
                     const double* A, int lda, double beta, double* C, int ldc, void* ws,
                     size_t ws_bytes) {
  pool_t pl = {.used = 0};
  node_t* t = syrk_tree(&pl, variant, uplo, trans, n, k, alpha, A, lda, beta, C, ldc);
  return t ? run_tree(t, ws, ws_bytes) : -1;
}

/* ---- TRSM variants (trsm.cpp:72-111) -------------------------------------------------- */
static node_t* trsm_tree(pool_t* pl, const char* v, int side, int uplo, int trans, int diag,
                         int m, int n, double alpha, const double* A, int lda, double* B,
                         int ldb) {
  if (strlen(v) != 2) return NULL;
  for (int i = 0; i < 2; ++i)
    if (v[i] != 'T' && v[i] != 'F') return NULL;
  int left = side == ORC_LEFT, lower = uplo == ORC_LOWER, t = trans == ORC_OP_T;
  const int unit = diag == ORC_UNIT;
  const int na = left ? m : n;
  node_t* a = mk_leaf(pl, A, na, na, lda);
  node_t* b = mk_leaf(pl, B, m, n, ldb);
  if (v[1] == 'T') { /* transpose_A: A^T in scratch, flip trans and uplo */
    t = !t; lower = !lower;
    a = mk_move(pl, a, 1.0, 1, 1);
  }
  if (v[0] == 'T') { /* swap_side: op(A) X = aB  <=>  X^T op(A)^T = a B^T */
    t = !t; left = !left;
    node_t* bt = mk_move(pl, b, 1.0, 1, 1);
    node_t* s = mk(pl, K_TRS_ALLOC);
    s->op[0] = a; s->op[1] = bt; s->nops = 2; s->out_operand = 1;
    s->f0 = left; s->f1 = lower; s->f2 = t; s->f3 = unit; s->alpha = alpha;
    node_t* b2 = mk_leaf(pl, B, m, n, ldb);
    return mk_accumulate(pl, s, b2, 1.0, 0.0, 1);
  }
  node_t* s = mk(pl, K_TRS);
  s->op[0] = a; s->op[1] = b; s->nops = 2; s->out_operand = 1;
  s->f0 = left; s->f1 = lower; s->f2 = t; s->f3 = unit; s->alpha = alpha;
  return s;
}

long orc_trsm_workspace(const char* variant, int side, int uplo, int trans, int diag, int m,
                        int n, int lda, int ldb) {
  pool_t pl = {.used = 0};
  node_t* t = trsm_tree(&pl, variant, side, uplo, trans, diag, m, n, 1.0, NULL, lda, NULL, ldb);
  return t ? (long)(node_workspace_req(t) * sizeof(double)) : -1;
}

int orc_trsm_variant(const char* variant, int side, int uplo, int trans, int diag, int m, int n,
                     double alpha, const double* A, int lda, double* B, int ldb, void* ws,
                     size_t ws_bytes) {
  pool_t pl = {.used = 0};
  node_t* t = trsm_tree(&pl, variant, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb);
  return t ? run_tree(t, ws, ws_bytes) : -1;
}
