/*
 * plain_c_host.c -- a host program in plain C that uses libcublasLt.so the way its real callers do.
 *
 * ZLUDA's tracing interposer opens the library it wraps with dlopen(path, RTLD_LAZY | RTLD_LOCAL)
 * (zluda_trace_common/src/lib.rs:67-71, path from ZLUDA_BLASLT_LIB: zluda_trace_blaslt/src/lib.rs:6-11)
 * and then resolves every cublasLt* export by name with dlsym on each call
 * (zluda_trace_blaslt/src/lib.rs:24); a missing name becomes CUBLAS_STATUS_INTERNAL_ERROR for the
 * application.  A CUDA application does the same through the dynamic linker.  Neither has a Python
 * interpreter, a torch allocator or an initialised HIP runtime in the process before the first call.
 *
 *   plain_c_host <libcublasLt.so> symbols <name>...   every name must resolve (no GPU needed)
 *   plain_c_host <libcublasLt.so> matmul              int8 -> int32 problems through
 *       cublasLtCreate / descriptors / AlgoGetHeuristic / Matmul, device memory from the HIP runtime
 *       the library itself brought in, results compared bit for bit with a loop on the host
 *
 * Only include/cublaslt_abi.h is used: function-pointer types are taken from its declarations, so a
 * declaration that drifts from the library shows up here as a wrong result or a compile error.
 */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "cublaslt_abi.h"

#define FN(name) __typeof__(&name) p_##name = (__typeof__(&name))must_sym(lib, #name)

static void *must_sym(void *lib, const char *name) {
  void *p = dlsym(lib, name);
  if (!p) {
    fprintf(stderr, "missing export %s\n", name);
    exit(2);
  }
  return p;
}

/* the four HIP runtime calls a host needs for device memory; hipMemcpyKind: 1 = to device, 2 = to host */
typedef int (*hip_malloc_t)(void **, size_t);
typedef int (*hip_memcpy_t)(void *, const void *, size_t, int);
typedef int (*hip_sync_t)(void);
typedef int (*hip_free_t)(void *);
static hip_malloc_t hip_malloc;
static hip_memcpy_t hip_memcpy;
static hip_sync_t hip_sync;
static hip_free_t hip_free;

static uint64_t rng_state;
static uint32_t rng_next(void) { /* splitmix64, upper half */
  uint64_t z = (rng_state += 0x9e3779b97f4a7c15ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return (uint32_t)((z ^ (z >> 31)) >> 32);
}

#define CHECK(call)                                                       \
  do {                                                                    \
    unsigned st_ = (unsigned)(call);                                      \
    if (st_ != 0) {                                                       \
      fprintf(stderr, "%s:%d: %s -> %u\n", __FILE__, __LINE__, #call, st_); \
      exit(3);                                                            \
    }                                                                     \
  } while (0)

typedef struct {
  const char *name;
  int m, n, k, transa, transb, with_c;
  int32_t alpha, beta;
  size_t workspace;
} problem_t;

/* column-major storage everywhere (the default order): op(A) is m x k, op(B) is k x n */
static int run_problem(void *lib, const problem_t *pr) {
  FN(cublasLtCreate);
  FN(cublasLtDestroy);
  FN(cublasLtMatmulDescCreate);
  FN(cublasLtMatmulDescSetAttribute);
  FN(cublasLtMatmulDescDestroy);
  FN(cublasLtMatrixLayoutCreate);
  FN(cublasLtMatrixLayoutDestroy);
  FN(cublasLtMatmulPreferenceCreate);
  FN(cublasLtMatmulPreferenceSetAttribute);
  FN(cublasLtMatmulPreferenceDestroy);
  FN(cublasLtMatmulAlgoGetHeuristic);
  FN(cublasLtMatmul);

  const int m = pr->m, n = pr->n, k = pr->k;
  const int a_rows = pr->transa ? k : m, a_cols = pr->transa ? m : k;
  const int b_rows = pr->transb ? n : k, b_cols = pr->transb ? k : n;
  const size_t a_bytes = (size_t)a_rows * a_cols, b_bytes = (size_t)b_rows * b_cols;
  const size_t d_bytes = (size_t)m * n * sizeof(int32_t);
  int8_t *A = malloc(a_bytes), *B = malloc(b_bytes);
  int32_t *Cm = malloc(d_bytes), *D = malloc(d_bytes), *ref = malloc(d_bytes);
  for (size_t i = 0; i < a_bytes; i++) A[i] = (int8_t)rng_next();
  for (size_t i = 0; i < b_bytes; i++) B[i] = (int8_t)rng_next();
  for (size_t i = 0; i < (size_t)m * n; i++) Cm[i] = (int32_t)(rng_next() % 2001u) - 1000;
  for (int j = 0; j < n; j++)
    for (int i = 0; i < m; i++) {
      int32_t acc = 0;
      for (int l = 0; l < k; l++) {
        const int8_t a = pr->transa ? A[(size_t)i * a_rows + l] : A[(size_t)l * a_rows + i];
        const int8_t b = pr->transb ? B[(size_t)l * b_rows + j] : B[(size_t)j * b_rows + l];
        acc += (int32_t)a * (int32_t)b;
      }
      /* 32-bit wrap-around arithmetic, as the integer epilogue computes it */
      uint32_t v = (uint32_t)pr->alpha * (uint32_t)acc;
      if (pr->with_c) v += (uint32_t)pr->beta * (uint32_t)Cm[(size_t)j * m + i];
      ref[(size_t)j * m + i] = (int32_t)v;
    }

  void *dA, *dB, *dC = NULL, *dD, *dW = NULL;
  CHECK(hip_malloc(&dA, a_bytes));
  CHECK(hip_malloc(&dB, b_bytes));
  CHECK(hip_malloc(&dD, d_bytes));
  if (pr->with_c) CHECK(hip_malloc(&dC, d_bytes));
  if (pr->workspace) CHECK(hip_malloc(&dW, pr->workspace));
  CHECK(hip_memcpy(dA, A, a_bytes, 1));
  CHECK(hip_memcpy(dB, B, b_bytes, 1));
  if (pr->with_c) CHECK(hip_memcpy(dC, Cm, d_bytes, 1));
  memset(D, 0x5a, d_bytes);
  CHECK(hip_memcpy(dD, D, d_bytes, 1));

  cublasLtHandle_t handle;
  cublasLtMatmulDesc_t desc;
  cublasLtMatrixLayout_t la, lb, lc;
  cublasLtMatmulPreference_t pref;
  CHECK(p_cublasLtCreate(&handle));
  CHECK(p_cublasLtMatmulDescCreate(&desc, CUBLAS_COMPUTE_32I, CUDA_R_32I));
  const int32_t ta = pr->transa ? CUBLAS_OP_T : CUBLAS_OP_N, tb = pr->transb ? CUBLAS_OP_T : CUBLAS_OP_N;
  CHECK(p_cublasLtMatmulDescSetAttribute(desc, CUBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof ta));
  CHECK(p_cublasLtMatmulDescSetAttribute(desc, CUBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof tb));
  CHECK(p_cublasLtMatrixLayoutCreate(&la, CUDA_R_8I, (uint64_t)a_rows, (uint64_t)a_cols, a_rows));
  CHECK(p_cublasLtMatrixLayoutCreate(&lb, CUDA_R_8I, (uint64_t)b_rows, (uint64_t)b_cols, b_rows));
  CHECK(p_cublasLtMatrixLayoutCreate(&lc, CUDA_R_32I, (uint64_t)m, (uint64_t)n, m));
  CHECK(p_cublasLtMatmulPreferenceCreate(&pref));
  const uint64_t ws = pr->workspace;
  CHECK(p_cublasLtMatmulPreferenceSetAttribute(pref, CUBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof ws));

  cublasLtMatmulHeuristicResult_t res[4];
  int found = 0;
  memset(res, 0, sizeof res);
  CHECK(p_cublasLtMatmulAlgoGetHeuristic(handle, desc, la, lb, lc, lc, pref, 4, res, &found));
  if (found < 1 || res[0].state != CUBLAS_STATUS_SUCCESS || res[0].workspaceSize > pr->workspace) {
    fprintf(stderr, "%s: heuristic returned %d results, state %u, workspace %zu\n", pr->name, found,
            res[0].state, res[0].workspaceSize);
    exit(4);
  }
  printf("%s: m %d n %d k %d, %d algorithms, first: kernel %u variant %u workspace %zu\n", pr->name, m, n, k,
         found, (unsigned)(res[0].algo.data[0] & 0xffffffffu), (unsigned)res[0].algo.data[1], res[0].workspaceSize);
  fflush(stdout);
  CHECK(p_cublasLtMatmul(handle, desc, &pr->alpha, dA, la, dB, lb, &pr->beta, pr->with_c ? dC : dD, lc, dD, lc,
                         &res[0].algo, dW, pr->workspace, NULL));
  CHECK(hip_sync());
  CHECK(hip_memcpy(D, dD, d_bytes, 2));
  size_t bad = 0;
  for (size_t i = 0; i < (size_t)m * n; i++) bad += D[i] != ref[i];
  printf("%s: %zu of %zu outputs differ from the host loop\n", pr->name, bad, (size_t)m * n);

  CHECK(p_cublasLtMatmulPreferenceDestroy(pref));
  CHECK(p_cublasLtMatrixLayoutDestroy(la));
  CHECK(p_cublasLtMatrixLayoutDestroy(lb));
  CHECK(p_cublasLtMatrixLayoutDestroy(lc));
  CHECK(p_cublasLtMatmulDescDestroy(desc));
  CHECK(p_cublasLtDestroy(handle));
  hip_free(dA), hip_free(dB), hip_free(dD);
  if (dC) hip_free(dC);
  if (dW) hip_free(dW);
  free(A), free(B), free(Cm), free(D), free(ref);
  return bad != 0;
}

int main(int argc, char **argv) {
  if (argc < 3) {
    fprintf(stderr, "usage: %s <libcublasLt.so> symbols <name>... | matmul\n", argv[0]);
    return 64;
  }
  void *lib = dlopen(argv[1], RTLD_LAZY | RTLD_LOCAL);
  if (!lib) {
    fprintf(stderr, "dlopen: %s\n", dlerror());
    return 1;
  }
  if (!strcmp(argv[2], "symbols")) {
    int missing = 0;
    for (int i = 3; i < argc; i++)
      if (!dlsym(lib, argv[i])) {
        fprintf(stderr, "missing export %s\n", argv[i]);
        missing++;
      }
    printf("%d names, %d missing\n", argc - 3, missing);
    return missing != 0;
  }
  if (strcmp(argv[2], "matmul")) return 64;

  /* the HIP runtime the library was linked against is already in the process */
  void *hip = dlopen("libamdhip64.so.7", RTLD_LAZY | RTLD_NOLOAD);
  if (!hip) hip = dlopen("libamdhip64.so", RTLD_LAZY | RTLD_NOLOAD);
  if (!hip) {
    fprintf(stderr, "the library did not bring a HIP runtime with it: %s\n", dlerror());
    return 1;
  }
  hip_malloc = (hip_malloc_t)must_sym(hip, "hipMalloc");
  hip_memcpy = (hip_memcpy_t)must_sym(hip, "hipMemcpy");
  hip_sync = (hip_sync_t)must_sym(hip, "hipDeviceSynchronize");
  hip_free = (hip_free_t)must_sym(hip, "hipFree");

  static const problem_t problems[] = {
      /* 256^3, A:N B:T, alpha 1, beta 0: the configuration the reference's CPU backend can run */
      {"a_n_b_t_256", 256, 256, 256, 0, 1, 0, 1, 0, 0},
      {"a_t_b_n_ragged", 520, 392, 336, 1, 0, 1, 3, -2, 0},
      {"a_n_b_n_with_c", 264, 200, 144, 0, 0, 1, -1, 5, 0},
      {"skinny_split_k", 1024, 16, 4096, 1, 0, 0, 2, 0, (size_t)8 << 20},
  };
  int failed = 0;
  for (size_t i = 0; i < sizeof problems / sizeof problems[0]; i++) {
    rng_state = 1000 + i;
    printf("problem %s\n", problems[i].name);
    fflush(stdout);
    failed += run_problem(lib, &problems[i]);
  }
  printf(failed ? "FAILED\n" : "plain C host ok\n");
  return failed != 0;
}
