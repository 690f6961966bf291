// The exported C ABI of libcublasLt.so: the 45 symbols of cuda_macros/src/cublaslt.rs:4-583.
//
// Host-only code.  Descriptors are plain heap objects owned by this library (the reference's are
// hipBLASLt pointers: zluda_blaslt/src/impl.rs:243-255, 360-374); the handle keeps the reference's
// cookie-checked boxing (zluda_common/src/lib.rs:1036-1107) so that a cublasHandle_t created by
// ZLUDA's libcublas, whose first payload word is an Lt handle (zluda_blas/src/impl.rs:17-23),
// is accepted wherever an Lt handle is.
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <new>

#include "../../include/cublaslt_abi.h"
#include "../../include/zluda_gemm_launch.h"

namespace {

constexpr uint64_t DESC_MAGIC = 0x5a4c44414d4d4431ull;    // matmul desc
constexpr uint64_t LAYOUT_MAGIC = 0x5a4c44414c41594full;  // matrix layout
constexpr uint64_t PREF_MAGIC = 0x5a4c444150524546ull;    // preference

struct LtHandle {
  size_t cookie;  // ZLUDA_BLASLT_HANDLE_COOKIE while alive, 0 after destroy
  uint64_t reserved;
};
struct BlasHandleView {  // zluda_blas/src/impl.rs:17-23 behind the LiveCheck cookie
  size_t cookie;
  cublasLtHandle_t blas_lt;
};

struct MatmulDescObj {
  uint64_t magic;
  zluda_matmul_desc d;
  int32_t sm_count_target;
};
struct LayoutObj {
  uint64_t magic;
  zluda_matrix_layout l;
};
struct PrefObj {
  uint64_t magic;
  uint32_t search_mode;
  uint64_t max_workspace;
  uint32_t min_align[4];
  uint32_t reduction_mask;
  float max_waves;
  uint64_t impl_mask;
};

// zluda_blaslt/src/impl.rs:57-73: a direct Lt handle, or a cuBLAS handle embedding one
LtHandle *resolve_handle(cublasLtHandle_t h) {
  if (!h) return nullptr;
  LtHandle *lt = reinterpret_cast<LtHandle *>(h);
  if (lt->cookie == ZLUDA_BLASLT_HANDLE_COOKIE) return lt;
  BlasHandleView *bh = reinterpret_cast<BlasHandleView *>(h);
  if (bh->cookie == ZLUDA_BLAS_HANDLE_COOKIE && bh->blas_lt) {
    LtHandle *inner = reinterpret_cast<LtHandle *>(bh->blas_lt);
    if (inner->cookie == ZLUDA_BLASLT_HANDLE_COOKIE) return inner;
  }
  return nullptr;
}

MatmulDescObj *as_desc(cublasLtMatmulDesc_t p) {
  auto *o = reinterpret_cast<MatmulDescObj *>(p);
  return (o && o->magic == DESC_MAGIC) ? o : nullptr;
}
LayoutObj *as_layout(cublasLtMatrixLayout_t p) {
  auto *o = reinterpret_cast<LayoutObj *>(p);
  return (o && o->magic == LAYOUT_MAGIC) ? o : nullptr;
}
PrefObj *as_pref(cublasLtMatmulPreference_t p) {
  auto *o = reinterpret_cast<PrefObj *>(p);
  return (o && o->magic == PREF_MAGIC) ? o : nullptr;
}

// typed attribute access ------------------------------------------------------------------------
template <class T>
cublasStatus_t set_val(T &dst, const void *buf, size_t size) {
  if (!buf || size != sizeof(T)) return CUBLAS_STATUS_INVALID_VALUE;
  memcpy(&dst, buf, sizeof(T));
  return CUBLAS_STATUS_SUCCESS;
}
template <class T>
cublasStatus_t get_val(const T &src, void *buf, size_t size, size_t *written) {
  if (size == 0 && !buf) {  // size query
    if (!written) return CUBLAS_STATUS_INVALID_VALUE;
    *written = sizeof(T);
    return CUBLAS_STATUS_SUCCESS;
  }
  if (!buf || size != sizeof(T)) return CUBLAS_STATUS_INVALID_VALUE;
  memcpy(buf, &src, sizeof(T));
  if (written) *written = sizeof(T);
  return CUBLAS_STATUS_SUCCESS;
}

// One accessor for set and get: `set` selects the direction.
template <class T>
cublasStatus_t access(bool set, T &field, const void *in, void *out, size_t size, size_t *written) {
  return set ? set_val(field, in, size) : get_val(field, out, size, written);
}

bool epilogue_supported(uint32_t e) {
  switch (e) {
  case CUBLASLT_EPILOGUE_DEFAULT: case CUBLASLT_EPILOGUE_RELU: case CUBLASLT_EPILOGUE_BIAS:
  case CUBLASLT_EPILOGUE_RELU_BIAS: case CUBLASLT_EPILOGUE_GELU: case CUBLASLT_EPILOGUE_GELU_BIAS:
  case CUBLASLT_EPILOGUE_BGRADA: case CUBLASLT_EPILOGUE_BGRADB:
  case CUBLASLT_EPILOGUE_GELU_AUX: case CUBLASLT_EPILOGUE_GELU_AUX_BIAS:
  case CUBLASLT_EPILOGUE_DGELU: case CUBLASLT_EPILOGUE_DGELU_BGRAD:
    return true;  // (the set zluda_common/src/lib.rs:762-804 maps; the ReLU bit-mask forms are not in it)
  default: return false;
  }
}

cublasStatus_t desc_attr(MatmulDescObj *o, uint32_t attr, bool set, const void *in, void *out,
                         size_t size, size_t *written) {
  zluda_matmul_desc &d = o->d;
  switch (attr) {
  case CUBLASLT_MATMUL_DESC_COMPUTE_TYPE: {
    int32_t v = (int32_t)d.compute_type;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) d.compute_type = (uint32_t)v;
    return st;
  }
  case CUBLASLT_MATMUL_DESC_SCALE_TYPE: {
    // zluda_blaslt/src/impl.rs:263-272 accepts only CUDA_R_32F; integer scaling (alpha, beta
    // int32 with COMPUTE_32I) is part of the int8 -> int32 contract and is accepted too.
    int32_t v = (int32_t)d.scale_type;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) {
      if (v != (int32_t)CUDA_R_32F && v != (int32_t)CUDA_R_32I) return CUBLAS_STATUS_NOT_SUPPORTED;
      d.scale_type = (uint32_t)v;
    }
    return st;
  }
  case CUBLASLT_MATMUL_DESC_POINTER_MODE: {
    int32_t v = d.pointer_mode;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) {
      if (v < CUBLASLT_POINTER_MODE_HOST || v > CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST)
        return CUBLAS_STATUS_INVALID_VALUE;
      d.pointer_mode = v;
    }
    return st;
  }
  case CUBLASLT_MATMUL_DESC_TRANSA:
  case CUBLASLT_MATMUL_DESC_TRANSB: {
    uint32_t &t = attr == CUBLASLT_MATMUL_DESC_TRANSA ? d.transa : d.transb;
    int32_t v = (int32_t)t;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) {
      // zluda_common/src/lib.rs:751-760: N, T, C only
      if (v < 0 || v > (int32_t)CUBLAS_OP_C) return CUBLAS_STATUS_INVALID_VALUE;
      t = (uint32_t)v;
    }
    return st;
  }
  case CUBLASLT_MATMUL_DESC_TRANSC: {
    int32_t v = 0;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st && v != 0) return CUBLAS_STATUS_NOT_SUPPORTED;
    return st;
  }
  case CUBLASLT_MATMUL_DESC_EPILOGUE: {
    uint32_t v = d.epilogue;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) {
      if (!epilogue_supported(v)) return CUBLAS_STATUS_NOT_SUPPORTED;
      d.epilogue = v;
    }
    return st;
  }
  case CUBLASLT_MATMUL_DESC_BIAS_POINTER: return access(set, d.bias, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_BIAS_BATCH_STRIDE: return access(set, d.bias_batch_stride, in, out, size, written);
  // (the reference maps these ids, zluda_common/src/lib.rs:664-674, but its set-attribute refuses them,
  // zluda_blaslt/src/impl.rs:302: the GELU_AUX / DGELU epilogues it forwards cannot be used through it)
  case CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_POINTER: return access(set, d.epilogue_aux, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_LD: return access(set, d.epilogue_aux_ld, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_BATCH_STRIDE: return access(set, d.epilogue_aux_batch_stride, in, out, size, written);
  // -1 or D's own type (what frameworks that set it pass for 16-bit outputs); which of the two it is can only be told
  // once D's layout is known, so the value is kept and the problem refused when it is lowered (planner.cpp)
  case CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_DATA_TYPE: return access(set, d.epilogue_aux_type, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_ALPHA_VECTOR_BATCH_STRIDE:
    return access(set, d.alpha_vector_batch_stride, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_SM_COUNT_TARGET: return access(set, o->sm_count_target, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_A_SCALE_POINTER: return access(set, d.a_scale, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_B_SCALE_POINTER: return access(set, d.b_scale, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_C_SCALE_POINTER: return access(set, d.c_scale, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_D_SCALE_POINTER: return access(set, d.d_scale, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_FAST_ACCUM: return access(set, d.fast_accum, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_BIAS_DATA_TYPE: return access(set, d.bias_type, in, out, size, written);
  case CUBLASLT_MATMUL_DESC_A_SCALE_MODE:
  case CUBLASLT_MATMUL_DESC_B_SCALE_MODE:
  case CUBLASLT_MATMUL_DESC_C_SCALE_MODE:
  case CUBLASLT_MATMUL_DESC_D_SCALE_MODE: {
    int32_t &m = attr == CUBLASLT_MATMUL_DESC_A_SCALE_MODE   ? d.a_scale_mode
                 : attr == CUBLASLT_MATMUL_DESC_B_SCALE_MODE ? d.b_scale_mode
                 : attr == CUBLASLT_MATMUL_DESC_C_SCALE_MODE ? d.c_scale_mode
                                                             : d.d_scale_mode;
    int32_t v = m;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) {
      const bool ab = attr == CUBLASLT_MATMUL_DESC_A_SCALE_MODE || attr == CUBLASLT_MATMUL_DESC_B_SCALE_MODE;
      const bool ok = v == CUBLASLT_MATMUL_MATRIX_SCALE_SCALAR_32F ||
                      (ab && (v == CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0 ||
                              v == CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F));
      if (!ok) return CUBLAS_STATUS_NOT_SUPPORTED;
      m = v;
    }
    return st;
  }
  default: return CUBLAS_STATUS_NOT_SUPPORTED;  // zluda_blaslt/src/impl.rs:302
  }
}

cublasStatus_t layout_attr(LayoutObj *o, uint32_t attr, bool set, const void *in, void *out,
                           size_t size, size_t *written) {
  zluda_matrix_layout &l = o->l;
  switch (attr) {
  case CUBLASLT_MATRIX_LAYOUT_TYPE: return access(set, l.type, in, out, size, written);
  case CUBLASLT_MATRIX_LAYOUT_ORDER: {
    int32_t v = l.order;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) {
      if (v != CUBLASLT_ORDER_COL && v != CUBLASLT_ORDER_ROW) return CUBLAS_STATUS_NOT_SUPPORTED;
      l.order = v;
    }
    return st;
  }
  case CUBLASLT_MATRIX_LAYOUT_ROWS: return access(set, l.rows, in, out, size, written);
  case CUBLASLT_MATRIX_LAYOUT_COLS: return access(set, l.cols, in, out, size, written);
  case CUBLASLT_MATRIX_LAYOUT_LD: return access(set, l.ld, in, out, size, written);
  case CUBLASLT_MATRIX_LAYOUT_BATCH_COUNT: {
    int32_t v = l.batch_count;
    cublasStatus_t st = access(set, v, in, out, size, written);
    if (set && !st) {
      if (v < 1) return CUBLAS_STATUS_INVALID_VALUE;
      l.batch_count = v;
    }
    return st;
  }
  case CUBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET: return access(set, l.batch_stride, in, out, size, written);
  default: return CUBLAS_STATUS_NOT_SUPPORTED;  // zluda_common/src/lib.rs:687-716
  }
}

cublasStatus_t pref_attr(PrefObj *o, uint32_t attr, bool set, const void *in, void *out,
                         size_t size, size_t *written) {
  switch (attr) {
  case CUBLASLT_MATMUL_PREF_SEARCH_MODE: return access(set, o->search_mode, in, out, size, written);
  case CUBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES: return access(set, o->max_workspace, in, out, size, written);
  // zluda_blaslt/src/impl.rs:346-353: the alignment hints are accepted (and remembered)
  case CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_A_BYTES: return access(set, o->min_align[0], in, out, size, written);
  case CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_B_BYTES: return access(set, o->min_align[1], in, out, size, written);
  case CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_C_BYTES: return access(set, o->min_align[2], in, out, size, written);
  case CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_D_BYTES: return access(set, o->min_align[3], in, out, size, written);
  case CUBLASLT_MATMUL_PREF_REDUCTION_SCHEME_MASK: return access(set, o->reduction_mask, in, out, size, written);
  case CUBLASLT_MATMUL_PREF_MAX_WAVES_COUNT: return access(set, o->max_waves, in, out, size, written);
  case CUBLASLT_MATMUL_PREF_IMPL_MASK: return access(set, o->impl_mask, in, out, size, written);
  default: return CUBLAS_STATUS_NOT_SUPPORTED;  // zluda_common/src/lib.rs:718-732
  }
}

// Initial contents of the three descriptor kinds.  They hold no pointers of their own, so they may
// live on the heap (Create) or in the caller's opaque storage (Init_internal: 256 bytes for a matmul
// descriptor, 64 for a layout or a preference, cuda_types/src/cublaslt.rs:43-83).
void init_layout(LayoutObj *o, cudaDataType_t type, uint64_t rows, uint64_t cols, int64_t ld) {
  o->magic = LAYOUT_MAGIC;
  o->l = zluda_matrix_layout{type, CUBLASLT_ORDER_COL, rows, cols, ld, 1, 0};
}
void init_desc(MatmulDescObj *o, cublasComputeType_t computeType, cudaDataType_t scaleType) {
  memset(o, 0, sizeof(*o));
  o->magic = DESC_MAGIC;
  o->d.compute_type = computeType;
  o->d.scale_type = scaleType;
  o->d.pointer_mode = CUBLASLT_POINTER_MODE_HOST;
  o->d.transa = o->d.transb = CUBLAS_OP_N;
  o->d.epilogue = CUBLASLT_EPILOGUE_DEFAULT;
  o->d.bias_type = -1;
  o->d.epilogue_aux_type = -1;
}
void init_pref(PrefObj *o) {
  memset(o, 0, sizeof(*o));
  o->magic = PREF_MAGIC;
  for (uint32_t &a : o->min_align) a = 256;
}
static_assert(sizeof(MatmulDescObj) <= 256 && alignof(MatmulDescObj) <= 8, "fits cublasLtMatmulDescOpaque_t");
static_assert(sizeof(LayoutObj) <= 64 && alignof(LayoutObj) <= 8, "fits cublasLtMatrixLayoutOpaque_t");
static_assert(sizeof(PrefObj) <= 64 && alignof(PrefObj) <= 8, "fits cublasLtMatmulPreferenceOpaque_t");

// descriptors -> problem.  Cdesc may be NULL (= Ddesc).
cublasStatus_t build_problem(cublasLtMatmulDesc_t op, cublasLtMatrixLayout_t A, cublasLtMatrixLayout_t B,
                             cublasLtMatrixLayout_t C, cublasLtMatrixLayout_t D, zluda_gemm_problem *p) {
  MatmulDescObj *o = as_desc(op);
  LayoutObj *a = as_layout(A), *b = as_layout(B), *d = as_layout(D);
  LayoutObj *c = C ? as_layout(C) : d;
  if (!o || !a || !b || !c || !d) return CUBLAS_STATUS_INVALID_VALUE;
  memset(p, 0, sizeof(*p));
  p->op = o->d;
  p->a = a->l; p->b = b->l; p->c = c->l; p->d = d->l;
  return CUBLAS_STATUS_SUCCESS;
}

void pack_algo(const zluda_gemm_plan &plan, cublasLtMatmulAlgo_t *algo) {
  memset(algo, 0, sizeof(*algo));
  algo->data[0] = ((uint64_t)ZLUDA_ALGO_MAGIC << 32) | plan.kernel;
  algo->data[1] = plan.variant;
  algo->data[2] = plan.workspace;
}
bool unpack_algo(const cublasLtMatmulAlgo_t *algo, uint32_t *kernel, int32_t *variant) {
  if ((algo->data[0] >> 32) != ZLUDA_ALGO_MAGIC) return false;
  *kernel = (uint32_t)(algo->data[0] & 0xffffffffu);
  *variant = (int32_t)algo->data[1];
  return *kernel >= ZLUDA_KERNEL_GENERIC && *kernel <= ZLUDA_KERNEL_MFMA_TR32;
}

// A/B forcing for measurements: ZLUDA_FORCE_KERNEL=<family>[:<variant>], read once per process (the
// first call that needs it), never on the per-call path afterwards
void env_force(uint32_t *kernel, int32_t *variant) {
  struct Forced { bool on; uint32_t kernel; int32_t variant; };
  static const Forced f = [] {
    Forced r{false, 0, -1};
    const char *e = getenv("ZLUDA_FORCE_KERNEL");
    if (e && *e) {
      r.on = true;
      r.kernel = (uint32_t)atoi(e);
      const char *c = strchr(e, ':');
      r.variant = c ? atoi(c + 1) : -1;
    }
    return r;
  }();
  if (!f.on) return;
  *kernel = f.kernel;
  *variant = f.variant;
}

} // namespace

extern "C" {

cublasStatus_t cublasLtCreate(cublasLtHandle_t *lightHandle) {
  if (!lightHandle) return CUBLAS_STATUS_INVALID_VALUE;
  LtHandle *h = new (std::nothrow) LtHandle{ZLUDA_BLASLT_HANDLE_COOKIE, 0};
  if (!h) return CUBLAS_STATUS_ALLOC_FAILED;
  *lightHandle = reinterpret_cast<cublasLtHandle_t>(h);
  return CUBLAS_STATUS_SUCCESS;
}

cublasStatus_t cublasLtDestroy(cublasLtHandle_t lightHandle) {
  if (!lightHandle) return CUBLAS_STATUS_INVALID_VALUE;
  LtHandle *lt = reinterpret_cast<LtHandle *>(lightHandle);
  if (lt->cookie != ZLUDA_BLASLT_HANDLE_COOKIE) {
    // zluda_blaslt/src/impl.rs:140-145: a cuBLAS handle: destroy its embedded Lt handle
    BlasHandleView *bh = reinterpret_cast<BlasHandleView *>(lightHandle);
    if (bh->cookie != ZLUDA_BLAS_HANDLE_COOKIE || !bh->blas_lt) return CUBLAS_STATUS_INVALID_VALUE;
    lt = reinterpret_cast<LtHandle *>(bh->blas_lt);
    if (lt->cookie != ZLUDA_BLASLT_HANDLE_COOKIE) return CUBLAS_STATUS_INVALID_VALUE;
  }
  // The cookie is cleared so that a second destroy (zluda_blas/src/impl.rs:551-559) or a stale
  // handle is reported as INVALID_VALUE; the 16-byte box itself stays allocated, which keeps that
  // check from reading freed memory.
  lt->cookie = 0;
  return CUBLAS_STATUS_SUCCESS;
}

const char *cublasLtGetStatusName(cublasStatus_t status) {
  switch (status) {
  case CUBLAS_STATUS_SUCCESS: return "CUBLAS_STATUS_SUCCESS";
  case CUBLAS_STATUS_NOT_INITIALIZED: return "CUBLAS_STATUS_NOT_INITIALIZED";
  case CUBLAS_STATUS_ALLOC_FAILED: return "CUBLAS_STATUS_ALLOC_FAILED";
  case CUBLAS_STATUS_INVALID_VALUE: return "CUBLAS_STATUS_INVALID_VALUE";
  case CUBLAS_STATUS_ARCH_MISMATCH: return "CUBLAS_STATUS_ARCH_MISMATCH";
  case CUBLAS_STATUS_MAPPING_ERROR: return "CUBLAS_STATUS_MAPPING_ERROR";
  case CUBLAS_STATUS_EXECUTION_FAILED: return "CUBLAS_STATUS_EXECUTION_FAILED";
  case CUBLAS_STATUS_INTERNAL_ERROR: return "CUBLAS_STATUS_INTERNAL_ERROR";
  case CUBLAS_STATUS_NOT_SUPPORTED: return "CUBLAS_STATUS_NOT_SUPPORTED";
  case CUBLAS_STATUS_LICENSE_ERROR: return "CUBLAS_STATUS_LICENSE_ERROR";
  default: return "CUBLAS_STATUS_UNKNOWN";
  }
}
const char *cublasLtGetStatusString(cublasStatus_t status) { return cublasLtGetStatusName(status); }

size_t cublasLtGetVersion(void) { return ZLUDA_CUBLAS_VERSION; }
size_t cublasLtGetCudartVersion(void) { return 13000; }
unsigned cublasLtDisableCpuInstructionsSetMask(unsigned mask) {
  static std::atomic<unsigned> cur{0};
  return cur.exchange(mask);
}
cublasStatus_t cublasLtGetProperty(libraryPropertyType type, int *value) {
  if (!value) return CUBLAS_STATUS_INVALID_VALUE;
  switch (type) {  // MAJOR_VERSION, MINOR_VERSION, PATCH_LEVEL
  case 0: *value = ZLUDA_CUBLAS_VERSION / 10000; return CUBLAS_STATUS_SUCCESS;
  case 1: *value = (ZLUDA_CUBLAS_VERSION / 100) % 100; return CUBLAS_STATUS_SUCCESS;
  case 2: *value = ZLUDA_CUBLAS_VERSION % 100; return CUBLAS_STATUS_SUCCESS;
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
}
cublasStatus_t cublasLtHeuristicsCacheGetCapacity(size_t *) { return CUBLAS_STATUS_NOT_SUPPORTED; }
cublasStatus_t cublasLtHeuristicsCacheSetCapacity(size_t) { return CUBLAS_STATUS_NOT_SUPPORTED; }

// ---- matrix layout -----------------------------------------------------------------------------
cublasStatus_t cublasLtMatrixLayoutCreate(cublasLtMatrixLayout_t *matLayout, cudaDataType_t type,
                                          uint64_t rows, uint64_t cols, int64_t ld) {
  if (!matLayout) return CUBLAS_STATUS_INVALID_VALUE;
  LayoutObj *o = new (std::nothrow) LayoutObj();
  if (!o) return CUBLAS_STATUS_ALLOC_FAILED;
  init_layout(o, type, rows, cols, ld);
  *matLayout = reinterpret_cast<cublasLtMatrixLayout_t>(o);
  return CUBLAS_STATUS_SUCCESS;
}
cublasStatus_t cublasLtMatrixLayoutDestroy(cublasLtMatrixLayout_t matLayout) {
  LayoutObj *o = as_layout(matLayout);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  o->magic = 0;
  delete o;
  return CUBLAS_STATUS_SUCCESS;
}
cublasStatus_t cublasLtMatrixLayoutSetAttribute(cublasLtMatrixLayout_t matLayout,
                                                cublasLtMatrixLayoutAttribute_t attr,
                                                const void *buf, size_t sizeInBytes) {
  LayoutObj *o = as_layout(matLayout);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  return layout_attr(o, attr, true, buf, nullptr, sizeInBytes, nullptr);
}
cublasStatus_t cublasLtMatrixLayoutGetAttribute(cublasLtMatrixLayout_t matLayout,
                                                cublasLtMatrixLayoutAttribute_t attr, void *buf,
                                                size_t sizeInBytes, size_t *sizeWritten) {
  LayoutObj *o = as_layout(matLayout);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  return layout_attr(o, attr, false, nullptr, buf, sizeInBytes, sizeWritten);
}
// what the cublasLtMatrixLayoutInit() inline of the CUDA header calls with the caller's own storage
cublasStatus_t cublasLtMatrixLayoutInit_internal(cublasLtMatrixLayout_t matLayout, size_t size,
                                                 cudaDataType_t type, uint64_t rows, uint64_t cols,
                                                 int64_t ld) {
  if (!matLayout || size < sizeof(LayoutObj)) return CUBLAS_STATUS_INVALID_VALUE;
  init_layout(reinterpret_cast<LayoutObj *>(matLayout), type, rows, cols, ld);
  return CUBLAS_STATUS_SUCCESS;
}

// ---- matmul descriptor -----------------------------------------------------------------------
cublasStatus_t cublasLtMatmulDescCreate(cublasLtMatmulDesc_t *matmulDesc,
                                        cublasComputeType_t computeType, cudaDataType_t scaleType) {
  if (!matmulDesc) return CUBLAS_STATUS_INVALID_VALUE;
  MatmulDescObj *o = new (std::nothrow) MatmulDescObj();
  if (!o) return CUBLAS_STATUS_ALLOC_FAILED;
  init_desc(o, computeType, scaleType);
  *matmulDesc = reinterpret_cast<cublasLtMatmulDesc_t>(o);
  return CUBLAS_STATUS_SUCCESS;
}
cublasStatus_t cublasLtMatmulDescDestroy(cublasLtMatmulDesc_t matmulDesc) {
  MatmulDescObj *o = as_desc(matmulDesc);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  o->magic = 0;
  delete o;
  return CUBLAS_STATUS_SUCCESS;
}
cublasStatus_t cublasLtMatmulDescSetAttribute(cublasLtMatmulDesc_t matmulDesc,
                                              cublasLtMatmulDescAttributes_t attr, const void *buf,
                                              size_t sizeInBytes) {
  MatmulDescObj *o = as_desc(matmulDesc);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  return desc_attr(o, attr, true, buf, nullptr, sizeInBytes, nullptr);
}
cublasStatus_t cublasLtMatmulDescGetAttribute(cublasLtMatmulDesc_t matmulDesc,
                                              cublasLtMatmulDescAttributes_t attr, void *buf,
                                              size_t sizeInBytes, size_t *sizeWritten) {
  MatmulDescObj *o = as_desc(matmulDesc);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  return desc_attr(o, attr, false, nullptr, buf, sizeInBytes, sizeWritten);
}
cublasStatus_t cublasLtMatmulDescInit_internal(cublasLtMatmulDesc_t matmulDesc, size_t size,
                                               cublasComputeType_t computeType, cudaDataType_t scaleType) {
  if (!matmulDesc || size < sizeof(MatmulDescObj)) return CUBLAS_STATUS_INVALID_VALUE;
  init_desc(reinterpret_cast<MatmulDescObj *>(matmulDesc), computeType, scaleType);
  return CUBLAS_STATUS_SUCCESS;
}

// ---- preference ----------------------------------------------------------------------------------
cublasStatus_t cublasLtMatmulPreferenceCreate(cublasLtMatmulPreference_t *pref) {
  if (!pref) return CUBLAS_STATUS_INVALID_VALUE;
  PrefObj *o = new (std::nothrow) PrefObj();
  if (!o) return CUBLAS_STATUS_ALLOC_FAILED;
  init_pref(o);
  *pref = reinterpret_cast<cublasLtMatmulPreference_t>(o);
  return CUBLAS_STATUS_SUCCESS;
}
cublasStatus_t cublasLtMatmulPreferenceDestroy(cublasLtMatmulPreference_t pref) {
  PrefObj *o = as_pref(pref);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  o->magic = 0;
  delete o;
  return CUBLAS_STATUS_SUCCESS;
}
cublasStatus_t cublasLtMatmulPreferenceSetAttribute(cublasLtMatmulPreference_t pref,
                                                    cublasLtMatmulPreferenceAttributes_t attr,
                                                    const void *buf, size_t sizeInBytes) {
  PrefObj *o = as_pref(pref);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  return pref_attr(o, attr, true, buf, nullptr, sizeInBytes, nullptr);
}
cublasStatus_t cublasLtMatmulPreferenceGetAttribute(cublasLtMatmulPreference_t pref,
                                                    cublasLtMatmulPreferenceAttributes_t attr,
                                                    void *buf, size_t sizeInBytes, size_t *sizeWritten) {
  PrefObj *o = as_pref(pref);
  if (!o) return CUBLAS_STATUS_INVALID_VALUE;
  return pref_attr(o, attr, false, nullptr, buf, sizeInBytes, sizeWritten);
}
cublasStatus_t cublasLtMatmulPreferenceInit_internal(cublasLtMatmulPreference_t pref, size_t size) {
  if (!pref || size < sizeof(PrefObj)) return CUBLAS_STATUS_INVALID_VALUE;
  init_pref(reinterpret_cast<PrefObj *>(pref));
  return CUBLAS_STATUS_SUCCESS;
}

// ---- heuristic and matmul ----------------------------------------------------------------------
cublasStatus_t cublasLtMatmulAlgoGetHeuristic(
    cublasLtHandle_t lightHandle, cublasLtMatmulDesc_t operationDesc, cublasLtMatrixLayout_t Adesc,
    cublasLtMatrixLayout_t Bdesc, cublasLtMatrixLayout_t Cdesc, cublasLtMatrixLayout_t Ddesc,
    cublasLtMatmulPreference_t preference, int requestedAlgoCount,
    cublasLtMatmulHeuristicResult_t *heuristicResultsArray, int *returnAlgoCount) {
  if (!resolve_handle(lightHandle)) return CUBLAS_STATUS_INVALID_VALUE;
  if (!heuristicResultsArray || !returnAlgoCount || requestedAlgoCount < 1) return CUBLAS_STATUS_INVALID_VALUE;
  PrefObj *pref = as_pref(preference);
  if (!pref) return CUBLAS_STATUS_INVALID_VALUE;
  zluda_gemm_problem p;
  cublasStatus_t st = build_problem(operationDesc, Adesc, Bdesc, Cdesc, Ddesc, &p);
  if (st) return st;
  *returnAlgoCount = 0;
  p.workspace_size = pref->max_workspace;  // what split-K may count on
  const uint32_t cus = zluda_gemm_device_cu_count();
  // candidates, best first: the planner's own choice, then the generic kernel
  uint32_t forced = ZLUDA_KERNEL_AUTO;
  int32_t forced_variant = -1;
  env_force(&forced, &forced_variant);
  const uint32_t families[2] = {forced, ZLUDA_KERNEL_GENERIC};
  uint32_t first_kernel = 0;
  cublasStatus_t last = CUBLAS_STATUS_NOT_SUPPORTED;
  for (int c = 0; c < 2 && *returnAlgoCount < requestedAlgoCount; c++) {
    zluda_gemm_plan plan;
    st = zluda_gemm_plan_problem(&p, families[c], c == 0 ? forced_variant : -1, cus, &plan);
    if (st) { last = st; continue; }
    if (c == 1 && plan.kernel == first_kernel) continue;
    if (plan.workspace > pref->max_workspace) continue;
    cublasLtMatmulHeuristicResult_t *r = &heuristicResultsArray[*returnAlgoCount];
    memset(r, 0, sizeof(*r));
    pack_algo(plan, &r->algo);
    r->workspaceSize = plan.workspace;
    r->state = CUBLAS_STATUS_SUCCESS;
    r->wavesCount = plan.waves;
    if (c == 0) first_kernel = plan.kernel;
    (*returnAlgoCount)++;
  }
  if (*returnAlgoCount == 0) return last == CUBLAS_STATUS_SUCCESS ? CUBLAS_STATUS_NOT_SUPPORTED : last;
  return CUBLAS_STATUS_SUCCESS;
}

cublasStatus_t cublasLtMatmulAlgoCheck(cublasLtHandle_t lightHandle, cublasLtMatmulDesc_t operationDesc,
                                       cublasLtMatrixLayout_t Adesc, cublasLtMatrixLayout_t Bdesc,
                                       cublasLtMatrixLayout_t Cdesc, cublasLtMatrixLayout_t Ddesc,
                                       const cublasLtMatmulAlgo_t *algo,
                                       cublasLtMatmulHeuristicResult_t *result) {
  if (!resolve_handle(lightHandle) || !algo || !result) return CUBLAS_STATUS_INVALID_VALUE;
  zluda_gemm_problem p;
  cublasStatus_t st = build_problem(operationDesc, Adesc, Bdesc, Cdesc, Ddesc, &p);
  if (st) return st;
  uint32_t kernel;
  int32_t variant;
  if (!unpack_algo(algo, &kernel, &variant)) return CUBLAS_STATUS_INVALID_VALUE;
  zluda_gemm_plan plan;
  st = zluda_gemm_plan_problem(&p, kernel, variant, zluda_gemm_device_cu_count(), &plan);
  if (st) return st;
  memset(result, 0, sizeof(*result));
  pack_algo(plan, &result->algo);
  result->workspaceSize = plan.workspace;
  result->state = CUBLAS_STATUS_SUCCESS;
  result->wavesCount = plan.waves;
  return CUBLAS_STATUS_SUCCESS;
}

cublasStatus_t cublasLtMatmul(cublasLtHandle_t lightHandle, cublasLtMatmulDesc_t computeDesc,
                              const void *alpha, const void *A, cublasLtMatrixLayout_t Adesc,
                              const void *B, cublasLtMatrixLayout_t Bdesc, const void *beta,
                              const void *C, cublasLtMatrixLayout_t Cdesc, void *D,
                              cublasLtMatrixLayout_t Ddesc, const cublasLtMatmulAlgo_t *algo,
                              void *workspace, size_t workspaceSizeInBytes, cudaStream_t stream) {
  if (!resolve_handle(lightHandle)) return CUBLAS_STATUS_INVALID_VALUE;
  zluda_gemm_problem p;
  cublasStatus_t st = build_problem(computeDesc, Adesc, Bdesc, Cdesc, Ddesc, &p);
  if (st) return st;
  p.alpha = alpha; p.beta = beta;
  p.A = A; p.B = B; p.C = C; p.D = D;
  p.workspace = workspace; p.workspace_size = workspaceSizeInBytes;
  // split-K needs 16-byte aligned scratch: without it the problem is planned unsplit instead of refused
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15)) { p.workspace = nullptr; p.workspace_size = 0; }

  uint32_t kernel = ZLUDA_KERNEL_AUTO;
  int32_t variant = -1;
  if (algo) {
    if (!unpack_algo(algo, &kernel, &variant)) return CUBLAS_STATUS_INVALID_VALUE;
  } else {
    env_force(&kernel, &variant);  // algo == NULL: the library's own first choice
  }
  const uint32_t cus = zluda_gemm_device_cu_count();
  if (cus == 0) return CUBLAS_STATUS_NOT_INITIALIZED;  // no usable HIP device: there is no CPU path
  zluda_gemm_plan plan;
  st = zluda_gemm_plan_problem(&p, kernel, variant, cus, &plan);
  if (st == CUBLAS_STATUS_NOT_SUPPORTED && kernel != ZLUDA_KERNEL_AUTO && kernel != ZLUDA_KERNEL_GENERIC) {
    // The algo was chosen from the descriptors alone (the heuristic assumes the MIN_ALIGNMENT_*
    // preferences hold); the real pointers do not qualify for it.  Run the layout-agnostic kernel
    // rather than failing the call.
    st = zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_GENERIC, -1, cus, &plan);
  }
  if (st) return st;
  st = zluda_gemm_launch(&p, &plan, stream);
  return st;
}

// ---- not supported, exactly like the reference's release build (zluda_blaslt/src/impl.rs:83-86) ----
cublasStatus_t cublasLtMatrixTransform(cublasLtHandle_t, cublasLtMatrixTransformDesc_t, const void *,
                                       const void *, cublasLtMatrixLayout_t, const void *,
                                       const void *, cublasLtMatrixLayout_t, void *,
                                       cublasLtMatrixLayout_t, cudaStream_t) {
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
cublasStatus_t cublasLtMatrixTransformDescInit_internal(cublasLtMatrixTransformDesc_t, size_t, cudaDataType_t) {
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
cublasStatus_t cublasLtMatrixTransformDescCreate(cublasLtMatrixTransformDesc_t *, cudaDataType_t) {
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
cublasStatus_t cublasLtMatrixTransformDescDestroy(cublasLtMatrixTransformDesc_t) {
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
cublasStatus_t cublasLtMatrixTransformDescSetAttribute(cublasLtMatrixTransformDesc_t,
                                                       cublasLtMatrixTransformDescAttributes_t,
                                                       const void *, size_t) {
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
cublasStatus_t cublasLtMatrixTransformDescGetAttribute(cublasLtMatrixTransformDesc_t,
                                                       cublasLtMatrixTransformDescAttributes_t, void *,
                                                       size_t, size_t *) {
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
// ---- algorithm enumeration (cuda_macros/src/cublaslt.rs:397-518; `unimplemented` in the reference) ----
// An algorithm id is a kernel family (ZLUDA_KERNEL_*); its one tunable, the tile variant, is exposed
// as CUBLASLT_ALGO_CONFIG_CUSTOM_OPTION (0 = let the planner choose, v + 1 = variant v).

// the families that can run a type combination at all (layouts decide the rest at AlgoCheck time)
static int families_for_types(uint32_t computeType, uint32_t scaleType, uint32_t A, uint32_t B, uint32_t C,
                              uint32_t D, int *ids) {
  zluda_gemm_problem p;
  memset(&p, 0, sizeof(p));
  p.op.compute_type = computeType; p.op.scale_type = scaleType; p.op.bias_type = -1; p.op.epilogue_aux_type = -1;
  p.op.transa = CUBLAS_OP_T; p.op.transb = CUBLAS_OP_N; p.op.epilogue = CUBLASLT_EPILOGUE_DEFAULT;
  const uint64_t n = 1024;
  p.a = {A, CUBLASLT_ORDER_COL, n, n, (int64_t)n, 1, (int64_t)(n * n)};
  p.b = {B, CUBLASLT_ORDER_COL, n, n, (int64_t)n, 1, (int64_t)(n * n)};
  p.c = {C, CUBLASLT_ORDER_COL, n, n, (int64_t)n, 1, (int64_t)(n * n)};
  p.d = {D, CUBLASLT_ORDER_COL, n, n, (int64_t)n, 1, (int64_t)(n * n)};
  if (A == CUDA_R_4F_E2M1) p.op.a_scale_mode = p.op.b_scale_mode = CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0;
  int count = 0;
  zluda_gemm_plan plan;
  // 1024^3 A:T B:N admits every square-GEMM family; the decode family wants a skinny shape
  for (uint32_t k = ZLUDA_KERNEL_GENERIC; k <= ZLUDA_KERNEL_MFMA_MXF4; k++)
    if (zluda_gemm_plan_problem(&p, k, -1, 256, &plan) == CUBLAS_STATUS_SUCCESS) ids[count++] = (int)k;
  if (zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_MFMA_H16, -1, 256, &plan) == CUBLAS_STATUS_SUCCESS)
    ids[count++] = ZLUDA_KERNEL_MFMA_H16;
  if (zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_MFMA_F32, -1, 256, &plan) == CUBLAS_STATUS_SUCCESS)
    ids[count++] = ZLUDA_KERNEL_MFMA_F32;
  p.b.cols = p.c.cols = p.d.cols = 16;
  if (zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_DECODE_W8A8, -1, 256, &plan) == CUBLAS_STATUS_SUCCESS)
    ids[count++] = ZLUDA_KERNEL_DECODE_W8A8;
  // the transposing kernels are what runs the layouts with A or B not K-contiguous
  p.b.cols = p.c.cols = p.d.cols = n;
  p.op.transa = CUBLAS_OP_N;
  if (zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_MFMA_TR8, -1, 256, &plan) == CUBLAS_STATUS_SUCCESS)
    ids[count++] = ZLUDA_KERNEL_MFMA_TR8;
  if (zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_MFMA_TR16, -1, 256, &plan) == CUBLAS_STATUS_SUCCESS)
    ids[count++] = ZLUDA_KERNEL_MFMA_TR16;
  if (zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_MFMA_TR32, -1, 256, &plan) == CUBLAS_STATUS_SUCCESS)
    ids[count++] = ZLUDA_KERNEL_MFMA_TR32;
  return count;
}

cublasStatus_t cublasLtMatmulAlgoGetIds(cublasLtHandle_t lightHandle, cublasComputeType_t computeType,
                                        cudaDataType_t scaleType, cudaDataType_t Atype, cudaDataType_t Btype,
                                        cudaDataType_t Ctype, cudaDataType_t Dtype, int requestedAlgoCount,
                                        int *algoIdsArray, int *returnAlgoCount) {
  if (!resolve_handle(lightHandle) || !algoIdsArray || !returnAlgoCount || requestedAlgoCount < 0)
    return CUBLAS_STATUS_INVALID_VALUE;
  int ids[8];
  const int n = families_for_types(computeType, scaleType, Atype, Btype, Ctype, Dtype, ids);
  *returnAlgoCount = n < requestedAlgoCount ? n : requestedAlgoCount;
  for (int i = 0; i < *returnAlgoCount; i++) algoIdsArray[i] = ids[i];
  return CUBLAS_STATUS_SUCCESS;
}

cublasStatus_t cublasLtMatmulAlgoInit(cublasLtHandle_t lightHandle, cublasComputeType_t computeType,
                                      cudaDataType_t scaleType, cudaDataType_t Atype, cudaDataType_t Btype,
                                      cudaDataType_t Ctype, cudaDataType_t Dtype, int algoId,
                                      cublasLtMatmulAlgo_t *algo) {
  if (!resolve_handle(lightHandle) || !algo) return CUBLAS_STATUS_INVALID_VALUE;
  int ids[8];
  const int n = families_for_types(computeType, scaleType, Atype, Btype, Ctype, Dtype, ids);
  for (int i = 0; i < n; i++)
    if (ids[i] == algoId) {
      zluda_gemm_plan plan;
      memset(&plan, 0, sizeof(plan));
      plan.kernel = (uint32_t)algoId;
      plan.variant = (uint32_t)-1;  // planner's choice until CUSTOM_OPTION says otherwise
      pack_algo(plan, algo);
      return CUBLAS_STATUS_SUCCESS;
    }
  return CUBLAS_STATUS_INVALID_VALUE;  // "algoId is not a valid id for these types" in cuBLASLt's terms
}

static int variants_of(uint32_t kernel) { return (int)zluda_gemm_variant_count(kernel); }

cublasStatus_t cublasLtMatmulAlgoCapGetAttribute(const cublasLtMatmulAlgo_t *algo,
                                                 cublasLtMatmulAlgoCapAttributes_t attr, void *buf,
                                                 size_t sizeInBytes, size_t *sizeWritten) {
  uint32_t kernel;
  int32_t variant;
  if (!algo || !unpack_algo(algo, &kernel, &variant)) return CUBLAS_STATUS_INVALID_VALUE;
  int32_t i32 = 0;
  uint32_t u32 = 0;
  uint64_t u64 = 0;
  switch (attr) {
  case 0 /* SPLITK_SUPPORT */: i32 = 0; return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  case 1 /* REDUCTION_SCHEME_MASK */: u32 = 0; return access(false, u32, nullptr, buf, sizeInBytes, sizeWritten);
  case 2 /* CTA_SWIZZLING_SUPPORT */: u32 = 0; return access(false, u32, nullptr, buf, sizeInBytes, sizeWritten);
  case 3 /* STRIDED_BATCH_SUPPORT */: i32 = 1; return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  case 4 /* OUT_OF_PLACE_RESULT_SUPPORT */: i32 = 1; return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  case 5 /* UPLO_SUPPORT */: i32 = 0; return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  case 6 /* TILE_IDS */: case 13 /* STAGES_IDS */:
    u32 = 0;  // one entry, CUBLASLT_MATMUL_TILE_UNDEFINED / STAGES_UNDEFINED: tiles are chosen through CUSTOM_OPTION
    return access(false, u32, nullptr, buf, sizeInBytes, sizeWritten);
  case 7 /* CUSTOM_OPTION_MAX */: i32 = variants_of(kernel); return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  case 10 /* CUSTOM_MEMORY_ORDER */: i32 = 0; return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  case 11 /* POINTER_MODE_MASK */: u32 = 0x1f; return access(false, u32, nullptr, buf, sizeInBytes, sizeWritten);
  case 12 /* EPILOGUE_MASK */:
    u32 = CUBLASLT_EPILOGUE_DEFAULT | CUBLASLT_EPILOGUE_RELU | CUBLASLT_EPILOGUE_BIAS | CUBLASLT_EPILOGUE_GELU;
    return access(false, u32, nullptr, buf, sizeInBytes, sizeWritten);
  case 14 /* LD_NEGATIVE */: i32 = 0; return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  case 15 /* NUMERICAL_IMPL_FLAGS */: u64 = ~0ull; return access(false, u64, nullptr, buf, sizeInBytes, sizeWritten);
  case 16: case 17: /* MIN_ALIGNMENT_A/B_BYTES */
    u32 = kernel == ZLUDA_KERNEL_GENERIC ? 1 : (kernel == ZLUDA_KERNEL_MFMA_TR8 || kernel == ZLUDA_KERNEL_MFMA_TR16 || kernel == ZLUDA_KERNEL_MFMA_TR32 ? 4 : 16);
    return access(false, u32, nullptr, buf, sizeInBytes, sizeWritten);
  case 18: case 19: /* MIN_ALIGNMENT_C/D_BYTES */ u32 = 1; return access(false, u32, nullptr, buf, sizeInBytes, sizeWritten);
  case 21 /* POINTER_ARRAY_BATCH_SUPPORT */: case 22 /* FLOATING_POINT_EMULATION_SUPPORT */:
    i32 = 0;
    return access(false, i32, nullptr, buf, sizeInBytes, sizeWritten);
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
}

// CONFIG attributes: ID (read-only) and CUSTOM_OPTION carry information; the others only accept /
// report the one value this implementation has (no split-K, no swizzle option, undefined tile and
// stage ids, automatic inner and cluster shapes).
static cublasStatus_t algo_config(cublasLtMatmulAlgo_t *algo, uint32_t attr, bool set, const void *in, void *out,
                                  size_t size, size_t *written) {
  uint32_t kernel;
  int32_t variant;
  if (!algo || !unpack_algo(algo, &kernel, &variant)) return CUBLAS_STATUS_INVALID_VALUE;
  switch (attr) {
  case 0 /* ID */: {
    int32_t id = (int32_t)kernel;
    if (set) return CUBLAS_STATUS_INVALID_VALUE;
    return access(false, id, nullptr, out, size, written);
  }
  case 5 /* CUSTOM_OPTION */: {
    uint32_t opt = variant < 0 ? 0u : (uint32_t)variant + 1;
    cublasStatus_t st = access(set, opt, in, out, size, written);
    if (set && !st) {
      if ((int)opt > variants_of(kernel)) return CUBLAS_STATUS_INVALID_VALUE;
      algo->data[1] = opt == 0 ? (uint64_t)(uint32_t)-1 : opt - 1;
    }
    return st;
  }
  case 2 /* SPLITK_NUM */: {
    int32_t v = 1;
    cublasStatus_t st = access(set, v, in, out, size, written);
    return (set && !st && v != 1 && v != 0) ? CUBLAS_STATUS_NOT_SUPPORTED : st;
  }
  case 1 /* TILE_ID */: case 3 /* REDUCTION_SCHEME */: case 4 /* CTA_SWIZZLING */: case 6 /* STAGES_ID */: {
    uint32_t v = 0;
    cublasStatus_t st = access(set, v, in, out, size, written);
    return (set && !st && v != 0) ? CUBLAS_STATUS_NOT_SUPPORTED : st;
  }
  case 7 /* INNER_SHAPE_ID */: case 8 /* CLUSTER_SHAPE_ID */: {
    uint16_t v = 0;
    cublasStatus_t st = access(set, v, in, out, size, written);
    return (set && !st && v != 0) ? CUBLAS_STATUS_NOT_SUPPORTED : st;
  }
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
}

cublasStatus_t cublasLtMatmulAlgoConfigSetAttribute(cublasLtMatmulAlgo_t *algo,
                                                    cublasLtMatmulAlgoConfigAttributes_t attr, const void *buf,
                                                    size_t sizeInBytes) {
  if (!buf) return CUBLAS_STATUS_INVALID_VALUE;
  return algo_config(algo, attr, true, buf, nullptr, sizeInBytes, nullptr);
}
cublasStatus_t cublasLtMatmulAlgoConfigGetAttribute(const cublasLtMatmulAlgo_t *algo,
                                                    cublasLtMatmulAlgoConfigAttributes_t attr, void *buf,
                                                    size_t sizeInBytes, size_t *sizeWritten) {
  return algo_config(const_cast<cublasLtMatmulAlgo_t *>(algo), attr, false, nullptr, buf, sizeInBytes, sizeWritten);
}
cublasStatus_t cublasLtLoggerSetCallback(cublasLtLoggerCallback_t) { return CUBLAS_STATUS_NOT_SUPPORTED; }
cublasStatus_t cublasLtLoggerSetFile(FILE *) { return CUBLAS_STATUS_NOT_SUPPORTED; }
cublasStatus_t cublasLtLoggerOpenFile(const char *) { return CUBLAS_STATUS_NOT_SUPPORTED; }
cublasStatus_t cublasLtLoggerSetLevel(int) { return CUBLAS_STATUS_NOT_SUPPORTED; }
cublasStatus_t cublasLtLoggerSetMask(int) { return CUBLAS_STATUS_NOT_SUPPORTED; }
cublasStatus_t cublasLtLoggerForceDisable(void) { return CUBLAS_STATUS_NOT_SUPPORTED; }

} // extern "C"
