// The extern "C" launch layer: lowers a problem, picks the template instantiation the plan names
// and enqueues it on the caller's stream.  Only the HIP runtime is used (hipLaunchKernel).
#include <atomic>
#include <hip/hip_runtime.h>

#include <cstring>

#include "decode_launch.hpp"
#include "launch_util.hpp"
#include "kernels/aux_epilogue.hpp"
#include "kernels/bgrad_reduce.hpp"
#include "kernels/decode_w8a8.hpp"
#include "kernels/gemm_generic.hpp"
#include "kernels/splitk_reduce.hpp"
#include "mfma_launch.hpp"
#include "mfma_tr_launch.hpp"
#include "planner.hpp"

using namespace zluda_amd;

namespace zluda_amd {
uint32_t launch_decode_stream_i8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s) {
  return launch_decode_stream_variant<KIND_I8>(prm, plan, nb, s);
}
uint32_t launch_decode_slab_i8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s) {
  return launch_decode_slab<KIND_I8>(prm, plan, nb, s);
}
} // namespace zluda_amd

namespace {

inline int f8_fmt(uint32_t t) { return t == CUDA_R_8F_E5M2 ? 1 : 0; }

// `ws` / `ws_size`: the scratch that holds split-K partial tiles (the caller's workspace, or the library's own)
uint32_t launch_mfma(const Lowered &l, const zluda_gemm_plan &plan_in, void *ws, uint64_t ws_size, hipStream_t s) {
  MfmaParams prm;
  prm.g = l.g;
  if (plan_in.variant >= (uint32_t)kNumMfmaVariants) return CUBLAS_STATUS_INVALID_VALUE;
  zluda_gemm_plan plan = plan_in;
  if (kMfmaVariants[plan.variant].w4) {
    // The four-wave kernel carries three epilogues.  What the call turns out to ask for beyond them (a beta that is not
    // zero, a D that is not 16-byte aligned: known only now) runs on the eight-wave kernel with the same tile, which
    // needs no workspace either.
    const uint32_t cus = zluda_gemm_device_cu_count();
    const int epi = w4_epilogue_class(l, false);
    const int np = plan.swapped ? l.g.N : l.g.M, nq = plan.swapped ? l.g.M : l.g.N;
    const uint64_t all = (uint64_t)((np + 255) / 256) * ((nq + 255) / 256) * l.g.batch;
    if (epi != W4_CLASS_NONE) {
      const uint32_t slots = cus >= 8 ? cus / 8 * 8 : cus;
      if (plan.grid_x == 0 || plan.grid_x > all || plan.grid_x > slots || plan.grid_y != 1 || plan.grid_z > 1) return CUBLAS_STATUS_INVALID_VALUE;
      prm.swapped = plan.swapped;
      prm.tiles_p = (np + 255) / 256; prm.tiles_q = (nq + 255) / 256;
      prm.group_p = 8;
      prm.splits = 1; prm.split_stages = 0; prm.ws = nullptr;
      return plan.kernel == ZLUDA_KERNEL_MFMA_I8     ? launch_mfma_w4_i8(prm, epi, plan.grid_x, s)
             : plan.kernel == ZLUDA_KERNEL_MFMA_MXF4 ? launch_mfma_w4_mxf4(prm, epi, plan.grid_x, s)
             : plan.kernel == ZLUDA_KERNEL_MFMA_H16  ? (l.g.a_type == CUDA_R_16BF ? launch_mfma_w4_bf16(prm, epi, plan.grid_x, s)
                                                                                   : launch_mfma_w4_f16(prm, epi, plan.grid_x, s))
                                                     : launch_mfma_w4_f8(prm, epi, plan.grid_x, plan.swapped ? f8_fmt(l.g.a_type) : f8_fmt(l.g.b_type),
                                                                         plan.swapped ? f8_fmt(l.g.b_type) : f8_fmt(l.g.a_type), s);
    }
    plan.variant = plan.kernel == ZLUDA_KERNEL_MFMA_MXF4 ? 0 : 8;  // (MXFP4 has no 16x16 eight-wave form)
    plan.grid_x = (uint32_t)(all / l.g.batch); plan.grid_y = l.g.batch; plan.grid_z = 1;
    plan.block = 512;
    plan.workspace = 0;
  }
  prm.swapped = plan.swapped;
  const MfmaVariant &v = kMfmaVariants[plan.variant];
  const int np = plan.swapped ? l.g.N : l.g.M, nq = plan.swapped ? l.g.M : l.g.N;
  prm.tiles_p = (np + v.bp - 1) / v.bp;
  prm.tiles_q = (nq + v.bq - 1) / v.bq;
  prm.group_p = 8;
  prm.splits = 1; prm.split_stages = 0; prm.ws = nullptr;
  if ((uint32_t)(prm.tiles_p * prm.tiles_q) != plan.grid_x) return CUBLAS_STATUS_INVALID_VALUE;
  if (plan.grid_z > 1) {
    // split-K: partial tiles go through the caller's workspace
    const uint64_t need = (uint64_t)plan.grid_z * l.g.batch * prm.tiles_p * v.bp * prm.tiles_q * v.bq * 4;
    if (!ws || (((uintptr_t)ws) & 15) || ws_size < need || plan.workspace != need) return CUBLAS_STATUS_INVALID_VALUE;
    const bool mx = plan.kernel == ZLUDA_KERNEL_MFMA_MXF4;
    const int kbytes = mx ? l.g.K / 2 : (plan.kernel == ZLUDA_KERNEL_MFMA_H16 ? l.g.K * 2 : plan.kernel == ZLUDA_KERNEL_MFMA_F32 ? l.g.K * 4 : l.g.K);
    const int stages = (kbytes + v.bkb - 1) / v.bkb;
    prm.splits = (int32_t)plan.grid_z;
    prm.split_stages = (stages + prm.splits - 1) / prm.splits;
    if (mx) {  // whole scale chunks (32 scale bytes = 512 fp4 bytes per row) per share
      const int ch = 512 / v.bkb;
      prm.split_stages = (prm.split_stages + ch - 1) / ch * ch;
    }
    prm.ws = ws;
  }
  uint32_t st;
  switch (plan.kernel) {
  case ZLUDA_KERNEL_MFMA_I8: st = launch_mfma_i8(prm, plan, s); break;
  case ZLUDA_KERNEL_MFMA_MXF4: st = launch_mfma_mxf4(prm, plan, s); break;
  case ZLUDA_KERNEL_MFMA_H16: st = launch_mfma_h16(prm, plan, l.g.a_type == CUDA_R_16BF, s); break;
  case ZLUDA_KERNEL_MFMA_F32: st = launch_mfma_f32(prm, plan, s); break;
  case ZLUDA_KERNEL_MFMA_F8: {
    // MFMA operand "A" is Q, operand "B" is P (see gemm_mfma.hpp)
    const int fa = f8_fmt(l.g.a_type), fb = f8_fmt(l.g.b_type);
    st = launch_mfma_f8(prm, plan, plan.swapped ? fa : fb, plan.swapped ? fb : fa, s);
    break;
  }
  default: return CUBLAS_STATUS_INTERNAL_ERROR;
  }
  if (st || prm.splits == 1) return st;
  SplitKReduceParams rp;
  rp.g = l.g;
  rp.swapped = plan.swapped;
  rp.splits = prm.splits;
  rp.acc_is_int = plan.kernel == ZLUDA_KERNEL_MFMA_I8;
  rp.ws_np = prm.tiles_p * v.bp;
  rp.ws_nq = prm.tiles_q * v.bq;
  rp.ws = (const int32_t *)ws;
  return launch_kernel(splitk_reduce_kernel, dim3((np + 1023) / 1024, nq, l.g.batch), dim3(256), s, rp);
}

uint32_t launch_tr(const Lowered &l, const zluda_gemm_plan &plan, void *ws, uint64_t ws_size, hipStream_t s) {
  if (plan.variant >= (uint32_t)kNumTrVariants) return CUBLAS_STATUS_INVALID_VALUE;
  const TrVariant &v = kTrVariants[plan.variant];
  MfmaParams prm;
  prm.g = l.g;
  prm.swapped = plan.swapped;
  const int np = plan.swapped ? l.g.N : l.g.M, nq = plan.swapped ? l.g.M : l.g.N;
  prm.tiles_p = (np + v.bp - 1) / v.bp;
  prm.tiles_q = (nq + v.bq - 1) / v.bq;
  prm.group_p = 8;
  prm.splits = 1; prm.split_stages = 0; prm.ws = nullptr;
  if ((uint32_t)(prm.tiles_p * prm.tiles_q) != plan.grid_x) return CUBLAS_STATUS_INVALID_VALUE;
  if (plan.grid_z > 1) {
    // split-K: partial tiles go through the caller's workspace (64 K bytes per stage)
    const uint64_t need = (uint64_t)plan.grid_z * l.g.batch * prm.tiles_p * v.bp * prm.tiles_q * v.bq * 4;
    if (!ws || (((uintptr_t)ws) & 15) || ws_size < need || plan.workspace != need) return CUBLAS_STATUS_INVALID_VALUE;
    const int stages = (l.g.K * (plan.kernel == ZLUDA_KERNEL_MFMA_TR16 ? 2 : plan.kernel == ZLUDA_KERNEL_MFMA_TR32 ? 4 : 1) + 63) / 64;
    prm.splits = (int32_t)plan.grid_z;
    prm.split_stages = (stages + prm.splits - 1) / prm.splits;
    prm.ws = ws;
  }
  // P is op(A) for a column-major D, op(B)^T otherwise
  const bool pkc = plan.swapped ? l.b_kcontig : l.a_kcontig, qkc = plan.swapped ? l.a_kcontig : l.b_kcontig;
  uint32_t st;
  if (l.g.a_type == CUDA_R_8I) {
    st = launch_tr_i8(prm, plan, pkc, qkc, s);
  } else if (l.g.a_type == CUDA_R_16F) {
    st = launch_tr_f16(prm, plan, pkc, qkc, s);
  } else if (l.g.a_type == CUDA_R_16BF) {
    st = launch_tr_bf16(prm, plan, pkc, qkc, s);
  } else if (l.g.a_type == CUDA_R_32F) {
    st = launch_tr_f32(prm, plan, pkc, qkc, s);
  } else {
    const int fa = f8_fmt(l.g.a_type), fb = f8_fmt(l.g.b_type);
    st = launch_tr_f8(prm, plan, plan.swapped ? fa : fb, plan.swapped ? fb : fa, pkc, qkc, s);
  }
  if (st || prm.splits == 1) return st;
  SplitKReduceParams rp;
  rp.g = l.g;
  rp.swapped = plan.swapped;
  rp.splits = prm.splits;
  rp.acc_is_int = l.g.a_type == CUDA_R_8I;
  rp.ws_np = prm.tiles_p * v.bp;
  rp.ws_nq = prm.tiles_q * v.bq;
  rp.ws = (const int32_t *)ws;
  return launch_kernel(splitk_reduce_kernel, dim3((np + 1023) / 1024, nq, l.g.batch), dim3(256), s, rp);
}

template <int NW, int STEPS>
uint32_t launch_decode_variant(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, bool full, hipStream_t s) {
  dim3 grid(plan.grid_x, plan.grid_y, 1), block(NW * 64);
  if (nb == 1) {
    return full ? launch_kernel(decode_w8a8_kernel<NW, STEPS, 1, true>, grid, block, s, prm)
                : launch_kernel(decode_w8a8_kernel<NW, STEPS, 1, false>, grid, block, s, prm);
  } else if constexpr (STEPS <= 8) {  // two token blocks double the fragment registers
    return full ? launch_kernel(decode_w8a8_kernel<NW, STEPS, 2, true>, grid, block, s, prm)
                : launch_kernel(decode_w8a8_kernel<NW, STEPS, 2, false>, grid, block, s, prm);
  }
  return CUBLAS_STATUS_NOT_SUPPORTED;
}

uint32_t launch_decode(const Lowered &l, const zluda_gemm_plan &plan, hipStream_t s) {
  if (plan.variant >= (uint32_t)kNumDecodeVariants) return CUBLAS_STATUS_INVALID_VALUE;
  const DecodeVariant &v = kDecodeVariants[plan.variant];
  DecodeParams prm;
  prm.g = l.g;
  prm.swapped = plan.swapped;
  prm.rows_base = prm.rows_rem = prm.full_rounds = 0;
  const int T = plan.swapped ? l.g.M : l.g.N;
  const int ksteps = (l.g.K + 63) / 64;
  prm.spw = (ksteps + v.nw - 1) / v.nw;
  prm.nchunks = (prm.spw + v.steps - 1) / v.steps;
  const bool full = l.g.K == v.nw * v.steps * 64;
  const int nb = (T + 15) / 16;
  const bool h16 = l.g.a_type == CUDA_R_16F || l.g.a_type == CUDA_R_16BF;
  if (h16 && v.stream != 2) return CUBLAS_STATUS_NOT_SUPPORTED;  // 16-bit weights: the slab kernel only
  if (v.stream == 2) {
    // slab kernel: one block of tokens (two in the shapes of up to two units), nw slabs of K, W and X through 2 GiB buffer windows, at most
    // kSlabMaxBlocks blocks per workgroup: full_rounds round-robin blocks, then an even share (in quads of 4)
    // of the rows that are left
    const int64_t rows = plan.swapped ? l.g.N : l.g.M, ldw = plan.swapped ? l.g.b_sj : l.g.a_si;
    const int64_t ldx = plan.swapped ? l.g.a_si : l.g.b_sj;
    const int64_t esz = h16 ? 2 : 1, kb = l.g.K * esz;  // the kernel counts K and the pitches in bytes
    if (nb > (v.nw == 8 && v.steps <= 16 ? 2 : 1) || kb > v.nw * v.steps * 64 || (kb & 15) || rows * ldw * esz >= 0x7fffffffll ||
        ((int64_t)(T - 1) * ldx + l.g.K) * esz >= 0x7fffffffll || plan.grid_x == 0)
      return CUBLAS_STATUS_NOT_SUPPORTED;
    const int64_t G = plan.grid_x;
    prm.full_rounds = (int32_t)(rows / (16 * G));
    const int64_t left = rows - 16 * G * prm.full_rounds, quads = (left + 3) / 4;
    if (prm.full_rounds + (left > 0 ? 1 : 0) > kSlabMaxBlocks) return CUBLAS_STATUS_NOT_SUPPORTED;
    prm.rows_base = (int32_t)(quads / G);
    prm.rows_rem = (int32_t)(quads % G);
    prm.spw = (int32_t)((kb + v.nw * 128 - 1) / (v.nw * 128)) * 2;  // a wave's slab: K bytes / nw, rounded up to 128 bytes
    if (h16) return launch_decode_slab_h16(prm, plan, nb, l.g.a_type == CUDA_R_16BF, s);
    return l.g.a_type == CUDA_R_8I ? launch_decode_slab_i8(prm, plan, nb, s) : launch_decode_slab_f8(prm, plan, nb, s);
  }
  if (v.stream) {
    // the kernel addresses W through one 2 GiB buffer window and covers K <= nw * steps * 64
    const int64_t rows = plan.swapped ? l.g.N : l.g.M, ldw = plan.swapped ? l.g.b_sj : l.g.a_si;
    if (l.g.K > v.nw * v.steps * 64 || (l.g.K & 15) || rows * ldw >= 0x7fffffffll || plan.grid_x > (uint32_t)((rows + 15) / 16))
      return CUBLAS_STATUS_NOT_SUPPORTED;
    const int64_t quads = (rows + 3) / 4;  // the kernel splits the rows in quads of 4
    prm.rows_base = (int32_t)(quads / plan.grid_x);
    prm.rows_rem = (int32_t)(quads % plan.grid_x);
    return l.g.a_type == CUDA_R_8I ? launch_decode_stream_i8(prm, plan, nb, s) : launch_decode_stream_f8(prm, plan, nb, s);
  }
  if (l.g.a_type != CUDA_R_8I) return CUBLAS_STATUS_NOT_SUPPORTED;  // the register-streaming kernel is int8 only
  if (nb > 2 || (nb == 2 && v.steps > 8)) return CUBLAS_STATUS_NOT_SUPPORTED;
  switch (plan.variant) {
  case 0: return launch_decode_variant<8, 8>(prm, plan, nb, full, s);
  case 1: return launch_decode_variant<8, 16>(prm, plan, nb, full, s);
  case 2: return launch_decode_variant<4, 16>(prm, plan, nb, full, s);
  case 3: return launch_decode_variant<4, 8>(prm, plan, nb, full, s);
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
}

} // namespace

extern "C" uint32_t zluda_gemm_device_cu_count(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  static std::atomic<int> cached[64];  // zero-initialised; any thread may fill an entry (same value)
  if (dev >= 0 && dev < 64) {
    const int c = cached[dev].load(std::memory_order_relaxed);
    if (c) return (uint32_t)c;
  }
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
  return (uint32_t)cus;
}

namespace zluda_amd {

// BGRADA / BGRADB: the K sums of one operand into the bias buffer, behind the matmul on its stream
static uint32_t launch_bgrad(const GemmArgs &g, hipStream_t s) {
  BgradParams b;
  const bool of_a = g.bgrad_src == 1;
  b.src = of_a ? g.A : g.B;
  b.type = of_a ? g.a_type : g.b_type;
  b.rows = of_a ? g.M : g.N;
  b.K = g.K;
  b.batch = g.batch;
  b.s_row = of_a ? g.a_si : g.b_sj;
  b.s_k = of_a ? g.a_sk : g.b_sk;
  b.s_b = of_a ? g.a_sb : g.b_sb;
  b.out = g.bgrad;
  b.out_type = g.bias_type;
  b.out_sb = g.bias_sb;
  if (b.s_k <= b.s_row) return launch_kernel(bgrad_rows_kernel, dim3(b.rows, b.batch), dim3(256), s, b);
  return launch_kernel(bgrad_cols_kernel, dim3((b.rows + 255) / 256, b.batch), dim3(256), s, b);
}

uint32_t launch_planned(const zluda_gemm_problem *p, const zluda_gemm_plan *plan, void *ws, uint64_t ws_size, void *stream) {
  hipStream_t s = (hipStream_t)stream;
  Lowered l;
  uint32_t st = lower_problem(p, false, &l);
  if (st) return st;
  if (!family_supports(plan->kernel, l)) return CUBLAS_STATUS_INVALID_VALUE;
  if (ws_size < plan->workspace) return CUBLAS_STATUS_INVALID_VALUE;
  if (zluda_gemm_device_cu_count() == 0) return CUBLAS_STATUS_NOT_INITIALIZED;
  // GELU_AUX: the GEMM kernel writes the GELU input where the caller wants it kept, unscaled; the second pass
  // below reads it back and writes D.  (DGELU: the kernel writes D as usual and the second pass rewrites it.)
  const GemmArgs whole = l.g;
  if (whole.aux_mode == 1) {
    l.g.D = whole.aux;
    l.g.d_si = whole.aux_si; l.g.d_sj = whole.aux_sj; l.g.d_sb = whole.aux_sb;
    l.g.d_scale = nullptr;
  }
  switch (plan->kernel) {
  case ZLUDA_KERNEL_GENERIC: {
    dim3 grid(plan->grid_x, plan->grid_y, plan->grid_z);
    const bool int_acc = l.g.a_type == CUDA_R_8I;
    st = int_acc ? launch_kernel(gemm_generic_kernel<true>, grid, dim3(256), s, l.g)
                 : launch_kernel(gemm_generic_kernel<false>, grid, dim3(256), s, l.g);
    break;
  }
  case ZLUDA_KERNEL_MFMA_I8: case ZLUDA_KERNEL_MFMA_F8: case ZLUDA_KERNEL_MFMA_MXF4: case ZLUDA_KERNEL_MFMA_H16:
  case ZLUDA_KERNEL_MFMA_F32:
    st = launch_mfma(l, *plan, ws, ws_size, s);
    break;
  case ZLUDA_KERNEL_DECODE_W8A8: st = launch_decode(l, *plan, s); break;
  case ZLUDA_KERNEL_MFMA_TR8: case ZLUDA_KERNEL_MFMA_TR16: case ZLUDA_KERNEL_MFMA_TR32: st = launch_tr(l, *plan, ws, ws_size, s); break;
  default: return CUBLAS_STATUS_NOT_SUPPORTED;
  }
  if (st == CUBLAS_STATUS_SUCCESS && l.g.bgrad_src) st = launch_bgrad(l.g, s);
  if (st == CUBLAS_STATUS_SUCCESS && whole.aux_mode == 1)
    st = launch_kernel(aux_gelu_kernel, dim3((uint32_t)(((int64_t)whole.M * whole.N + 255) / 256), whole.batch), dim3(256), s, whole);
  if (st == CUBLAS_STATUS_SUCCESS && whole.aux_mode == 2)
    st = launch_kernel(aux_dgelu_kernel, dim3((whole.M + (whole.d_si == 1 ? 63 : 3)) / (whole.d_si == 1 ? 64 : 4), whole.batch), dim3(256), s, whole);
  return st;
}

} // namespace zluda_amd

extern "C" uint32_t zluda_gemm_launch(const zluda_gemm_problem *p, const zluda_gemm_plan *plan,
                                      void *stream) {
  if (!p || !plan) return CUBLAS_STATUS_INVALID_VALUE;
  return launch_planned(p, plan, p->workspace, p->workspace_size, stream);
}

// ---- cublasGemmEx-shaped entry points --------------------------------------------------------
extern "C" uint32_t zluda_gemm_strided_batched_ex(uint32_t transa, uint32_t transb, int32_t m, int32_t n,
                                                  int32_t k, const void *alpha, const void *A, uint32_t a_type,
                                                  int64_t lda, int64_t stride_a, const void *B, uint32_t b_type,
                                                  int64_t ldb, int64_t stride_b, const void *beta, void *C,
                                                  uint32_t c_type, int64_t ldc, int64_t stride_c,
                                                  int32_t batch_count, uint32_t compute_type, void *stream) {
  if (m < 0 || n < 0 || k < 0 || batch_count < 0) return CUBLAS_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0 || batch_count == 0) return CUBLAS_STATUS_SUCCESS;  // nothing to write
  if (k == 0) return CUBLAS_STATUS_NOT_SUPPORTED;  // C = beta * C only: not a matmul problem of this layer
  const bool int_path = compute_type == CUBLAS_COMPUTE_32I || compute_type == CUBLAS_COMPUTE_32I_PEDANTIC;
  zluda_gemm_problem p;
  memset(&p, 0, sizeof(p));
  p.op.compute_type = compute_type;
  p.op.scale_type = int_path ? CUDA_R_32I : CUDA_R_32F;
  p.op.pointer_mode = CUBLASLT_POINTER_MODE_HOST;
  p.op.transa = transa; p.op.transb = transb;
  p.op.epilogue = CUBLASLT_EPILOGUE_DEFAULT;
  p.op.bias_type = -1;
  p.op.epilogue_aux_type = -1;
  const bool ta = transa != CUBLAS_OP_N, tb = transb != CUBLAS_OP_N;
  p.a = {a_type, CUBLASLT_ORDER_COL, (uint64_t)(ta ? k : m), (uint64_t)(ta ? m : k), lda, batch_count, stride_a};
  p.b = {b_type, CUBLASLT_ORDER_COL, (uint64_t)(tb ? n : k), (uint64_t)(tb ? k : n), ldb, batch_count, stride_b};
  p.c = {c_type, CUBLASLT_ORDER_COL, (uint64_t)m, (uint64_t)n, ldc, batch_count, stride_c};
  p.d = p.c;
  p.alpha = alpha; p.beta = beta;
  p.A = A; p.B = B; p.C = C; p.D = C;
  zluda_gemm_plan plan;
  uint32_t st = zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_AUTO, -1, zluda_gemm_device_cu_count(), &plan);
  if (st == CUBLAS_STATUS_SUCCESS) st = zluda_gemm_launch(&p, &plan, stream);
  if (st == CUBLAS_STATUS_NOT_SUPPORTED || st == CUBLAS_STATUS_INVALID_VALUE) {
    // the chosen family may refuse the actual pointers (alignment): the generic kernel takes anything valid
    if (zluda_gemm_plan_problem(&p, ZLUDA_KERNEL_GENERIC, -1, zluda_gemm_device_cu_count(), &plan) == CUBLAS_STATUS_SUCCESS)
      st = zluda_gemm_launch(&p, &plan, stream);
  }
  return st;
}

extern "C" uint32_t zluda_gemm_ex(uint32_t transa, uint32_t transb, int32_t m, int32_t n, int32_t k,
                                  const void *alpha, const void *A, uint32_t a_type, int64_t lda, const void *B,
                                  uint32_t b_type, int64_t ldb, const void *beta, void *C, uint32_t c_type,
                                  int64_t ldc, uint32_t compute_type, void *stream) {
  return zluda_gemm_strided_batched_ex(transa, transb, m, n, k, alpha, A, a_type, lda, 0, B, b_type, ldb, 0, beta, C,
                                       c_type, ldc, 0, 1, compute_type, stream);
}
