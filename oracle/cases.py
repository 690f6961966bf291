"""TEST INFRASTRUCTURE.  Shared machinery of the parity tests, the smoke test and the benchmark's
cpu_baseline leg: seeded inputs, the oracle run, the GPU run through the
C ABI, and the comparison.  The same `spec` dict drives zluda_amd.cublaslt.MatmulCall (GPU) and the
zluda_gemm_problem handed to the CPU oracle."""
import ctypes as C

import numpy as np

import oracle
from zluda_amd import abi
from zluda_amd.cublaslt import MatmulCall

NP_OF = {abi.CUDA_R_32F: np.float32, abi.CUDA_R_32I: np.int32, abi.CUDA_R_16F: np.uint16,
         abi.CUDA_R_16BF: np.uint16, abi.CUDA_R_8I: np.int8, abi.CUDA_R_8F_E4M3: np.uint8,
         abi.CUDA_R_8F_E5M2: np.uint8}


def _layout(spec, tag, rows, cols):
    order = spec.get("order_" + tag, abi.CUBLASLT_ORDER_COL)
    ld = spec.get("ld" + tag, rows if order == abi.CUBLASLT_ORDER_COL else cols)
    lead = cols if order == abi.CUBLASLT_ORDER_COL else rows
    stride = spec.get("stride_" + tag, ld * lead)
    return order, ld, stride


def _encode(values, typ):
    """float32 values -> storage codes of `typ` (not FP4)."""
    if typ == abi.CUDA_R_32F:
        return values.astype(np.float32)
    if typ == abi.CUDA_R_16F:
        return oracle.encode_f16(values)
    if typ == abi.CUDA_R_16BF:
        return oracle.encode_bf16(values)
    if typ == abi.CUDA_R_8F_E4M3:
        return oracle.encode_e4m3(values)
    if typ == abi.CUDA_R_8F_E5M2:
        return oracle.encode_e5m2(values)
    raise ValueError(typ)


def decode_storage(buf, typ):
    """storage codes -> float64 values (outputs)."""
    if typ == abi.CUDA_R_32F:
        return buf.astype(np.float64)
    if typ in (abi.CUDA_R_32I, abi.CUDA_R_8I):
        return buf.astype(np.float64)
    if typ == abi.CUDA_R_16BF:
        return oracle.decode_bf16(buf).astype(np.float64)
    if typ == abi.CUDA_R_16F:
        return buf.view(np.float16).astype(np.float64)
    if typ == abi.CUDA_R_8F_E4M3:
        return oracle.decode_table("e4m3")[buf].astype(np.float64)
    if typ == abi.CUDA_R_8F_E5M2:
        return oracle.decode_table("e5m2")[buf].astype(np.float64)
    raise ValueError(typ)


class Case:
    """Host-side data of one matmul."""

    def __init__(self, spec, seed, int_dist="uniform", value_scale=1.0):
        self.spec = s = dict(spec)
        rng = np.random.default_rng(seed)
        m, n, k = s["m"], s["n"], s["k"]
        batch = s.get("batch", 1)
        ta, tb = s.get("transa", 0) != 0, s.get("transb", 0) != 0
        s.setdefault("c_type", s["d_type"])
        self.batch = batch
        self.a_scale = self.b_scale = self.c_scale = self.d_scale = self.bias = None

        def operand(tag, typ, rows, cols, k_is_rows, scale_mode):
            """returns (storage array, block scale array or None)"""
            order, ld, stride = _layout(s, tag, rows, cols)
            total = stride * (batch - 1) + ld * (cols if order == abi.CUBLASLT_ORDER_COL else rows)
            if typ == abi.CUDA_R_4F_E2M1:
                # K must be the contiguous dimension
                contig_rows = order == abi.CUBLASLT_ORDER_COL
                assert contig_rows == k_is_rows, "FP4 operands must be K-contiguous"
                nvec = cols if contig_rows else rows  # number of K-vectors (M or N)
                store = rng.integers(0, 256, size=(total + 1) // 2, dtype=np.uint8)
                if "mx_scale_range" in s:
                    # random E2M1 codes under scale bytes drawn independently per row and K block: a scale
                    # tensor read in any other order than [row][K/32] changes nearly every output
                    lo, hi = s["mx_scale_range"]
                    return store, rng.integers(lo, hi, size=(batch, nvec, k // 32), dtype=np.uint8)
                scales = np.empty((batch, nvec, k // 32), np.uint8)
                for b in range(batch):
                    x = (rng.standard_normal((nvec, k)) * value_scale).astype(np.float32)
                    q, sc = oracle.quantize_mxfp4(x)
                    scales[b] = sc
                    for v in range(nvec):
                        off = (stride * b + v * ld) // 2
                        store[off:off + k // 2] = q[v]
                return store, scales
            if typ == abi.CUDA_R_8I:
                if int_dist == "uniform":
                    store = rng.integers(-128, 128, size=total, dtype=np.int8)
                else:  # round(N(0, 32)) clipped to +-127
                    store = np.clip(np.rint(rng.standard_normal(total) * 32.0), -127, 127).astype(np.int8)
                return store, None
            vals = (rng.standard_normal(total) * value_scale).astype(np.float32)
            if s.get("f8_amax_quant", False) and typ in (abi.CUDA_R_8F_E4M3, abi.CUDA_R_8F_E5M2):
                # per-tensor quantisation: q = fp8(x * fmax / max|x|), scale = max|x| / fmax
                fmax = 448.0 if typ == abi.CUDA_R_8F_E4M3 else 57344.0
                amax = float(np.abs(vals).max())
                return _encode(vals * np.float32(fmax / amax), typ), np.array([amax / fmax], np.float32)
            store = _encode(vals, typ)
            scales = None
            if scale_mode == abi.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0:
                nvec = cols if k_is_rows else rows
                scales = rng.integers(120, 135, size=(batch, nvec, k // 32), dtype=np.uint8)
            return store, scales

        self.A, a_blk = operand("a", s["a_type"], k if ta else m, m if ta else k, ta, s.get("a_scale_mode", 0))
        self.B, b_blk = operand("b", s["b_type"], n if tb else k, k if tb else n, not tb, s.get("b_scale_mode", 0))
        # C and D
        _, ldc, sc = _layout(s, "c", m, n)
        _, ldd, sd = _layout(s, "d", m, n)
        oc = s.get("order_c", 0)
        od = s.get("order_d", 0)
        ctot = sc * (batch - 1) + ldc * (n if oc == 0 else m)
        dtot = sd * (batch - 1) + ldd * (n if od == 0 else m)
        self.has_c = s.get("with_c", False)
        if self.has_c:
            if s["c_type"] == abi.CUDA_R_32I:
                self.Cm = rng.integers(-1000, 1000, size=ctot, dtype=np.int32)
            elif s["c_type"] == abi.CUDA_R_8I:
                self.Cm = rng.integers(-128, 128, size=ctot, dtype=np.int8)
            else:
                self.Cm = _encode(rng.standard_normal(ctot).astype(np.float32), s["c_type"])
        else:
            self.Cm = None
        self.dtot = dtot
        self.d_np = NP_OF[s["d_type"]]

        # alpha / beta
        pm = s.get("pointer_mode", abi.CUBLASLT_POINTER_MODE_HOST)
        int_scale = s["scale_type"] == abi.CUDA_R_32I
        sdt = np.int32 if int_scale else np.float32
        avs = s.get("alpha_vector_batch_stride", 0)
        alpha_vec = pm in (abi.CUBLASLT_POINTER_MODE_DEVICE_VECTOR,
                           abi.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
                           abi.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST)
        nalpha = (m + avs * (batch - 1)) if alpha_vec else 1
        if "alpha" in s:
            self.alpha = np.full(nalpha, s["alpha"], dtype=sdt)
        elif int_scale:
            self.alpha = rng.integers(-3, 4, size=nalpha).astype(np.int32)
            self.alpha[self.alpha == 0] = 1
        else:
            lo, hi = s.get("alpha_range", (0.5, 1.5))
            self.alpha = rng.uniform(lo, hi, size=nalpha).astype(np.float32)
        nbeta = m if pm == abi.CUBLASLT_POINTER_MODE_DEVICE_VECTOR else 1
        if not self.has_c:
            self.beta = np.zeros(nbeta, dtype=sdt)
        elif int_scale:
            self.beta = rng.integers(1, 3, size=nbeta).astype(np.int32)
        else:
            self.beta = rng.uniform(0.5, 1.5, size=nbeta).astype(np.float32)
        self.alpha_on_device = pm != abi.CUBLASLT_POINTER_MODE_HOST
        self.beta_on_device = pm in (abi.CUBLASLT_POINTER_MODE_DEVICE, abi.CUBLASLT_POINTER_MODE_DEVICE_VECTOR)

        # scales
        def scale(mode, blk, n_outer, rng_range):
            if mode == abi.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0:
                return blk
            if blk is not None and blk.dtype == np.float32:   # per-tensor scale that came with the quantisation
                return blk
            if mode == abi.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F:
                return rng.uniform(*rng_range, size=n_outer).astype(np.float32)
            if s.get("with_scalar_scales", False):
                return rng.uniform(*rng_range, size=1).astype(np.float32)
            return None
        sr = s.get("scale_range", (0.5, 2.0))
        self.a_scale = scale(s.get("a_scale_mode", 0), a_blk, m, sr)
        self.b_scale = scale(s.get("b_scale_mode", 0), b_blk, n, sr)
        if s.get("with_cd_scales", False):
            self.c_scale = rng.uniform(0.5, 2.0, size=1).astype(np.float32)
            self.d_scale = rng.uniform(0.5, 2.0, size=1).astype(np.float32)

        # bias
        epi = s.get("epilogue", abi.CUBLASLT_EPILOGUE_DEFAULT)
        if epi in (abi.CUBLASLT_EPILOGUE_BIAS, abi.CUBLASLT_EPILOGUE_RELU_BIAS, abi.CUBLASLT_EPILOGUE_GELU_BIAS,
                   abi.CUBLASLT_EPILOGUE_GELU_AUX_BIAS):
            bt = s.get("bias_type", -1)
            if bt < 0:
                bt = abi.CUDA_R_32F if s["d_type"] in (abi.CUDA_R_8I, abi.CUDA_R_32I, abi.CUDA_R_8F_E4M3,
                                                       abi.CUDA_R_8F_E5M2) else s["d_type"]
            nb = m + s.get("bias_batch_stride", 0) * (batch - 1)
            bvals = (rng.standard_normal(nb) * s.get("bias_std", 0.5)).astype(np.float32)
            self.bias = _encode(bvals, bt)
        # bias-gradient epilogues: the bias buffer is an output (M sums for BGRADA, N for BGRADB); it starts as a
        # canary, the oracle's result lands in self.bgrad_ref and the GPU's in self.bgrad_got
        # (3: DGELU_BGRAD, the sums of D's rows)
        self.bgrad = {abi.CUBLASLT_EPILOGUE_BGRADA: 1, abi.CUBLASLT_EPILOGUE_BGRADB: 2, abi.CUBLASLT_EPILOGUE_DGELU_BGRAD: 3}.get(epi, 0)
        if self.bgrad:
            bt = s.get("bias_type", -1)
            if bt < 0:
                bt = abi.CUDA_R_32F if s["d_type"] in (abi.CUDA_R_8I, abi.CUDA_R_32I, abi.CUDA_R_8F_E4M3,
                                                       abi.CUDA_R_8F_E5M2) else s["d_type"]
            self.bgrad_type = bt
            nb = (n if self.bgrad == 2 else m) + s.get("bias_batch_stride", 0) * (batch - 1)
            self.bias = np.frombuffer(bytes([0xCD]) * (nb * (4 if bt == abi.CUDA_R_32F else 2)),
                                      dtype=np.float32 if bt == abi.CUDA_R_32F else np.uint16).copy()
        # The aux matrix of GELU_AUX[_BIAS] (output: the GELU input, starts as a canary) and DGELU[_BGRAD] (input:
        # random values): D's type and order, leading dimension spec["aux_ld"] (default: tight), batches
        # spec["aux_batch_stride"] apart (default: tight).  self.aux_mode 1 = written, 2 = read.
        self.aux = None
        self.aux_mode = {abi.CUBLASLT_EPILOGUE_GELU_AUX: 1, abi.CUBLASLT_EPILOGUE_GELU_AUX_BIAS: 1,
                         abi.CUBLASLT_EPILOGUE_DGELU: 2, abi.CUBLASLT_EPILOGUE_DGELU_BGRAD: 2}.get(epi, 0)
        if self.aux_mode:
            col = s.get("order_d", abi.CUBLASLT_ORDER_COL) == abi.CUBLASLT_ORDER_COL
            lead, other = (m, n) if col else (n, m)
            self.aux_ld = s.setdefault("aux_ld", lead)
            self.aux_stride = s.setdefault("aux_batch_stride", self.aux_ld * other)
            tot = self.aux_stride * (batch - 1) + self.aux_ld * other
            if self.aux_mode == 1:
                self.aux = np.frombuffer(bytes([0xCD]) * (tot * np.dtype(self.d_np).itemsize), dtype=self.d_np).copy()
            else:
                self.aux = _encode((rng.standard_normal(tot) * s.get("aux_std", 1.5)).astype(np.float32), s["d_type"])

    def new_d(self):
        """output storage pre-filled with a canary pattern"""
        return np.frombuffer(bytes([0xCD]) * (self.dtot * np.dtype(self.d_np).itemsize), dtype=self.d_np).copy()

    # ---- CPU oracle ---------------------------------------------------------------------------
    def problem(self, ptrs):
        """zluda_gemm_problem with the given pointer dict (host or device addresses)."""
        s = self.spec
        m, n, k = s["m"], s["n"], s["k"]
        ta, tb = s.get("transa", 0) != 0, s.get("transb", 0) != 0
        p = abi.zluda_gemm_problem()

        def lay(dst, tag, typ, rows, cols):
            order, ld, stride = _layout(s, tag, rows, cols)
            dst.type, dst.order, dst.rows, dst.cols, dst.ld = typ, order, rows, cols, ld
            dst.batch_count, dst.batch_stride = self.batch, stride
        lay(p.a, "a", s["a_type"], k if ta else m, m if ta else k)
        lay(p.b, "b", s["b_type"], n if tb else k, k if tb else n)
        lay(p.c, "c", s["c_type"], m, n)
        lay(p.d, "d", s["d_type"], m, n)
        o = p.op
        o.compute_type, o.scale_type = s["compute_type"], s["scale_type"]
        o.pointer_mode = s.get("pointer_mode", 0)
        o.transa, o.transb = s.get("transa", 0), s.get("transb", 0)
        o.epilogue = s.get("epilogue", abi.CUBLASLT_EPILOGUE_DEFAULT)
        o.bias_type = s.get("bias_type", -1)
        o.bias_batch_stride = s.get("bias_batch_stride", 0)
        o.alpha_vector_batch_stride = s.get("alpha_vector_batch_stride", 0)
        o.a_scale_mode, o.b_scale_mode = s.get("a_scale_mode", 0), s.get("b_scale_mode", 0)
        o.bias, o.a_scale, o.b_scale = ptrs.get("bias"), ptrs.get("a_scale"), ptrs.get("b_scale")
        o.c_scale, o.d_scale = ptrs.get("c_scale"), ptrs.get("d_scale")
        o.epilogue_aux = ptrs.get("aux")
        o.epilogue_aux_ld, o.epilogue_aux_batch_stride = s.get("aux_ld", 0), s.get("aux_batch_stride", 0)
        o.epilogue_aux_type = s.get("aux_type", -1)
        p.alpha, p.beta = ptrs["alpha"], ptrs["beta"]
        p.A, p.B, p.C, p.D = ptrs["A"], ptrs["B"], ptrs.get("C"), ptrs["D"]
        return p

    def run_oracle(self):
        d = self.new_d()
        hp = lambda x: x.ctypes.data if x is not None else None
        bias = self.bias
        if self.bgrad:   # the oracle writes it: keep the canary for the GPU run
            bias = self.bgrad_ref = self.bias.copy()
        aux = self.aux
        if self.aux_mode == 1:   # the oracle writes it: keep the canary for the GPU run
            aux = self.aux_ref = self.aux.copy()
        ptrs = {"A": hp(self.A), "B": hp(self.B), "C": hp(self.Cm), "D": hp(d), "alpha": hp(self.alpha),
                "beta": hp(self.beta), "bias": hp(bias), "a_scale": hp(self.a_scale),
                "b_scale": hp(self.b_scale), "c_scale": hp(self.c_scale), "d_scale": hp(self.d_scale), "aux": hp(aux)}
        p = self.problem(ptrs)
        st = oracle.gemm(p)
        assert st == 0, "oracle status %d" % st
        return d

    # ---- GPU through the C ABI ------------------------------------------------------------------
    def upload(self, offset_bytes=0):
        """copies every host array to cuda:0; returns (tensors to keep alive, address dict, D tensor)"""
        import torch
        dev = torch.device("cuda:0")

        def up(x, off=0):
            if x is None:
                return None, None
            raw = np.frombuffer(x.tobytes(), dtype=np.uint8)
            t = torch.empty(raw.size + off + 16, dtype=torch.uint8, device=dev)
            t[off:off + raw.size] = torch.from_numpy(raw.copy()).to(dev)
            return t, t.data_ptr() + off
        keep, ptr = [], {}
        for name, arr, off in (("A", self.A, offset_bytes), ("B", self.B, offset_bytes), ("C", self.Cm, 0),
                               ("bias", self.bias, 0), ("a_scale", self.a_scale, 0),
                               ("b_scale", self.b_scale, 0), ("c_scale", self.c_scale, 0),
                               ("d_scale", self.d_scale, 0), ("alpha_dev", self.alpha, 0),
                               ("beta_dev", self.beta, 0), ("aux", self.aux, 0)):
            t, p = up(arr, off)
            keep.append(t)
            ptr[name] = p
        # D sits between two canary-filled guard regions at least as large as what a 256-column tile
        # hanging over the end of the matrix could reach; download() checks that both are intact
        d_host = self.new_d()
        esz = d_host.dtype.itemsize
        _, ldd, _ = _layout(self.spec, "d", self.spec["m"], self.spec["n"])
        guard = (max(256 * ldd * esz, 4096) + 255) // 256 * 256
        dt = torch.full((guard + d_host.nbytes + guard,), 0xCD, dtype=torch.uint8, device=dev)
        dt[guard:guard + d_host.nbytes] = torch.from_numpy(np.frombuffer(d_host.tobytes(), dtype=np.uint8).copy()).to(dev)
        self._guard = guard
        ptr["D"] = dt.data_ptr() + guard
        return keep, ptr, dt

    def scalars(self, ptr):
        """alpha / beta arguments as cublasLtMatmul wants them for this pointer mode"""
        if self.alpha_on_device:
            alpha = ptr["alpha_dev"]
        else:
            alpha = (C.c_int32 if self.alpha.dtype == np.int32 else C.c_float)(self.alpha[0].item())
        if self.beta_on_device:
            beta = ptr["beta_dev"]
        else:
            beta = (C.c_int32 if self.beta.dtype == np.int32 else C.c_float)(self.beta[0].item())
        return alpha, beta

    def download(self, dt):
        nbytes = self.dtot * np.dtype(self.d_np).itemsize
        g = self._guard
        assert bool((dt[:g] == 0xCD).all()) and bool((dt[g + nbytes:] == 0xCD).all()), \
            "bytes outside the storage of D were written"
        return dt[g:g + nbytes].cpu().numpy().view(self.d_np).copy()

    def run_gpu(self, api, forced_kernel=None, forced_variant=-1, offset_bytes=0, workspace_bytes=0):
        """Returns (status, D storage, kernel family, variant).  offset_bytes misaligns A and B;
        workspace_bytes > 0 offers that much workspace (preference and call), which is what lets the
        planner split K.  self.last_workspace_needed = what the heuristic asked for."""
        import torch
        keep, ptr, dt = self.upload(offset_bytes)
        call = MatmulCall(api, self.spec, forced_kernel=forced_kernel, forced_variant=forced_variant,
                          max_workspace=workspace_bytes)
        ws = torch.empty(max(workspace_bytes, 16), dtype=torch.uint8, device="cuda:0") if workspace_bytes else None
        self.last_workspace_needed = call.heuristic[0].workspaceSize if call.heuristic else None
        try:
            call.set_pointers(bias=ptr["bias"], a_scale=ptr["a_scale"], b_scale=ptr["b_scale"],
                              c_scale=ptr["c_scale"], d_scale=ptr["d_scale"], aux=ptr["aux"])
            alpha, beta = self.scalars(ptr)
            stream = torch.cuda.current_stream().cuda_stream
            st = call.run(alpha, ptr["A"], ptr["B"], beta, ptr["C"], ptr["D"],
                          ws.data_ptr() if ws is not None else None, workspace_bytes, stream)
            torch.cuda.synchronize()
            if self.bgrad:
                self.bgrad_got = keep[3][:self.bias.nbytes].cpu().numpy().view(self.bias.dtype).copy()
            if self.aux_mode == 1:
                self.aux_got = keep[10][:self.aux.nbytes].cpu().numpy().view(self.aux.dtype).copy()
            return st, self.download(dt), call.kernel, call.variant
        finally:
            call.close()

    def run_gpu_plan(self, api, forced_kernel, forced_variant=-1, grid_x=None):
        """The same problem through the inner launch layer (zluda_gemm_plan_problem + zluda_gemm_launch), with the
        plan's grid_x overridden when given: a smaller grid makes every workgroup of the row-streaming decode
        kernel walk several 16-row blocks without needing a matrix of tens of thousands of rows.
        Returns (status, D storage, plan)."""
        import torch
        keep, ptr, dt = self.upload()
        host = {"alpha": self.alpha.ctypes.data, "beta": self.beta.ctypes.data}
        ptrs = dict(ptr)
        ptrs["alpha"] = ptr["alpha_dev"] if self.alpha_on_device else host["alpha"]
        ptrs["beta"] = ptr["beta_dev"] if self.beta_on_device else host["beta"]
        p = self.problem(ptrs)
        plan = abi.zluda_gemm_plan()
        st = api.zluda_gemm_plan_problem(C.byref(p), forced_kernel, forced_variant, api.zluda_gemm_device_cu_count(), C.byref(plan))
        if st:
            return st, None, plan
        if grid_x is not None:
            plan.grid_x = grid_x
        st = api.zluda_gemm_launch(C.byref(p), C.byref(plan), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return st, self.download(dt), plan

    def run_hipblaslt(self):
        """The reference's forwarded path.  Returns (D storage or None, reason)."""
        import torch
        from oracle.hipblaslt_replay import Replay
        keep, ptr, dt = self.upload()
        rp = Replay(self.spec)
        try:
            if rp.why:
                return None, rp.why
            if not rp.set_pointers(bias=ptr["bias"], a_scale=ptr["a_scale"], b_scale=ptr["b_scale"],
                                   c_scale=ptr["c_scale"], d_scale=ptr["d_scale"], aux=ptr["aux"]):
                return None, rp.why
            if not rp.find_algo():
                return None, rp.why
            alpha, beta = self.scalars(ptr)
            st = rp.run(alpha, ptr["A"], ptr["B"], beta, ptr["C"], ptr["D"], torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            if st:
                return None, "hipblasLtMatmul status %d" % st
            if self.bgrad:
                self.bgrad_theirs = keep[3][:self.bias.nbytes].cpu().numpy().view(self.bias.dtype).copy()
            if self.aux_mode == 1:
                self.aux_theirs = keep[10][:self.aux.nbytes].cpu().numpy().view(self.aux.dtype).copy()
            return self.download(dt), ""
        finally:
            rp.close()

    # ---- comparison -------------------------------------------------------------------------------
    def compare_aux(self, got, ref, tol=1e-2):
        """the aux matrix of GELU_AUX[_BIAS]: its padding keeps the canary, its elements (the GELU input) agree within
        `tol` relative to max(|ref|, 1e-2 * rms)"""
        s = self.spec
        m, n = s["m"], s["n"]
        col = s.get("order_d", abi.CUBLASLT_ORDER_COL) == abi.CUBLASLT_ORDER_COL
        i, j = np.meshgrid(np.arange(m), np.arange(n), indexing="ij")
        one = (j * self.aux_ld + i) if col else (i * self.aux_ld + j)
        idx = np.concatenate([(one + b * self.aux_stride).ravel() for b in range(self.batch)])
        mask = np.ones(got.size, bool)
        mask[idx] = False
        assert np.array_equal(got[mask], ref[mask]), "padding of the aux matrix was overwritten"
        g, r = decode_storage(got[idx], s["d_type"]), decode_storage(ref[idx], s["d_type"])
        assert np.isfinite(g).all() and np.isfinite(r).all()
        rms = float(np.sqrt(np.mean(r * r)))
        err = float(np.max(np.abs(g - r) / np.maximum(np.abs(r), 1e-2 * rms if rms > 0 else 1.0)))
        print("aux matrix: max rel err %.3e" % err)
        assert err <= tol, "aux matrix: max relative error %.3e > %.1e" % (err, tol)
        return err

    def compare_bgrad(self, got, ref, exact=False, floor_frac=1e-2):
        """bias gradients as stored (bias data type): bit-exact when `exact` (integer operands: the sums are
        exact in int32 and convert the same way), else within 1e-2 of max(|ref|, floor_frac * rms(ref)) -- the fp32
        summation order of the GPU kernel is its own and the output may be a 16-bit float.  (DGELU_BGRAD sums
        the elements of D as its two passes rounded them, hundreds of terms of either sign: callers pass
        floor_frac=1, i.e. an absolute bound of 1 % of the rms of the sums.)"""
        g, r = decode_storage(got, self.bgrad_type), decode_storage(ref, self.bgrad_type)
        assert g.shape == r.shape
        if exact:
            np.testing.assert_array_equal(got, ref)
            return
        floor = floor_frac * float(np.sqrt(np.mean(r * r))) + 1e-30
        err = np.abs(g - r) / np.maximum(np.abs(r), floor)
        print("bias gradient: max relative error %.3g" % float(err.max()), flush=True)
        assert err.max() <= 1e-2

    def logical_index(self):
        """flat storage indices of D(i, j, batch) as an int64 array [batch, m, n]"""
        s = self.spec
        m, n = s["m"], s["n"]
        order, ld, stride = _layout(s, "d", m, n)
        i = np.arange(m)[:, None]
        j = np.arange(n)[None, :]
        base = (i + j * ld) if order == abi.CUBLASLT_ORDER_COL else (i * ld + j)
        return np.stack([base + b * stride for b in range(self.batch)])

    def compare(self, got, ref, tol=None, floor_frac=None):
        """bit-exact for integer outputs (whole storage incl. padding); otherwise padding must be
        untouched and max |got-ref| / max(|ref|, floor) <= tol with floor = floor_frac * rms(ref).

        floor_frac defaults to 1e-2, and to 1e-1 for FP8 inputs when `ref` is the float64 oracle:
        v_mfma_f32_32x32x64_f8f6f4 does not keep every bit of the fp32 running sum for 8-bit float
        operands (measured against an exact fp64 sum: deviations up to 1.3e-4 * rms of the output, where
        the scalar fp32 kernel shows none; the FP4 forms of the same instruction are exact), so outputs
        that nearly cancel, |ref| < 0.1 * rms, cannot meet a 1e-2 bound relative to their own magnitude.
        Comparisons of two GPU results that both come from that instruction pass floor_frac=1e-2.

        Returns the error figure under the floor used; self.last_errors = {"strict": figure with
        floor 1e-2 * rms, "relaxed": figure with floor 1e-1 * rms, "max_abs_over_rms": ...} whatever the
        outcome, and the figures are printed (pytest -s shows them)."""
        s = self.spec
        if s["d_type"] in (abi.CUDA_R_32I, abi.CUDA_R_8I) and s["scale_type"] == abi.CUDA_R_32I:
            bad = np.nonzero(got != ref)[0]
            assert bad.size == 0, "%d mismatching int32 elements, first at %d: %d vs %d" % (
                bad.size, bad[0], got[bad[0]], ref[bad[0]])
            return 0.0
        idx = self.logical_index().ravel()
        mask = np.ones(got.size, bool)
        mask[idx] = False
        assert np.array_equal(got[mask], ref[mask]), "padding between ld and rows was overwritten"
        g = decode_storage(got[idx], s["d_type"])
        r = decode_storage(ref[idx], s["d_type"])
        assert np.isfinite(g).all() and np.isfinite(r).all()
        rms = float(np.sqrt(np.mean(r * r)))
        f8_in = s["a_type"] in (abi.CUDA_R_8F_E4M3, abi.CUDA_R_8F_E5M2)
        if floor_frac is None:
            floor_frac = 1e-1 if f8_in else 1e-2
        diff = np.abs(g - r)

        def figure(frac):
            return float(np.max(diff / np.maximum(np.abs(r), frac * rms if rms > 0 else 1.0)))
        self.last_errors = {"strict": figure(1e-2), "relaxed": figure(1e-1),
                            "max_abs_over_rms": float(diff.max() / rms) if rms > 0 else float(diff.max())}
        floor = floor_frac * rms if rms > 0 else 1.0
        err = figure(floor_frac)
        print("max rel err: %.3e with floor 1e-2*rms (strict), %.3e with floor 1e-1*rms; max |diff| / rms %.3e; "
              "gate uses floor %.0e*rms" % (self.last_errors["strict"], self.last_errors["relaxed"],
                                            self.last_errors["max_abs_over_rms"], floor_frac), flush=True)
        if tol is None:
            tol = 1e-2
        if s["d_type"] == abi.CUDA_R_8I:
            assert np.max(np.abs(g - r)) <= 1, "int8 outputs differ by more than one step"
            return err
        if err > tol:
            rel = diff / np.maximum(np.abs(r), floor)
            bad = np.nonzero(rel > tol)[0]
            m = s["m"]
            rows = (idx[bad] % (self.dtot // self.batch)) % max(_layout(s, "d", m, s["n"])[1], 1)
            raise AssertionError("max relative error %.3e > %.1e: %d of %d outputs off, logical positions %d..%d, "
                                 "storage offsets mod ld: min %d max %d (%d distinct)" %
                                 (err, tol, bad.size, rel.size, bad[0], bad[-1], rows.min(), rows.max(), np.unique(rows).size))
        return err
