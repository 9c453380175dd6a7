"""The kernels as Python functions over torch tensors on the GPU.

Every function checks on the host that shapes, element types and devices are what
the kernel and its grid assume, before anything is launched; a size that a kernel
does not take is refused with an error that names it. Tensors are only memory
here: the work is done by the HIP library loaded through ``ctypes`` on the
current torch stream. If the library cannot be built or loaded this raises; there
is no other implementation behind these functions.
"""
from __future__ import annotations

import ctypes
import os
import sys
from dataclasses import dataclass

import torch

from . import library

CORE_SOURCES = ["error.hip", "elementwise.hip", "gemm_generic.hip", "gemm_skinny_bf16.hip", "gemm_fewrows_bf16.hip", "attention_generic.hip",
                "sampling.hip", "measure.hip"]
BLAS_SOURCES = ["error.hip", "gemm_library.hip"]                                                   # the vendor's matrix library, algorithm by number
BLAS_LINK = ["-lhipblaslt"]
ATTENTION_SOURCES = ["error.hip", "attention_decode_bf16.hip", "attention_prefill_bf16.hip"]      # compiled once per head size
ATTENTION_HEAD_DIMS_BUILT_AHEAD = [16, 32, 48, 64, 80, 96, 112, 128, 256]

F32, BF16 = 0, 1
# a measured choice for a matrix product: the own kernel, or what the rule gives (0, 1, ...: that algorithm of the library's list)
OWN, RULE = -1, -2
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    """A kernel refused its arguments or failed to launch."""


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported (float32 and bfloat16 are)") from None


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
# torch.mm takes out_dtype (a float32 result from bfloat16 operands) from version 2.8 on
_MM_GIVES_FLOAT32 = tuple(int(p) for p in torch.__version__.split("+")[0].split(".")[:2]) >= (2, 8)


def _stream():
    """torch's current stream of the current device, as the kernels' launch argument (asked for before every
    kernel: the direct call takes a tenth of the time of building a ``torch.cuda.Stream`` object)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg) -> None:
    """``msg``: the message, or a function that makes it (the checks run before every kernel: a message that
    has to be formatted is only formatted when the check fails)."""
    if not cond:
        raise KernelError(msg() if callable(msg) else msg)


def _dense(t: torch.Tensor, name: str, shape: tuple | None = None, dtype=None) -> None:
    want = backend().device_type
    if t.device.type != want:
        raise KernelError(f"{name}: must live on a '{want}' device, is on {t.device}")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)} but {tuple(shape)} is needed")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: element type {t.dtype} but {dtype} is needed")


@dataclass
class AttentionBatch:
    """What attention has to know about the step's batch (device tensors are int32)."""

    num_tokens: int
    num_requests: int
    token_req: torch.Tensor        # [T] request index of every token
    positions: torch.Tensor        # [T] absolute position of every token
    cu_seqlens_q: torch.Tensor     # [B+1] first token of every request in the batch
    context_lens: torch.Tensor     # [B] keys of the request after this step
    max_q_len: int
    max_context_len: int


class NativeBackend:
    """ctypes calls into the HIP library."""

    name = "hip"
    device_type = "cuda"
    few_rows = 16                 # up to this many rows the own matrix kernels are the rule
    library_rows = 64             # up to this many rows the way a product is done may be chosen by measurement (see _choose)
    library_algorithms = 48       # so many of the library's algorithms are asked for and tried
    library_workspace = 32 << 20  # bytes of scratch memory the library's algorithms may use
    own_kernels_only = False      # True: no library call (matrix products of up to 64 rows take the own kernels)
    planned_context = 0           # > 0 while a HIP graph is recorded: the lengths to plan for (the batch's own are bounds)
    covered_context = 0           # and the longest context that the recorder will let the graph meet
    measure_linears = False       # True: a product of few rows and a shape not seen before is timed in every way there is (see _choose)
    measure_many_rows = True      # a product of more than library_rows rows is timed in the third step that meets its shape
    measuring_allowed = True      # False: nothing is ever timed; a shape follows the table that was loaded, or the rule
    fuse_norms = True             # products of up to few_rows rows may take over the residual addition and the norm around them (see Summed, Normed)
    step_number = 0               # counted by the engine, one per eager step

    def __init__(self):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to torch; the HIP kernels are the only implementation")
        self.lib = library.load_library("nhv_core", CORE_SOURCES)
        self.lib.nhv_last_error.restype = ctypes.c_char_p
        self._attention_libs: dict[int, ctypes.CDLL] = {}
        # (M, N, K, float result, gated) of a product -> OWN, RULE or a library algorithm, measured. ``chosen`` is the
        # table in force: the process-wide one that engines share by default (a shape is timed once per process), or
        # the table of the engine that runs now (see ``use_choices``)
        self.shared_chosen: dict[tuple, int] = {}
        self.chosen: dict[tuple, int] = self.shared_chosen
        self._blas = None
        self._plans: dict[tuple, tuple[int, int]] = {}
        self.times: dict[tuple, tuple[float, float]] = {}   # measured shape -> (ms of the own kernel, ms of the library's best), cold
        self._met: dict[tuple, tuple[int, int]] = {}        # shape of many rows -> (steps that met it, the last of them)
        self._workspace = None
        self._sweep = None                                  # scratch memory whose reading empties the caches before a measurement

    def _call(self, fn_name: str, *args, lib=None) -> None:
        lib = lib or self.lib
        rc = getattr(lib, fn_name)(*args)
        if rc != 0:
            raise KernelError(lib.nhv_last_error().decode())

    def attention_lib(self, head_dim: int) -> ctypes.CDLL:
        """The bfloat16 attention kernels are compiled per head size, when a model first needs them."""
        lib = self._attention_libs.get(head_dim)
        if lib is None:
            lib = library.load_library(f"nhv_attention_d{head_dim}", ATTENTION_SOURCES, [f"-DNHV_HEAD_DIM={head_dim}"])
            lib.nhv_last_error.restype = ctypes.c_char_p
            self._attention_libs[head_dim] = lib
        return lib

    # -- each method launches one kernel; arguments were checked by the caller --
    def embed(self, ids, table, out, scale=1.0):
        T, H = out.shape
        self._call("nhv_embed", _ptr(ids), _ptr(table), _ptr(out), T, H, table.shape[0], dtype_code(table),
                   ctypes.c_float(scale), _stream())

    def soft_cap(self, x, cap):
        self._call("nhv_soft_cap", _ptr(x), ctypes.c_size_t(x.numel()), ctypes.c_float(cap), _stream())

    def rmsnorm(self, x, residual, residual_mode, w, y, eps):
        T, H = x.shape
        self._call("nhv_rmsnorm", _ptr(x), _ptr(residual), residual_mode,
                   F32 if residual is None else dtype_code(residual), _ptr(w), _ptr(y), T, H, ctypes.c_float(eps),
                   dtype_code(x), dtype_code(w), _stream())

    def silu_mul(self, gu, out):
        T, I = out.shape
        self._call("nhv_silu_mul", _ptr(gu), _ptr(out), T, I, dtype_code(gu), _stream())

    def gather_rows(self, x, rows, out):
        self._call("nhv_gather_rows", _ptr(x), _ptr(rows), _ptr(out), out.shape[0], x.shape[1], x.shape[0],
                   dtype_code(x), _stream())

    def qk_rope_write(self, qkv, bias, q_norm_w, k_norm_w, eps, cos_sin, rot, positions, slot_mapping,
                      q_out, k_cache, v_cache, Hq, Hkv, D, write_kv, pair_axes=None):
        wd = dtype_code(q_norm_w) if q_norm_w is not None else dtype_code(qkv)
        self._call("nhv_qk_rope_write", _ptr(qkv), _ptr(bias), _ptr(q_norm_w), _ptr(k_norm_w), ctypes.c_float(eps),
                   _ptr(cos_sin), rot, 0 if cos_sin is None else cos_sin.shape[0], _ptr(positions), _ptr(pair_axes),
                   _ptr(slot_mapping),
                   _ptr(q_out), _ptr(k_cache), _ptr(v_cache), qkv.shape[0], Hq, Hkv, D, int(write_kv),
                   dtype_code(qkv), wd, _stream())

    def paged_attention(self, q, k_cache, v_cache, out, batch: AttentionBatch, block_tables, scale, window):
        T, Hq, D = q.shape
        _, page_size, Hkv, _ = k_cache.shape
        if (q.dtype == torch.bfloat16 and batch.max_q_len == 1 and D % 16 == 0 and D <= 256 and Hq // Hkv <= 16
                and T <= 65535):
            return self._decode_attention(q, k_cache, v_cache, out, batch, block_tables, scale, window)
        if q.dtype == torch.bfloat16 and D % 16 == 0 and D <= 256 and batch.num_requests <= 65535 and Hkv <= 65535:
            # prompt portions (and whatever single tokens share their batch) on the matrix cores
            return self._call("nhv_prefill_attention_bf16", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out),
                              _ptr(batch.cu_seqlens_q), _ptr(batch.context_lens), _ptr(block_tables),
                              block_tables.shape[1], batch.num_requests, batch.max_q_len, Hq, Hkv, page_size,
                              ctypes.c_float(scale), window, _stream(), lib=self.attention_lib(D))
        self._call("nhv_paged_attention_generic", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out),
                   _ptr(batch.token_req), _ptr(batch.positions), _ptr(block_tables), block_tables.shape[1], T, Hq, Hkv,
                   D, page_size, ctypes.c_float(scale), window, dtype_code(q), _stream())

    def _decode_attention(self, q, k_cache, v_cache, out, batch, block_tables, scale, window):
        """Single tokens in bfloat16: keys split over waves, then merged."""
        T, Hq, D = q.shape
        _, page_size, Hkv, _ = k_cache.shape
        # inside a graph the lengths are only bounded (by max_model_len): the recorder says what to plan for
        span = min(self.planned_context, batch.max_context_len) if self.planned_context else batch.max_context_len
        if window:
            span = min(span, window + 64)
        # One wave per SIMD of the chip (about a thousand) is the fastest while that leaves splits of up to 256
        # keys, half as many waves again from there on (a wave takes its keys one round after the other), and no
        # split is longer than 1,024 keys. Measured at 2,176 and 8,192 keys, 1 to 64 requests, 8 key/value heads: the
        # best split length is 64 to 128 keys for 8 x 2,176 keys in all, 256 for 32 x 2,176 (62 against 64 us with
        # 512), 512 for 48 and 64 x 2,176 (110 against 118 us with 1,024) and for 16 x 8,192, 1,024 for 32 x 8,192.
        want = max(1, T * Hkv * span // 1024)
        want = min(want, max(256, want * 2 // 3))
        # (splits of one round of 32 keys for one request of 2,100 keys, 525 waves: 3.64 against 3.66 ms a step; for two
        # requests 3.77 against 3.75: not taken)
        split_len = 64
        while split_len * 2 <= want and split_len < 1024:
            split_len *= 2
        # the splits cover the longest context this launch can meet: outside a graph the batch's own; inside one, what
        # the recorder says it will let the graph meet (``covered_context``: it replaces a graph before its contexts
        # outgrow that), not the bound of the block tables (max_model_len), whose splits would nearly all be empty blocks
        covered = batch.max_context_len
        if self.planned_context and self.covered_context:
            covered = min(covered, self.covered_context)
        n_splits = -(-covered // split_len)
        part_o = torch.empty((T, Hq, n_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, Hq, n_splits, 2), dtype=torch.float32, device=q.device)
        self._call("nhv_decode_attention_bf16", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(part_o),
                   _ptr(part_ml), _ptr(batch.token_req), _ptr(batch.positions), _ptr(block_tables),
                   block_tables.shape[1], T, Hq, Hkv, page_size, ctypes.c_float(scale), window, split_len, n_splits,
                   _stream(), lib=self.attention_lib(D))

    # -- matrix products of few rows: own kernel or one of the library's algorithms, by measurement --
    def blas_lib(self) -> ctypes.CDLL:
        """The wrapper of the vendor's matrix library, loaded when a product is first given to it."""
        if self._blas is None:
            self._blas = library.load_library("nhv_blas", BLAS_SOURCES, link=BLAS_LINK)
            self._blas.nhv_last_error.restype = ctypes.c_char_p
        return self._blas

    def _library_plan(self, M: int, N: int, K: int, float_result: bool) -> tuple[int, int]:
        """(plan, number of algorithms) of the library for this shape."""
        key = (M, N, K, float_result)
        got = self._plans.get(key)
        if got is None:
            plan, count = ctypes.c_int(), ctypes.c_int()
            self._call("nhv_library_gemm_plan", M, N, K, F32 if float_result else BF16, self.library_algorithms,
                       ctypes.c_size_t(self.library_workspace), ctypes.byref(plan), ctypes.byref(count), lib=self.blas_lib())
            got = self._plans[key] = (plan.value, count.value)
        return got

    def _library_product(self, x, w, out, algorithm: int) -> None:
        plan, _ = self._library_plan(x.shape[0], w.shape[0], x.shape[1], out.dtype == torch.float32)
        if self._workspace is None:
            self._workspace = torch.empty(self.library_workspace, dtype=torch.uint8, device=x.device)
        self._call("nhv_library_gemm", plan, algorithm, _ptr(x), _ptr(w), _ptr(out), _ptr(self._workspace),
                   ctypes.c_size_t(self.library_workspace), _stream(), lib=self.blas_lib())

    def _time_cold(self, run, repeats: int) -> float:
        """The shortest of ``repeats`` runs in milliseconds, each alone and after a read of 512 MB has swept the
        caches (the memory-side one holds 256 MB): in a decoding step a weight comes from memory, and a weight
        left in a cache by the run before would be measured 15 to 20 % too fast, by an amount that differs from
        kernel to kernel. The sweep reads, as the step before a product does: after a sweep that writes, the
        caches are full of lines that have to go back to memory while the product runs, which adds 10 to 35 us."""
        times = []
        for _ in range(repeats):
            self._sweep.sum()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            run()
            end.record()
            end.synchronize()
            times.append(start.elapsed_time(end))
        return min(times)

    def _choose(self, x, w, out, gated: bool = False) -> int | None:
        """How this product is done: ``OWN`` (the own kernel; with ``gated`` the one that also does the
        SiLU-and-multiply), the number of one of the library's algorithms (``gated``: followed by the
        SiLU-and-multiply kernel), ``RULE`` (measured, and nothing beat what the rule gives), or ``None`` if the
        shape was never measured (then the rule holds too: own kernel up to ``few_rows`` rows, ``torch.mm`` above).
        Which is fastest depends on the shape in ways no rule here captures, and the library's own first guess is
        often far from its best (a 5120 x 17408 weight against 8 rows: 112 us by its first guess, 37 us by another
        of its algorithms, 50 us by the own kernel; a 4096 x 12288 weight: 22, 22 and 25 us; the same weight
        against 128 rows: 67 us by ``torch.mm``, 43 us by the library's sixth guess; against 2,048 rows the first
        guess is as good as any). So a shape is timed in
        every way there is, once, and the answer is kept for the life of the process: a shape of up to
        ``library_rows`` rows while ``measure_linears`` is set (the run before a graph is recorded), a shape of
        more rows (a portion of a prompt) in the third step that meets it, since only the sizes that come again
        and again (portions that fill the token budget) are worth the 50 ms. An algorithm whose result differs
        from the trusted way's (own kernel, ``torch.mm``) by more than rounding, or from its own on a second run,
        is left out. The trusted way stays unless a library algorithm takes less than 0.95 of its time (0.90 for the
        gated projection)."""
        M, K = x.shape
        N = w.shape[0]
        float_result = out.dtype == torch.float32
        key = (M, N, K, float_result, gated)
        known = self.chosen.get(key)
        if known is not None or not self.measuring_allowed or torch.cuda.is_current_stream_capturing():
            return known
        many = M > self.library_rows
        if many:
            met, step = self._met.get(key, (0, -1))
            if step != self.step_number:                     # (a model's layers meet the same shape in one step)
                met += 1
                self._met[key] = (met, self.step_number)
            if not self.measure_many_rows or (met < 3 and not self.measure_linears):
                return None                                  # (before a graph is recorded every new shape is measured at once)
        elif not self.measure_linears:
            return None
        try:
            how = self._measure(x, w, out, gated, many)
        except torch.OutOfMemoryError:
            how = RULE if many else None                     # no room to measure: the rule
        finally:
            if many:
                self._sweep = None                           # (a step of prompt portions is followed by no end_measurements)
        if how is not None:
            self.chosen[key] = how
            if gated and how >= 0:
                self.chosen[(M, N, K, False, False)] = how   # the packed product that follows a refusal of gated_linear
        return how

    def _measure(self, x, w, out, gated: bool, many: bool) -> int:
        M, K = x.shape
        N = w.shape[0]
        float_result = out.dtype == torch.float32
        if self._sweep is None:
            self._sweep = torch.zeros(128 << 20, dtype=torch.float32, device="cuda")      # (a sum of floats is one kernel and no copy)
        packed = torch.empty((M, N), dtype=x.dtype, device=x.device) if gated else out

        def trusted():
            if many:
                torch.mm(x, w.t(), out=out)
            elif gated:
                self._call("nhv_gemm_skinny_glu_bf16", _ptr(x), _ptr(w), _ptr(out), M, N // 2, K, dtype_code(out), _stream())
            else:
                self._call("nhv_gemm_skinny_bf16", _ptr(x), _ptr(w), None, _ptr(out), M, N, K, dtype_code(out), _stream())

        def by_library(algorithm):
            def run():
                self._library_product(x, w, packed, algorithm)
                if gated:
                    self.silu_mul(packed, out)
            return run

        trusted()
        reference = out.clone()
        bound = (1e-3 if float_result else 2e-2) * max(float(reference.abs().max()), 1e-30)
        incumbent = RULE if many else OWN
        runs = {incumbent: trusted} if many or M <= self.few_rows else {}
        _, count = self._library_plan(M, N, K, float_result and not gated)
        for algorithm in range(min(count, 16) if many else count):
            run = by_library(algorithm)
            try:
                out.zero_()
                run()
                first = out.clone()
                out.zero_()
                run()
            except KernelError:
                continue
            if torch.equal(first, out) and float((out - reference).abs().max()) <= bound:
                runs[algorithm] = run
            del first
        if not runs:
            return RULE                                      # the library has no algorithm for this shape that holds
        # every way once; then the four fastest, and the trusted way whatever its place, eight times more each (the
        # shortest run counts: a single run is off by up to a tenth, and a choice made on it changes from one start of
        # the engine to the next, by up to 5 % of a decoding step)
        once = sorted((self._time_cold(run, 1), how) for how, run in runs.items())
        finalists = once[:4] + [(t, h) for t, h in once[4:] if h == incumbent]
        best = sorted((min(t, self._time_cold(runs[how], 8)), how) for t, how in finalists)
        how = best[0][1]
        incumbent_time = next((t for t, h in best + once if h == incumbent), None)
        # (the fused gated kernel gives way only to a clear win: the library's way is two kernels, and the second one's
        # cost inside a step is the harder one to measure alone)
        if incumbent_time is not None and how != incumbent and best[0][0] >= (0.90 if gated else 0.95) * incumbent_time:
            how = incumbent
        library_times = [t for t, h in best + once if h >= 0]
        if incumbent_time is not None and library_times:
            self.times[(M, N, K, float_result, gated)] = (incumbent_time, min(library_times))
        if os.environ.get("NHV_SHOW_MEASUREMENTS"):
            name = {OWN: "own", RULE: "torch.mm"}
            first_guess = next((t for t, h in once if h == 0), float("nan"))
            print(f"[nanohybrid_vlm_amd] {'gated ' if gated else ''}product {M} x {K} . {N} x {K}: {name[incumbent]} "
                  f"{'-' if incumbent_time is None else format(1e3 * incumbent_time, '.1f')} us, library's first guess "
                  f"{1e3 * first_guess:.1f} us, fastest {1e3 * best[0][0]:.1f} us ({name.get(best[0][1], best[0][1])} "
                  f"of {len(runs)} ways); taken: {name.get(how, how)}", file=sys.stderr, flush=True)
        return how

    # -- the table of choices, so that a process can run by what another one measured --
    def choices_table(self, chosen: dict | None = None) -> dict[str, int]:
        """A table of choices (default: the one in force), by shape: "M,N,K,float result,gated" -> -1 (own kernel),
        -2 (the rule: ``torch.mm``) or the number of a library algorithm."""
        chosen = self.chosen if chosen is None else chosen
        return {",".join(str(int(v)) for v in key): how for key, how in sorted(chosen.items())}

    def parse_choices(self, table: dict[str, int]) -> dict[tuple, int]:
        """A table as ``choices_table`` gives it, as a table of this backend's own kind. Every entry is checked
        now: its shape's form, and a library algorithm's number against the library's list for that shape."""
        out = {}
        for text, how in table.items():
            parts = text.split(",")
            if len(parts) != 5:
                raise KernelError(f"a product's shape is 'M,N,K,float result,gated', got '{text}'")
            M, N, K, f, g = (int(v) for v in parts)
            if not isinstance(how, int) or how < RULE:
                raise KernelError(f"choice {how!r} for the product '{text}' is neither -1, -2 nor an algorithm's number")
            if how >= 0:
                _, count = self._library_plan(M, N, K, bool(f) and not bool(g))
                if how >= count:
                    raise KernelError(f"choice {how} for the product '{text}': the library names {count} algorithms for this shape")
            out[(M, N, K, bool(f), bool(g))] = how
        return out

    def use_choices(self, table: dict | None, measuring: bool) -> None:
        """Puts an engine's table in force (None: the process-wide one) and says whether shapes that it lacks may be timed."""
        self.chosen = self.shared_chosen if table is None else table
        self.measuring_allowed = bool(measuring)

    def end_measurements(self) -> None:
        """Gives the scratch memory of the measurements back (what was measured stays known)."""
        self._sweep = None

    def linear(self, x, w, bias, out):
        M, K = x.shape
        N = w.shape[0]
        if x.dtype == torch.bfloat16 and K % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0:
            if bias is None and not self.own_kernels_only and (M <= self.library_rows or out.dtype == torch.bfloat16):
                how = self._choose(x, w, out)
                if how is not None and how >= 0:
                    return self._library_product(x, w, out, how)
            if M <= self.few_rows or (M <= 64 and self.own_kernels_only):
                return self._call("nhv_gemm_skinny_bf16", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), M, N, K,
                                  dtype_code(out), _stream())
            if out.dtype == torch.bfloat16 and bias is None and not self.own_kernels_only:
                # many rows: the library's matrix product (the reference's linears are library calls too,
                # nanovllm/layers/linear.py:88,192)
                torch.mm(x, w.t(), out=out)
                return None
            if out.dtype == torch.float32 and bias is None and not self.own_kernels_only and _MM_GIVES_FLOAT32:
                # the logits of many rows: the library's product with float sums and a float result (270 us for 64
                # rows of the 8B head against 400 us of the own kernel for 17 to 64 rows, which takes 64 rows a call)
                torch.mm(x, w.t(), out_dtype=torch.float32, out=out)
                return None
            if out.dtype == torch.float32:
                for m0 in range(0, M, 64):          # float32 output (logits), or more rows than a graph may hold in one call
                    m1 = min(M, m0 + 64)
                    self._call("nhv_gemm_skinny_bf16", _ptr(x[m0:m1]), _ptr(w), _ptr(bias), _ptr(out[m0:m1]),
                               m1 - m0, N, K, dtype_code(out), _stream())
                return None
        self._call("nhv_gemm_generic", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), M, N, K, dtype_code(x),
                   dtype_code(out), _stream())

    norm_kernel_ms = 0.003        # what a norm's own kernel costs in a decoding step, about

    def _measured(self, x, w, gated: bool):
        """(the choice for this shape, (ms of the own kernel, ms of the library's best) or None); the shape is
        measured here if it is due, as ``linear`` would have it measured."""
        M, K = x.shape
        key = (M, w.shape[0], K, False, gated)
        how = self.chosen.get(key)
        if how is None and self.measure_linears and self.measuring_allowed and not torch.cuda.is_current_stream_capturing():
            scratch = torch.empty((M, w.shape[0] // 2 if gated else w.shape[0]), dtype=x.dtype, device=x.device)
            how = self._choose(x, w, scratch, gated=gated)
        return how, self.times.get(key)

    def fusion_pays(self, x, w, gated: bool = False) -> bool:
        """For a product whose rows come as a sum that still lacks its norm's scales: whether the own kernel, which
        scales its sums itself, beats what this shape is otherwise done by. Where a measurement chose a library
        algorithm for the shape, that algorithm and a kernel that scales the rows first have to be slower together
        than the own kernel alone."""
        if self.own_kernels_only:
            return True
        how, times = self._measured(x, w, gated)
        if how is None or how < 0:
            return True
        if times is None:
            return False                                     # (a choice from a table: followed as it stands)
        own, library = times
        return own <= library + self.norm_kernel_ms

    def addition_pays(self, x, w, reader_w=None, reader_gated: bool = False) -> bool:
        """For a product whose result is about to be added to the residual stream and normed: whether the own
        kernel, which makes the addition itself, is the one to take. That saves the norm's kernel only if the product
        that reads the norm (``reader_w``, of the same rows) scales its rows itself, so the two are priced together:
        own kernels for both, against each one's best way and the norm's kernel between them. Without times for both
        shapes the own kernel is taken where it is this shape's choice anyway."""
        if self.own_kernels_only:
            return True
        how, times = self._measured(x, w, False)
        if how is None or how < 0:
            return True
        if times is None or reader_w is None:
            return False
        reader_how = self.chosen.get((x.shape[0], reader_w.shape[0], reader_w.shape[1], False, reader_gated))
        reader_times = self.times.get((x.shape[0], reader_w.shape[0], reader_w.shape[1], False, reader_gated))
        if reader_how is None:
            return False                                     # (the reader's shape is not measured yet: next time)
        if reader_times is None:
            if reader_how >= 0:
                return False
            reader_times = (0.0, 0.0)                        # the own kernel is the reader's way whatever is fused
        own, library = times
        reader_own, reader_library = reader_times
        return own + reader_own <= min(own, library) + self.norm_kernel_ms + min(reader_own, reader_library)

    def fused_linear(self, x, w, bias, out, gated=False, row_scales=None, residual=None, sum_out=None, ss_out=None, next_w=None):
        """The own few-rows product with what it may take over. ``row_scales`` = (squares [M, tiles], eps): x is a
        sum whose rows still lack their norm's scales, which are applied to the finished sums. ``residual``: the
        result is added to it (in place); ``sum_out`` gets the sum times ``next_w`` (the next norm's weight), rounded,
        and ``ss_out`` the tiles' shares of the rows' sums of squares (``out`` is then not written)."""
        M, K = x.shape
        N = w.shape[0] // 2 if gated else w.shape[0]
        ss, eps = row_scales if row_scales is not None else (None, 0.0)
        self._call("nhv_gemm_fewrows_fused_bf16", _ptr(x), _ptr(ss), 0 if ss is None else ss.shape[1], ctypes.c_float(eps),
                   _ptr(w), _ptr(bias), _ptr(out), M, N, K, BF16 if out is None else dtype_code(out), int(gated),
                   _ptr(residual), F32 if residual is None else dtype_code(residual), _ptr(sum_out), _ptr(ss_out),
                   _ptr(next_w), F32 if next_w is None else dtype_code(next_w), _stream())

    def scale_rows(self, x, squares, eps, out):
        self._call("nhv_scale_rows", _ptr(x), _ptr(squares), squares.shape[1], ctypes.c_float(eps), _ptr(out), x.shape[0],
                   x.shape[1], _stream())

    def gated_linear(self, x, w, out) -> bool:
        """silu(x Wg^T) * (x Wu^T) in one kernel, if this batch is one for the few-rows kernel; else False."""
        M, K = x.shape
        if (x.dtype == torch.bfloat16 and K % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
                and (M <= self.few_rows or (M <= 64 and self.own_kernels_only))):
            if M <= self.few_rows and not self.own_kernels_only:
                how = self._choose(x, w, out, gated=True)
                if how is not None and how >= 0:
                    return False                             # the library's product, then silu_mul
            self._call("nhv_gemm_skinny_glu_bf16", _ptr(x), _ptr(w), _ptr(out), M, out.shape[1], K, dtype_code(out),
                       _stream())
            return True
        return False

    def sample(self, logits, temperatures, keys, tokens):
        n, V = logits.shape
        pieces = self.lib.nhv_sample_pieces(V)
        piece_value = torch.empty((n, pieces), dtype=torch.float32, device=logits.device)
        piece_index = torch.empty((n, pieces), dtype=torch.int32, device=logits.device)
        self._call("nhv_sample", _ptr(logits), _ptr(temperatures), _ptr(keys), _ptr(tokens), n, V, _ptr(piece_value),
                   _ptr(piece_index), _stream())


def measured_peaks(device="cuda:0", read_bytes: int = 4 << 30, gemm_size: int = 8192) -> dict:
    """What this very GPU gives, for fractions beside those of the published peaks: the rate of a kernel that only
    reads ``read_bytes`` from memory (each byte once, far more than the caches hold), and the rate of a bfloat16
    matrix product of ``gemm_size``^3 by the vendor's library. The shortest of five runs each."""
    b = backend()
    data = torch.empty(read_bytes // 1024 * 1024, dtype=torch.uint8, device=device).zero_()
    sink = torch.zeros(1, dtype=torch.float32, device=device)

    def shortest(run, n=5):
        best = float("inf")
        for _ in range(n + 1):                      # (the first run is a warm-up)
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            run()
            end.record()
            end.synchronize()
            best = min(best, start.elapsed_time(end) * 1e-3)
        return best

    read_s = shortest(lambda: b._call("nhv_measure_read", _ptr(data), _ptr(sink), ctypes.c_size_t(data.numel()), _stream()))
    del data
    a = torch.randn(gemm_size, gemm_size, dtype=torch.bfloat16, device=device)
    c = torch.empty_like(a)
    gemm_s = shortest(lambda: torch.mm(a, a.t(), out=c))
    return {"hbm_read_GBs": read_bytes // 1024 * 1024 / read_s / 1e9, "gemm_bf16_TFLOPs": 2.0 * gemm_size ** 3 / gemm_s / 1e12}


class KernelTimes:
    """Per-kernel device time of everything launched inside ``with kernel_times() as t`` (events around every
    call into the library; not for use while a graph is recorded). ``t.table()`` after the block."""

    def __init__(self):
        self.records: list[tuple[str, torch.cuda.Event, torch.cuda.Event]] = []

    def summary(self) -> dict[str, tuple[int, float]]:
        torch.cuda.synchronize()
        out: dict[str, tuple[int, float]] = {}
        for name, start, end in self.records:
            n, ms = out.get(name, (0, 0.0))
            out[name] = (n + 1, ms + start.elapsed_time(end))
        return out

    def table(self) -> str:
        rows = sorted(self.summary().items(), key=lambda kv: -kv[1][1])
        total = sum(ms for _, (_, ms) in rows) or 1.0
        lines = [f"{'kernel':40s} {'calls':>7s} {'total ms':>10s} {'mean us':>9s} {'share':>6s}"]
        for name, (n, ms) in rows:
            lines.append(f"{name:40s} {n:7d} {ms:10.3f} {ms / n * 1e3:9.1f} {100 * ms / total:5.1f}%")
        return "\n".join(lines)


class kernel_times:
    def __enter__(self) -> KernelTimes:
        self.times = KernelTimes()
        b = backend()
        self._old = b._call
        times = self.times

        def timed_call(fn_name, *args, lib=None):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            self._old(fn_name, *args, lib=lib)
            end.record()
            times.records.append((fn_name, start, end))

        b._call = timed_call
        return self.times

    def __exit__(self, *exc):
        backend()._call = self._old
        return False


_backend = None


def backend():
    global _backend
    if _backend is None:
        _backend = NativeBackend()
    return _backend


def set_backend(obj) -> None:
    """Replace the kernel library (tests of the engine's logic on a machine
    without a GPU put a stand-in here; the engine itself never does)."""
    global _backend
    _backend = obj


# ------------------------------------------------------------------ work that a product takes over from its neighbours
@dataclass
class AddTo:
    """What a part is handed in place of nothing when its result is about to be added to the residual stream and
    normed: the stream, the weight and eps of the norm that follows, and (if known) the first product of the part
    that reads that norm, as (weight, gated): whether making the addition in the product's kernel pays depends on
    whether that reader scales its rows itself."""

    residual: torch.Tensor
    norm_weight: torch.Tensor
    eps: float
    reader: tuple | None = None


@dataclass
class Summed:
    """What ``linear(..., add_to=AddTo(...))`` returns where the product's own kernel has made the addition: the
    residual stream holds the sum already. ``weighted`` is the sum times the weight of the norm that follows, in
    the rows' element type; ``squares`` [rows, tiles] holds every tile's share of each row's sum of squares. What the
    norm still has to do is scale the rows: a product that reads ``Normed(summed)`` does that itself."""

    weighted: torch.Tensor
    squares: torch.Tensor
    residual: torch.Tensor
    norm_weight: torch.Tensor
    eps: float

    @property
    def shape(self):
        return self.weighted.shape


@dataclass
class Normed:
    """The norm of a ``Summed`` with the scaling of its rows left to the product that reads it (``linear``,
    ``gated_linear``: a product is linear in its rows, so it scales its own sums). ``tensor()`` is the norm as a
    tensor, for any other reader (one small kernel)."""

    summed: Summed

    @property
    def shape(self):
        return self.summed.weighted.shape

    def tensor(self) -> torch.Tensor:
        s = self.summed
        out = torch.empty_like(s.weighted)
        backend().scale_rows(s.weighted, s.squares, float(s.eps), out)
        return out


def dense(x):
    """``x`` as a tensor, whatever work was left undone in it."""
    if isinstance(x, Normed):
        return x.tensor()
    if isinstance(x, Summed):
        raise KernelError("a sum that was made for a norm (ops.Summed) goes through that norm, not anywhere else")
    return x


def _may_fuse(x: torch.Tensor, w: torch.Tensor) -> bool:
    b = backend()
    return (getattr(b, "fuse_norms", False) and hasattr(b, "fused_linear") and x.dtype == torch.bfloat16
            and x.shape[0] <= getattr(b, "few_rows", 0) and x.shape[1] % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def _fusion_pays(x: torch.Tensor, w: torch.Tensor, gated: bool) -> bool:
    pays = getattr(backend(), "fusion_pays", None)
    return True if pays is None else pays(x, w, gated=gated)


def _addition_pays(x: torch.Tensor, w: torch.Tensor, add_to: AddTo) -> bool:
    pays = getattr(backend(), "addition_pays", None)
    if pays is None:
        return True
    reader_w, reader_gated = add_to.reader if add_to.reader is not None else (None, False)
    return pays(x, w, reader_w, reader_gated)


# ------------------------------------------------------------------ checked entry points
def embed(ids: torch.Tensor, table: torch.Tensor, scale: float | None = None) -> torch.Tensor:
    """Rows of ``table``; with ``scale`` each row times it (multiplied in float, rounded once)."""
    _need(table.dim() == 2, "embed: the table must be [vocab, width]")
    _dense(table, "embed: table")
    _dense(ids, "embed: ids", (ids.shape[0],), torch.int32)
    dtype_code(table)
    out = torch.empty((ids.shape[0], table.shape[1]), dtype=table.dtype, device=table.device)
    if scale is None:
        backend().embed(ids, table, out)
    else:
        backend().embed(ids, table, out, float(scale))
    return out


def soft_cap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    _dense(logits, "soft_cap: logits", dtype=torch.float32)
    _need(cap > 0, lambda: f"soft_cap: the cap must be positive, got {cap}")
    if logits.numel():
        backend().soft_cap(logits, float(cap))
    return logits


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, residual: torch.Tensor | None = None,
            start_residual: bool = False, residual_float32: bool = True):
    """``rmsnorm(x, w, eps)``: the norm of x.
    ``residual=r``: r += x in place (the sum is taken in float and normed unrounded; r keeps it in its own element
    type) and the norm of the sum is returned.
    ``start_residual=True``: returns (norm of x, the residual that later norms add to): a new float32 tensor holding
    x, or, with ``residual_float32=False``, x itself (which later calls then add to in place)."""
    _need(x.dim() == 2, "rmsnorm: x must be [tokens, width]")
    _dense(x, "rmsnorm: x")
    _dense(w, "rmsnorm: weight", (x.shape[1],))
    _need(w.dtype == x.dtype or w.dtype == torch.float32,
          lambda: f"rmsnorm: weight of {w.dtype} with activations of {x.dtype}")
    dtype_code(x)
    y = torch.empty_like(x)
    if start_residual:
        _need(residual is None, "rmsnorm: a residual is either started or added to")
        if not residual_float32 and x.dtype != torch.float32:
            backend().rmsnorm(x, None, 0, w, y, float(eps))
            return y, x
        residual = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        backend().rmsnorm(x, residual, 2, w, y, float(eps))
        return y, residual
    if residual is not None:
        _dense(residual, "rmsnorm: residual", tuple(x.shape))
        _need(residual.dtype == x.dtype or residual.dtype == torch.float32,
              lambda: f"rmsnorm: residual of {residual.dtype} with rows of {x.dtype}")
        backend().rmsnorm(x, residual, 1, w, y, float(eps))
        return y
    backend().rmsnorm(x, None, 0, w, y, float(eps))
    return y


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "silu_mul: input must be [tokens, 2 * width]")
    _dense(gate_up, "silu_mul: input")
    dtype_code(gate_up)
    out = torch.empty((gate_up.shape[0], gate_up.shape[1] // 2), dtype=gate_up.dtype, device=gate_up.device)
    backend().silu_mul(gate_up, out)
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    _need(x.dim() == 2, "gather_rows: x must be [tokens, width]")
    _dense(x, "gather_rows: x")
    _dense(rows, "gather_rows: rows", (rows.shape[0],), torch.int32)
    dtype_code(x)
    out = torch.empty((rows.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    backend().gather_rows(x, rows, out)
    return out


def qk_rope_write(qkv, bias, q_norm_w, k_norm_w, eps, cos_sin, positions, slot_mapping, k_cache, v_cache,
                  num_heads: int, num_kv_heads: int, head_dim: int, write_kv: bool = True,
                  pair_axes: torch.Tensor | None = None) -> torch.Tensor:
    """Splits the packed projection, norms and turns q and k, stores k and v in the
    paged cache and returns q as [tokens, heads, head_dim].
    ``positions``: [tokens], or [axes, tokens] with ``pair_axes`` [rotary size / 2] (int32): the axis whose
    coordinate turns each pair (without ``pair_axes`` every pair turns by the first axis)."""
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _dense(qkv, "qk_rope_write: qkv", (T, width))
    dtype_code(qkv)
    if bias is not None:
        _dense(bias, "qk_rope_write: bias", (width,), qkv.dtype)
    for name, w in (("q_norm", q_norm_w), ("k_norm", k_norm_w)):
        if w is not None:
            _dense(w, f"qk_rope_write: {name} weight", (head_dim,))
            _need(w.dtype == qkv.dtype or w.dtype == torch.float32, lambda: f"qk_rope_write: {name} weight of {w.dtype}")
    _need((q_norm_w is None) == (k_norm_w is None), "qk_rope_write: q and k norm weights come together")
    if q_norm_w is not None:
        _need(q_norm_w.dtype == k_norm_w.dtype, "qk_rope_write: q and k norm weights differ in element type")
    rot = 0
    if cos_sin is not None:
        _need(cos_sin.dim() == 2, "qk_rope_write: rotation table must be [positions, rotary size]")
        _dense(cos_sin, "qk_rope_write: rotation table", dtype=torch.float32)
        rot = cos_sin.shape[1]
        _need(rot % 2 == 0 and rot <= head_dim, lambda: f"qk_rope_write: rotary size {rot} with head size {head_dim}")
    if positions.dim() == 1:
        _dense(positions, "qk_rope_write: positions", (T,), torch.int32)
    else:
        _need(positions.dim() == 2 and positions.shape[1] == T and positions.shape[0] >= 1,
              lambda: f"qk_rope_write: positions {tuple(positions.shape)} for {T} tokens (want [axes, tokens])")
        _dense(positions, "qk_rope_write: positions", dtype=torch.int32)
    if pair_axes is not None:
        _need(cos_sin is not None, "qk_rope_write: axes of pairs without a rotation table")
        _dense(pair_axes, "qk_rope_write: pair_axes", (rot // 2,), torch.int32)
        _need(positions.dim() == 2, "qk_rope_write: pair_axes go with positions [axes, tokens]")
    if write_kv:
        _dense(slot_mapping, "qk_rope_write: slot_mapping", (T,), torch.int32)
        _need(k_cache.dim() == 4 and tuple(k_cache.shape[2:]) == (num_kv_heads, head_dim),
              lambda: f"qk_rope_write: cache shape {tuple(k_cache.shape)} does not fit {num_kv_heads} heads of {head_dim}")
        _dense(k_cache, "qk_rope_write: k_cache", dtype=qkv.dtype)
        _dense(v_cache, "qk_rope_write: v_cache", tuple(k_cache.shape), qkv.dtype)
    q_out = torch.empty((T, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    backend().qk_rope_write(qkv, bias, q_norm_w, k_norm_w, float(eps), cos_sin, rot, positions,
                            slot_mapping if write_kv else None, q_out, k_cache if write_kv else None,
                            v_cache if write_kv else None, num_heads, num_kv_heads, head_dim, write_kv,
                            **({} if pair_axes is None else {"pair_axes": pair_axes}))
    return q_out


def paged_attention(q, k_cache, v_cache, batch: AttentionBatch, block_tables, scale: float,
                    window: int | None = None) -> torch.Tensor:
    _need(q.dim() == 3, "attention: q must be [tokens, heads, head_dim]")
    T, Hq, D = q.shape
    _dense(q, "attention: q")
    dtype_code(q)
    _need(k_cache.dim() == 4 and k_cache.shape[3] == D, lambda: f"attention: cache shape {tuple(k_cache.shape)} with head size {D}")
    _dense(k_cache, "attention: k_cache", dtype=q.dtype)
    _dense(v_cache, "attention: v_cache", tuple(k_cache.shape), q.dtype)
    Hkv = k_cache.shape[2]
    _need(Hq % Hkv == 0, lambda: f"attention: {Hq} query heads are not a multiple of {Hkv} key heads")
    _need(T == batch.num_tokens, lambda: f"attention: {T} tokens but the batch has {batch.num_tokens}")
    _dense(batch.token_req, "attention: token_req", (T,), torch.int32)
    _dense(batch.positions, "attention: positions", (T,), torch.int32)
    _need(block_tables.dim() == 2 and block_tables.shape[0] == batch.num_requests,
          lambda: f"attention: block tables {tuple(block_tables.shape)} for {batch.num_requests} requests")
    _dense(block_tables, "attention: block_tables", dtype=torch.int32)
    page_size = k_cache.shape[1]
    _need(block_tables.shape[1] * page_size >= batch.max_context_len,
          lambda: f"attention: block tables of {block_tables.shape[1]} pages of {page_size} are too short for "
          f"{batch.max_context_len} keys")
    out = torch.empty_like(q)
    backend().paged_attention(q, k_cache, v_cache, out, batch, block_tables, float(scale), int(window or 0))
    return out


def linear(x, w: torch.Tensor, bias: torch.Tensor | None = None, out_dtype=None, add_to: AddTo | None = None):
    """x[M, K] . w[N, K]^T (+ bias), accumulated in float. ``out_dtype`` may be
    float32 for bfloat16 inputs (the logits).
    ``x`` may be a ``Normed``: where the product's kernel can, it scales the rows itself.
    ``add_to``: the residual stream [M, N] that the caller is about to add the result to, and the norm that follows.
    Where the product's kernel can, it makes the addition itself (in float; the stream is rewritten) and a ``Summed``
    is returned, which that norm takes; otherwise the plain result is returned and the stream is left alone."""
    normed = x if isinstance(x, Normed) else None
    if normed is not None:
        x = normed.summed.weighted
        _dense(w, "linear: w", dtype=x.dtype)
        if not (_may_fuse(x, w) and _fusion_pays(x, w, False)):
            x, normed = normed.tensor(), None
    _need(x.dim() == 2 and w.dim() == 2, "linear: x must be [rows, in] and w [out, in]")
    _need(x.shape[1] == w.shape[1], lambda: f"linear: x has {x.shape[1]} columns but w has {w.shape[1]}")
    _dense(x, "linear: x")
    _dense(w, "linear: w", dtype=x.dtype)
    dtype_code(x)
    if bias is not None:
        _dense(bias, "linear: bias", (w.shape[0],), x.dtype)
    out_dtype = out_dtype or x.dtype
    _need(out_dtype == x.dtype or out_dtype == torch.float32, lambda: f"linear: output of {out_dtype} from {x.dtype}")
    M, N = x.shape[0], w.shape[0]
    scales = None if normed is None else (normed.summed.squares, float(normed.summed.eps))
    if add_to is not None and out_dtype == x.dtype and _may_fuse(x, w) and (normed is not None or _addition_pays(x, w, add_to)):
        residual = add_to.residual
        _dense(residual, "linear: residual", (M, N))
        _need(residual.dtype == x.dtype or residual.dtype == torch.float32, lambda: f"linear: residual of {residual.dtype} with rows of {x.dtype}")
        _dense(add_to.norm_weight, "linear: the next norm's weight", (N,))
        dtype_code(add_to.norm_weight)
        weighted = torch.empty((M, N), dtype=x.dtype, device=x.device)
        squares = torch.empty((M, (N + 15) // 16), dtype=torch.float32, device=x.device)
        backend().fused_linear(x, w, bias, None, row_scales=scales, residual=residual, sum_out=weighted, ss_out=squares,
                               next_w=add_to.norm_weight)
        return Summed(weighted, squares, residual, add_to.norm_weight, add_to.eps)
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if normed is not None:
        backend().fused_linear(x, w, bias, out, row_scales=scales)
    else:
        backend().linear(x, w, bias, out)
    return out


def gated_linear(x, w: torch.Tensor) -> torch.Tensor:
    """silu(x . w[:I]^T) * (x . w[I:]^T) for a packed gate | up matrix w[2 I, K]: fused into one kernel for
    few rows, else the matrix product followed by ``silu_mul``. ``x`` may be a ``Normed`` (see ``linear``)."""
    if isinstance(x, Normed):
        normed, x = x, x.summed.weighted
        _need(w.dim() == 2 and w.shape[0] % 2 == 0 and x.shape[1] == w.shape[1], "gated_linear: w must be [2 * out, in]")
        _dense(w, "gated_linear: w", dtype=x.dtype)
        if _may_fuse(x, w) and _fusion_pays(x, w, True):
            out = torch.empty((x.shape[0], w.shape[0] // 2), dtype=x.dtype, device=x.device)
            backend().fused_linear(x, w, None, out, gated=True, row_scales=(normed.summed.squares, float(normed.summed.eps)))
            return out
        x = normed.tensor()
    _need(x.dim() == 2 and w.dim() == 2 and w.shape[0] % 2 == 0, "gated_linear: x must be [rows, in] and w [2 * out, in]")
    _need(x.shape[1] == w.shape[1], lambda: f"gated_linear: x has {x.shape[1]} columns but w has {w.shape[1]}")
    _dense(x, "gated_linear: x")
    _dense(w, "gated_linear: w", dtype=x.dtype)
    dtype_code(x)
    fused = getattr(backend(), "gated_linear", None)
    if fused is not None:
        out = torch.empty((x.shape[0], w.shape[0] // 2), dtype=x.dtype, device=x.device)
        if fused(x, w, out):
            return out
    return silu_mul(linear(x, w))


def sample(logits: torch.Tensor, temperatures: torch.Tensor, keys: torch.Tensor) -> torch.Tensor:
    _need(logits.dim() == 2, "sample: logits must be [rows, vocab]")
    n = logits.shape[0]
    _dense(logits, "sample: logits", dtype=torch.float32)
    _dense(temperatures, "sample: temperatures", (n,), torch.float32)
    _dense(keys, "sample: keys", (n,), torch.int64)
    tokens = torch.empty((n,), dtype=torch.int32, device=logits.device)
    backend().sample(logits, temperatures, keys, tokens)
    return tokens
