"""The ``runtime.launch()`` executor seam for the gfx950 lane.

Tessera dispatches a compiled artifact by looking ``(target, compiler_path)`` up
in its execution matrix and calling the executor function the row names
(``python/tessera/runtime.py:31008-31077``,
``python/tessera/compiler/execution_matrix.py:38-77,4095-4111``).  Adding a lane
is three pieces — an executor function, a ``KNOWN_EXECUTORS`` entry and an
``ExecutionRow`` — and this module holds all three for target ``rocm_gfx950``,
in the reference's own shapes, so a maintainer can paste the rows into the matrix
and the functions into the executor table unchanged.

Executor contract (``runtime.py:2078-2143, 6582-6766, 7229-7475, 1826-1902``):
``executor(artifact, args) -> ndarray | (ndarray, execution_kind)``; metadata
carries ``target``, ``compiler_path``, ``executable``, ``arg_names``,
``output_name`` and ``ops = [{op_name, result, operands, kwargs}]``;
``ValueError`` for a bad op / dtype / shape, ``RuntimeError`` for a device
failure, :class:`~tessera_amd.lane.LaneUnavailable` when the lane is absent;
:func:`launch` turns any raise into ``runtime_status="invalid_artifact"``.
"""
from __future__ import annotations

import hashlib
import time
from dataclasses import dataclass, field
from typing import Any, Callable, Mapping, Optional

import numpy as np

from . import bf16 as _bf16
from . import lane as _lane
from . import ops as _ops
from .lane import LaneUnavailable

TARGET = "rocm_gfx950"


@dataclass
class RuntimeArtifact:
    """The fields of ``tessera.runtime.RuntimeArtifact`` the executors read
    (``runtime.py:141-149``)."""
    graph_ir: str = ""
    schedule_ir: str = ""
    tile_ir: str = ""
    target_ir: str = ""
    metadata: Optional[dict] = None
    abi_signature: str = ""

    @property
    def artifact_hash(self) -> str:
        h = hashlib.sha256()
        for part in (self.graph_ir, self.schedule_ir, self.tile_ir, self.target_ir, repr(sorted(
                (k, repr(v)) for k, v in (self.metadata or {}).items()))):
            h.update(part.encode())
        return h.hexdigest()


@dataclass(frozen=True)
class ExecutionRow:
    """Same fields as ``compiler/execution_matrix.py:38-77`` (forward rows)."""
    target: str
    compiler_path: str
    execution_kind: str
    executable: bool
    executor_id: Optional[str]
    runtime_status: str
    reason: str = ""
    execution_mode: str = ""
    direction: str = "forward"
    op_family: str = ""


#: docstring registry, as ``KNOWN_EXECUTORS`` (``execution_matrix.py:103``).
KNOWN_EXECUTORS: dict[str, str] = {
    "gfx950_gemm": "single tessera.matmul/gemm/fused_epilogue op, rank-2, f16/bf16 -> f32 (optional bias[N] "
                   "+ relu/gelu/silu fused) or int8 -> int32, hand-written CDNA4 MFMA GEMM "
                   "(tessera_gfx950_gemm_* C ABI)",
    "gfx950_flash_attn": "flash_attn / multi_head / gqa / mqa attention forward, f16/bf16 -> f32, "
                         "causal + GQA, MFMA FA-2 (tessera_gfx950_flash_attn_gqa_* C ABI)",
    "gfx950_flash_attn_bwd": "flash_attn_bwd / flash_attn_vjp: (dO, Q, K, V) -> (dQ, dK, dV) f32, causal + GQA, "
                             "forward recomputed on device (tessera_gfx950_flash_attn_bwd_* C ABI)",
    "gfx950_moe_transport": "tessera.moe_dispatch / moe_combine / grouped_gemm / grouped_swiglu on "
                            "device gather, slot-ordered scatter-add and grouped MFMA GEMM",
    "gfx950_quant_gemm": "tessera.fp8_gemm (e4m3 codes + per-tensor scales) and tessera.w8a8_gemm "
                         "(int8 + per-row / per-column scales)",
}

_COMMON = dict(target=TARGET, execution_kind="native_gpu", executable=True, runtime_status="success",
               execution_mode="hip_runtime")
#: The lane's execution-matrix rows as plain field dicts (the fields of the reference's
#: ``ExecutionRow``, ``compiler/execution_matrix.py:38-77``), so they can be built with
#: whichever row class the host hands to :func:`tessera_amd.install.install`.
ROW_FIELDS: tuple = (
    dict(_COMMON, compiler_path="gfx950_gemm", executor_id="gfx950_gemm",
         reason="matmul runs the hand-written gfx950 MFMA GEMM through the "
                "tessera_gfx950_gemm_{f16,bf16,i8_i32} C ABI symbols"),
    dict(_COMMON, compiler_path="gfx950_flash_attn", executor_id="gfx950_flash_attn",
         reason="attention forward runs the hand-written gfx950 MFMA FA-2 kernel (causal, GQA, LSE)"),
    dict(_COMMON, compiler_path="gfx950_flash_attn_bwd", executor_id="gfx950_flash_attn_bwd",
         reason="attention backward runs the gfx950 MFMA dQ and dK/dV kernels; O and the "
                "log-sum-exp are recomputed by the forward kernel (nothing saved)",
         direction="backward", op_family="flash_attn"),
    dict(_COMMON, compiler_path="gfx950_moe_transport", executor_id="gfx950_moe_transport",
         reason="MoE dispatch / combine / grouped GEMM / grouped SwiGLU on the gfx950 lane"),
    dict(_COMMON, compiler_path="gfx950_quant_gemm", executor_id="gfx950_quant_gemm",
         reason="fp8-e4m3 and int8 W8A8 GEMM on the gfx950 MFMA lane"),
)
EXECUTION_ROWS: dict[tuple[str, str], ExecutionRow] = {
    (f["target"], f["compiler_path"]): ExecutionRow(**f) for f in ROW_FIELDS}


def lookup(target: str, compiler_path: str) -> Optional[ExecutionRow]:
    return EXECUTION_ROWS.get((target, compiler_path))


def lane_default_available() -> bool:
    """The cached host probe a ``JitFn._uses_<lane>_default()`` predicate consults
    before stamping an artifact executable (``compiler/jit.py:302-326``)."""
    return _lane.available()


# ---- argument plumbing -----------------------------------------------------------------
# What the reference's launch does with its ``args`` (runtime.py:44363-44384): a mapping is
# taken by name, a bare value is one positional argument, positions follow ``arg_names``,
# and a short argument list is a ValueError naming what is absent.

def _named_args(args: Any, arg_names: list) -> dict:
    if isinstance(args, Mapping):
        return {key: args[key] for key in args}
    positional = [] if args is None else list(args) if isinstance(args, (list, tuple)) else [args]
    absent = arg_names[len(positional):]
    if absent:
        raise ValueError("launch args missing value(s): " + ", ".join(absent))
    return dict(zip(arg_names, positional))


def _host_array(value: Any):
    """The numpy view of an operand: tensor wrappers are unwrapped (a ``numpy()`` method,
    else a ``_data`` payload), bf16 arrays pass through as they are."""
    to_numpy = getattr(value, "numpy", None)
    if callable(to_numpy):
        return np.asarray(to_numpy())
    payload = getattr(value, "_data", value)
    return payload if _bf16.is_bf16(payload) else np.asarray(payload)


def _single_op(artifact: RuntimeArtifact, allowed: tuple, who: str) -> dict:
    ops = list((artifact.metadata or {}).get("ops") or [])
    name = str(ops[0].get("op_name", "")) if len(ops) == 1 else ""
    if len(ops) != 1 or name not in allowed:
        raise ValueError(f"{who} executor handles exactly one of {allowed}; got {[o.get('op_name') for o in ops]!r}")
    return ops[0]


# ---- executors -------------------------------------------------------------------------

def execute_gfx950_gemm(artifact: RuntimeArtifact, args: Any):
    """One ``tessera.matmul`` / ``tessera.gemm`` / ``tessera.fused_epilogue`` op:
    rank-2 operands with matching K; f16/bf16 storage -> f32 result, int8 -> int32
    result.  An optional third operand is the per-output-column bias ``[N]`` and
    ``kwargs["activation"]`` (none / relu / gelu / silu) selects the fused
    activation — float only (``runtime.py:6603-6660``)."""
    md = artifact.metadata or {}
    op = _single_op(artifact, ("tessera.matmul", "tessera.gemm", "tessera.fused_epilogue"), "gfx950_gemm")
    values = _named_args(args, list(md.get("arg_names") or []))
    names = [str(n) for n in op.get("operands", [])]
    kwargs = op.get("kwargs") or {}
    activation = str(kwargs.get("activation") or "none")
    if activation not in ("none", "relu", "gelu", "silu"):
        raise ValueError(f"gfx950 epilogue activation must be one of none/relu/gelu/silu; got {activation!r}")
    if len(names) not in (2, 3):
        raise ValueError(f"matmul takes two operands (a, b) plus an optional third bias operand; got {len(names)}")
    has_bias = len(names) == 3
    a, b = _host_array(values[names[0]]), _host_array(values[names[1]])
    if a.ndim != 2 or b.ndim != 2 or a.shape[1] != b.shape[0]:
        raise ValueError(f"gfx950 matmul needs rank-2 operands with matching K; got {a.shape} @ {b.shape}")
    if a.dtype == np.int8 and b.dtype == np.int8:
        if has_bias or activation != "none":
            raise ValueError("gfx950 fused epilogue (bias/activation) is float-only; got integer dtype int8")
        return _ops.gemm_i8(a, b)
    if not has_bias and activation == "none":
        return _ops.gemm(a, b, out="f32")
    bias = None
    if has_bias:
        bias = np.ascontiguousarray(np.asarray(_host_array(values[names[2]])), dtype=np.float32)
        if bias.shape != (b.shape[1],):
            raise ValueError(f"bias must have shape ({b.shape[1]},) (one per output column); got {bias.shape}")
    return _ops.fused_gemm(a, b, bias, activation)


_FA_OPS = ("tessera.flash_attn", "tessera.multi_head_attention", "tessera.gqa_attention", "tessera.mqa_attention",
           "tessera.attn_sliding_window")


def execute_gfx950_flash_attn(artifact: RuntimeArtifact, args: Any):
    """Attention forward: Q ``[..., Hq, Sq, D]``, K/V ``[..., Hkv, Sk, D]`` in
    f16/bf16 -> f32 O shaped like Q; an optional fourth operand is the additive
    attention bias, broadcastable to ``[..., Hq, Sq, Sk]`` (``runtime.py:7270-7274``).
    ``kwargs``: ``causal``, ``scale``, ``window`` (a positive width; required by
    ``tessera.attn_sliding_window``) and ``logit_softcap`` (``runtime.py:7312-7340``)."""
    md = artifact.metadata or {}
    op = _single_op(artifact, _FA_OPS, "gfx950_flash_attn")
    names = [str(n) for n in op.get("operands", [])]
    if len(names) < 3:
        raise ValueError("flash_attn requires Q, K, V operands")
    if len(names) > 4:
        raise ValueError(f"flash_attn takes Q, K, V plus an optional attn_bias operand; got {len(names)}")
    values = _named_args(args, list(md.get("arg_names") or []))
    q, k, v = (_host_array(values[n]) for n in names[:3])
    bias = np.asarray(_host_array(values[names[3]])) if len(names) == 4 else None
    kwargs = op.get("kwargs") or {}
    if kwargs.get("dropout_p"):
        raise ValueError("gfx950 flash_attn lane does not implement `dropout_p`")
    window = int(kwargs.get("window") or 0)
    if window < 0:
        raise ValueError(f"gfx950 flash_attn window must be a non-negative width; got {window}")
    if str(op.get("op_name")) == "tessera.attn_sliding_window" and window <= 0:
        raise ValueError(f"tessera.attn_sliding_window requires a positive `window` width kwarg; got {window}")
    softcap = kwargs.get("logit_softcap")
    softcap = float(softcap) if softcap else 0.0
    if softcap < 0:
        raise ValueError(f"gfx950 flash_attn logit_softcap must be non-negative; got {softcap}")
    # the windowed kernel of the reference is implicitly causal (runtime.py:7318-7321)
    causal = bool(kwargs.get("causal", False)) or window > 0
    return _ops.gqa_attention(q, k, v, scale=kwargs.get("scale"), causal=causal, out="f32", window=window,
                              logit_softcap=softcap, attn_bias=bias)


_FA_BWD_OPS = ("tessera.flash_attn_bwd", "tessera.flash_attn_vjp")


def execute_gfx950_flash_attn_bwd(artifact: RuntimeArtifact, args: Any):
    """Attention backward: operands ``(dO, Q, K, V)`` -> the tuple ``(dQ, dK, dV)``
    in f32 shaped like ``(Q, K, V)`` (``runtime.py:7598-7665``).  ``kwargs``:
    ``causal``, ``scale``; an additive bias, sliding window or logit soft-cap is
    not on this lane and is rejected."""
    md = artifact.metadata or {}
    op = _single_op(artifact, _FA_BWD_OPS, "gfx950_flash_attn_bwd")
    names = [str(n) for n in op.get("operands", [])]
    if len(names) != 4:
        raise ValueError("gfx950 flash_attn backward requires exactly the (dO, Q, K, V) operands")
    values = _named_args(args, list(md.get("arg_names") or []))
    do, q, k, v = (_host_array(values[n]) for n in names)
    kwargs = op.get("kwargs") or {}
    if kwargs.get("window") or kwargs.get("logit_softcap") or kwargs.get("attn_bias") is not None:
        raise ValueError("gfx950 flash_attn backward handles scale + causal only (no bias / window / soft-cap)")
    return _ops.flash_attn_backward(do, q, k, v, scale=kwargs.get("scale"), causal=bool(kwargs.get("causal", False)))


def _plan_to_transport(plan: Any) -> _ops.MoETransport:
    """Accept the lane's own :class:`MoETransport` or a stdlib ``DispatchPlan``-like
    object (``expert_ids``, ``weights``, ``sort_perm``, ``group_sizes``,
    ``num_tokens``, ``top_k``) and lower it as ``descriptor_from_dispatch_plan``
    does (``compiler/moe_transport.py:194-227``), with the same validation."""
    if isinstance(plan, _ops.MoETransport):
        return plan
    expert_ids = np.asarray(plan.expert_ids)
    weights = np.asarray(plan.weights)
    perm = np.asarray(plan.sort_perm, np.int64).reshape(-1)
    groups = np.asarray(plan.group_sizes, np.int64).reshape(-1)
    T, k = int(plan.num_tokens), int(plan.top_k)
    if expert_ids.shape != (T, k):
        raise ValueError("MoE expert_ids shape disagrees with T/top_k")
    if weights.shape != expert_ids.shape:
        raise ValueError("MoE weights must match expert_ids")
    total = T * k
    if perm.size and (int(perm.min()) < 0 or int(perm.max()) >= total):
        raise ValueError("MoE sort permutation contains an invalid slot")
    if np.unique(perm).size != perm.size:
        raise ValueError("MoE sort permutation contains duplicate slots")
    kept = getattr(plan, "kept_mask", None)
    if kept is not None and not np.array_equal(np.sort(perm), np.flatnonzero(np.asarray(kept).reshape(-1))):
        raise ValueError("MoE sort permutation does not cover exactly the kept slots")
    if total > np.iinfo(np.int32).max:
        raise ValueError("MoE metadata exceeds the int32 device ABI")
    flat_e = expert_ids.reshape(-1)
    offsets = np.concatenate((np.zeros(1, np.int64), np.cumsum(groups))).astype(np.int32)
    return _ops.MoETransport(
        T, k, int(groups.size), getattr(plan, "capacity", None),
        (perm // k).astype(np.int32), flat_e[perm].astype(np.int32),
        weights.astype(np.float32).reshape(-1)[perm].astype(np.float32),
        groups.astype(np.int32), offsets)


def execute_gfx950_moe_transport(artifact: RuntimeArtifact, args: Any):
    """``tessera.moe_dispatch`` / ``moe_combine`` / ``grouped_gemm`` /
    ``grouped_swiglu`` → ``(output, "native_gpu")``."""
    md = artifact.metadata or {}
    values = dict(args) if isinstance(args, Mapping) else _named_args(args, list(md.get("arg_names") or ["x", "plan"]))
    ops = list(md.get("ops") or [])
    name = str(ops[0].get("op_name", "")) if len(ops) == 1 else ""

    def need(*keys):
        try:
            return tuple(values[k] for k in keys)
        except KeyError as exc:
            raise ValueError(f"missing {name.split('.')[-1]} argument {exc.args[0]!r}") from exc

    if name == "tessera.moe_dispatch":
        x, plan = need("x", "plan")
        return (_ops.moe_dispatch(_host_array(x), _plan_to_transport(plan)), "native_gpu")
    if name == "tessera.moe_combine":
        partials, plan = need("partials", "plan")
        return (_ops.moe_combine(_host_array(partials), _plan_to_transport(plan)), "native_gpu")
    if name == "tessera.grouped_gemm":
        x, w, gs = need("x", "weights", "group_sizes")
        return (_ops.grouped_gemm(_host_array(x), _host_array(w), gs, out="f32"), "native_gpu")
    if name == "tessera.grouped_swiglu":
        x, wg, wu, wd, gs = need("x_packed", "w_gate", "w_up", "w_down", "group_sizes")
        return (_ops.moe_swiglu_block(*map(_host_array, (x, wg, wu, wd)), gs), "native_gpu")
    raise ValueError("gfx950_moe_transport executor handles tessera.moe_dispatch, tessera.moe_combine, "
                     f"tessera.grouped_gemm, or tessera.grouped_swiglu; got {name!r}")


def execute_gfx950_quant_gemm(artifact: RuntimeArtifact, args: Any):
    """``tessera.fp8_gemm``: operands (a_codes, b_codes), kwargs scale_a/scale_b/out/format;
    ``tessera.w8a8_gemm``: operands (x_q, w_q, a_scale, w_scale)."""
    md = artifact.metadata or {}
    op = _single_op(artifact, ("tessera.fp8_gemm", "tessera.w8a8_gemm"), "gfx950_quant_gemm")
    values = _named_args(args, list(md.get("arg_names") or []))
    names = [str(n) for n in op.get("operands", [])]
    kwargs = op.get("kwargs") or {}
    if op["op_name"] == "tessera.fp8_gemm":
        if len(names) != 2:
            raise ValueError("fp8_gemm requires two operands")
        return _ops.gemm_fp8(values[names[0]], values[names[1]], float(kwargs.get("scale_a", 1.0)),
                             float(kwargs.get("scale_b", 1.0)), out=str(kwargs.get("out", "bf16")),
                             format=str(kwargs.get("format", "e4m3")))
    if len(names) != 4:
        raise ValueError("w8a8_gemm requires x_q, w_q, a_scale, w_scale")
    return _ops.w8a8_gemm(*(values[n] for n in names))


def executor_table() -> dict[str, Callable[[RuntimeArtifact, Any], Any]]:
    """executor_id -> function, as ``_executor_table()`` (``runtime.py:30515``)."""
    return {
        "gfx950_gemm": execute_gfx950_gemm,
        "gfx950_flash_attn": execute_gfx950_flash_attn,
        "gfx950_flash_attn_bwd": execute_gfx950_flash_attn_bwd,
        "gfx950_moe_transport": execute_gfx950_moe_transport,
        "gfx950_quant_gemm": execute_gfx950_quant_gemm,
    }


@dataclass
class DispatchLog:
    """``(target, compiler_path, status)`` of each launch — the lane's analogue of
    ``runtime.dispatch_fallback_log``."""
    entries: list = field(default_factory=list)


DISPATCH_LOG = DispatchLog()


def launch(kernel: RuntimeArtifact, args: Any, stream: Any = None) -> dict:
    """Matrix-driven dispatch with the result dict of ``runtime.launch``
    (``runtime.py:30993-31077``): ``ok``, ``runtime_status``, ``compiler_path``,
    ``execution_kind``, ``execution_mode``, ``artifact_hash``, ``output``,
    ``telemetry``, ``profile``."""
    start_ns = time.perf_counter_ns()
    md = kernel.metadata or {}
    target = str(md.get("target", "cpu") or "cpu")
    path = str(md.get("compiler_path", "") or "")
    row = lookup(target, path)
    table = executor_table()
    if row is None or not row.executable or md.get("executable") is not True or row.executor_id not in table:
        DISPATCH_LOG.entries.append((target, path, "unimplemented"))
        return {"ok": False, "runtime_status": "unimplemented", "compiler_path": path,
                "execution_kind": "artifact_only", "artifact_hash": kernel.artifact_hash,
                "reason": f"no gfx950 executor for ({target!r}, {path!r}) or artifact not stamped executable"}
    kid = str(md.get("kernel_id", row.executor_id))
    try:
        output = table[row.executor_id](kernel, args)
    except Exception as exc:                       # mapped, never re-raised: runtime.py:31021-31041
        DISPATCH_LOG.entries.append((target, path, "invalid_artifact"))
        return {"ok": False, "runtime_status": "invalid_artifact", "compiler_path": row.compiler_path,
                "execution_kind": row.execution_kind, "artifact_hash": kernel.artifact_hash, "reason": str(exc),
                "telemetry": {"event": "runtime.launch", "arch": row.target, "kernel_id": kid,
                              "status": "invalid_artifact", "unavailable": isinstance(exc, LaneUnavailable)}}
    exec_kind = row.execution_kind
    if isinstance(output, tuple) and len(output) == 2 and isinstance(output[1], str):
        output, exec_kind = output
    elapsed_ms = (time.perf_counter_ns() - start_ns) / 1e6
    DISPATCH_LOG.entries.append((target, path, "ok"))
    return {"ok": True, "runtime_status": "success", "compiler_path": row.compiler_path,
            "execution_kind": exec_kind, "execution_mode": row.execution_mode,
            "artifact_hash": kernel.artifact_hash, "output": output,
            "telemetry": {"event": "runtime.launch", "source": "runtime", "op": "artifact_launch", "arch": row.target,
                          "kernel_id": kid, "latency_ms": elapsed_ms, "status": "ok",
                          "metadata": {"compiler_path": row.compiler_path, "execution_kind": exec_kind,
                                       "execution_mode": row.execution_mode}},
            "profile": {"cpu_wall_ms": elapsed_ms, "launch_overhead_ms": elapsed_ms}}


def make_artifact(op_name: str, arg_names: list, operands: list, compiler_path: str, kwargs: Optional[dict] = None,
                  executable: Optional[bool] = None) -> RuntimeArtifact:
    """The metadata ``JitFn._build_runtime_artifact`` stamps for a single-op
    program on this lane (``compiler/jit.py:2188-2217``).  ``executable``
    defaults to the cached host probe, so off-device artifacts stay
    ``artifact_only``."""
    if executable is None:
        executable = lane_default_available()
    return RuntimeArtifact(metadata={
        "target": TARGET, "compiler_path": compiler_path, "executable": bool(executable),
        "execution_kind": "native_gpu" if executable else "artifact_only",
        "arg_names": list(arg_names), "output_name": "out",
        "ops": [{"op_name": op_name, "result": "out", "operands": list(operands), "kwargs": dict(kwargs or {})}],
    })
