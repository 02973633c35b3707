"""Plug the gfx950 lane into a Tessera host.

Tessera programs pick a lane up through ``runtime.launch()`` and the measured
arbiter without change to the programs.  In the reference that takes these
registrations, each into an object the host owns:

* arbiter candidates and the grouped-GEMM op kind
  (``tessera.compiler.emit.candidate``: ``register_op_kind`` ``:81-87``,
  ``register_candidate`` ``:206-236``);
* execution-matrix rows (``tessera.compiler.execution_matrix._MATRIX``, rows as at
  ``:2495-2537``) and their catalogue entries (``KNOWN_EXECUTORS``, ``:103``);
* executor functions under the ids those rows name (``runtime._executor_table()``,
  ``python/tessera/runtime.py:30515``; ``launch`` resolves a row's ``executor_id``
  through it, ``:31008-31020``);
* optionally, the submit hook for typed native artifacts
  (``runtime.register_native_launcher``, ``python/tessera/runtime.py:279-306``).

:func:`install` does those registrations into whatever objects it is handed, and
nothing else: it owns no registry and restates none of the host's machinery.
"""
from __future__ import annotations

from typing import Any, Callable, MutableMapping, Optional

from . import candidates as _cand
from . import executors as _ex
from . import native_launcher as _native


def _rows_into(matrix_owner: Any) -> list:
    """Add the lane's rows to the host's matrix and catalogue.  ``matrix_owner`` is the
    host's ``execution_matrix`` module (or any object with ``ExecutionRow``, ``_MATRIX``
    and, optionally, ``KNOWN_EXECUTORS``)."""
    row_cls = matrix_owner.ExecutionRow
    matrix: MutableMapping = matrix_owner._MATRIX
    added = []
    for fields in _ex.ROW_FIELDS:
        row = row_cls(**fields)
        matrix[(row.target, row.compiler_path)] = row
        added.append((row.target, row.compiler_path))
    catalogue = getattr(matrix_owner, "KNOWN_EXECUTORS", None)
    if catalogue is not None:
        catalogue.update(_ex.KNOWN_EXECUTORS)
    return added


def _executors_into(table_owner: Any) -> list:
    """Make the lane's executor functions reachable under their ids.  ``table_owner``
    is either a mutable mapping ``executor_id -> function`` or an object whose
    ``_executor_table()`` returns such a mapping afresh on every call (the reference's
    ``runtime`` module): that function is then wrapped so its result carries the
    lane's entries too."""
    ours = _ex.executor_table()
    if isinstance(table_owner, MutableMapping):
        table_owner.update(ours)
        return sorted(ours)
    inner: Optional[Callable[[], dict]] = getattr(table_owner, "_executor_table", None)
    if not callable(inner):
        raise TypeError("executor_table must be a mutable mapping or expose a callable _executor_table()")
    if getattr(inner, "_gfx950_wrapped", False):
        return sorted(ours)

    def _executor_table_with_gfx950() -> dict:
        table = dict(inner())
        table.update(ours)
        return table

    _executor_table_with_gfx950._gfx950_wrapped = True
    table_owner._executor_table = _executor_table_with_gfx950
    return sorted(ours)


def install(candidate_api: Any = None, execution_matrix: Any = None, executor_table: Any = None,
            native_launchers: Any = None) -> dict:
    """Register the lane with a host; every argument is optional and independent.

    ``candidate_api``     the host's candidate module / namespace -> op kind + five candidates
    ``execution_matrix``  the host's execution-matrix module / namespace -> five rows + catalogue
    ``executor_table``    a mapping, or the host's runtime module -> five executor functions
    ``native_launchers``  the host's runtime module (``register_native_launcher``) -> the typed-descriptor
                          submit hook for target ``rocm_gfx950``

    Returns what was registered: ``{"candidates": [names], "rows": [(target, path)],
    "executors": [ids], "native_launcher": target or None}``.  Safe to call again (everything is keyed by name)."""
    report: dict = {"candidates": [], "rows": [], "executors": [], "native_launcher": None}
    if candidate_api is not None:
        report["candidates"] = [c.name for c in _cand.register(candidate_api)]
    if execution_matrix is not None:
        report["rows"] = _rows_into(execution_matrix)
    if executor_table is not None:
        report["executors"] = _executors_into(executor_table)
    if native_launchers is not None:
        report["native_launcher"] = _native.register(native_launchers, replace=True)
    return report


def install_into_tessera() -> dict:
    """:func:`install` into an importable ``tessera`` package — the three objects
    named in the module docstring."""
    from tessera import runtime
    from tessera.compiler import execution_matrix
    from tessera.compiler.emit import candidate
    return install(candidate, execution_matrix, runtime, runtime)
