"""The source-text seam of the emitters: every C spelling decision goes through a ``RenderTarget``.

Same protocol as the reference's (emmy/compiler/render_target.py:24-80): ``type_name``, ``literal``,
``convert``, ``intrinsic``, ``has_native_op``, ``vector_type``, all over canonical dtype tokens
(``"f32"``, ``"bf16"``, ``"f16"``, ``"i32"``).  The reference's only implementation is
``CudaRenderTarget`` (emmy/compiler/backend/cuda/render_target.py); a backend that wants to share the
statement renderer supplies its own.  Here the emitters (``deplodock_amd/emit``) and the expression
renderer (``deplodock_amd/ir/expr.py``) consult the target instead of keeping type and intrinsic tables
of their own; ``HipRenderTarget`` (``deplodock_amd/backend/hip/render_target.py``) is the gfx950 one.
"""

from __future__ import annotations

from typing import Protocol, runtime_checkable


@runtime_checkable
class RenderTarget(Protocol):
    """Per-target spelling helpers consulted while kernel source is written."""

    def type_name(self, dtype: str) -> str:
        """C type of a scalar of ``dtype`` (``"f32"`` -> ``"float"``)."""

    def literal(self, text: str, dtype: str) -> str:
        """A numeric literal ``text`` (written as an fp32 literal) as a value of ``dtype``."""

    def convert(self, value: str, src_dt: str, dst_dt: str) -> str:
        """``value`` (an expression of ``src_dt``) as ``dst_dt``; unchanged when they are equal."""

    def intrinsic(self, op_name: str, result_dt: str) -> str:
        """Function spelling of abstract op ``op_name`` at ``result_dt`` (``("exp", "f32")`` ->
        ``"expf"``); the op name itself when the target has no special form."""

    def has_native_op(self, op_name: str, dtype: str) -> bool:
        """Whether ``op_name`` is evaluated natively at ``dtype`` (otherwise the renderer widens to
        fp32, applies the fp32 form and rounds back)."""

    def vector_type(self, dtype: str, n: int) -> tuple[str, str] | None:
        """``(vector C type, element C type)`` of ``n`` elements of ``dtype``, or ``None``."""


_current: RenderTarget | None = None


def current() -> RenderTarget:
    """The render target the emitters write for (the gfx950 one unless ``use`` installed another)."""
    global _current
    if _current is None:
        from deplodock_amd.backend.hip.render_target import HipRenderTarget

        _current = HipRenderTarget()
    return _current


def use(target: RenderTarget | None) -> RenderTarget | None:
    """Install ``target`` (``None`` = back to the default); returns the previous one."""
    global _current
    old, _current = _current, target
    return old


class _Proxy:
    """Module-level handle that always forwards to ``current()`` (so ``use`` takes effect everywhere)."""

    def __getattr__(self, name):
        return getattr(current(), name)


rt = _Proxy()

__all__ = ["RenderTarget", "current", "use", "rt"]
