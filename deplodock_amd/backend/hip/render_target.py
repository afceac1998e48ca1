"""gfx950 implementation of :class:`deplodock_amd.render_target.RenderTarget`.

Owns every HIP / clang spelling the emitters use, where the reference's
``CudaRenderTarget`` (emmy/compiler/backend/cuda/render_target.py) owns CUDA's:

* scalar types are clang's native ones — ``float``, ``__bf16``, ``_Float16`` (the reference's table has
  no bf16 entry: there bf16 rides in ``float`` registers), so conversions are plain C casts that the
  compiler lowers to the hardware's round-to-nearest-even converts (``v_cvt_pk_bf16_f32`` on gfx950);
* vectors are ``ext_vector_type`` typedefs (declared by the emitters' prelude): element access is
  ``v[i]``, and a 16-byte vector of any element type is one ``global_load_dwordx4`` / ``ds_read_b128``;
* fp32 intrinsics are the precise libm-style device functions (``expf``, ``rsqrtf``, true division):
  fp32 results must match eager to rtol 1e-5, so nothing here maps to a fast-math form.  The ``fast_*``
  ops are the explicit opt-ins the emitters use where a result is rounded to 16 bits straight away;
* 16-bit arithmetic is never native: every op is evaluated in fp32 and rounded at the points eager
  rounds (``has_native_op`` is False for bf16 / f16), which is what keeps parity with eager's per-op
  rounding without packed 16-bit math.
"""

from __future__ import annotations

_TYPE_NAME = {"f32": "float", "bf16": "__bf16", "f16": "_Float16", "i32": "int", "i64": "long long", "u32": "unsigned int"}
_VEC_PREFIX = {"f32": "f32", "bf16": "bf16", "f16": "f16", "u32": "u32"}
_VEC_WIDTHS = {"f32": (2, 4, 8, 16), "bf16": (2, 4, 8), "f16": (2, 4, 8), "u32": (2, 4)}

# abstract op -> fp32 spelling ("{a}" / "{b}" are the operands; a bare name is a function)
_INTRINSIC_F32 = {
    "exp": "expf",
    "exp2": "exp2f",
    "fast_exp": "__expf",
    "fast_exp2": "__builtin_amdgcn_exp2f",
    "fast_div": "__fdividef",
    "rsqrt": "rsqrtf",
    "sqrt": "sqrtf",
    "tanh": "tanhf",
    "fabs": "fabsf",
    "abs": "fabsf",
    "fmax": "fmaxf",
    "max": "fmaxf",
    "fmin": "fminf",
    "min": "fminf",
    "pow": "powf",
    "erf": "erff",
    "fma": "__builtin_fmaf",
}
_NATIVE_F32 = frozenset({"add", "sub", "subtract", "mul", "multiply", "div", "divide", "neg", "maximum", "minimum", *_INTRINSIC_F32})


class HipRenderTarget:
    """C spellings for clang-HIP on gfx950."""

    name = "hip-gfx950"

    def type_name(self, dtype: str) -> str:
        try:
            return _TYPE_NAME[dtype]
        except KeyError as exc:
            raise KeyError(f"HipRenderTarget: no C type for dtype {dtype!r}") from exc

    def literal(self, text: str, dtype: str) -> str:
        return text if dtype == "f32" else f"(({self.type_name(dtype)})({text}))"

    def convert(self, value: str, src_dt: str, dst_dt: str) -> str:
        if src_dt == dst_dt:
            return value
        return f"(({self.type_name(dst_dt)})({value}))"

    def intrinsic(self, op_name: str, result_dt: str) -> str:
        if result_dt == "f32":
            return _INTRINSIC_F32.get(op_name, op_name)
        return op_name  # 16-bit types have no native forms here: the renderer widens to fp32

    def has_native_op(self, op_name: str, dtype: str) -> bool:
        return dtype == "f32" and op_name in _NATIVE_F32

    def vector_type(self, dtype: str, n: int) -> tuple[str, str] | None:
        if n == 1 and dtype in _TYPE_NAME:
            return (_TYPE_NAME[dtype], _TYPE_NAME[dtype])
        if dtype not in _VEC_PREFIX or n not in _VEC_WIDTHS[dtype]:
            return None
        return (f"{_VEC_PREFIX[dtype]}x{n}", _TYPE_NAME[dtype])

    # -- what the emitters build from the protocol ----------------------------------------------------
    def round_trip(self, value: str, dtype: str) -> str:
        """``value`` (fp32) rounded to ``dtype`` storage precision and widened back."""
        return self.convert(self.convert(value, "f32", dtype), dtype, "f32")


__all__ = ["HipRenderTarget"]
