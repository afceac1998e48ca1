"""The layout-change kernel's host side: which of its two forms is chosen, that both compile for gfx950, and that a
view reaching past its buffer is refused before anything could be launched."""

import pytest

from deplodock_amd.dtype import BF16, F32
from deplodock_amd.emit.copy import emit_strided_copy
from deplodock_amd.emit.errors import LoweringError
from deplodock_amd.ir.tile import StridedCopy


def _copy(axes, dtype=F32, offset=0, numel=None):
    reach = offset + sum((se - 1) * st for _, se, st in axes)
    return StridedCopy(src="X", out="out", dtype=dtype, src_offset=offset, src_numel=reach + 1 if numel is None else numel, axes=tuple(axes))


@pytest.mark.parametrize(
    "axes, dtype, mode",
    [
        ([(2048, 2048, 1), (1024, 1024, 2048)], F32, "tile64"),  # [K, N] read as [N, K]
        ([(40, 37, 1), (104, 100, 37)], F32, "tile64"),  # the same, ragged and padded
        ([(6, 6, 9100), (132, 130, 1), (72, 70, 130)], BF16, "tile64"),
        ([(128, 128, 64), (16, 16, 8192), (64, 64, 1)], F32, "rows"),  # heads <-> tokens: the unit-stride axis stays last
        ([(5, 5, 1650), (36, 33, 50), (56, 50, 1)], F32, "rows"),
        ([(4, 4, 0), (16, 16, 16), (16, 16, 1)], F32, "rows"),  # a broadcast (stride 0) leading axis
        ([(1, 1, 1), (300, 300, 1)], F32, "rows"),
    ],
)
def test_form_and_compile(launcher_lib, axes, dtype, mode):
    from deplodock_amd.backend.hip import hiprtc

    hip = emit_strided_copy(_copy(axes, dtype), "k_copy_probe")
    assert hip.knobs == {"COPY": mode}
    hiprtc.compile_to_hsaco(hip.kernel_source, hip.kernel_name)
    total = 1
    for de, _, _ in axes:
        total *= de
    blocks = hip.grid[0][0]
    assert blocks * (1024 if mode == "rows" else 4096) >= total


def test_views_past_the_buffer_are_refused():
    with pytest.raises(LoweringError, match="reaches element"):
        emit_strided_copy(_copy([(8, 8, 16), (16, 16, 1)], numel=100), "k")
    with pytest.raises(LoweringError, match="source extent"):
        emit_strided_copy(_copy([(8, 9, 16), (16, 16, 1)], numel=1000), "k")
    with pytest.raises(LoweringError, match="32-bit"):
        emit_strided_copy(_copy([(1 << 16, 1 << 16, 1 << 16), (1 << 16, 1 << 16, 1)]), "k")
