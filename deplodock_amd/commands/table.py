"""Plain-text tables for the CLI."""

from __future__ import annotations


def render_table(headers: list[str], rows: list[list[str]], align: str | None = None) -> list[str]:
    """Lines of a column-aligned table; ``align`` holds one of ``l``/``r`` per column."""
    align = align or "l" * len(headers)
    widths = [max(len(str(h)), *(len(str(r[i])) for r in rows)) if rows else len(str(h)) for i, h in enumerate(headers)]

    def fmt(cells) -> str:
        return "  ".join(str(c).rjust(w) if a == "r" else str(c).ljust(w) for c, w, a in zip(cells, widths, align)).rstrip()

    rule = "  ".join("-" * w for w in widths)
    return [fmt(headers), rule, *(fmt(r) for r in rows)]
