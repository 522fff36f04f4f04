"""The example programs of the HIP back-end, and what it takes to build each.

The counterpart of the reference's examples/ directory and of its generate_evals.py:13-48, which prints the
whole set into generated/: `python -m prism_amd.examples [directory]` writes `<name>.hip` (kernel or device
function as `generate()` prints it) for every program, and `<kernel>_launcher.hip` (helpers, kernel and C
launcher, what `build()` compiles) for every global kernel. The committed copies under
prism_amd/examples/generated are compared with fresh output by the tests, so a change of the emitter shows
up as a change of text.
"""
from __future__ import annotations

import sys
from pathlib import Path
from typing import Dict, List, Optional, Tuple

# global kernel -> (module, workgroup size, template arguments)
KERNELS: Dict[str, Tuple[str, int, Optional[List[int]]]] = {
    "add_m_blocks": ("add_m", 256, None),
    "add_m_by_wavefronts": ("add_m", 256, None),
    "naive_sgemm": ("sgemm", 256, None),
    "remapped_sgemm": ("sgemm", 1024, None),
    "tiled_sgemm": ("sgemm", 1024, [32]),
    "thread_tile_sgemm": ("sgemm", 256, [64, 64, 8, 4, 4]),
    "vector_tile_sgemm": ("sgemm", 256, [128, 128, 8, 8, 8]),
    "staged_sgemm": ("sgemm", 256, [64, 64, 8, 4, 4, 256]),
    "mfma_tile_sgemm": ("sgemm", 256, None),
    "one_mfma_per_wavefront": ("mfma", 256, None),
    "one_bf16_mfma_per_wavefront": ("mfma", 256, None),
    "row_scan32": ("scan", 256, None),
    "lookback_scan": ("scan", 256, None),
    "lookback_scan_by_parts": ("scan", 256, None),
    "lookback_scan_wide": ("scan", 256, None),
    "lookback_scan_striped": ("scan", 1024, None),
    "scaled_sum_all": ("basics", 256, None),
    "two_roles": ("basics", 256, None),
    "gather_columns": ("basics", 256, None),
    "handed_over_gemm": ("handover", 320, None),
    "handed_over_gemm_big": ("handover", 512, None),
    "handed_over_sgemm": ("handover", 768, None),
    "pipelined_sgemm": ("pipelined", 1024, None),
    "pipelined_gemm_bf16": ("pipelined", 512, None),
}
# device functions, printed on their own as well (the reference prints its scan's helpers one file each)
DEVICE_FUNCTIONS: Dict[str, str] = {
    "lane_load": "add_m", "lane_store": "add_m", "wave_load": "add_m", "wave_store": "add_m",
    "stage_tiles": "sgemm", "multiply_tiles": "sgemm", "scaled_sum": "basics",
    "lane_shift_up": "scan", "shift_up_in_wavefront": "scan", "take_ticket": "scan", "publish": "scan",
    "look_back": "scan", "scan_rows": "scan", "collect_row_ends": "scan", "scan_row_ends": "scan", "write_back": "scan",
    "fill_slot": "handover", "multiply_slot": "handover", "fill_slot_f32": "handover", "multiply_slot_f32": "handover",
    "look_back_wide": "scan", "value_of_last_lane": "scan",
    "fill_stage_f32": "pipelined", "multiply_stage_f32": "pipelined",
    "fill_stage_bf16": "pipelined", "multiply_stage_bf16": "pipelined",
}
GENERATED = Path(__file__).resolve().parent / "generated"


def load() -> None:
    """Imports every example module, which registers its programs."""
    import importlib
    for module in sorted(set(m for m, _, _ in KERNELS.values()) | set(DEVICE_FUNCTIONS.values())):
        importlib.import_module(f"{__name__}.{module}")


def texts() -> Dict[str, str]:
    """File name -> generated text for the whole set."""
    from ..hipgen import generate, generate_launcher
    load()
    out: Dict[str, str] = {}
    for name in list(DEVICE_FUNCTIONS) + list(KERNELS):
        out[f"{name}.hip"] = generate(name)
    for name, (_, block_size, template) in KERNELS.items():
        out[f"{name}_launcher.hip"] = generate_launcher(name, block_size, template)
    return out


def write(directory: Optional[str] = None) -> List[Path]:
    d = Path(directory) if directory else GENERATED
    d.mkdir(parents=True, exist_ok=True)
    written = []
    for file_name, text in texts().items():
        path = d / file_name
        path.write_text(text)
        written.append(path)
    return written


def main(argv: Optional[List[str]] = None) -> int:
    args = sys.argv[1:] if argv is None else argv
    for path in write(args[0] if args else None):
        print(f"  {path}")
    return 0
