"""MI355X (gfx950) SpMM operator behind the entry points and data formats of
Ritt2020/hopper_spmm.  The product is the C-ABI library `libhspmm.so`
(include/hspmm.h); this package is its thin ctypes driver plus the synthetic
matrix generators the benchmark configurations name."""
from .capi import (FP16, TF32, BF16, IDX_MAX, ROW_WINDOW, HspmmError, Plan, build_library, library_path,
                   load_library, mtx_load, csr_to_btcf, btcf_relayout, csr_to_bitmap, bitmap_expand, bitmap_to_grouped,
                   BITS_PER_TILE, BITS_AS_REFERENCE, partition_preview, partition_preview_aligned, panel_units_preview, configure, get_config,
                   set_kernel_mode, get_kernel_mode, set_window_pairing, set_panel_stream, has_experimental, set_group_cuts, cli_path)

__all__ = ["FP16", "TF32", "BF16", "IDX_MAX", "ROW_WINDOW", "HspmmError", "Plan", "build_library", "library_path",
           "load_library", "mtx_load", "csr_to_btcf", "btcf_relayout", "csr_to_bitmap", "bitmap_expand", "bitmap_to_grouped",
           "BITS_PER_TILE", "BITS_AS_REFERENCE", "partition_preview", "partition_preview_aligned", "panel_units_preview", "configure", "get_config",
           "set_kernel_mode", "get_kernel_mode", "set_window_pairing", "set_panel_stream", "has_experimental", "set_group_cuts", "cli_path"]
