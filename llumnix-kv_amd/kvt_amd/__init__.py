"""Python (ctypes) binding of libkvt_hip.so, the MI355X KV-cache pack/unpack library.

The library itself is C++/HIP behind a C ABI (``include/kvt_hip.h``); this
module only loads it and offers thin helpers used by the tests, ``bench.py`` and
``__graft_entry__``. There is no CPU fallback: GPU entry points raise
``KvtError`` when the library or a gfx950 device is missing.
"""
from .binding import (KvtError, LIB_PATH, BlockLists, RunLists, Cache, Parser, Plan, Session, Stager,
                      WireLayout, WIRE_TCP, WIRE_RDMA_STAGED, block_object_lists, device_count,
                      lib, select_parser, compute_valid_ranks_pd, merge_interval, validate_bounds,
                      wire_layout_of, wire_parse_frame, wire_write_frame, set_copy_cu_usage,
                      get_copy_cu_usage, ObjectRing, PlanSlot, SlotLayout, copy_ticket_stats)
from . import ctypes_defs

__all__ = ["KvtError", "LIB_PATH", "BlockLists", "Cache", "Parser", "Plan", "Session", "Stager",
           "device_count", "lib", "select_parser", "compute_valid_ranks_pd", "merge_interval",
           "validate_bounds", "ctypes_defs", "WireLayout", "WIRE_TCP", "WIRE_RDMA_STAGED",
           "block_object_lists", "RunLists", "wire_layout_of", "wire_parse_frame", "wire_write_frame",
           "set_copy_cu_usage", "get_copy_cu_usage", "ObjectRing", "PlanSlot", "SlotLayout",
           "copy_ticket_stats"]
