"""ctypes mirrors of the plain-C types in ``include/kvt_types.h``.

Field order and widths must match the header exactly; ``tests/test_abi.py``
checks ``sizeof`` against the values the compiled library reports.
"""
import ctypes as C

MAX_TP_SIZE = 16
MAX_TENSORS = 8
MAX_SHAPE_DIMS = 4
MAX_CHANNEL_DIMS = 8

# cache shapes (reference: kvtransfer/include/envcfg.h:25-52)
SHAPE_RAGGED_FLASH = 1
SHAPE_FLASH = 2
SHAPE_QWEN3_NEXT_FLASH = 3
SHAPE_DPSK_V32_SPARSE_MLA = 4
SHAPE_FLASHINFER = 5
SHAPE_TURBOQUANT = 6
SHAPE_QWEN3_NEXT_FLASHINFER = 7
SHAPE_KIMI_K3_MLA = 8

TP_PEQD, TP_PLTD, TP_PGTD, TP_UNKNOWN = 0, 1, 2, 3

PARSER_NAMES = [
    "RAGGED_PEQD", "RAGGED_PGTD", "RAGGED_PGTD_DPSK", "RAGGED_PLTD",
    "FLASH_PEQD", "FLASH_PGTD",
    "HYBRID_PEQD", "HYBRID_PGTD", "HYBRID_PLTD",
    "DPSK_PEQD", "DPSK_PGTD", "DPSK_PLTD",
    "FLASHINFER_PEQD", "FLASHINFER_PGTD",
    "HYBRID_FI_PEQD", "HYBRID_FI_PGTD", "HYBRID_FI_PLTD",
    "KDA_PEQD", "KDA_PGTD", "KDA_PLTD",
    "KIMI_K3_PEQD", "KIMI_K3_PGTD", "KIMI_K3_PLTD",
    "TURBOQUANT_PEQD", "TURBOQUANT_PGTD",
]
PARSER = {name: i for i, name in enumerate(PARSER_NAMES)}

(OK, ERR_OUT_OF_RANGE, ERR_OVERFLOW, ERR_INVALID, ERR_UNSUPPORTED, ERR_HIP, ERR_NO_DEVICE,
 ERR_TIMEOUT) = range(8)


class IpcBlock(C.Structure):
    _fields_ = [("src_offset", C.c_uint64), ("dst_offset", C.c_uint64), ("length", C.c_uint64)]

    def astuple(self):
        return (self.src_offset, self.dst_offset, self.length)


class WorkerInfo(C.Structure):
    _fields_ = [
        ("engine_tp_size", C.c_uint32),
        ("worker_tp_rank", C.c_uint32),
        ("n_tensors", C.c_uint32),
        ("layer_num_blocks", C.c_uint32),
        ("block_sizes", C.c_uint64 * MAX_TENSORS),
        ("token_sizes", C.c_uint64 * MAX_TENSORS),
        ("num_layers", C.c_uint32),
        ("attn_kernel_blk_ntpb", C.c_uint32),
        ("indexer_blk_ntpb", C.c_uint32),
        ("attn_pack_size", C.c_uint32),
        ("num_kv_heads", C.c_int32),
        ("num_gdn_layers", C.c_uint32),
        ("hybrid_indexer_token_size", C.c_uint32),
        ("gdn_conv_elem_size", C.c_uint32),
        ("gdn_ssm_elem_size", C.c_uint32),
        ("n_conv_state_shape", C.c_uint32),
        ("conv_state_shape", C.c_uint64 * MAX_SHAPE_DIMS),
        ("n_ssm_state_shape", C.c_uint32),
        ("n_gdn_conv_channel_dims", C.c_uint32),
        ("ssm_state_shape", C.c_uint64 * MAX_SHAPE_DIMS),
        ("gdn_conv_channel_dims", C.c_uint64 * MAX_CHANNEL_DIMS),
        ("num_ple_layers", C.c_uint32),
        ("ple_block_group", C.c_uint32),
        ("ple_conv_elem_size", C.c_uint32),
        ("n_ple_conv_state_shape", C.c_uint32),
        ("ple_conv_state_shape", C.c_uint64 * MAX_SHAPE_DIMS),
        ("n_ple_conv_channel_dims", C.c_uint32),
        ("kda_conv_dim_first", C.c_uint32),
        ("ple_conv_channel_dims", C.c_uint64 * MAX_CHANNEL_DIMS),
        ("hybrid_attn_token_size", C.c_uint32),
        ("reserved0", C.c_uint32),
        ("kda_page_stride", C.c_uint64),
    ]


class Task(C.Structure):
    _fields_ = [
        ("seen_tokens", C.c_uint32),
        ("new_tokens", C.c_uint32),
        ("reach_last_token", C.c_uint32),
        ("n_src_groups", C.c_uint32),
        ("n_dst_groups", C.c_uint32),
        ("reserved0", C.c_uint32),
        ("src_blocks", C.POINTER(C.c_uint32)),
        ("src_group_len", C.POINTER(C.c_uint32)),
        ("dst_blocks", C.POINTER(C.c_uint32)),
        ("dst_group_len", C.POINTER(C.c_uint32)),
    ]


class ParseOpts(C.Structure):
    _fields_ = [("bf16_to_fp8", C.c_uint32), ("pad_last_attn_block", C.c_uint32)]


def make_worker_info(
    block_sizes,
    token_sizes,
    layer_num_blocks,
    tp=1,
    rank=0,
    num_layers=1,
    num_kv_heads=-1,
    attn_kernel_blk_ntpb=None,
    indexer_blk_ntpb=0,
    attn_pack_size=1,
    num_gdn_layers=3,
    hybrid_indexer_token_size=0,
    gdn_conv_elem_size=1,
    gdn_ssm_elem_size=1,
    conv_state_shape=(),
    ssm_state_shape=(),
    gdn_conv_channel_dims=(),
    num_ple_layers=0,
    ple_block_group=0,
    ple_conv_elem_size=1,
    ple_conv_state_shape=(),
    ple_conv_channel_dims=(),
    kda_conv_dim_first=False,
    hybrid_attn_token_size=0,
    kda_page_stride=0,
):
    """Builds a WorkerInfo the way the reference's Context does.

    ``attn_kernel_blk_ntpb`` defaults to block_sizes[0] / token_sizes[0] /
    attn_pack_size (reference: kvtransfer/src/context.cpp:37-65 with
    BLLM_KVTRANS_ATTN_KERNEL_BLK_SIZE unset).
    """
    w = WorkerInfo()
    w.engine_tp_size = tp
    w.worker_tp_rank = rank
    w.n_tensors = len(block_sizes)
    assert len(block_sizes) == len(token_sizes) <= MAX_TENSORS
    for i, (b, t) in enumerate(zip(block_sizes, token_sizes)):
        w.block_sizes[i] = b
        w.token_sizes[i] = t
    w.layer_num_blocks = layer_num_blocks
    w.num_layers = num_layers
    pack = attn_pack_size or 1
    if attn_kernel_blk_ntpb is None:
        attn_kernel_blk_ntpb = (block_sizes[0] // token_sizes[0] // pack) if block_sizes else 0
    w.attn_kernel_blk_ntpb = attn_kernel_blk_ntpb
    w.indexer_blk_ntpb = indexer_blk_ntpb
    w.attn_pack_size = attn_pack_size
    w.num_kv_heads = num_kv_heads
    w.num_gdn_layers = num_gdn_layers
    w.hybrid_indexer_token_size = hybrid_indexer_token_size
    w.gdn_conv_elem_size = gdn_conv_elem_size
    w.gdn_ssm_elem_size = gdn_ssm_elem_size
    for name, vals, cap in (
        ("conv_state_shape", conv_state_shape, MAX_SHAPE_DIMS),
        ("ssm_state_shape", ssm_state_shape, MAX_SHAPE_DIMS),
        ("gdn_conv_channel_dims", gdn_conv_channel_dims, MAX_CHANNEL_DIMS),
        ("ple_conv_state_shape", ple_conv_state_shape, MAX_SHAPE_DIMS),
        ("ple_conv_channel_dims", ple_conv_channel_dims, MAX_CHANNEL_DIMS),
    ):
        assert len(vals) <= cap
        setattr(w, "n_" + name, len(vals))
        arr = getattr(w, name)
        for i, v in enumerate(vals):
            arr[i] = v
    w.num_ple_layers = num_ple_layers
    w.ple_block_group = ple_block_group
    w.ple_conv_elem_size = ple_conv_elem_size
    w.kda_conv_dim_first = 1 if kda_conv_dim_first else 0
    w.hybrid_attn_token_size = hybrid_attn_token_size
    w.kda_page_stride = kda_page_stride
    return w


class TaskBuf:
    """Owns the arrays a ``Task`` struct points at."""

    def __init__(self, seen, new, last, src_groups, dst_groups):
        self.src_groups = [list(g) for g in src_groups]
        self.dst_groups = [list(g) for g in dst_groups]
        sflat = [b for g in self.src_groups for b in g]
        dflat = [b for g in self.dst_groups for b in g]
        self._s = (C.c_uint32 * max(1, len(sflat)))(*sflat)
        self._d = (C.c_uint32 * max(1, len(dflat)))(*dflat)
        self._sl = (C.c_uint32 * max(1, len(self.src_groups)))(*[len(g) for g in self.src_groups])
        self._dl = (C.c_uint32 * max(1, len(self.dst_groups)))(*[len(g) for g in self.dst_groups])
        t = Task()
        t.seen_tokens, t.new_tokens, t.reach_last_token = seen, new, 1 if last else 0
        t.n_src_groups, t.n_dst_groups = len(self.src_groups), len(self.dst_groups)
        t.src_blocks = C.cast(self._s, C.POINTER(C.c_uint32))
        t.dst_blocks = C.cast(self._d, C.POINTER(C.c_uint32))
        t.src_group_len = C.cast(self._sl, C.POINTER(C.c_uint32))
        t.dst_group_len = C.cast(self._dl, C.POINTER(C.c_uint32))
        self.struct = t


def task_array(bufs):
    arr = (Task * max(1, len(bufs)))()
    for i, b in enumerate(bufs):
        arr[i] = b.struct
    return arr
