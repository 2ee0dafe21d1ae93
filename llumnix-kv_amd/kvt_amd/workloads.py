"""Seeded synthetic workloads shaped like the five benchmark configurations.

A workload is plain host data (numpy / python): cache geometry, per-request
block tables and the ParseBlock inputs. Device memory is the caller's business.
Every builder takes scale parameters so that tests can run the same code on
small pools while bench.py uses the full sizes.
"""
from dataclasses import dataclass, field

import numpy as np

from .ctypes_defs import (PARSER, SHAPE_DPSK_V32_SPARSE_MLA, SHAPE_FLASH, SHAPE_FLASHINFER,
                          SHAPE_QWEN3_NEXT_FLASH, SHAPE_RAGGED_FLASH, TaskBuf, make_worker_info)


@dataclass
class Workload:
    name: str
    cache_shape: int
    parser: str
    n_layers: int
    src_info: dict                 # make_worker_info kwargs (sender)
    dst_info: dict                 # make_worker_info kwargs (receiver)
    tasks: list                    # [seen, new, last, src_groups, dst_groups] per request
    elem_dtype: str = "bf16"       # "bf16" | "fp8" | "f32"
    xform: tuple = None            # (heads, ntpb, row_bytes) for the HND<->NHD transposing pack
    seed: int = 0
    notes: dict = field(default_factory=dict)

    def worker_infos(self):
        return make_worker_info(**self.src_info), make_worker_info(**self.dst_info)

    def task_bufs(self):
        return [TaskBuf(*t) for t in self.tasks]

    @property
    def n_tensors(self):
        return len(self.src_info["block_sizes"])

    def capacities(self, side="src"):
        info = self.src_info if side == "src" else self.dst_info
        return [b * info["layer_num_blocks"] for b in info["block_sizes"]]


def _tables(rng, n_req, lens_tokens, ntpb, src_pool, dst_pool):
    """Block tables the way a paged allocator hands them out: every request gets blocks
    nobody else holds, drawn from one seeded permutation of the pool. Destination tables
    are always disjoint (a scatter into shared blocks would race). When the batch needs
    more source blocks than the source pool has, the permutation wraps around, i.e. the
    last requests share blocks with the first ones (reads only, as with a shared prefix)."""
    n_blocks = [(int(t) + ntpb - 1) // ntpb for t in lens_tokens]
    total = sum(n_blocks)
    if total > dst_pool:
        raise ValueError("destination pool too small for disjoint tables: %d > %d"
                         % (total, dst_pool))
    dperm = rng.permutation(dst_pool)[:total]
    sperm = rng.permutation(src_pool)
    src, dst, pos = [], [], 0
    for nb in n_blocks:
        if nb > src_pool:
            raise ValueError("request larger than the source pool")
        src.append([int(sperm[(pos + i) % src_pool]) for i in range(nb)])
        dst.append([int(x) for x in dperm[pos:pos + nb]])
        pos += nb
    return src, dst


def llama8b_single(n_layers=32, pool=1024, tokens=512, seed=20251):
    """Config 1: FlashAttention layout [2, pool, 16, 8, 128] bf16, one request."""
    rng = np.random.default_rng(seed)
    T, ntpb = 2 * 8 * 128 * 2, 16
    src, dst = _tables(rng, 1, [tokens], ntpb, pool, pool)
    info = dict(block_sizes=[T * ntpb], token_sizes=[T], layer_num_blocks=pool, num_kv_heads=8,
                num_layers=n_layers)
    return Workload("llama3-8b FA 1x%d tok" % tokens, SHAPE_FLASH, "FLASH_PEQD", n_layers, info,
                    dict(info), [[0, tokens, True, [src[0]], [dst[0]]]], seed=seed)


def llama8b_batch(n_layers=32, src_pool=16384, dst_pool=24576, n_req=64, min_tok=1024,
                  max_tok=8192, seed=20252):
    """Config 2: same geometry, 64 requests with lengths uniform in [1k, 8k]."""
    rng = np.random.default_rng(seed)
    T, ntpb = 4096, 16
    lens = rng.integers(min_tok, max_tok + 1, size=n_req)
    src, dst = _tables(rng, n_req, lens, ntpb, src_pool, dst_pool)
    s_info = dict(block_sizes=[T * ntpb], token_sizes=[T], layer_num_blocks=src_pool,
                  num_kv_heads=8, num_layers=n_layers)
    d_info = dict(s_info, layer_num_blocks=dst_pool)
    tasks = [[0, int(n), True, [s], [d]] for n, s, d in zip(lens, src, dst)]
    return Workload("llama3-8b FA %dreq x %d-%d tok" % (n_req, min_tok, max_tok), SHAPE_FLASH,
                    "FLASH_PEQD", n_layers, s_info, d_info, tasks, seed=seed,
                    notes=dict(tokens=int(lens.sum())))


def llama70b_flashinfer(n_layers=80, pool=8192, n_req=32, tokens=4096, transpose=True,
                        seed=20253, heads=8):
    """Config 3: FlashInfer pages, HND in the cache ([pool, 2, 8, 16, 128] bf16; `heads` KV
    heads instead of 8 for one rank of a tensor-parallel instance).

    transpose=True: whole-page plan (the page parse of the NHD page layout) with
    the HND->NHD transform applied while packing. transpose=False: the plain
    FlashInfer HND parse (per-head ranges, merged)."""
    rng = np.random.default_rng(seed)
    ntpb, row = 16, 256
    T = 2 * heads * row
    src, dst = _tables(rng, n_req, [tokens] * n_req, ntpb, pool, pool)
    info = dict(block_sizes=[T * ntpb], token_sizes=[T], layer_num_blocks=pool, num_kv_heads=heads,
                num_layers=n_layers, num_gdn_layers=0)
    tasks = [[0, tokens, True, [s], [d]] for s, d in zip(src, dst)]
    if transpose:
        return Workload("llama3-70b FlashInfer HND->NHD %dreq x %d tok" % (n_req, tokens),
                        SHAPE_QWEN3_NEXT_FLASH, "HYBRID_PEQD", n_layers, info, dict(info), tasks,
                        xform=(heads, ntpb, row), seed=seed)
    return Workload("llama3-70b FlashInfer HND %dreq x %d tok" % (n_req, tokens), SHAPE_FLASHINFER,
                    "FLASHINFER_PEQD", n_layers, info, dict(info), tasks, seed=seed)


def deepseek_mla(n_layers=61, pool=4608, n_req=16, tokens=16384, seed=20254):
    """Config 4: MLA latent (576 B/token) + DSA indexer keys (128 B/token), fp8, 64 tokens/block."""
    rng = np.random.default_rng(seed)
    ntpb = 64
    src, dst = _tables(rng, n_req, [tokens] * n_req, ntpb, pool, pool)
    info = dict(block_sizes=[576 * ntpb, 128 * ntpb], token_sizes=[576, 128],
                layer_num_blocks=pool, num_kv_heads=1, num_layers=n_layers)
    tasks = [[0, tokens, True, [s], [d]] for s, d in zip(src, dst)]
    return Workload("deepseek-v3 MLA+indexer fp8 %dreq x %d tok" % (n_req, tokens),
                    SHAPE_DPSK_V32_SPARSE_MLA, "DPSK_PEQD", n_layers, info, dict(info), tasks,
                    elem_dtype="fp8", seed=seed)


def qwen3next_attn(n_layers=12, pool=36864, n_req=128, tokens=4096, seed=20255):
    """Config 5, full-attention part: NHD pages of 2 KV heads x 256 bf16, 16 tokens (32 KiB)."""
    rng = np.random.default_rng(seed)
    T, ntpb = 2 * 2 * 256 * 2, 16
    src, dst = _tables(rng, n_req, [tokens] * n_req, ntpb, pool, pool)
    info = dict(block_sizes=[T * ntpb], token_sizes=[T], layer_num_blocks=pool, num_kv_heads=2,
                num_layers=n_layers, num_gdn_layers=0)
    tasks = [[0, tokens, True, [s], [d]] for s, d in zip(src, dst)]
    return Workload("qwen3-next full-attn pages %dreq x %d tok" % (n_req, tokens),
                    SHAPE_QWEN3_NEXT_FLASH, "HYBRID_PEQD", n_layers, info, dict(info), tasks,
                    seed=seed)


def qwen3next_gdn(n_layers=36, slots=256, n_req=128, seed=20256):
    """Config 5, linear-attention part: one 2 MiB fp32 state (32 x 128 x 128) per request and
    layer, kept in its own pool of state slots. A state is one whole page of that pool and is
    sent when the request completes (the whole-page rule of the hybrid P==D parser, with the
    page size set to the slot stride)."""
    rng = np.random.default_rng(seed)
    state = 32 * 128 * 128 * 4
    perm_s = rng.permutation(slots)[:n_req]
    perm_d = rng.permutation(slots)[:n_req]
    info = dict(block_sizes=[state], token_sizes=[state], layer_num_blocks=slots, num_kv_heads=2,
                num_layers=n_layers, num_gdn_layers=0)
    # one "token" per request in a pool whose page holds one token: exactly one whole page
    tasks = [[0, 1, True, [[int(s)]], [[int(d)]]] for s, d in zip(perm_s, perm_d)]
    return Workload("qwen3-next GDN state %dreq" % n_req, SHAPE_QWEN3_NEXT_FLASH, "HYBRID_PEQD",
                    n_layers, info, dict(info), tasks, elem_dtype="f32", seed=seed)


def qwen3next_uniform_pages(n_layers=12, pool=1024, n_req=128, tokens=4096, n_gdn=3, seed=20258):
    """Config 5 the way the reference itself lays a hybrid model out: ONE cache tensor per
    full-attention layer, shared with the n_gdn linear-attention layers in front of it, with
    one uniform page size (kvtbackend.py:994-1000). The page must hold a 2 MiB GDN state
    (32 x 128 x 128 fp32), so an attention page holds 1024 tokens of 2 KV heads x 256 bf16.
    Block groups per request: [gdn_0, .., gdn_{n-1}, attn]; a request sends its attention pages
    and, with its last token, one state page per GDN layer
    (parse_block_qwen3_next.cpp:865-955)."""
    rng = np.random.default_rng(seed)
    T, page = 2 * 2 * 256 * 2, 32 * 128 * 128 * 4
    ntpb = page // T
    n_attn = (tokens + ntpb - 1) // ntpb
    per_req = n_gdn + n_attn
    if per_req * n_req > pool:
        raise ValueError("pool too small for disjoint tables: %d > %d" % (per_req * n_req, pool))
    sperm, dperm = rng.permutation(pool), rng.permutation(pool)
    tasks = []
    for r in range(n_req):
        s = [int(x) for x in sperm[r * per_req:(r + 1) * per_req]]
        d = [int(x) for x in dperm[r * per_req:(r + 1) * per_req]]
        sg = [[s[g]] for g in range(n_gdn)] + [s[n_gdn:]]
        dg = [[d[g]] for g in range(n_gdn)] + [d[n_gdn:]]
        tasks.append([0, tokens, True, sg, dg])
    info = dict(block_sizes=[page], token_sizes=[T], layer_num_blocks=pool, num_kv_heads=2,
                num_layers=n_layers, num_gdn_layers=n_gdn)
    return Workload("qwen3-next hybrid, uniform 2 MiB pages %dreq x %d tok" % (n_req, tokens),
                    SHAPE_QWEN3_NEXT_FLASH, "HYBRID_PEQD", n_layers, info, dict(info), tasks,
                    seed=seed)


def qwen3next_tp_split(p_tp=2, d_tp=1, rank=0, n_layers=12, pool=1024, n_req=128, tokens=4096,
                       n_gdn=3, kv_heads=2, head_dim=256, key_heads=16, value_heads=32,
                       state_dim=128, conv_rows=3, kernel_block=16, seed=20259):
    """The hybrid model of config 5 between a TP`p_tp` prefill and a TP`d_tp` decode instance
    (p_tp > d_tp), in the reference's arrangement (one tensor per full-attention layer, uniform
    pages shared with `n_gdn` GDN layers). Every rank holds kv_heads / tp attention heads
    (bf16), conv state rows of 2 * key_dim + value_dim bf16 channels and an fp32 SSM state of
    value_heads / tp x state_dim x state_dim, so a sending rank's pieces interleave into the
    receiver's wider rows: per token and K / V for attention (inside kernel blocks of
    `kernel_block` tokens), per conv row and channel group (q, k, v) plus one SSM range for a
    GDN state (parse_block_qwen3_next.cpp:108-413, 532-711). `rank` is the sending rank."""
    if p_tp <= d_tp or p_tp % d_tp or kv_heads % p_tp or key_heads % p_tp or value_heads % p_tp:
        raise ValueError("need p_tp a multiple of d_tp and heads divisible by p_tp")
    rng = np.random.default_rng(seed)
    gn = p_tp // d_tp

    def side(tp):
        tok = 2 * (kv_heads // tp) * head_dim * 2
        key_dim, value_dim = key_heads // tp * state_dim, value_heads // tp * state_dim
        chans = [key_dim, key_dim, value_dim]
        conv = conv_rows * sum(chans) * 2
        ssm = (value_heads // tp) * state_dim * state_dim * 4
        return tok, chans, conv + ssm

    pT, p_ch, p_state = side(p_tp)
    dT, d_ch, d_state = side(d_tp)
    ntpb = -(-d_state // dT)                       # tokens per page: the page holds a D state
    ntpb = -(-ntpb // kernel_block) * kernel_block
    assert pT * ntpb >= p_state
    n_attn = (tokens + ntpb - 1) // ntpb
    per_req = n_gdn + n_attn
    if per_req * n_req > pool:
        raise ValueError("pool too small for disjoint tables: %d > %d" % (per_req * n_req, pool))
    sperm, dperm = rng.permutation(pool), rng.permutation(pool)
    tasks = []
    for r in range(n_req):
        s = [int(x) for x in sperm[r * per_req:(r + 1) * per_req]]
        d = [int(x) for x in dperm[r * per_req:(r + 1) * per_req]]
        tasks.append([0, tokens, True, [[s[g]] for g in range(n_gdn)] + [s[n_gdn:]],
                      [[d[g]] for g in range(n_gdn)] + [d[n_gdn:]]])

    def info(tp, rk, tok, chans):
        return dict(block_sizes=[tok * ntpb], token_sizes=[tok], layer_num_blocks=pool, tp=tp,
                    rank=rk, num_kv_heads=kv_heads, num_layers=n_layers, num_gdn_layers=n_gdn,
                    attn_kernel_blk_ntpb=kernel_block,
                    conv_state_shape=[pool, conv_rows, sum(chans)],
                    ssm_state_shape=[pool, value_heads // tp, state_dim, state_dim],
                    gdn_conv_channel_dims=chans, gdn_conv_elem_size=2, gdn_ssm_elem_size=4)

    return Workload("qwen3-next hybrid TP%d->TP%d, uniform pages %dreq x %d tok" %
                    (p_tp, d_tp, n_req, tokens), SHAPE_QWEN3_NEXT_FLASH, "HYBRID_PGTD", n_layers,
                    info(p_tp, rank, pT, p_ch), info(d_tp, rank // gn, dT, d_ch), tasks, seed=seed,
                    notes=dict(tokens=tokens * n_req, page_tokens=ntpb))


def tp_split(layout="flash", p_tp=2, d_tp=1, rank=0, n_layers=32, src_pool=16384,
             dst_pool=24576, n_req=64, min_tok=1024, max_tok=8192, total_heads=8, head_dim=128,
             ntpb=16, seed=20257, fp8_dst=False):
    """A TP-remapping batch (prefill TP != decode TP): every token's K and V rows are split
    between / gathered from several ranks, i.e. one short range per token (and per head for
    the HND page layout). layout = "flash" ([2, nblk, bs, h, d]), "hnd" ([nblk, 2, h, bs, d])
    or "ragged" ([nblk, bs, 2, h, d], the only one with a P<D parser); bf16. `rank` is the sending rank when p_tp > d_tp, the receiving rank otherwise.
    fp8_dst: the receiver's cache holds fp8 (half the token size); parse with fp8=True, the
    sender converts while it gathers."""
    rng = np.random.default_rng(seed)
    row = head_dim * 2
    pT = 2 * (total_heads // p_tp) * row
    dT = 2 * (total_heads // d_tp) * row // (2 if fp8_dst else 1)
    lens = rng.integers(min_tok, max_tok + 1, size=n_req)
    src, dst = _tables(rng, n_req, lens, ntpb, src_pool, dst_pool)
    gn = max(p_tp, d_tp) // min(p_tp, d_tp)
    p_rank, d_rank = (rank, rank // gn) if p_tp > d_tp else (rank // gn, rank)
    s_info = dict(block_sizes=[pT * ntpb], token_sizes=[pT], layer_num_blocks=src_pool, tp=p_tp,
                  rank=p_rank, num_kv_heads=total_heads, num_layers=n_layers)
    d_info = dict(block_sizes=[dT * ntpb], token_sizes=[dT], layer_num_blocks=dst_pool, tp=d_tp,
                  rank=d_rank, num_kv_heads=total_heads, num_layers=n_layers)
    tasks = [[0, int(n), True, [s], [d]] for n, s, d in zip(lens, src, dst)]
    kind = "PGTD" if p_tp > d_tp else "PLTD"
    shape, fam = {"flash": (SHAPE_FLASH, "FLASH"), "hnd": (SHAPE_FLASHINFER, "FLASHINFER"),
                  "ragged": (SHAPE_RAGGED_FLASH, "RAGGED")}[layout]
    if kind == "PLTD" and layout != "ragged":
        raise ValueError("the reference has a P<D parser only for the ragged layout")
    return Workload("%s TP%d->TP%d %dreq x %d-%d tok" % (layout, p_tp, d_tp, n_req, min_tok, max_tok),
                    shape, "%s_%s" % (fam, kind), n_layers, s_info, d_info, tasks, seed=seed,
                    notes=dict(tokens=int(lens.sum()), fp8=bool(fp8_dst)))


def parser_id(w):
    return PARSER[w.parser]
