"""Seeded generators of valid ParseBlock inputs for every parser family.

A *case* is a JSON-serialisable dict::

    {"name", "parser" (name), "src": {make_worker_info kwargs}, "dst": {...},
     "valid": mask, "tp_size", "tp_rank", "fp8": bool,
     "tasks": [[seen, new, last, src_groups, dst_groups], ...]}

The same cases feed (a) oracle-vs-compiled-reference comparison, (b) the golden
fixture writer in tests/golden/, (c) product-vs-oracle parity tests.
"""
import numpy as np

from kvt_amd.ctypes_defs import PARSER, TaskBuf, make_worker_info


def materialise(case):
    src = make_worker_info(**case["src"])
    dst = make_worker_info(**case["dst"])
    tasks = [TaskBuf(*t) for t in case["tasks"]]
    return PARSER[case["parser"]], src, dst, case["valid"], case["tp_size"], case["tp_rank"], tasks


def _ids(rng, pool, n):
    return [int(x) for x in rng.choice(pool, size=n, replace=False)]


def _token_plan(rng, ntpb, max_blocks=6):
    """-> list of (seen, new, last) chunk steps covering one request, n_blocks"""
    total = int(rng.integers(1, ntpb * max_blocks + 1))
    steps, seen = [], 0
    while seen < total:
        new = int(rng.integers(1, total - seen + 1))
        steps.append((seen, new, seen + new == total))
        seen += new
    return steps, (total + ntpb - 1) // ntpb, total


def _all_mask(tp):
    return (1 << tp) - 1


def _pick_steps(rng, steps):
    # one random chunk, plus always consider the whole request as one step
    return steps[int(rng.integers(0, len(steps)))]


def gen_token_walk(rng, parser):
    """RAGGED / FLASH / DPSK / FLASHINFER families."""
    fam, kind = parser.rsplit("_", 1) if not parser.endswith("_DPSK") else ("RAGGED", "PGTD_DPSK")
    ntpb = int(rng.choice([1, 2, 4, 16, 64]))
    elem = int(rng.choice([1, 2]))
    hd = int(rng.choice([8, 64, 128])) * elem          # bytes per head row
    n_tensors = 2 if fam == "DPSK" else 1
    pool_s, pool_d = int(rng.integers(8, 64)), int(rng.integers(8, 64))
    if kind == "PEQD":
        tp = int(rng.choice([1, 2, 4]))
        p_tp = d_tp = tp
    elif kind in ("PGTD", "PGTD_DPSK"):
        d_tp = int(rng.choice([1, 2, 4]))
        p_tp = d_tp * int(rng.choice([2, 4]))
    else:
        p_tp = int(rng.choice([1, 2, 4]))
        d_tp = p_tp * int(rng.choice([2, 4]))
    big, small = max(p_tp, d_tp), min(p_tp, d_tp)
    gn = big // small
    heads_small_side = int(rng.choice([1, 2, 4]))      # heads per rank on the larger-TP side
    total_heads = heads_small_side * big
    if fam == "FLASHINFER":
        # per-rank heads on P; D holds gn times more
        p_heads = total_heads // p_tp
        pT = 2 * p_heads * hd
        dT = 2 * (total_heads // d_tp) * hd
        toks_p, toks_d = [pT], [dT]
    elif fam == "DPSK":
        if kind == "PEQD" or (kind == "PGTD" and rng.random() < 0.4):
            toks_p = toks_d = [576 * elem, 128 * elem]     # replicated MLA: same token size
        else:
            base = [2 * heads_small_side * hd, 2 * hd]
            if kind == "PGTD":
                toks_p, toks_d = base, [t * gn for t in base]
            else:
                toks_d, toks_p = base, [t * gn for t in base]
    else:
        base = 2 * heads_small_side * hd
        if kind == "PEQD" or kind == "PGTD_DPSK":
            toks_p = toks_d = [base]
        elif kind == "PGTD":
            toks_p, toks_d = [base], [base * gn]
        else:
            toks_d, toks_p = [base], [base * gn]
    if kind == "PLTD":
        d_rank = int(rng.integers(0, d_tp))
        p_rank = d_rank // gn
    elif kind in ("PGTD", "PGTD_DPSK"):
        p_rank = int(rng.integers(0, p_tp))
        d_rank = p_rank // gn
        if kind == "PGTD_DPSK" or (fam == "DPSK" and toks_p == toks_d):
            p_rank = int(rng.choice([0, p_rank]))
            d_rank = 0 if p_rank == 0 else d_rank
    else:
        p_rank = d_rank = int(rng.integers(0, p_tp))
    src = dict(block_sizes=[t * ntpb for t in toks_p], token_sizes=toks_p, layer_num_blocks=pool_s,
               tp=p_tp, rank=p_rank, num_kv_heads=total_heads)
    dst = dict(block_sizes=[t * ntpb for t in toks_d], token_sizes=toks_d, layer_num_blocks=pool_d,
               tp=d_tp, rank=d_rank, num_kv_heads=total_heads)
    valid = _all_mask(p_tp)
    tasks = []
    for _ in range(int(rng.integers(1, 4))):
        steps, nblk, _ = _token_plan(rng, ntpb, max_blocks=min(6, pool_s, pool_d))
        seen, new, last = _pick_steps(rng, steps)
        tasks.append([seen, new, last, [_ids(rng, pool_s, nblk)], [_ids(rng, pool_d, nblk)]])
    return dict(parser=parser, src=src, dst=dst, valid=valid, tp_size=p_tp, tp_rank=p_rank,
                fp8=False, tasks=tasks)


def gen_hybrid(rng, parser):
    """QWEN3_NEXT_FLASH (HYBRID_*), QWEN3_NEXT_FLASHINFER (HYBRID_FI_*), TURBOQUANT_*."""
    fi = "_FI_" in parser
    kind = parser.rsplit("_", 1)[1]
    elem = 2
    if kind == "PEQD":
        p_tp = d_tp = int(rng.choice([1, 2, 4]))
    elif kind == "PGTD":
        d_tp = int(rng.choice([1, 2]))
        p_tp = d_tp * int(rng.choice([2, 4]))
    else:
        p_tp = int(rng.choice([1, 2]))
        d_tp = p_tp * int(rng.choice([2, 4]))
    big, small = max(p_tp, d_tp), min(p_tp, d_tp)
    gn = big // small
    # head regime: total heads >= big (fully split) most of the time; sometimes
    # replicated (heads <= small) for P<D; for P>D with few heads valid ranks thin out.
    regime = str(rng.choice(["split", "few", "mixed"])) if kind != "PEQD" else "split"
    if regime == "mixed" and not (kind == "PLTD" and gn == 4):
        regime = "split"
    hd = int(rng.choice([16, 64])) * elem
    if regime == "split":
        total_heads = big * int(rng.choice([1, 2]))
    elif regime == "mixed":
        total_heads = p_tp * 2                         # p_tp < heads < d_tp
    else:
        total_heads = small if kind == "PLTD" else int(rng.choice([h for h in (1, 2, 4) if h < p_tp and p_tp % h == 0 and (d_tp % h == 0 or h % d_tp == 0)]))
    pack = int(rng.choice([1, 1, 2])) if not fi else 1
    kb = int(rng.choice([4, 8, 16]))                  # kernel-block tokens
    per_layer_ntpb = kb * (int(rng.choice([1, 2])) if not fi else 1)
    ntpb = per_layer_ntpb * pack                       # tokens per physical page (all pack members)

    def heads_per_rank(tp):
        return max(1, total_heads // tp)

    pT = 2 * heads_per_rank(p_tp) * hd
    dT = 2 * heads_per_rank(d_tp) * hd
    pB, dB = pT * ntpb, dT * ntpb
    # valid ranks as the reference computes them
    from checkers import oracle
    valid = oracle().kvto_valid_ranks(p_tp, d_tp, total_heads)
    tp_size = bin(valid).count("1")
    if kind == "PLTD":
        d_rank = int(rng.integers(0, d_tp))
        p_rank = d_rank // gn
    elif kind == "PGTD":
        p_rank = int(rng.integers(0, p_tp))
        d_rank = p_rank // gn
    else:
        p_rank = d_rank = int(rng.integers(0, p_tp))
    tp_rank = bin(valid & ((1 << p_rank) - 1)).count("1")
    n_gdn = int(rng.choice([0, 1, 3]))
    has_indexer = bool(rng.random() < 0.4)
    n_ple = int(rng.choice([0, 0, 1, 2]))
    # GDN state geometry on the side with the larger TP ("narrow"), scaled by gn on the other
    rows = int(rng.choice([2, 3]))
    chan_narrow = [int(rng.choice([2, 4])) * 2 for _ in range(3)]
    ssm_narrow = (1, int(rng.choice([1, 2])), 2, 4)
    conv_e, ssm_e = 2, 4

    def gdn_meta(scale):
        ch = [c * scale for c in chan_narrow]
        return dict(conv_state_shape=[8, rows, sum(ch)], ssm_state_shape=[8, ssm_narrow[1] * scale, ssm_narrow[2], ssm_narrow[3]],
                    gdn_conv_channel_dims=ch, gdn_conv_elem_size=conv_e, gdn_ssm_elem_size=ssm_e)

    p_scale = gn if kind == "PLTD" else 1
    d_scale = gn if kind == "PGTD" else 1
    ple_shape = [8, 2, 3]
    idx_tok = 16
    idx_ntpb_p = (pB // idx_tok) if has_indexer else 0
    idx_ntpb_d = (dB // idx_tok) if has_indexer else 0
    if has_indexer and kind == "PEQD":
        idx_ntpb_p = idx_ntpb_d = int(rng.choice([per_layer_ntpb, per_layer_ntpb * 2]))
    if has_indexer and kind == "PLTD" and pT == dT:
        idx_ntpb_p = idx_ntpb_d = per_layer_ntpb
    pool_s, pool_d = int(rng.integers(24, 64)), int(rng.integers(24, 64))
    common = dict(num_kv_heads=total_heads, attn_pack_size=pack, num_gdn_layers=n_gdn,
                  hybrid_indexer_token_size=idx_tok if has_indexer else 0,
                  num_ple_layers=n_ple, ple_block_group=n_gdn + (1 if has_indexer else 0) + 1,
                  ple_conv_elem_size=2, ple_conv_state_shape=ple_shape,
                  attn_kernel_blk_ntpb=kb if not fi else ntpb)
    src = dict(block_sizes=[pB], token_sizes=[pT], layer_num_blocks=pool_s, tp=p_tp, rank=p_rank,
               indexer_blk_ntpb=idx_ntpb_p, **common, **gdn_meta(p_scale))
    dst = dict(block_sizes=[dB], token_sizes=[dT], layer_num_blocks=pool_d, tp=d_tp, rank=d_rank,
               indexer_blk_ntpb=idx_ntpb_d, **common, **gdn_meta(d_scale))
    # state pages must fit into a page on both sides
    state_p = rows * sum(chan_narrow) * p_scale * conv_e + ssm_narrow[1] * p_scale * 8 * ssm_e
    state_d = rows * sum(chan_narrow) * d_scale * conv_e + ssm_narrow[1] * d_scale * 8 * ssm_e
    if state_p > pB or state_d > dB:
        return gen_hybrid(rng, parser)
    tasks = []
    for _ in range(int(rng.integers(1, 3))):
        steps, nblk, total = _token_plan(rng, per_layer_ntpb, max_blocks=5)
        seen, new, last = _pick_steps(rng, steps)
        extra = int(rng.choice([0, 0, 1]))           # spec-decode trailing blocks
        sg, dg = [], []
        used_s, used_d = set(), set()

        def take(pool, used, n):
            avail = [i for i in range(pool) if i not in used]
            got = [int(x) for x in rng.choice(avail, size=n, replace=False)]
            used.update(got)
            return got

        for _g in range(n_gdn):
            sg.append(take(pool_s, used_s, 1))
            dg.append(take(pool_d, used_d, 1))
        if has_indexer:
            n_i_s = max(1, -(-(total) // max(1, idx_ntpb_p)))
            n_i_d = max(1, -(-(total) // max(1, idx_ntpb_d)))
            if kind == "PEQD" or (kind == "PLTD" and pT == dT):
                n_i_s = n_i_d = max(n_i_s, n_i_d)
            sg.append(take(pool_s, used_s, n_i_s))
            dg.append(take(pool_d, used_d, n_i_d))
        sg.append(take(pool_s, used_s, nblk + extra))
        dg.append(take(pool_d, used_d, nblk + extra))
        for _g in range(n_ple):
            sg.append(take(pool_s, used_s, 1))
            dg.append(take(pool_d, used_d, 1))
        tasks.append([seen, new, last, sg, dg])
    return dict(parser=parser, src=src, dst=dst, valid=int(valid), tp_size=tp_size, tp_rank=tp_rank,
                fp8=False, tasks=tasks)


def gen_kda(rng, parser):
    """KDA state pages (KDA_*) and Kimi-K3 (KDA groups + one replicated MLA group)."""
    kimi = parser.startswith("KIMI")
    kind = parser.rsplit("_", 1)[1]
    if kind == "PEQD":
        p_tp = d_tp = int(rng.choice([1, 2, 4]))
    elif kind == "PGTD":
        d_tp = int(rng.choice([1, 2]))
        p_tp = d_tp * int(rng.choice([2, 4]))
    else:
        p_tp = int(rng.choice([1, 2]))
        d_tp = p_tp * int(rng.choice([2, 4]))
    gn = max(p_tp, d_tp) // min(p_tp, d_tp)
    if kind == "PLTD":
        d_rank = int(rng.integers(0, d_tp))
        p_rank = d_rank // gn
    elif kind == "PGTD":
        p_rank = int(rng.integers(0, p_tp))
        d_rank = p_rank // gn
    else:
        p_rank = d_rank = int(rng.integers(0, p_tp))
    dim_first = bool(rng.random() < 0.5)
    state_len = int(rng.choice([2, 3, 4]))
    narrow_ch = [int(rng.choice([2, 4, 6])) for _ in range(3)]
    narrow_rec = (int(rng.choice([1, 2])), 2, int(rng.choice([2, 4])))
    conv_e, rec_e = int(rng.choice([1, 2])), 4

    def meta(scale):
        ch = [c * scale for c in narrow_ch]
        qkv = sum(ch)
        shape = [8, qkv, state_len] if dim_first else [8, state_len, qkv]
        rec = [8, narrow_rec[0] * scale, narrow_rec[1], narrow_rec[2]]
        size = state_len * qkv * conv_e + rec[1] * rec[2] * rec[3] * rec_e
        return dict(conv_state_shape=shape, ssm_state_shape=rec, gdn_conv_channel_dims=ch,
                    gdn_conv_elem_size=conv_e, gdn_ssm_elem_size=rec_e,
                    kda_conv_dim_first=dim_first), size

    p_meta, p_size = meta(gn if kind == "PLTD" else 1)
    d_meta, d_size = meta(gn if kind == "PGTD" else 1)
    n_gdn = int(rng.choice([1, 2, 3]))
    mla_tok = 16 * int(rng.choice([1, 2, 4]))
    kernel_ntpb = int(rng.choice([2, 4]))
    s_mgr = kernel_ntpb * int(rng.choice([1, 2]))
    d_mgr = s_mgr if kind == "PEQD" else kernel_ntpb * int(rng.choice([1, 2, 4]))
    # physical page must hold the KDA state and, for Kimi, the MLA prefix of a manager block
    s_page = -(-max(p_size, s_mgr * mla_tok if kimi else 0) // 64) * 64 + 64 * int(rng.integers(0, 3))
    d_page = -(-max(d_size, d_mgr * mla_tok if kimi else 0) // 64) * 64 + 64 * int(rng.integers(0, 3))
    if kind == "PEQD":
        d_page = s_page
    use_stride = bool(rng.random() < 0.5) or kimi
    pool_s, pool_d = int(rng.integers(16, 48)), int(rng.integers(16, 48))
    if kimi:
        # logical MLA blocks: block_sizes[0] = manager tokens x registered token size
        reg_tok = mla_tok
        s_blk, d_blk, s_tok, d_tok = s_mgr * reg_tok, d_mgr * reg_tok, reg_tok, reg_tok
        # capacity of the registered tensor must cover pool * physical page
        s_lnb = -(-pool_s * s_page // s_blk)
        d_lnb = -(-pool_d * d_page // d_blk)
    else:
        s_blk, d_blk, s_tok, d_tok = s_page, d_page, s_page, d_page
        s_lnb, d_lnb = pool_s, pool_d
    common = dict(num_kv_heads=1, num_gdn_layers=n_gdn, attn_kernel_blk_ntpb=kernel_ntpb,
                  hybrid_attn_token_size=mla_tok if kimi else 0, attn_pack_size=1)
    src = dict(block_sizes=[s_blk], token_sizes=[s_tok], layer_num_blocks=s_lnb, tp=p_tp,
               rank=p_rank, kda_page_stride=s_page if use_stride else 0, **common, **p_meta)
    dst = dict(block_sizes=[d_blk], token_sizes=[d_tok], layer_num_blocks=d_lnb, tp=d_tp,
               rank=d_rank, kda_page_stride=d_page if use_stride else 0, **common, **d_meta)
    from checkers import oracle
    valid = oracle().kvto_valid_ranks(p_tp, d_tp, 1)
    tp_size = bin(valid).count("1")
    tp_rank = bin(valid & ((1 << p_rank) - 1)).count("1")
    tasks = []
    for _ in range(int(rng.integers(1, 3))):
        used_s, used_d = set(), set()

        def take(pool, used, n):
            avail = [i for i in range(pool) if i not in used]
            got = [int(x) for x in rng.choice(avail, size=n, replace=False)]
            used.update(got)
            return got

        sg = [take(pool_s, used_s, 1) for _ in range(n_gdn)]
        dg = [take(pool_d, used_d, 1) for _ in range(n_gdn)]
        steps, _, total = _token_plan(rng, s_mgr, max_blocks=4)
        seen, new, last = _pick_steps(rng, steps)
        if kimi:
            extra = int(rng.choice([0, 1]))
            n_s = -(-total // s_mgr) + extra
            n_d = -(-total // d_mgr) + extra
            if kind == "PEQD":
                n_d = n_s
            sg.append(take(pool_s, used_s, n_s))
            dg.append(take(pool_d, used_d, n_d))
        tasks.append([seen, new, last, sg, dg])
    return dict(parser=parser, src=src, dst=dst, valid=int(valid), tp_size=tp_size, tp_rank=tp_rank,
                fp8=False, tasks=tasks)


TOKEN_WALK = ["RAGGED_PEQD", "RAGGED_PGTD", "RAGGED_PGTD_DPSK", "RAGGED_PLTD", "FLASH_PEQD",
              "FLASH_PGTD", "DPSK_PEQD", "DPSK_PGTD", "DPSK_PLTD", "FLASHINFER_PEQD",
              "FLASHINFER_PGTD"]
HYBRID = ["HYBRID_PEQD", "HYBRID_PGTD", "HYBRID_PLTD", "HYBRID_FI_PEQD", "HYBRID_FI_PGTD",
          "HYBRID_FI_PLTD", "TURBOQUANT_PEQD", "TURBOQUANT_PGTD"]
KDA = ["KDA_PEQD", "KDA_PGTD", "KDA_PLTD", "KIMI_K3_PEQD", "KIMI_K3_PGTD", "KIMI_K3_PLTD"]
ALL_PARSERS = TOKEN_WALK + HYBRID + KDA


def gen_case(parser, seed):
    rng = np.random.default_rng(seed)
    if parser in TOKEN_WALK:
        c = gen_token_walk(rng, parser)
    elif parser in KDA:
        c = gen_kda(rng, parser)
    else:
        base = parser.replace("TURBOQUANT", "HYBRID")
        c = gen_hybrid(rng, base)
        c["parser"] = parser
    c["name"] = "%s/seed%d" % (parser, seed)
    return c


def gen_synthetic_runs(seed, cap, run_dtype):
    """Strided runs that no parser would emit (odd lengths, zero source strides, three full
    levels, lengths around 4 KiB, many distinct shapes). Destination ranges never overlap."""
    rng = np.random.default_rng(seed)
    runs = np.zeros(int(rng.integers(1, 40)), dtype=run_dtype)
    d_cursor = 0
    for r in runs:
        length = int(rng.choice([16, 48, 256, 1000, 1024, 4080, 4096, 5000, 20]))
        n = [int(rng.integers(1, 4)), int(rng.integers(1, 9)), int(rng.integers(1, 4))]
        unit = 16 if rng.random() < 0.8 else 4
        # destination: dense nest laid out from a running cursor, so that ranges never overlap
        d2 = (length + unit - 1) // unit * unit + unit * int(rng.integers(0, 3))
        d1 = d2 * n[2] + unit * int(rng.integers(0, 3))
        d0 = d1 * n[1] + unit * int(rng.integers(0, 3))
        r["length"], r["n"] = length, n
        r["dst_offset"] = d_cursor
        r["dst_stride"] = [d0, d1, d2]
        d_cursor += d0 * n[0] + 64
        # source: anything inside the buffer, repeats allowed (strides may be zero)
        s_str = [unit * int(rng.integers(0, 600)), unit * int(rng.integers(0, 80)),
                 unit * int(rng.integers(0, 40))]
        span = sum(s * (k - 1) for s, k in zip(s_str, n)) + length
        r["src_offset"] = unit * int(rng.integers(0, (cap - span) // unit))
        r["src_stride"] = s_str
    assert d_cursor < cap
    return runs
