"""Writes tests/golden/parse_golden.json from the COMPILED REFERENCE.

Run in the authoring container only (needs /root/reference):

    make -C oracle ref && python tests/golden/make_golden.py

For every parser family it takes seeded cases from tests/cases.py, runs the
reference's own ParseBlock function through oracle/_ref/libkvt_ref.so and stores
inputs + expected (src_offset, dst_offset, length) triples. The bf16->fp8
variants need the reference's process-wide environment switch, so they are
produced in a child process with BLLM_KVTRANS_BF162FP8_CONV=1.

The fixture holds data only (inputs and expected outputs).
"""
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [os.path.join(ROOT, "llumnix-kv_amd"), os.path.join(ROOT, "tests")]

import cases  # noqa: E402
import checkers  # noqa: E402

SEEDS = [0, 1, 2, 3, 4, 5]
FP8_PARSERS = ["RAGGED_PEQD", "RAGGED_PGTD", "RAGGED_PLTD", "FLASH_PEQD", "FLASH_PGTD", "DPSK_PGTD",
               "DPSK_PLTD"]


def config_shaped():
    """Small samples with the geometry of the benchmark configurations."""
    out = []
    # FLASH, T=4096, B=65536, pool 1024
    w = dict(block_sizes=[65536], token_sizes=[4096], layer_num_blocks=1024, num_kv_heads=8)
    out.append(dict(name="cfg/flash_llama8b", parser="FLASH_PEQD", src=w, dst=w, valid=1, tp_size=1,
                    tp_rank=0, fp8=False, tasks=[[0, 40, True, [[7, 3, 900]], [[0, 1, 2]]]]))
    # FlashInfer HND 8 heads x 128 bf16
    out.append(dict(name="cfg/flashinfer_hnd", parser="FLASHINFER_PEQD", src=w, dst=w, valid=1,
                    tp_size=1, tp_rank=0, fp8=False, tasks=[[0, 20, True, [[5, 2]], [[1, 0]]]]))
    # DeepSeek V3.2: MLA 576 B/token + indexer 128 B/token, 64 tokens per block
    m = dict(block_sizes=[36864, 8192], token_sizes=[576, 128], layer_num_blocks=64, num_kv_heads=1)
    out.append(dict(name="cfg/dpsk_v32", parser="DPSK_PEQD", src=m, dst=m, valid=1, tp_size=1,
                    tp_rank=0, fp8=False, tasks=[[10, 150, True, [[9, 3, 4]], [[7, 8, 1]]]]))
    # Qwen3-Next hybrid pages: 3 GDN groups + attention group, 2 KV heads x 256 bf16, 16 tokens
    q = dict(block_sizes=[32768], token_sizes=[2048], layer_num_blocks=256, num_kv_heads=2,
             num_gdn_layers=3)
    out.append(dict(name="cfg/qwen3_next_chunk", parser="HYBRID_PEQD", src=q, dst=q, valid=1,
                    tp_size=1, tp_rank=0, fp8=False,
                    tasks=[[0, 40, False, [[6], [7], [8], [3, 4, 5]], [[10], [11], [12], [7, 8, 9]]],
                           [5, 50, True, [[16], [17], [18], [13, 14, 15, 19]],
                            [[20], [21], [22], [23, 24, 25, 26]]]]))
    # the reference's own hybrid arrangement (uniform pages shared by attention and GDN states),
    # at P == D and between a TP2 prefill and a TP1 decode instance; a FLASH TP2 -> TP1 batch
    from kvt_amd import workloads
    for tag, w in (("cfg/qwen3_next_uniform_pages", workloads.qwen3next_uniform_pages(
                        n_layers=1, pool=40, n_req=3, tokens=2500)),
                   ("cfg/qwen3_next_tp2_to_tp1_rank0", workloads.qwen3next_tp_split(
                        2, 1, 0, n_layers=1, pool=16, n_req=1, tokens=200, head_dim=64, state_dim=32)),
                   ("cfg/qwen3_next_tp2_to_tp1_rank1", workloads.qwen3next_tp_split(
                        2, 1, 1, n_layers=1, pool=16, n_req=1, tokens=200, head_dim=64, state_dim=32)),
                   ("cfg/flash_tp2_to_tp1", workloads.tp_split(
                        "flash", 2, 1, 1, n_layers=1, src_pool=32, dst_pool=48, n_req=2,
                        min_tok=20, max_tok=100))):
        out.append(workload_case(tag, w))
    return out


def workload_case(name, w, fp8=False):
    """A kvt_amd.workloads.Workload as a golden case (dispatch values from the oracle's
    restatement of refresh_dst_info, which the valid-rank known answers pin)."""
    src, dst = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    assert rc == 0
    from kvt_amd.ctypes_defs import PARSER
    parser = [k for k, v in PARSER.items() if v == pid][0]
    return dict(name=name, parser=parser, src=w.src_info, dst=w.dst_info, valid=int(valid),
                tp_size=int(tps), tp_rank=int(tpr), fp8=fp8, tasks=w.tasks)


def run_cases(case_list):
    res = []
    for c in case_list:
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(c)
        rc, outs = checkers.ref_parse(pid, src, dst, valid, tps, tpr, tasks)
        c = dict(c)
        c["rc"] = rc
        c["expect"] = [o.tolist() for o in outs]
        res.append(c)
    return res


def main():
    if "--child-fp8" in sys.argv:
        assert os.environ.get("BLLM_KVTRANS_BF162FP8_CONV") == "1"
        lst = []
        for p in FP8_PARSERS:
            for s in SEEDS[:4]:
                c = cases.gen_case(p, 100 + s)
                c["fp8"] = True
                c["name"] += "/fp8"
                # the converting path reads 2x the length at the source: give the source pool room
                lst.append(c)
        from kvt_amd import workloads
        lst.append(workload_case("cfg/flash_tp2_to_tp1/fp8", workloads.tp_split(
            "flash", 2, 1, 1, n_layers=1, src_pool=32, dst_pool=48, n_req=2, min_tok=20,
            max_tok=100, fp8_dst=True), fp8=True))
        json.dump(run_cases(lst), sys.stdout)
        return
    assert checkers.ref() is not None, "build oracle/_ref first (make -C oracle ref)"
    lst = config_shaped()
    for p in cases.ALL_PARSERS:
        for s in SEEDS:
            lst.append(cases.gen_case(p, s))
    golden = run_cases(lst)
    env = dict(os.environ, BLLM_KVTRANS_BF162FP8_CONV="1")
    child = subprocess.run([sys.executable, os.path.abspath(__file__), "--child-fp8"], env=env,
                           stdout=subprocess.PIPE, check=True)
    text = child.stdout.decode()
    golden += json.loads(text[text.index("[{"):])
    path = os.path.join(HERE, "parse_golden.json")
    with open(path, "w") as f:
        json.dump(golden, f, separators=(",", ":"))
    print("wrote", path, len(golden), "cases", os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
