"""Layer tensors larger than 4 GiB: every offset that crosses 2^32 has to survive
the plan tables, the strided record arithmetic and the int64 launcher arrays.
On a 288 GB part a per-layer KV tensor of 6-8 GiB is the normal case (a 32-layer
model given 200 GB of cache holds 6.25 GiB per layer), so these are ordinary
inputs, not a stress test. Checked against torch's own index_select /
index_copy over 16-byte rows, bit-exact. Needs a real MI355X with ~40 GiB free."""
import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import pipeline, workloads
from test_gpu_full_size import _gathered_equals, _oracle_lists, _scatter, _unit_index

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

GIB = 1 << 30


@pytest.fixture(autouse=True)
def _release_hbm():
    yield
    torch.cuda.empty_cache()


def _random_bytes(n, seed):
    """n seeded random bytes on the GPU, generated 1 GiB at a time."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    out = torch.empty(n, dtype=torch.uint8, device="cuda")
    for a in range(0, n, GIB):
        m = min(GIB, n - a)
        out[a:a + m] = torch.randint(0, 256, (m,), generator=g, device="cuda", dtype=torch.uint8)
    return out


def _pack_unpack_and_compare(plan, ranges, src, dst, s_cap, d_cap):
    """One layer, one tensor: pack from src, unpack into dst, both compared with torch's
    gather / scatter of the 16-byte rows the ranges cover."""
    sc = kvt_amd.Cache(0, [[src]], [s_cap])
    dc = kvt_amd.Cache(0, [[dst]], [d_cap])
    nb = int(ranges[:, 2].sum())
    assert plan.tensor_bytes(0) == nb
    packed = torch.zeros(plan.layer_bytes, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, 1, packed, plan.layer_bytes)
    plan.unpack(dc, 0, 1, packed, plan.layer_bytes)
    torch.cuda.synchronize()
    s_idx = torch.from_numpy(_unit_index(ranges[:, 0], ranges[:, 2])).cuda()
    d_idx = torch.from_numpy(_unit_index(ranges[:, 1], ranges[:, 2])).cuda()
    assert len(torch.unique(d_idx)) == len(d_idx)          # the scatter is race-free
    blob = packed[:nb].view(-1, 16)
    assert _gathered_equals(src.view(-1, 16), s_idx, blob)
    exp = torch.full_like(dst, 0xA5).view(-1, 16)
    _scatter(exp, d_idx, blob)
    assert torch.equal(dst.view(-1, 16), exp)


def test_plain_plan_with_6_and_8_gib_layer_tensors():
    # FLASH layout: K region [0, cap/2), V region [cap/2, cap): every V offset of the
    # 8 GiB destination lies beyond 2^32, and so do the upper K blocks of both sides
    w = workloads.llama8b_batch(n_layers=1, src_pool=98304, dst_pool=131072, n_req=6,
                                min_tok=700, max_tok=2500)
    assert w.capacities("src")[0] == 6 * GIB and w.capacities("dst")[0] == 8 * GIB
    runs = _oracle_lists(w)[0]
    assert (runs[:, 0] >= 2**32).sum() > 50 and (runs[:, 1] >= 2**32).sum() > 50
    assert runs[:, 1].max() > 7 * GIB
    plan, lists = pipeline.build_plan(w, 0)
    assert np.array_equal(lists.tensor(0), runs)
    src = _random_bytes(6 * GIB, 11)
    dst = torch.full((8 * GIB,), 0xA5, device="cuda", dtype=torch.uint8)
    _pack_unpack_and_compare(plan, runs, src, dst, 6 * GIB, 8 * GIB)


def test_run_plan_strided_records_beyond_4_gib():
    # TP2 -> TP1: one 1 KiB K and V row per token, evaluated inside the kernel from
    # (base, stride) records; source 6 GiB (32 KiB blocks), destination 8 GiB
    w = workloads.tp_split("flash", 2, 1, 1, n_layers=1, src_pool=196608, dst_pool=131072,
                           n_req=5, min_tok=300, max_tok=1500)
    assert w.capacities("src")[0] == 6 * GIB and w.capacities("dst")[0] == 8 * GIB
    plan, runs = pipeline.build_plan_runs(w, 0)
    assert plan.num_strided_chunks > 0
    src_i, dst_i = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src_i, dst_i)
    assert rc == 0 and kind != 0
    rc, outs = checkers.oracle_parse(pid, src_i, dst_i, valid, tps, tpr, w.task_bufs())
    assert rc == 0
    ranges = outs[0]
    assert np.array_equal(runs.expand().tensor(0), ranges)
    assert (ranges[:, 0] >= 2**32).sum() > 500 and (ranges[:, 1] >= 2**32).sum() > 500
    src = _random_bytes(6 * GIB, 12)
    dst = torch.full((8 * GIB,), 0xA5, device="cuda", dtype=torch.uint8)
    _pack_unpack_and_compare(plan, ranges, src, dst, 6 * GIB, 8 * GIB)


def test_int64_launcher_arrays_beyond_4_gib():
    # the reference-shaped launchers take offsets as int64 device arrays
    cap = 6 * GIB
    rng = np.random.default_rng(13)
    n = 400
    lens = (rng.integers(1, 40, size=n) * 1024).astype(np.int64)
    slots = np.sort(rng.choice(cap // 65536 - 1, size=n, replace=False)).astype(np.int64)
    gpu_off = slots * 65536
    assert (gpu_off >= 2**32).sum() > 50
    contig = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int64)
    total = int(lens.sum())
    src = _random_bytes(cap, 14)
    out = torch.zeros(total, dtype=torch.uint8, device="cuda")
    so, do, ln = (torch.from_numpy(a).cuda() for a in (gpu_off, contig, lens))
    lib = kvt_amd.lib()
    rc = lib.kvt_launch_copy_d2h_direct(src.data_ptr(), out.data_ptr(), so.data_ptr(),
                                        do.data_ptr(), ln.data_ptr(), n, 0, 0, None)
    assert rc == 0, lib.kvt_last_error()
    torch.cuda.synchronize()
    idx = torch.from_numpy(_unit_index(gpu_off.astype(np.uint64), lens.astype(np.uint64))).cuda()
    assert torch.equal(out.view(-1, 16), src.view(-1, 16).index_select(0, idx))
    dst = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda")
    rc = lib.kvt_launch_copy_h2d_direct(out.data_ptr(), dst.data_ptr(), do.data_ptr(),
                                        so.data_ptr(), ln.data_ptr(), n, 0, 0, None)
    assert rc == 0, lib.kvt_last_error()
    torch.cuda.synchronize()
    exp = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda").view(-1, 16)
    exp.index_copy_(0, idx, out.view(-1, 16))
    assert torch.equal(dst.view(-1, 16), exp)
    del exp, dst
    # converting gather: lens count bf16 elements, source offsets in bytes
    elems = lens // 2
    fp8_off = np.concatenate([[0], np.cumsum(elems)[:-1]]).astype(np.int64)
    out8 = torch.zeros(int(elems.sum()), dtype=torch.uint8, device="cuda")
    do8, ln8 = torch.from_numpy(fp8_off).cuda(), torch.from_numpy(elems).cuda()
    rc = lib.kvt_launch_copy_d2h_bf16_to_fp8(src.data_ptr(), out8.data_ptr(), so.data_ptr(),
                                             do8.data_ptr(), ln8.data_ptr(), n, 0, 0, None)
    assert rc == 0, lib.kvt_last_error()
    torch.cuda.synchronize()
    gathered = src.view(-1, 16).index_select(0, idx).view(-1)        # the bf16 bytes, in order
    table = np.array([checkers.oracle().kvto_bf16_to_fp8(b) for b in range(65536)], dtype=np.uint8)
    lut = torch.from_numpy(table).cuda()
    bits = gathered.view(torch.int16).to(torch.int32) & 0xFFFF
    assert torch.equal(out8, lut[bits.long()])


def test_transposing_pack_with_a_6_gib_page_pool():
    # HND pages -> NHD blob and back; page bases beyond 2^32
    w = workloads.llama70b_flashinfer(n_layers=1, pool=98304, n_req=3, tokens=2048)
    heads, ntpb, row = w.xform
    cap = w.capacities("src")[0]
    assert cap == 6 * GIB
    plan, lists = pipeline.build_plan(w, 0)
    runs = _oracle_lists(w)[0]
    assert np.array_equal(lists.tensor(0), runs)
    assert (runs[:, 0] >= 2**32).sum() > 20 and (runs[:, 1] >= 2**32).sum() > 20
    B = 2 * heads * ntpb * row
    nblk = cap // B
    s_ids = torch.from_numpy(np.concatenate(
        [np.arange(r[0] // B, (r[0] + r[2]) // B) for r in runs]).astype(np.int64)).cuda()
    d_ids = torch.from_numpy(np.concatenate(
        [np.arange(r[1] // B, (r[1] + r[2]) // B) for r in runs]).astype(np.int64)).cuda()
    assert len(torch.unique(d_ids)) == len(d_ids)
    src = _random_bytes(cap, 15)
    dst = torch.full((cap,), 0xA5, device="cuda", dtype=torch.uint8)
    sc, dc = kvt_amd.Cache(0, [[src]], [cap]), kvt_amd.Cache(0, [[dst]], [cap])
    stride = plan.layer_bytes
    assert stride == len(s_ids) * B
    packed = torch.zeros(stride, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, 1, packed, stride)
    plan.unpack(dc, 0, 1, packed, stride)
    torch.cuda.synchronize()
    picked = src.view(nblk, 2, heads, ntpb, row).index_select(0, s_ids)
    want = picked.permute(0, 1, 3, 2, 4).contiguous()
    assert torch.equal(packed, want.view(-1))
    exp = torch.full_like(dst, 0xA5).view(nblk, 2, heads, ntpb, row)
    exp.index_copy_(0, d_ids, picked)
    assert torch.equal(dst.view(nblk, 2, heads, ntpb, row), exp)
