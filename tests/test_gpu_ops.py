"""GPU parity of the remaining multi-tensor operations against the CPU oracle:
scale/cast copies for every dtype pair, zero fill, read-only norm, one-pass unscale+pack,
the plan-free single-tensor entry point, pointer updates and the two-call step."""
import math

import pytest
import torch

from oracle import gradpath as oracle
from rannc_amd import _lib
from rannc_amd.multi_tensor import TensorPlan, copy_cast_, fill_zero_
from tests.helpers import TORCH_DTYPE, assert_bits_equal, place_in_arena

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAIRS = [(s, d) for s in ("f32", "f16", "bf16") for d in ("f32", "f16", "bf16")]
SHAPES = [(0,), (1,), (5,), (8,), (63,), (64,), (65,), (127,), (1023,), (1024,), (1025,), (2047,), (3, 1000), (16385,), (70001,)]


def special_values(dtype):
    vals = [0.0, -0.0, 1.0, -1.0, 65504.0, 65520.0, 70000.0, 1e-8, 5.96e-8, 2.98e-8, 6.1e-5, 3.4e38, -3.4e38,
            1e-40, float("inf"), float("-inf"), float("nan"), 1.0 + 2 ** -8, 1.0 + 2 ** -9, 1.0 + 3 * 2 ** -9,
            1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, 0.1, 1 / 3]
    return torch.tensor(vals, dtype=torch.float32).to(dtype)


def _inputs(dtype, seed):
    g = torch.Generator().manual_seed(seed)
    ts = [(torch.randn(s, generator=g) * 10 ** float(torch.randint(-6, 6, (1,), generator=g))).to(dtype) for s in SHAPES]
    ts.append(special_values(dtype))
    return ts


@pytest.mark.parametrize("src_name,dst_name", PAIRS)
@pytest.mark.parametrize("scale", [1.0, 0.37])
def test_scale_cast_all_pairs(src_name, dst_name, scale):
    sdt, ddt = TORCH_DTYPE[src_name], TORCH_DTYPE[dst_name]
    srcs_cpu = _inputs(sdt, 11)
    srcs = place_in_arena(srcs_cpu, DEV, 1, 3)
    dsts = place_in_arena([torch.full(t.shape, 9.0, dtype=ddt) for t in srcs_cpu], DEV, 3, 1, fill=9.0)
    plan = TensorPlan(srcs, dsts, chunk_elems=2048)
    plan.scale_cast(scale)
    torch.cuda.synchronize()
    for s, d in zip(srcs_cpu, dsts):
        if scale == 1.0:
            want = oracle.cast(s, ddt)
        else:
            want = (s.float() * torch.tensor(scale)).to(ddt)
        assert_bits_equal(d.cpu(), want, f"{src_name}->{dst_name}")
    plan.close()


def test_same_dtype_copy_preserves_every_bit_pattern():
    # raw copy: NaN payloads and signalling NaNs included
    bits = torch.arange(-2 ** 15, 2 ** 15, dtype=torch.int32).to(torch.int16)
    for dt in (torch.float16, torch.bfloat16):
        src = bits.view(dt).to(DEV)
        dst = torch.zeros_like(src)
        TensorPlan([src], [dst]).scale_cast(1.0)
        assert torch.equal(dst.cpu().view(torch.int16), bits)
    f = torch.tensor([0x7F800001, 0x7FC00000, 0xFFC12345, 0x00000001, 0x80000000], dtype=torch.int64).to(torch.int32)
    src = f.view(torch.float32).to(DEV)
    dst = torch.zeros_like(src)
    TensorPlan([src], [dst]).scale_cast(1.0)
    assert torch.equal(dst.cpu().view(torch.int32), f)


def test_zero_over_back_to_back_destinations_and_after_they_move_apart():
    """Destinations that lie back to back in plan order (the views of a bucket, of mixed widths here) are cleared as one
    flat range; once an update moves one of them away the table-driven pass takes over.  Either way exactly the
    destinations' bytes change."""
    arena = torch.full((1 << 20,), 0x55, dtype=torch.uint8, device=DEV)
    specs = [(torch.float16, 1002), (torch.float32, 0), (torch.float32, 30000), (torch.bfloat16, 6), (torch.float32, 4099)]

    def views(start, gap_before=None, gap=0):
        out, o = [], start
        for i, (dt, n) in enumerate(specs):
            if i == gap_before:
                o += gap
            es = torch.empty((), dtype=dt).element_size()
            out.append(arena[o:o + n * es].view(dt))
            o += n * es
        return out, o

    def check(dsts):
        torch.cuda.synchronize()
        covered = torch.zeros(arena.numel(), dtype=torch.bool)
        base = arena.data_ptr()
        for d in dsts:
            covered[d.data_ptr() - base:d.data_ptr() - base + d.numel() * d.element_size()] = True
        got = arena.cpu()
        assert bool((got[covered] == 0).all()) and bool((got[~covered] == 0x55).all())
        arena.fill_(0x55)

    dsts, _ = views(4)                                    # 4-byte aligned start, off the 128-byte grid
    plan = TensorPlan([None] * len(dsts), dsts, chunk_elems=2048)
    plan.zero()
    check(dsts)
    moved, _ = views(4, gap_before=3, gap=64)            # the last two move 64 bytes up: no longer one range
    plan.update(dsts=moved)
    plan.zero()
    check(moved)
    back, _ = views(260)                                  # one range again, elsewhere
    plan.update(dsts=back)
    plan.zero()
    check(back)
    plan.close()


def test_zero_of_scattered_destinations_of_a_streaming_size():
    """Above 1.5 GiB the table-driven clear holds every tile's wavefronts for a moment before they store (pacing);
    the bytes it writes are the same: every destination zero, every gap between them untouched."""
    k, n, gap = 26, (16 << 20) + 5, 37                       # 26 tensors of 64 MiB + 20 B, 148-byte gaps: 1.63 GiB
    arena = torch.full((k * (n + gap) + gap,), 3.0, dtype=torch.float32, device=DEV)
    dsts = [arena[gap + i * (n + gap):gap + i * (n + gap) + n] for i in range(k)]
    plan = TensorPlan([None] * k, dsts)
    plan.zero()
    torch.cuda.synchronize()
    assert int((arena == 0).sum()) == k * n
    assert all(bool((d == 0).all()) for d in dsts)
    assert int((arena == 3.0).sum()) == (k + 1) * gap
    plan.close()


@pytest.mark.parametrize("dst_name", ["f32", "f16", "bf16"])
def test_zero_fills_only_the_destinations(dst_name):
    ddt = TORCH_DTYPE[dst_name]
    shapes = [(0,), (1,), (7,), (100,), (5000,), (70001,)]
    dsts = place_in_arena([torch.full(s, 3.0, dtype=ddt) for s in shapes], DEV, 5, 2, fill=3.0)
    arena_before = dsts[0].untyped_storage()
    plan = TensorPlan([None] * len(dsts), dsts, chunk_elems=2048)
    plan.zero()
    torch.cuda.synchronize()
    for d in dsts:
        assert bool((d == 0).all())
    whole = torch.empty(0, dtype=ddt, device=DEV).set_(arena_before)
    total = sum(d.numel() for d in dsts)
    assert int((whole == 3.0).sum()) == whole.numel() - total     # gaps untouched
    t = torch.full((12345,), 2.0, device=DEV)[1:]
    fill_zero_(t.contiguous())


@pytest.mark.parametrize("src_name", ["f32", "f16", "bf16"])
def test_grad_norm_measures_the_source_as_stored(src_name):
    sdt = TORCH_DTYPE[src_name]
    g = torch.Generator().manual_seed(12)
    cpu = [(torch.randn(s, generator=g)).to(sdt) for s in SHAPES]
    dev = place_in_arena(cpu, DEV, 1, 1)
    # destination dtype differs on purpose: it must not influence the norm of the source
    dsts = [torch.empty(t.shape, dtype=torch.bfloat16 if sdt != torch.bfloat16 else torch.float16, device=DEV) for t in cpu]
    plan = TensorPlan(dev, dsts, chunk_elems=4096)
    plan.grad_norm()
    res = plan.result()
    want = oracle.per_tensor_norms(cpu)
    for a, b in zip(plan.tensor_norms(), want):
        assert math.isclose(a, b, rel_tol=1e-6, abs_tol=1e-30)
    assert math.isclose(res.norm, oracle.grad_global_l2_norm(cpu), rel_tol=1e-6)
    assert res.overflow == 0 and res.clipped == 0
    plan.close()
    # norm-only plan without destinations
    plan = TensorPlan(dev)
    plan.grad_norm()
    assert math.isclose(plan.result().norm, oracle.grad_global_l2_norm(cpu), rel_tol=1e-6)


def test_norm_closed_forms_on_device():
    a = torch.full((4096,), 0.5, device=DEV)
    b = torch.full((64, 64), -0.25, dtype=torch.bfloat16, device=DEV)
    plan = TensorPlan([a, b])
    plan.grad_norm()
    assert plan.tensor_norms() == [32.0, 16.0]
    assert plan.result().norm == math.sqrt(32.0 ** 2 + 16.0 ** 2)


@pytest.mark.parametrize("src_name,dst_name", [("f16", "f32"), ("bf16", "f32"), ("f32", "f32"), ("f16", "f16")])
def test_unscale_pack_matches_apex_semantics(src_name, dst_name):
    sdt, ddt = TORCH_DTYPE[src_name], TORCH_DTYPE[dst_name]
    g = torch.Generator().manual_seed(13)
    cpu = [(torch.randn(s, generator=g) * 128.0).to(sdt) for s in SHAPES]
    dev = place_in_arena(cpu, DEV, 1, 1)
    dsts = place_in_arena([torch.zeros(t.shape, dtype=ddt) for t in cpu], DEV, 2, 1)
    plan = TensorPlan(dev, dsts, chunk_elems=2048)
    plan.unscale_pack(1.0 / 128.0)
    res = plan.result()
    want, flag = oracle.unscale_and_check(cpu, 1.0 / 128.0, ddt)
    assert res.overflow == flag == 0
    for d, w in zip(dsts, want):
        assert_bits_equal(d.cpu(), w, "unscale_pack")
    assert math.isclose(res.norm, oracle.grad_global_l2_norm(want), rel_tol=1e-6)
    # with a non-finite input the values are still written (Apex writes them) and the flag is set
    cpu[3][2] = float("inf")
    dev[3].copy_(cpu[3])
    plan.unscale_pack(1.0 / 128.0)
    res = plan.result()
    want, flag = oracle.unscale_and_check(cpu, 1.0 / 128.0, ddt)
    assert res.overflow == flag == 1
    for d, w in zip(dsts, want):
        assert_bits_equal(d.cpu(), w, "unscale_pack overflow")
    plan.close()


@pytest.mark.parametrize("src_name,dst_name", PAIRS)
def test_single_tensor_entry_point(src_name, dst_name):
    sdt, ddt = TORCH_DTYPE[src_name], TORCH_DTYPE[dst_name]
    g = torch.Generator().manual_seed(14)
    for n in (0, 1, 1023, 1024, 16384, 16385, 100003):
        s = (torch.randn(n + 1, generator=g) * 3).to(sdt)
        sd = s.to(DEV)[1:]                       # off the allocation's alignment
        dd = torch.full((n + 2,), 5.0, dtype=ddt, device=DEV)
        copy_cast_(dd[1:n + 1], sd)
        out = dd.cpu()
        assert_bits_equal(out[1:n + 1], oracle.cast(s[1:], ddt), "single")
        assert out[0] == 5.0 and out[n + 1] == 5.0
    z = torch.full((5001,), 5.0, dtype=ddt, device=DEV)
    copy_cast_(z[1:], None)
    assert float(z[0]) == 5.0 and bool((z[1:] == 0).all())


def test_pointer_update_moves_the_table():
    g = torch.Generator().manual_seed(15)
    a = [torch.randn(3000, generator=g), torch.randn(17, generator=g)]
    b = [torch.randn(3000, generator=g), torch.randn(17, generator=g)]
    da, db = [t.to(DEV) for t in a], [t.to(DEV) for t in b]
    out1 = [torch.zeros_like(t) for t in da]
    out2 = [torch.zeros_like(t) for t in da]
    plan = TensorPlan(da, out1)
    plan.scale_cast(2.0)
    plan.update(srcs=db, dsts=out2)
    plan.scale_cast(2.0)
    plan.update(srcs=da)
    plan.scale_cast(0.5)
    torch.cuda.synchronize()
    for x, o in zip(a, out1):
        assert_bits_equal(o.cpu(), x * 2.0, "first table")
    for x, o in zip(a, out2):
        assert_bits_equal(o.cpu(), x * 0.5, "third call overwrote the second")
    with pytest.raises(ValueError):
        plan.update(srcs=[da[0][:10], da[1]])


def test_two_call_step_equals_fused_step():
    g = torch.Generator().manual_seed(16)
    cpu = [(torch.randn(s, generator=g) * 1e-2 * 1024).to(torch.float16) for s in [(50000,), (33,), (4096,)]]
    dev = [t.to(DEV) for t in cpu]
    o1 = [torch.zeros(t.shape, device=DEV) for t in cpu]
    o2 = [torch.zeros(t.shape, device=DEV) for t in cpu]
    p1, p2 = TensorPlan(dev, o1), TensorPlan(dev, o2)
    p1.fused_step(1 / 1024.0, 0.3)
    p2.step_begin(1 / 1024.0)
    mid = p2.result()
    assert mid.clipped == 0 and mid.coef == 1.0 and mid.overflow == 0
    p2.step_finish(0.3)
    r1, r2 = p1.result(), p2.result()
    assert (r1.norm, r1.coef, r1.clipped) == (r2.norm, r2.coef, r2.clipped) and r1.clipped == 1
    for a, b in zip(o1, o2):
        assert_bits_equal(a.cpu(), b.cpu(), "two-call")
    with pytest.raises(ValueError, match="pending"):
        p2.step_finish(0.3)


def test_error_paths():
    a = torch.zeros(10, device=DEV)
    with pytest.raises(ValueError, match="contiguous"):
        TensorPlan([torch.zeros(10, 10, device=DEV).t()], [torch.zeros(10, 10, device=DEV)])
    with pytest.raises(ValueError, match="GPU"):
        TensorPlan([torch.zeros(10)], [a])
    with pytest.raises(ValueError, match="elements"):
        TensorPlan([a], [torch.zeros(11, device=DEV)])
    with pytest.raises(ValueError, match="dtype"):
        TensorPlan([torch.zeros(10, dtype=torch.float64, device=DEV)], [a])
    p = TensorPlan([a])
    with pytest.raises(ValueError, match="destination"):
        p.scale_cast(1.0)
    with pytest.raises(ValueError, match="inv_scale"):
        TensorPlan([a], [torch.zeros(10, device=DEV)]).fused_step(0.0, 1.0)
    with pytest.raises(ValueError, match="in place"):
        TensorPlan([a], [a.view(torch.int32).view(torch.float32)]).plan  # same dtype in place is fine
        b16 = torch.zeros(20, dtype=torch.bfloat16, device=DEV)
        _lib.scale_cast_single(b16.data_ptr(), b16.data_ptr(), 10, _lib.RG_BF16, _lib.RG_F32, 1.0, 0, 0)


@pytest.mark.parametrize("src_name,dst_name", [("f16", "f32"), ("bf16", "f32"), ("f32", "f32"), ("f16", "f16"), ("f32", "bf16")])
def test_accumulate_and_unscale_accumulate(src_name, dst_name):
    sdt, ddt = TORCH_DTYPE[src_name], TORCH_DTYPE[dst_name]
    g = torch.Generator().manual_seed(17)
    model = [(torch.randn(s, generator=g) * 64.0).to(sdt) for s in SHAPES]
    master = [torch.randn(s, generator=g).to(ddt) for s in SHAPES]
    srcs = place_in_arena(model, DEV, 1, 3)
    dsts = place_in_arena(master, DEV, 2, 1)
    plan_srcs = list(srcs)
    plan_srcs[4] = None                                   # a parameter without a gradient adds nothing
    plan = TensorPlan(plan_srcs, dsts, chunk_elems=2048)
    want = [m.clone() for m in master]
    model_with_hole = [None if i == 4 else x for i, x in enumerate(model)]
    for step in range(2):                                 # accumulate twice
        plan.unscale_accumulate(1.0 / 64.0)
        flag = oracle.unscale_accumulate(want, model_with_hole, 1.0 / 64.0)
        res = plan.result()
        assert res.overflow == flag == 0
        for d, w in zip(dsts, want):
            assert_bits_equal(d.cpu(), w, f"unscale_accumulate step {step}")
        assert math.isclose(res.norm, oracle.grad_global_l2_norm(want), rel_tol=1e-6)
    plan.accumulate(0.25)                                 # plain axpy, no flag / norm
    oracle.unscale_accumulate(want, model_with_hole, 0.25)
    for d, w in zip(dsts, want):
        assert_bits_equal(d.cpu(), w, "accumulate")
    model[2][1] = float("inf")
    srcs[2].copy_(model[2])
    plan.unscale_accumulate(1.0 / 64.0)
    assert plan.result().overflow == 1
    with pytest.raises(ValueError, match="itself"):
        TensorPlan([dsts[5]], [dsts[5]]).accumulate(1.0)
    plan.close()


def test_unscale_accumulate_checks_the_incoming_gradients_only():
    """Apex's unscale_with_stashed passes "check only arg 0, the incoming model grads" to its axpby kernel: an
    inf already sitting in the stashed master gradient makes the result (and the norm) non-finite but does
    not raise the flag."""
    g = torch.Generator().manual_seed(19)
    model = [(torch.randn(5000, generator=g) * 64.0).to(torch.float16), (torch.randn(300, generator=g) * 64.0).to(torch.float16)]
    master = [torch.randn(5000, generator=g), torch.randn(300, generator=g)]
    master[0][4321] = float("inf")
    srcs, dsts = place_in_arena(model, DEV, 1, 3), place_in_arena(master, DEV, 2, 1)
    plan = TensorPlan(srcs, dsts)
    plan.unscale_accumulate(1.0 / 64.0)
    res = plan.result()
    want = [m.clone() for m in master]
    assert oracle.unscale_accumulate(want, model, 1.0 / 64.0) == 0
    assert res.overflow == 0 and math.isinf(res.norm)
    for d, w in zip(dsts, want):
        assert_bits_equal(d.cpu(), w, "accumulated onto a non-finite master gradient")
    plan.close()


@pytest.mark.parametrize("dst_name", ["f32", "bf16"])
def test_chunk_boundaries_follow_the_destination_alignment(dst_name):
    """Chunk boundaries inside a tensor sit on 128-byte boundaries of its destination, so the
    first chunk may be longer than the others and the last one empty; the number of chunks
    must not depend on the addresses (pointer updates keep the table's size)."""
    ddt = TORCH_DTYPE[dst_name]
    chunk = 2048
    per_line = 128 // torch.empty(0, dtype=ddt).element_size()
    g = torch.Generator().manual_seed(21)
    # sizes around multiples of the chunk: a tensor that fits in the lengthened first chunk,
    # one that needs exactly one more element, and a long one
    sizes = [chunk, chunk + 1, chunk + per_line - 1, chunk + per_line, 2 * chunk + 3, 10 * chunk + per_line // 2, 7]
    cpu = [(torch.randn(n, generator=g) * 8).to(torch.float16) for n in sizes]
    total = sum(sizes) + 4 * per_line
    src_arena = torch.zeros(total + 64, dtype=torch.float16, device=DEV)
    plan = None
    for dst_off in (0, 1, per_line // 2 + 1, per_line - 1):
        dst_arena = torch.full((total,), 7.0, dtype=ddt, device=DEV)
        srcs, dsts, o = [], [], dst_off
        for t in cpu:
            s = src_arena[o + 3:o + 3 + t.numel()]
            s.copy_(t)
            srcs.append(s)
            dsts.append(dst_arena[o:o + t.numel()])
            o += t.numel()                                    # no padding: only the first tensor's offset is chosen
        if plan is None:
            plan = TensorPlan(srcs, dsts, chunk_elems=chunk)
            n_chunks = plan.plan.num_chunks
        else:
            plan.update(srcs=srcs, dsts=dsts)
            assert plan.plan.num_chunks == n_chunks
        plan.fused_step(0.125, math.inf)
        res = plan.result()
        want, _ = oracle.unscale_and_check(cpu, 0.125, ddt)
        assert math.isclose(res.norm, oracle.grad_global_l2_norm(want), rel_tol=1e-6) and res.clipped == 0
        for d, w in zip(dsts, want):
            assert_bits_equal(d.cpu(), w, f"offset {dst_off}")
        out = dst_arena.cpu()
        assert bool((out[:dst_off] == 7.0).all()) and bool((out[o:] == 7.0).all())      # nothing outside was touched
        plan.unscale_pack(0.5)
        want2, _ = oracle.unscale_and_check(cpu, 0.5, ddt)
        for d, w in zip(dsts, want2):
            assert_bits_equal(d.cpu(), w, f"unscale_pack offset {dst_off}")
        plan.zero()
        out = dst_arena.cpu()
        assert bool((out[dst_off:o] == 0).all()) and bool((out[:dst_off] == 7.0).all()) and bool((out[o:] == 7.0).all())
    plan.close()


def test_plan_tune_changes_only_the_time():
    """rg_plan_tune measures the block -> XCD orders on the plan's tensors; whatever it picks, a pass writes the
    same bits.  The destinations are overwritten by the measurement itself (cast of the sources)."""
    g = torch.Generator().manual_seed(33)
    cpu = [(torch.randn(n, generator=g) * 8).to(torch.float16) for n in (300001, 17, 70001, 4096, 1)]
    srcs = place_in_arena(cpu, DEV, 1, 3)
    dsts = [torch.full((t.numel(),), 7.0, dtype=torch.float32, device=DEV) for t in cpu]
    plan = TensorPlan(srcs, dsts)
    plan.scale_cast(0.5)
    before = [d.cpu().clone() for d in dsts]
    order = plan.tune()
    assert order in (0, 64, 256, -1)
    for d, c in zip(dsts, cpu):
        assert_bits_equal(d.cpu(), c.float(), "what the measurement leaves behind")
    plan.scale_cast(0.5)
    for d, b in zip(dsts, before):
        assert_bits_equal(d.cpu(), b, "same bits under the tuned order")
    plan.fused_step(0.125, 1.0)
    res = plan.result()
    want = oracle.fused_step(cpu, ["f32"] * len(cpu), 0.125, 1.0)
    assert math.isclose(res.norm, want.norm, rel_tol=1e-6) and res.clipped == 1
    plan.close()
    # in place: left alone
    t = torch.randn(5000, device=DEV)
    keep = t.clone()
    p2 = TensorPlan([t], [t])
    p2.tune()
    assert torch.equal(t, keep)
    p2.close()


@pytest.mark.parametrize("nbytes", [0, 1, 15, 16, 17, 127, 128, 129, 4095, 4096, 4097, 8 * 4096 * 64 + 5, (1 << 20) + 3])
@pytest.mark.parametrize("offset", [0, 1, 2, 16, 127, 129])
def test_fill_zero_writes_exactly_its_bytes(nbytes, offset):
    """``rg_fill_zero`` over a flat byte range at any address: every byte of the range is zero afterwards and no
    byte outside it is touched (tiles are laid out from the first 128-byte boundary; the bytes before it and
    behind the last whole 16 are written one at a time)."""
    from rannc_amd import _lib
    from rannc_amd.multi_tensor import stream_handle
    guard = 256
    arena = torch.full((guard + offset + nbytes + guard,), 0xAB, dtype=torch.uint8, device=DEV)
    _lib.fill_zero(arena.data_ptr() + guard + offset, nbytes, 0, stream_handle(torch.device(DEV)))
    torch.cuda.synchronize()
    lo, hi = guard + offset, guard + offset + nbytes
    assert int(arena[lo:hi].count_nonzero()) == 0
    assert int((arena[:lo] == 0xAB).sum()) == lo
    assert int((arena[hi:] == 0xAB).sum()) == arena.numel() - hi


def test_fill_zero_of_a_streaming_size():
    """Above 256 MiB the fill uses streaming stores; same contract."""
    from rannc_amd import _lib
    from rannc_amd.multi_tensor import stream_handle
    nbytes, offset, guard = (300 << 20) + 5, 3, 256
    arena = torch.full((guard + offset + nbytes + guard,), 0x5C, dtype=torch.uint8, device=DEV)
    _lib.fill_zero(arena.data_ptr() + guard + offset, nbytes, 0, stream_handle(torch.device(DEV)))
    torch.cuda.synchronize()
    lo, hi = guard + offset, guard + offset + nbytes
    assert int(arena[lo:hi].count_nonzero()) == 0
    assert int((arena[:lo] == 0x5C).sum()) == lo and int((arena[hi:] == 0x5C).sum()) == guard
