"""The bookkeeping behind repeated layers (kllm_amd/engine/repeat.py), without a GPU: which
descriptions are alike, which tensors a run may name, how a second run's commands are
explained from the first's, and how what a block gave is handed on in another run's name."""

from dataclasses import dataclass

import numpy as np
import torch

from kllm_amd.engine import repeat as R
from kllm_amd.parts import LayerSpec, Part, PartSpec
from kllm_amd.parts.base import PagedCacheView, Runtime


def layer(i, window=0, eps=1e-5, names=None):
    rotary = PartSpec("rotary", head_dim=16, theta=1e4)
    mixer = PartSpec("attention", f"l{i}.attn", hidden=64, heads=4, window=window, position=rotary)
    if names:
        mixer.params["names"] = names
    return LayerSpec(mixer=mixer, feed_forward=PartSpec("gated_mlp", f"l{i}.mlp", hidden=64, intermediate=176),
                     norm_mixer=PartSpec("rmsnorm", f"l{i}.n1", size=64, eps=eps),
                     norm_feed_forward=PartSpec("rmsnorm", f"l{i}.n2", size=64, eps=eps))


def test_descriptions_that_differ_in_names_only_are_alike():
    assert R._alike(layer(0)) == R._alike(layer(5)) == R._alike(layer(2, names={"o_proj.weight": "elsewhere"}))
    assert R._alike(layer(0)) != R._alike(layer(1, window=8))
    assert R._alike(layer(0)) != R._alike(layer(1, eps=1e-6))
    a, b = layer(0), layer(1)
    b.block_params = {"scale": 2.0}
    assert R._alike(a) != R._alike(b)
    assert R._alike(object()) != R._alike(object())       # what is not understood is alike to itself only
    hash(R._alike(layer(0)))


class Holder:
    def __init__(self, t):
        self.data = t


class ToyPart(Part):
    def __init__(self, seed, rt, child=None):
        super().__init__(PartSpec("toy"), rt)
        g = torch.Generator().manual_seed(seed)
        self.w = torch.randn(8, 16, generator=g)
        self.rows = self.w[2:4]                          # a view is held beside the tensor it is cut from
        self.more = {"gu": Holder(torch.randn(32, generator=g)), "list": [torch.randn(4, generator=g)]}
        self.empty = torch.empty(0)
        self.child = child
        self.eps = 1e-5


def names_of(seed, rt, with_next=True):
    block = ToyPart(seed, rt, child=ToyPart(seed + 100, rt))
    nxt = ToyPart(seed + 200, rt) if with_next else None
    return R._Names(block, nxt), block, nxt


def test_every_tensor_and_part_of_a_run_has_a_path():
    rt = Runtime(device=torch.device("cpu"), dtype=torch.float32)
    n, block, nxt = names_of(1, rt)
    assert set(n.parts) == {("b",), ("b", "child"), ("n",)}
    assert n.parts[("b", "child")] is block.child and n.path_of[id(nxt)] == ("n",)
    assert ("b", "more", "'gu'", "data") in n.tensors and ("b", "child", "more", "'list'", 0) in n.tensors
    assert ("b", "empty") not in n.address
    # an address inside a tensor is found with its offset; one inside a view as well (either name will do:
    # the other run's tensor of that name lies at the same place in its own)
    path, off = n.find(block.w.data_ptr() + 4 * 5)
    assert (path, off) == (("b", "w"), 20) or (path, off) == (("b", "rows"), 20 - 4 * 32)
    path, off = n.find(block.w.data_ptr() + 4 * 40)
    assert n.address[path] + off == block.w.data_ptr() + 160
    assert n.find(block.w.data_ptr() + 4 * 8 * 16) is None or n.find(block.w.data_ptr() + 4 * 8 * 16)[0] != ("b", "w")
    assert n.find(12345) is None
    # the same block as its own successor: nothing is named twice
    again = R._Names(block, block)
    assert set(again.parts) == {("b",), ("b", "child")}


def words_of(n: R._Names, view, scratch):
    """Commands as a run with these names might write them: headers, sizes, addresses."""
    return np.array([(3 << 32) | (2 << 16) | 7, n.address[("b", "w")] + 64, scratch, 128,
                     (4 << 32) | (3 << 16) | 9, n.address[("n", "more", "'gu'", "data")], view.pages.data_ptr() + 256,
                     view.block_table.data_ptr(), np.float32(0.5).view(np.uint32)], dtype=np.uint64)


def test_a_second_run_is_explained_by_its_own_tensors():
    rt = Runtime(device=torch.device("cpu"), dtype=torch.float32)
    (na, _, _), (nb, _, _), (nc, _, _) = names_of(1, rt), names_of(2, rt), names_of(3, rt)
    table = torch.zeros(4, dtype=torch.int32)
    va, vb = (PagedCacheView(torch.zeros(1024), table, 16) for _ in range(2))
    held = torch.zeros(8)
    scratch = held.data_ptr()
    wa, wb = words_of(na, va, scratch), words_of(nb, vb, scratch)
    found = R._StepRepeater._explain(wa, wb, na, nb, va, vb)
    assert [(i, p) for i, p, _ in found if p[0] != "c"] == [(1, ("b", "w")), (5, ("n", "more", "'gu'", "data"))]
    # (the table both views share is the same word in both runs: it may be named or left as it is)
    in_views = sorted((i, p, o) for i, p, o in found if p[0] == "c")
    assert in_views[0] == (6, ("c", "pages"), 256) and in_views[1:] in ([], [(7, ("c", "block_table"), 0)])
    assert [o for i, p, o in found if i == 1] == [64]
    # a word that differs and is no tensor's address (a scratch buffer that alternates): no
    other = wb.copy()
    other[2] = wb[2] + np.uint64(1 << 20)
    assert R._StepRepeater._explain(wa, other, na, nb, va, vb) is None
    # a word that names a tensor of the first run's layer, where the second names another tensor of its own: no
    other = wb.copy()
    other[1] = nb.address[("b", "child", "w")] + 64
    assert R._StepRepeater._explain(wa, other, na, nb, va, vb) is None
    # a tensor that both layers share is its own counterpart
    nb.address[("b", "w")] = na.address[("b", "w")]
    other = wb.copy()
    other[1] = wa[1]
    assert R._StepRepeater._explain(wa, other, na, nb, va, vb) is not None
    # a cache view with other fields: no
    @dataclass
    class OtherView:
        pages: torch.Tensor
    assert R._StepRepeater._explain(wa, wb, na, nb, va, OtherView(vb.pages)) is None


@dataclass
class Pending:
    x: torch.Tensor
    norm: Part
    parts: int = 3


def test_what_a_block_gave_is_handed_on_in_another_runs_name():
    rt = Runtime(device=torch.device("cpu"), dtype=torch.float32)
    (na, ba, nxa), (nb, bb, nxb) = names_of(1, rt), names_of(2, rt)
    x = torch.zeros(4, 8)
    gave_a, gave_b = (x, Pending(x[1:], nxa)), (x, Pending(x[1:], nxb))
    assert R._shape(gave_a, na) == R._shape(gave_b, nb)
    assert R._shape(gave_a, na) != R._shape((x, Pending(x[2:], nxa)), na)
    assert R._shape(gave_a, na) != R._shape((x, Pending(x[1:], ba.child)), na)
    moved = R._moved(gave_a, na, nb)
    assert moved[0] is x and moved[1].norm is nxb and moved[1].x is gave_a[1].x and moved[1].parts == 3
    assert gave_a[1].norm is nxa                                   # a copy, the first run's own is as it was
    stranger = ToyPart(9, rt)
    try:
        R._shape((x, Pending(x, stranger)), na)
        raise AssertionError("a part that the run cannot name was taken")
    except R._Unnamed:
        pass
    try:
        R._shape((x, rt), na)
        raise AssertionError
    except R._Unnamed:
        pass


def test_recorded_commands_are_copied_and_added_with_their_step_values():
    """The recording side of repeated layers: commands written inside ``copy_recorded`` are also
    kept apart, with the places of the step's values in them, and ``add_recorded`` puts such
    commands behind what was recorded, the places moved along.  Nothing is launched here: the
    recording is dropped, not run (the library is only asked for its table of entry points)."""
    import pytest
    from kllm_amd import kernels as K
    try:
        K._ops()
    except Exception as exc:                       # no built library where this runs
        pytest.skip(f"the kernel library is not there: {exc}")
    rec = K._Recorder(stream=0, chunk=10 ** 9, keep=True)
    K._scoped.recorder = rec
    try:
        n_args = K._ops()["kllm_attn_prefill"].nargs
        dynamic = K._ops()["kllm_attn_prefill"].dynamic
        args = [1000 + i for i in range(n_args)]
        args[14] = 0.125                                              # the scale, a float
        args[dynamic[0]], args[dynamic[1]] = K.StepValue(777, "keys.total"), K.StepValue(55, "keys.longest")
        K._launch("kllm_attn_prefill", "before", *args)
        first = rec.at
        with K.copy_recorded() as copied:
            K._launch("kllm_attn_prefill", "attention", *args)
            K._launch("kllm_silu_mul", "gate", 1, 2, 3, 4, 5, 6, 7, 8, 9, 0)
        assert copied.whole and copied.run.names == ["attention", "gate"]
        assert bytes(copied.run.data) == bytes(rec.buf[first:rec.at])
        assert copied.run.patches == [(8 + 8 * dynamic[0], "keys.total"), (8 + 8 * dynamic[1], "keys.longest")]
        assert rec.patches[2:] == [(first + off, name) for off, name in copied.run.patches]
        # the same commands again, as a layer that is alike would add them
        words = np.frombuffer(bytes(copied.run.data), dtype=np.uint64).copy()
        words[1] = 424242                                              # the first argument of the first command
        second = rec.at
        K.add_recorded(words.tobytes(), copied.run.names, copied.run.patches)
        assert rec.names == ["before", "attention", "gate", "attention", "gate"]
        assert int(np.frombuffer(bytes(rec.buf[second:second + 16]), dtype=np.uint64)[1]) == 424242
        assert bytes(rec.buf[second + 16:rec.at]) == bytes(copied.run.data[16:])
        assert rec.patches[4:] == [(second + off, name) for off, name in copied.run.patches]
        # something launched past the recording inside: the copy is not whole
        with K.copy_recorded() as broken:
            K._launch("kllm_silu_mul", "gate", 1, 2, 3, 4, 5, 6, 7, 8, 9, 0)
            rec.bypassed = True                                        # (what bypass_recorded and direct_launches leave)
        assert not broken.whole and rec.bypassed
        # outside a recording there is nothing to copy
        K._scoped.recorder = None
        with K.copy_recorded() as nothing:
            pass
        assert nothing.run is None and not nothing.whole
    finally:
        rec.names = []                                                 # dropped, not run
        K._scoped.recorder = None
