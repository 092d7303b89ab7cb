"""What a recipe says as data, checked without a GPU: parameters that are rows of a larger checkpoint tensor,
paged needs with a page length of their own, and the scheduler's page accounting over such groups."""
import pytest
import torch

from arle_amd.cache import CacheManager, OutOfPages, PagedNeed
from arle_amd.parts import Part, PartSpec, Rows, WeightDecl, build_part, expected_tensors, register
from arle_amd.parts.base import Runtime


@register("feed_forward", "cpu_two_mats")
class TwoMats(Part):
    @classmethod
    def declare_weights(cls, params):
        return {"a": WeightDecl((params["rows_a"], params["cols"])), "b": WeightDecl((params["rows_b"], params["cols"])),
                "scale": WeightDecl((params["cols"],), init="ones")}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.tensors = tensors


def test_parameters_may_be_rows_of_one_checkpoint_tensor():
    params = {"rows_a": 3, "rows_b": 5, "cols": 4}
    spec = PartSpec("cpu_two_mats", params, {"a": Rows("ab", 0, 3, 8), "b": Rows("ab", 3, 8, 8), "scale": "s"})
    want = expected_tensors("feed_forward", spec)
    assert set(want) == {"ab", "s"} and tuple(want["ab"].shape) == (8, 4) and want["ab"].init == "normal"
    whole = torch.arange(32.0).reshape(8, 4)
    part = build_part("feed_forward", spec, {"ab": whole, "s": torch.ones(4)}.__getitem__,
                      Runtime(torch.device("cpu"), torch.float32))
    assert torch.equal(part.tensors["a"], whole[:3]) and torch.equal(part.tensors["b"], whole[3:])
    assert part.tensors["b"].data_ptr() == whole[3:].data_ptr()        # a view of the loaded tensor, no copy


def test_rows_that_do_not_fit_their_parameter_or_their_tensor_are_refused():
    params = {"rows_a": 3, "rows_b": 5, "cols": 4}
    with pytest.raises(ValueError, match="rows 0:4"):
        expected_tensors("feed_forward", PartSpec("cpu_two_mats", params,
                                                  {"a": Rows("ab", 0, 4, 8), "b": Rows("ab", 3, 8, 8), "scale": "s"}))
    with pytest.raises(ValueError, match="two shapes"):
        expected_tensors("feed_forward", PartSpec("cpu_two_mats", params,
                                                  {"a": Rows("ab", 0, 3, 8), "b": Rows("ab", 3, 8, 9), "scale": "s"}))
    with pytest.raises(ValueError, match="do not lie"):
        Rows("ab", 5, 9, 8)


def test_a_paged_need_may_have_a_page_length_of_its_own():
    needs = [PagedNeed(2, 16), PagedNeed(1, 8, page_size=16), PagedNeed(2, 16)]
    c = CacheManager(needs, page_size=4, num_pages=32, max_slots=3, max_request_tokens=70)
    assert [(g.page_size, g.pool.num_pages) for g in c.groups] == [(4, 32), (16, 8)]     # the same 128 tokens each
    assert c.pool_tokens() == 128 and c.request_capacity == 72       # 18 pages of 4, 5 of 16: the shorter reach
    assert c.pages_for_length(33) == [9, 3]
    c.admit("a")
    c.append([("a", 33)])
    assert c.free_pages() == [32 - 9, 8 - 3]
    assert c.view(0).page_size == 4 and c.view(1).page_size == 16 and c.view(2).page_size == 4
    assert c.pages_needed([("a", 15)]) == [3, 0]        # 48 tokens: 12 pages of 4, still 3 of 16
    c.admit("b")
    with pytest.raises(OutOfPages):                     # the coarse group runs out first: 5 pages left, 6 asked for
        c.append([("b", 16 * 5 + 1)])
    assert c.length("b") == 0 and c.free_pages() == [23, 5]
    with pytest.raises(OutOfPages, match="longest request"):
        c.append([("a", 40)])
    c.check()
    c.release("a")
    c.release("b")
    assert c.free_pages() == [32, 8]
    c.check()


def test_admission_counts_pages_group_by_group():
    """Two groups with pages of 4 and of 16 tokens over the same 64 tokens: a prompt of 17 tokens + 1 takes 5 of 16
    fine pages but 2 of 4 coarse ones, so the coarse group admits two such requests and defers the third."""
    from test_scheduler import FakeSampler, expected_output, prompt
    from arle_amd.engine.scheduler import Scheduler, SchedulerConfig
    from test_scheduler import FakeEngine

    eng = FakeEngine(slots=4)
    eng.cache = CacheManager([PagedNeed(1, 16), PagedNeed(1, 16, page_size=16)], page_size=4, num_pages=16, max_slots=4,
                             max_request_tokens=64)
    s = Scheduler(eng, FakeSampler(), SchedulerConfig(num_slots=4))
    ids = [s.submit(prompt(17, k), max_tokens=3) for k in range(3)]
    s.iteration()
    assert len(eng.cache.slot_of) == 2 and len(s.waiting) == 1
    s.run_until_done()
    for k, rid in enumerate(ids):
        assert s.finished[rid].generated == expected_output(prompt(17, k), 3)
    assert eng.cache.free_pages() == [16, 4] and not eng.cache.slot_of


def test_a_product_table_is_parsed_and_looked_up_by_widths_and_rows():
    """The table that says which kernel runs a matrix product (what `bench.py --tune-products` writes): keys are the
    widths, entries are looked up by the first row count that is not smaller; the tables that come with the package
    parse, name known kernels only and are sorted by row count."""
    import json
    import os

    from arle_amd.kernels import ops

    saved = dict(ops._PRODUCT_TABLE)
    try:
        ops.clear_product_table()
        ops.load_product_table({"640,320,0,1": [[64, "stream", [1], 4], [16, "rows", [], 0]], "640,320,1,1": [[8, "rounds", [], 0]]})
        entries = ops._PRODUCT_TABLE[(640, 320, False, True)]
        assert [m for m, _ in entries] == [16, 64] and entries[1][1] == ops.ProductChoice("stream", (1,), 4)
        assert (640, 320, True, True) in ops._PRODUCT_TABLE
        with pytest.raises(ops.ShapeError):
            ops.load_product_table({"8,8,0,0": [[4, "magic", [], 0]]})
        ops.clear_product_table()
        assert ops.load_shipped_product_tables() >= 1
        for name in os.listdir(ops.PRODUCT_TABLE_DIR):
            table = json.load(open(os.path.join(ops.PRODUCT_TABLE_DIR, name)))
            for key, rows in table.items():
                assert len(key.split(",")) == 4 and [r[0] for r in rows] == sorted(r[0] for r in rows)
                assert all(r[1] in ops.PRODUCT_KERNELS for r in rows)
    finally:
        ops.clear_product_table()
        ops._PRODUCT_TABLE.update(saved)
