"""The torch.ops.hgcalml.* ops have fake ("meta") implementations: output shapes and dtypes follow from
the input shapes alone, so torch.compile / torch.export can trace through them. Checked on meta tensors:
no kernel runs, no GPU is needed."""
import pytest
import torch


@pytest.fixture(scope="module")
def ops():
    from hgcalml_amd import ops
    return ops


def m(*shape, dtype=torch.float32):
    return torch.empty(shape, dtype=dtype, device="meta")


def describe(outs):
    outs = outs if isinstance(outs, (tuple, list)) else (outs,)
    return [(tuple(o.shape), o.dtype, o.device.type) for o in outs]


def test_fake_implementations_give_the_reference_output_shapes(ops):
    i32, f32, u8 = torch.int32, torch.float32, torch.uint8
    N, K, F, C = 50, 8, 16, 4
    h = torch.ops.hgcalml
    assert describe(h.bin_by_coordinates(m(N, 3), m(3, dtype=i32), m(1), m(3, dtype=i32), 125, True)) == \
        [((N, 4), i32, "meta"), ((N,), i32, "meta"), ((125,), i32, "meta")]
    assert describe(h.binned_select_knn(m(N, C), m(N, dtype=i32), m(N, 4, dtype=i32), m(126, dtype=i32), m(3, dtype=i32),
                                        m(1), m(N, dtype=i32), K, False, False)) == \
        [((N, K), i32, "meta"), ((N, K), f32, "meta")]
    assert describe(h.index_replacer(m(N, K, dtype=i32), m(N, dtype=i32))) == [((N, K), i32, "meta")]
    assert describe(h.accumulate_knn(m(N, K), m(N, F), m(N, K, dtype=i32), 0, True)) == \
        [((N, 2 * F), f32, "meta"), ((N, F), i32, "meta")]
    assert describe(h.accumulate_knn(m(N, K), m(N, F), m(N, K, dtype=i32), 0, False)) == \
        [((N, F), f32, "meta"), ((N, F), i32, "meta")]
    assert describe(h.accumulate_knn_slots(m(N, K), m(N, F), m(N, K, dtype=i32), 0, True)) == \
        [((N, 2 * F), f32, "meta"), ((N, F), i32, "meta"), ((N, F), u8, "meta")]
    assert describe(h.accumulate_knn_slots(m(N, 300), m(N, F), m(N, 300, dtype=i32), 0, True))[2] == ((0,), u8, "meta")
    assert describe(h.accumulate_knn_exp_slots(m(N, K), m(N, F), m(N, K, dtype=i32), 0, True)) == \
        [((N, 2 * F), f32, "meta"), ((N, F), i32, "meta"), ((N, F), u8, "meta"), ((N, K), f32, "meta")]
    grads = [((N, K), f32, "meta"), ((N, F), f32, "meta")]
    assert describe(h.accumulate_knn_grad(m(N, 2 * F), m(N, K), m(N, F), m(N, K, dtype=i32), m(N, F, dtype=i32),
                                          m(N + 1, dtype=i32), m(N * K, dtype=i32))) == grads
    assert describe(h.accumulate_knn_grad_slots(m(N, 2 * F), m(N, K), m(N, F), m(N, K, dtype=i32), m(N, F, dtype=i32),
                                                m(N, F, dtype=u8), m(N + 1, dtype=i32), m(N * K, dtype=i32))) == grads
    assert describe(h.select_knn_grad(m(N, K), m(N, K, dtype=i32), m(N, K), m(N, C))) == [((N, C), f32, "meta")]
    assert describe(h.local_distance(m(N, C), m(N, K, dtype=i32))) == [((N, K), f32, "meta")]
    assert describe(h.push_knn(m(N, K), m(N, F), m(N, K, dtype=i32))) == [((N, F), f32, "meta")]
    assert describe(h.push_knn_grad(m(N, F), m(N, K), m(N, F), m(N, K, dtype=i32))) == grads
    NH, R = 20, 2
    assert describe(h.binned_assign_to_condensates(
        m(N, C), m(N), m(N), m(N, dtype=i32), m(N, dtype=i32), m(126, dtype=i32), m(N, dtype=i32), m(NH, dtype=i32),
        m(R + 1, dtype=i32), m(3, dtype=i32), m(1), m(NH, C), m(NH), m(NH), m(NH, dtype=i32), m(R + 1, dtype=i32), 0.1,
        True)) == [((NH,), i32, "meta"), ((N,), i32, "meta"), ((NH,), i32, "meta"), ((N,), i32, "meta"),
                   ((R + 1,), i32, "meta")]


def test_an_op_traces_under_fake_tensor_mode(ops):
    """what torch.compile does first: run the graph on FakeTensors"""
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        w, x = torch.empty(30, 6), torch.empty(30, 12)
        idx = torch.empty(30, 6, dtype=torch.int32)
        out, maxidx = torch.ops.hgcalml.accumulate_knn(w, x, idx, 0, True)
        assert tuple(out.shape) == (30, 24) and tuple(maxidx.shape) == (30, 12)
