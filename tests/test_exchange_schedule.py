"""The multi-resolution exchange module runs the layers of its parallel paths side by side when the
layer namespace offers group calls (conv_group / residual_group / add_group).  Checked here on the
CPU with dense layers and group calls that simply loop: the side-by-side schedule has to give
exactly what the path-after-path schedule gives, run every layer exactly once per frame, and keep
the order of each output's sum."""
import types

import pytest
import torch

from deltacnn_amd.networks import DenseLayers, _HRModule


def _namespace(log):
    """DenseLayers + group calls that run their items one by one and note what they were given."""
    def conv_group(convs, inputs):
        log.append(("conv", len(convs)))
        return [c(x) for c, x in zip(convs, inputs)]

    def residual_group(adds, residuals, convs, inputs):
        log.append(("residual", len(convs)))
        return [a(r, c(x)) for a, r, c, x in zip(adds, residuals, convs, inputs)]

    def add_group(adds, firsts, seconds, upsamples):
        log.append(("add", len(adds)))
        return [a(x, y if up is None else up(y)) for a, x, y, up in zip(adds, firsts, seconds, upsamples)]

    names = {k: v for k, v in vars(DenseLayers).items() if not k.startswith("__")}
    return types.SimpleNamespace(**names, conv_group=conv_group, residual_group=residual_group, add_group=add_group)


@pytest.mark.parametrize("channels,multi", [([8, 16], True), ([8, 16, 24], True), ([8, 16, 24, 32], True),
                                            ([8, 16, 24, 32], False)])
def test_side_by_side_schedule_equals_path_after_path(channels, multi):
    torch.manual_seed(len(channels) + int(multi))
    log = []
    plain = _HRModule(DenseLayers, channels, blocks=2, multi_scale_output=multi).eval()
    grouped = _HRModule(_namespace(log), channels, blocks=2, multi_scale_output=multi).eval()
    grouped.load_state_dict(plain.state_dict())
    xs = [torch.randn(2, c, 32 >> k, 32 >> k) for k, c in enumerate(channels)]
    calls = {}
    for name, m in grouped.named_modules():
        if not list(m.children()) and not isinstance(m, torch.nn.Identity):
            m.register_forward_hook(lambda mod, a, b, name=name: calls.__setitem__(name, calls.get(name, 0) + 1))
    with torch.no_grad():
        want = plain([x.clone() for x in xs])
        got = grouped([x.clone() for x in xs])
    assert len(got) == len(want) == (len(channels) if multi else 1)
    for g, w in zip(got, want):
        assert torch.equal(g, w)
    # every leaf layer (the identity placeholders of the exchange aside) ran exactly once
    assert calls and all(n == 1 for n in calls.values()), {k: v for k, v in calls.items() if v != 1}
    leaves = [n for n, m in grouped.named_modules() if not list(m.children()) and not isinstance(m, torch.nn.Identity)]
    assert sorted(calls) == sorted(leaves)
    n = len(channels)
    # the branches: per block one group of first convolutions and one of sum-carrying second ones
    assert log[:4] == [("conv", n), ("residual", n)] * 2
    # the sums of the exchange: one call per level (term j of every output), sizes shrink by the carried ones
    adds = [k for kind, k in log if kind == "add"]
    outputs = n if multi else 1
    assert adds == [min(j + 1, outputs) for j in range(1, n)]
