"""The kernel tables against the layer's own validation (CPU).

The reference's layers accept a ``config=`` only if its ``_layer_key`` equals the key the
layer computes for itself (jigsaw/_core/config.py:6-34, called from
jigsaw/modules/convolution/_conv/base.py:193-205 and _conv_transpose/base.py:197-207), and
they rebuild it as ``type(config)(channel_group, bias, kernel_size, stride, device,
channel_comm, groups)`` when resharded (_conv/base.py:572-580). Both steps are restated
here (the reference is not imported) and replayed against the HIP tables.
"""

import pytest
import torch

from jigsaw_amd import conv as jc
from jigsaw_amd import conv_transpose as jct


def check_config(config, expected):
    """jigsaw/_core/config.py:26-34."""
    diff = [f"{k}={config._layer_key[k]!r} (layer: {v!r})" for k, v in expected.items() if config._layer_key[k] != v]
    if diff:
        raise ValueError("config was built for a different layer: " + ", ".join(diff) + ".")


def layer_side_key(channel_group, bias, kernel_size, stride, groups):
    """What the layer computes for itself (jigsaw/modules/convolution/_common/config.py:37-43)."""
    return {
        "n_spatial": len(kernel_size),
        "bias": bias is not None,
        "kernel_size == stride": tuple(kernel_size) == tuple(stride),
        "groups": groups,
        "channel group size": channel_group.size(),
    }


CLASSES = [jc.HipConvNdConfig, jct.HipConvTransposeNdConfig]


@pytest.mark.parametrize("cls", CLASSES)
@pytest.mark.parametrize("kernel,stride", [((3, 3), (1, 1)), ((3, 3, 3), (1, 1, 1)), ((2, 2), (2, 2)), ((3,), (1,))])
@pytest.mark.parametrize("with_bias", [True, False])
def test_config_passes_the_layers_check(cls, kernel, stride, with_bias):
    group = jc.TileGroup(1, 0)
    bias = torch.zeros(4) if with_bias else None
    cfg = cls(group, bias, kernel, stride, torch.device("cuda"))
    check_config(cfg, layer_side_key(group, bias, kernel, stride, 1))
    assert cfg.n_spatial == len(kernel) and cfg.channel_comm == "all_to_all"
    assert cfg.channel_local and cfg.groups_local == 1 and cfg.groups == 1 and cfg.vmapped is False
    assert (cfg.grad_bias(torch.zeros(1)) is None) if not with_bias else cfg.grad_bias == cfg._sum_grad_bias


@pytest.mark.parametrize("cls", CLASSES)
def test_mismatched_layer_is_rejected(cls):
    group = jc.TileGroup(1, 0)
    cfg = cls(group, torch.zeros(4), (3, 3), (1, 1), torch.device("cuda"))
    for other in (
        layer_side_key(group, None, (3, 3), (1, 1), 1),            # layer without a bias
        layer_side_key(group, torch.zeros(4), (3, 3, 3), (1, 1, 1), 1),  # 3-D layer
        layer_side_key(group, torch.zeros(4), (2, 2), (2, 2), 1),   # patchify layer
        layer_side_key(group, torch.zeros(4), (3, 3), (1, 1), 2),   # grouped layer
        layer_side_key(jc.TileGroup(2, 0), torch.zeros(4), (3, 3), (1, 1), 1),  # channel-sharded layer
    ):
        with pytest.raises(ValueError, match="different layer"):
            check_config(cfg, other)


@pytest.mark.parametrize("cls", CLASSES)
def test_rebuild_from_type_keeps_the_options(cls):
    """The layer's reshard path: ``type(config)(...)`` with positional arguments."""
    exchange = object()
    bound = cls.bound(halo_exchange=exchange, fused_fold=False)
    group = jc.TileGroup(1, 0)
    cfg = bound(group, None, (3, 3), (1, 1), torch.device("cuda"), "auto", 1)
    again = type(cfg)(group, torch.zeros(2), (3, 3), (1, 1), torch.device("cuda"), cfg.channel_comm, 1)
    assert again.halo_exchange is exchange and again.fused_fold is False
    assert again._layer_key["bias"] is True and cfg._layer_key["bias"] is False
    assert isinstance(again, cls)
    with pytest.raises(TypeError):
        cls.bound(no_such_option=1)
    with pytest.raises(TypeError):
        cls(group, None, (3, 3), (1, 1), None, no_such_option=1)


def test_short_form_and_unsupported_layers():
    cfg = jc.HipConvNdConfig.for_rank(3, None, framed=True)
    assert cfg.framed and cfg._layer_key["n_spatial"] == 3 and not cfg._layer_key["kernel_size == stride"]
    with pytest.raises(NotImplementedError):
        jc.HipConvNdConfig(jc.TileGroup(2, 1), None, (3, 3), (1, 1), torch.device("cuda"))
    grouped = jc.HipConvNdConfig(jc.TileGroup(1, 0), None, (3, 3), (1, 1), torch.device("cuda"), groups=2)
    assert grouped.groups == 2 and grouped.groups_local == 2 and grouped.channel_local and grouped._layer_key["groups"] == 2
    with pytest.raises(ValueError):
        jc.HipConvNdConfig(jc.TileGroup(1, 0), None, (3, 3), (1, 1), torch.device("cuda"), channel_comm="carrier_pigeon")
    with pytest.raises(ValueError):
        jc.HipConvNdConfig(jc.TileGroup(1, 0), None, (3, 3), (1, 1), torch.device("cpu"), channel_comm="all_to_all")
    assert jc.HipConvNdConfig(jc.TileGroup(1, 0), None, (3, 3), (1, 1), torch.device("cpu")).channel_comm == "batch_isend_irecv"
    assert jc.HipConvNdConfig(jc.TileGroup(1, 0), None, (3, 3), (1, 1), None, "all_gather").channel_comm == "all_gather"
