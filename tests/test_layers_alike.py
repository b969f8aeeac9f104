"""Which entries of a run order may run from one layer's launch list (no GPU): only layers that would launch
the same kernels with the same numbers. A layer that differs in one constant, or entries that do not each have a
cache plane of their own (or all read one), must run their own code."""

import dataclasses

from conftest import TINY_B

import tie_amd  # noqa: F401  (registers the architecture and the parts)
from tie_amd.config.registry import resolve_architecture
from tie_amd.models.builder import Model
from tie_amd.models.spec import LayerCall, PartSpec


def qwen3_spec(layers):
    arch = resolve_architecture(TINY_B)
    return arch.build_spec(arch.read_config(dict(TINY_B, num_hidden_layers=layers)))


def alike(spec):
    model = Model(spec)
    model._find_layers_alike()
    return model._alike


def with_layer(spec, index, **changes):
    layers = list(spec.layers)
    layers[index] = dataclasses.replace(layers[index], **changes)
    return dataclasses.replace(spec, layers=tuple(layers))


def test_layers_of_one_shape_are_alike():
    assert alike(qwen3_spec(7)) == {0: 7}
    assert alike(qwen3_spec(3)) == {}          # fewer than four gain nothing


def test_a_layer_with_another_constant_is_not_alike():
    spec = qwen3_spec(9)
    norms = dict(spec.layers[4].norms)
    norms["pre_mixer"] = PartSpec("rms_norm", dict(norms["pre_mixer"].params, eps=1e-3))
    assert alike(with_layer(spec, 4, norms=norms)) == {0: 4, 5: 9}
    mixer = spec.layers[6].mixer
    other_scale = PartSpec(mixer.kind, dict(mixer.params, scale=0.5))
    assert alike(with_layer(spec, 6, mixer=other_scale)) == {0: 6}
    position = PartSpec("rope_neox", dict(mixer.params["position"].params, theta=10000.0))
    other_theta = PartSpec(mixer.kind, dict(mixer.params, position=position))
    assert alike(with_layer(spec, 2, mixer=other_theta)) == {3: 9}
    eps = PartSpec(mixer.kind, dict(mixer.params, qk_norm=dict(mixer.params["qk_norm"], eps=1e-2)))
    assert alike(with_layer(spec, 8, mixer=eps)) == {0: 8}


def test_entries_that_share_some_cache_planes_are_not_alike():
    spec = qwen3_spec(8)
    own = tuple(LayerCall(l) for l in range(8))
    assert alike(dataclasses.replace(spec, order=own)) == {0: 8}
    # entries 4 and 5 read entry 3's keys and values, 6 and 7 read entry 2's: the readers are of one shape and
    # write nothing, but they do not all read one plane, nor each its own
    shared = own[:4] + (LayerCall(4, 3), LayerCall(5, 3), LayerCall(6, 2), LayerCall(7, 2))
    assert alike(dataclasses.replace(spec, order=shared)) == {0: 4}
    one_plane = own[:4] + tuple(LayerCall(l, 3) for l in range(4, 8))
    assert alike(dataclasses.replace(spec, order=one_plane)) == {0: 4, 4: 8}
