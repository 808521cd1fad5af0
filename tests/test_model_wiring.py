"""Which parts of a model are allowed to hand unfinished work to the part that follows them.

A mixer or feed-forward may leave its last product unmade (`ops.PendingProduct`) for the norm
that follows, and a norm may leave its rows' factors to the product that follows
(`ops.ScaledRows`), only where the receiving part says it takes them.  Inside a block the
block arranges this; between blocks the model does, looking at everything that follows a
block in the order of calls.  Built on the CPU: nothing here runs a kernel.
"""

import dataclasses

import torch

import tiny
from mini_infer_amd.models import DecoderModel, architecture_for
from mini_infer_amd.models.spec import LayerCall
from mini_infer_amd.parts.base import Norm
from mini_infer_amd.registry import register_norm


def _spec(cfg=tiny.TINY_B):
    arch = architecture_for(cfg)
    return arch.build_spec(arch.parse_config(cfg))


def test_built_in_parts_hand_work_on_in_every_layer():
    model = DecoderModel(_spec(), torch.bfloat16, "cpu")
    assert len(model.blocks) == 3
    for block in model.blocks:
        # attention -> norm -> feed-forward inside the block
        assert block.mixer.emit_pending_output and block.ffn_norm.emit_scaled_rows
        # feed-forward -> the next block's first norm -> its attention (the final norm after the last)
        assert block.feed_forward.emit_pending_output and block.mixer_norm.emit_scaled_rows
        assert block.takes_pending_products
    assert model.final_norm.takes_pending_products and not model.final_norm.emit_scaled_rows


class _PlainNorm(Norm):
    """A norm that knows tensors only."""

    def __init__(self, dtype, device):
        super().__init__(dtype, device)

    def param_specs(self, prefix):
        return {}

    def load_params(self, prefix, get):
        pass


@register_norm("test_wiring_plain_norm")
def _build_plain_norm(desc, dtype, device, shared=None):
    return _PlainNorm(dtype, device)


def test_a_block_hands_on_only_to_followers_that_all_take_it():
    spec = _spec()
    plain = dict(spec.layers[1].block)
    plain["norm"] = {"kind": "test_wiring_plain_norm"}
    layers = [spec.layers[0], dataclasses.replace(spec.layers[1], block=plain), spec.layers[2]]
    # layer 0 is followed by layer 1 (plain norms) and, the second time, by layer 2; layer 2 by
    # layer 0 and by the final norm; layer 1 by layer 2
    order = [LayerCall(0), LayerCall(1), LayerCall(2), LayerCall(0, reads_cache_of=0), LayerCall(2, reads_cache_of=2)]
    model = DecoderModel(dataclasses.replace(spec, layers=layers, order=order), torch.bfloat16, "cpu")
    first, middle, last = model.blocks
    assert not middle.takes_pending_products and not middle.mixer.emit_pending_output
    assert not middle.mixer_norm.emit_scaled_rows and not middle.ffn_norm.emit_scaled_rows
    assert not first.feed_forward.emit_pending_output  # one of its followers does not take it
    assert middle.feed_forward.emit_pending_output and last.feed_forward.emit_pending_output
    assert first.mixer.emit_pending_output and last.mixer.emit_pending_output  # inside their own blocks


def test_float32_models_are_wired_the_same_and_decide_at_run_time():
    # the flags say what a part MAY do; float32 parts then make every product themselves
    model = DecoderModel(_spec(tiny.TINY_A), torch.float32, "cpu")
    assert all(block.feed_forward.emit_pending_output for block in model.blocks)
