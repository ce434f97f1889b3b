"""The arrangement of a layer's parts.  ``prenorm_residual`` is the reference's wiring
(src/qwen.cc:574-589,741-759,797-798): r = h; x = norm(h); h = mixer(x) + r; r = h;
x = norm(h); h = feed_forward(x) + r.  The additions are folded into the next norm's kernel:
a branch's output waits in ``stream.pending`` until then.  A branch that says it takes scaled
rows (``takes_scaled_rows``) may be given ops.ScaledRows by a norm that offers them
(``offers_scaled_rows``); everyone else gets and returns tensors."""
from __future__ import annotations

from ..config.registry import BLOCKS
from .base import ResidualStream


@BLOCKS.register("prenorm_residual")
class PreNormResidualBlock:
    # the slots of this arrangement and the family each is built from; the model builds the
    # parts named in ``LayerSpec.parts`` and hands them over by slot name
    slots = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm",
             "feed_forward_norm": "norm"}

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    @staticmethod
    def _normed(norm, branch, stream: ResidualStream):
        if getattr(norm, "offers_scaled_rows", False) and getattr(branch, "takes_scaled_rows", False):
            return norm.add_norm(stream, scaled=True)
        return norm.add_norm(stream)

    def forward(self, stream: ResidualStream, site) -> None:
        x = self._normed(self.mixer_norm, self.mixer, stream)
        stream.pending = self.mixer.forward(x, site)
        x = self._normed(self.feed_forward_norm, self.feed_forward, stream)
        stream.pending = self.feed_forward.forward(x)
