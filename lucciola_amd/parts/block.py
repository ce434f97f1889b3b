"""The arrangement of a layer's parts.  ``prenorm_residual`` is the reference's wiring
(src/qwen.cc:574-589,741-759,797-798): r = h; x = norm(h); h = mixer(x) + r; r = h;
x = norm(h); h = feed_forward(x) + r.  The additions are folded into the next norm's kernel:
a branch's output waits in ``stream.pending`` until then."""
from __future__ import annotations

from ..config.registry import BLOCKS
from .base import ResidualStream


@BLOCKS.register("prenorm_residual")
class PreNormResidualBlock:
    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def forward(self, stream: ResidualStream, site) -> None:
        x = self.mixer_norm.add_norm(stream)
        stream.pending = self.mixer.forward(x, site)
        x = self.feed_forward_norm.add_norm(stream)
        stream.pending = self.feed_forward.forward(x)
