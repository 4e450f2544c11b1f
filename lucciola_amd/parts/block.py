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


@BLOCKS.register("prenorm_mixer")
class PreNormMixerBlock:
    """A layer without a feed-forward: h = h + mixer(norm(h))."""

    slots = {"mixer": "mixer", "mixer_norm": "norm"}

    def __init__(self, mixer, mixer_norm):
        self.mixer, self.mixer_norm = mixer, mixer_norm

    def forward(self, stream: ResidualStream, site) -> None:
        x = PreNormResidualBlock._normed(self.mixer_norm, self.mixer, stream)
        stream.pending = self.mixer.forward(x, site)


def _caching_index(parts, part) -> int:
    """Which of the site's caches belongs to ``part``: a site's caches follow the layer's caching parts
    in the order of the block's slots."""
    return [p for p in parts if p.cache_need() is not None].index(part)


@BLOCKS.register("prenorm_shift_residual")
class PreNormShiftResidualBlock:
    """The pre-norm residual arrangement with an input shift between the first norm and the mixer:
    h += mixer(shift(norm(h))); h += feed_forward(norm(h)).  The shift keeps state of its own beside the
    mixer's cache."""

    slots = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm",
             "feed_forward_norm": "norm", "mixer_shift": "input_shift"}

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, mixer_shift):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm, self.mixer_shift = mixer_norm, feed_forward_norm, mixer_shift
        order = (mixer, feed_forward, mixer_norm, feed_forward_norm, mixer_shift)
        self._mixer_at = _caching_index(order, mixer) if mixer.cache_need() is not None else None
        self._shift_at = _caching_index(order, mixer_shift)

    def forward(self, stream: ResidualStream, site) -> None:
        x = self.mixer_shift.add_norm_shift(self.mixer_norm, stream, site.part(self._shift_at))
        stream.pending = self.mixer.forward(x, site.part(self._mixer_at) if self._mixer_at is not None else site)
        x = PreNormResidualBlock._normed(self.feed_forward_norm, self.feed_forward, stream)
        stream.pending = self.feed_forward.forward(x)


@BLOCKS.register("prenorm_shift_mixer")
class PreNormShiftMixerBlock:
    """The same without a feed-forward: h += mixer(shift(norm(h)))."""

    slots = {"mixer": "mixer", "mixer_norm": "norm", "mixer_shift": "input_shift"}

    def __init__(self, mixer, mixer_norm, mixer_shift):
        self.mixer, self.mixer_norm, self.mixer_shift = mixer, mixer_norm, mixer_shift
        order = (mixer, mixer_norm, mixer_shift)
        self._mixer_at = _caching_index(order, mixer) if mixer.cache_need() is not None else None
        self._shift_at = _caching_index(order, mixer_shift)

    def forward(self, stream: ResidualStream, site) -> None:
        x = self.mixer_shift.add_norm_shift(self.mixer_norm, stream, site.part(self._shift_at))
        stream.pending = self.mixer.forward(x, site.part(self._mixer_at) if self._mixer_at is not None else site)


def _post_normed(norm, branch):
    """The branch output behind its norm: left to the next kernel that adds to the stream where
    the norm can say so (``behind``), else normed now."""
    if hasattr(norm, "behind"):
        return norm.behind(branch)
    from ..kernels import ops
    return norm.apply(ops.value(branch))


@BLOCKS.register("sandwich_residual")
class SandwichResidualBlock:
    """A norm before and behind each branch: h += post(mixer(pre(h))); h += post(ff(pre(h)))."""

    slots = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm",
             "mixer_post_norm": "norm", "feed_forward_norm": "norm", "feed_forward_post_norm": "norm"}

    def __init__(self, mixer, feed_forward, mixer_norm, mixer_post_norm, feed_forward_norm,
                 feed_forward_post_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.mixer_post_norm = mixer_norm, mixer_post_norm
        self.feed_forward_norm, self.feed_forward_post_norm = feed_forward_norm, feed_forward_post_norm

    def forward(self, stream: ResidualStream, site) -> None:
        x = self.mixer_norm.add_norm(stream)
        stream.pending = _post_normed(self.mixer_post_norm, self.mixer.forward(x, site))
        x = self.feed_forward_norm.add_norm(stream)
        stream.pending = _post_normed(self.feed_forward_post_norm, self.feed_forward.forward(x))


@BLOCKS.register("sandwich_mixer")
class SandwichMixerBlock:
    """The same without a feed-forward: h += post(mixer(pre(h)))."""

    slots = {"mixer": "mixer", "mixer_norm": "norm", "mixer_post_norm": "norm"}

    def __init__(self, mixer, mixer_norm, mixer_post_norm):
        self.mixer, self.mixer_norm, self.mixer_post_norm = mixer, mixer_norm, mixer_post_norm

    def forward(self, stream: ResidualStream, site) -> None:
        x = self.mixer_norm.add_norm(stream)
        stream.pending = _post_normed(self.mixer_post_norm, self.mixer.forward(x, site))
