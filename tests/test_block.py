"""The arrangement's protocol with its parts, on the CPU with stand-in parts: when a
norm is handed over without having run, when a part adds to the stream itself, and that
a part which knows nothing of either is called as it always was."""

import torch

from zig_ai_amd.parts.block import PreNormResidualBlock, apply_normed


class Norm:
    """Doubles what it norms; can defer only when told so."""

    def __init__(self, can_defer):
        self.can_defer = can_defer
        self.calls = []

    def add_forward(self, residual, delta, rows=None):
        self.calls.append("add_forward")
        if delta is not None:
            residual.add_(delta)
        return residual * 2

    def deferred(self, residual, rows=None):
        self.calls.append("deferred")
        return ("not yet", residual) if self.can_defer else None


class PlainPart:
    """Knows nothing of streams: forward(x, *args) -> y."""

    def forward(self, x, *args):
        assert isinstance(x, torch.Tensor)
        return x + 1


class StreamPart:
    takes_stream = True

    def __init__(self, adds):
        self.adds = adds
        self.saw = None

    def forward(self, x, *args, stream=None):
        self.saw = x
        if isinstance(x, tuple):            # the norm that has not run yet
            x = x[1] * 2
        y = x + 1
        if self.adds:
            stream.add_(y)
            return None
        return y


def test_a_part_without_takes_stream_is_called_as_before():
    residual, pending = torch.ones(2, 3), torch.full((2, 3), 2.0)
    norm = Norm(can_defer=True)
    y = apply_normed(norm, PlainPart(), residual, pending, "step")
    assert norm.calls == ["add_forward"]
    assert torch.equal(residual, torch.full((2, 3), 3.0)) and torch.equal(y, torch.full((2, 3), 7.0))


def test_a_norm_is_handed_over_only_when_nothing_is_pending():
    for pending in (None, torch.full((2, 3), 2.0)):
        residual = torch.ones(2, 3)
        norm, part = Norm(can_defer=True), StreamPart(adds=False)
        y = apply_normed(norm, part, residual, pending, "step")
        if pending is None:
            assert norm.calls == ["deferred"] and isinstance(part.saw, tuple)
            assert torch.equal(y, torch.full((2, 3), 3.0))
        else:
            assert norm.calls == ["add_forward"] and isinstance(part.saw, torch.Tensor)
            assert torch.equal(y, torch.full((2, 3), 7.0))


def test_a_norm_that_cannot_defer_runs():
    residual = torch.ones(2, 3)
    norm, part = Norm(can_defer=False), StreamPart(adds=False)
    apply_normed(norm, part, residual, None, "step")
    assert norm.calls == ["deferred", "add_forward"] and isinstance(part.saw, torch.Tensor)


def test_block_with_parts_that_add_to_the_stream_leaves_nothing_pending():
    for adds in (True, False):
        residual = torch.ones(2, 3)
        block = PreNormResidualBlock({"mixer_norm": Norm(True), "mixer": StreamPart(adds),
                                      "feed_forward_norm": Norm(True), "feed_forward": StreamPart(adds)})
        out, pending = block.forward(residual, None, "step", "cache")
        assert out is residual
        # h = x + (2x + 1) = 4; y = h + (2h + 1) = 13
        total = out if pending is None else out + pending
        assert (pending is None) == adds
        assert torch.equal(total, torch.full((2, 3), 13.0))


def test_a_runtime_that_forbids_additions_to_the_stream_hands_no_stream_over():
    from zig_ai_amd.parts import Runtime

    class Recording(StreamPart):
        def forward(self, x, *args, stream=None):
            self.stream = stream
            return super().forward(x, *args, stream=torch.zeros(2, 3) if stream is None else stream)

    for allowed in (True, False):
        part = Recording(adds=False)
        part.runtime = Runtime(device=torch.device("cpu"), dtype=torch.float32,
                               stream_additions=allowed)
        residual = torch.ones(2, 3)
        apply_normed(Norm(True), part, residual, None, "step")
        assert (part.stream is residual) == allowed
