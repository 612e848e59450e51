"""Which parts may describe themselves to the native step program: those whose `emit` describes
the `forward` they run. A subclass that replaces `forward` alone falls back to running one by one."""
from imparo_amd.parts import ffn, norm
from imparo_amd.parts.base import emits


def test_a_subclass_that_replaces_forward_does_not_inherit_the_description():
    class Louder(ffn.SwiGlu):
        def forward(self, ctx, n):
            return 2 * super().forward(ctx, n)

    class LouderAndSaysSo(Louder):
        def emit(self, program):
            raise NotImplementedError

    class Renamed(ffn.SwiGlu):
        pass

    new = lambda cls: cls.__new__(cls)
    assert emits(new(ffn.SwiGlu)) and emits(new(Renamed))
    assert not emits(new(Louder))
    assert emits(new(LouderAndSaysSo))


def test_the_head_norm_is_described_by_its_own_pair_of_methods():
    class OtherRows(norm.RmsNorm):
        def forward_rows(self, ctx, res, rows, out_dtype, name="normed_rows"):
            raise NotImplementedError

    new = lambda cls: cls.__new__(cls)
    assert emits(new(norm.RmsNorm), "emit_head", "forward_rows")
    assert not emits(new(OtherRows), "emit_head", "forward_rows")
    assert emits(new(OtherRows))            # its forward is still the one `emit` describes

    class NoEmit:
        def forward(self):
            pass
    assert not emits(NoEmit())
