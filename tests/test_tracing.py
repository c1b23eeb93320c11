"""The named ranges around the parts of a step: inert unless switched on, balanced when on."""
from tq_kv_amd import tracing


class _Recorder:
    def __init__(self):
        self.events = []

    def roctxRangePushA(self, name):
        self.events.append(("push", name.decode()))
        return len(self.events)

    def roctxRangePop(self):
        self.events.append(("pop",))
        return 0


def test_spans_are_inert_until_switched_on_and_balanced_when_on():
    old = dict(tracing._state)
    rec = _Recorder()
    try:
        tracing._state.update(on=False, lib=rec, tried=True)
        with tracing.span("model"):
            with tracing.span("attn"):
                pass
        assert rec.events == [] and not tracing.enabled()
        assert tracing.enable() and tracing.enabled()
        try:
            with tracing.span("model"):
                with tracing.span("attn"):
                    pass
                with tracing.span("attn-mlp"):
                    raise ValueError("inside")
        except ValueError:
            pass
        assert rec.events == [("push", "model"), ("push", "attn"), ("pop",), ("push", "attn-mlp"), ("pop",), ("pop",)]
        # switched off while a range is open: the range is still closed, later ones are not opened
        s = tracing.span("step")
        s.__enter__()
        tracing.enable(False)
        s.__exit__(None, None, None)
        with tracing.span("later"):
            pass
        assert rec.events[-2:] == [("push", "step"), ("pop",)]
        # no library: enabling says no and stays off
        tracing._state.update(on=False, lib=None, tried=True)
        assert tracing.enable() is False
        with tracing.span("x"):
            pass
    finally:
        tracing._state.clear()
        tracing._state.update(old)
