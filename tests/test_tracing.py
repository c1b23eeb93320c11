"""The named ranges around the parts of a step: inert unless switched on, balanced when on."""
from tq_kv_amd import tracing


def test_spans_are_inert_until_switched_on_and_balanced_when_on():
    events = []
    was_on = tracing.enabled()
    tracing.enable(False)
    tracing.set_sink(lambda name: events.append(("push", name.decode())), lambda: events.append(("pop",)))
    try:
        with tracing.span("model"):
            with tracing.span("attn"):
                pass
        assert events == [] and not tracing.enabled()
        assert tracing.enable() and tracing.enabled()
        try:
            with tracing.span("model"):
                with tracing.span("attn"):
                    pass
                with tracing.span("attn-mlp"):
                    raise ValueError("inside")
        except ValueError:
            pass
        assert events == [("push", "model"), ("push", "attn"), ("pop",), ("push", "attn-mlp"), ("pop",), ("pop",)]
        # switched off while a range is open: the range is still closed, later ones are not opened
        s = tracing.span("step")
        s.__enter__()
        tracing.enable(False)
        s.__exit__(None, None, None)
        with tracing.span("later"):
            pass
        assert events[-2:] == [("push", "step"), ("pop",)]
    finally:
        tracing.enable(False)
        tracing.set_sink(None, None)
        tracing.enable(was_on)


def test_the_engines_own_ranges_go_to_the_sink_too():
    """The ranges the library opens around a model's parts are the same mechanism: a model without a GPU runs
    nothing, so only the sink's plumbing is checked here (a step's ranges: tests/test_gpu_engine.py)."""
    events = []
    tracing.set_sink(lambda name: events.append(name.decode()), lambda: events.append("pop"))
    try:
        assert tracing.enable()
        with tracing.span("outer"):
            pass
        assert events == ["outer", "pop"]
    finally:
        tracing.enable(False)
        tracing.set_sink(None, None)
