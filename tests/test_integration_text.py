"""The integration notes quote the engine-side code of the batched step and of the local frame from oracle/integration_batched.inc, the file the
compiler sees (oracle/ref_shim_graph.c includes it against the reference's own structs).  The quotation must be the file."""
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_integration_md_quotes_the_compiled_file():
    with open(os.path.join(ROOT, "oracle", "integration_batched.inc")) as f:
        source = f.read()
    with open(os.path.join(ROOT, "INTEGRATION.md")) as f:
        doc = f.read()
    marker6, marker6b = "/* ---- section 6: the batched decoder step", "/* ---- section 6b: the local-transformer frame"
    part6 = source[source.index(marker6):source.index(marker6b)].strip()
    part6b = source[source.index(marker6b):].strip()
    assert part6 in doc, "the integration notes no longer quote the batched-step part of oracle/integration_batched.inc"
    assert part6b in doc, "the integration notes no longer quote the local-frame part of oracle/integration_batched.inc"
