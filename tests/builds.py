"""Kernel builds that only tests use: head sizes and head groupings of the kernel tests and of the tests'
own small models, and builds of the decode attention whose thresholds are lowered so that a test can
reach the kernels for long contexts and many sequences with inputs it can check.  `__graft_entry__.build()`
compiles them ahead together with the product's own list; a test that finds one missing compiles it then."""

ATTENTION = [(128, 16), (128, 1), (16, 3), (48, 3), (64, 1), (32, 16), (256, 4), (80, 3), (256, 2), (16, 1), (32, 2), (16, 6)]   # (head size, group)
EARLY_STREAM = [(128, 4), (48, 3), (16, 2)]      # the kernel for long contexts takes over at 1,024 keys
WHOLE_CONTEXTS = [(128, 4), (128, 16)]           # the whole-context kernel at few sequences


def test_builds():
    out = []
    for head_dim, group in ATTENTION:
        out.append(("attention_prefill", {"HEAD_DIM": head_dim}))
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group}))
    for head_dim, group in EARLY_STREAM:
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group, "STREAM_FROM": 1024}))
    for head_dim, group in WHOLE_CONTEXTS:
        out.append(("attention_decode", {"HEAD_DIM": head_dim, "GROUP": group, "RING_FROM_PAIRS": 1}))
    seen, unique = set(), []
    for name, defines in out:
        key = (name, tuple(sorted(defines.items())))
        if key not in seen:
            seen.add(key)
            unique.append((name, defines))
    return unique


test_builds.__test__ = False      # a list for the build step, not a test
