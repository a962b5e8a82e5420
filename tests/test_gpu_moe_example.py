"""The forward-MoE example over the delivery profiles the reference runs
(tests/distributed/test_acceptance.py:17-28), at world_size == 1."""

import pytest

from nanoep_amd.examples import moe

pytestmark = pytest.mark.gpu

# name, layout, tokens, hidden, topk, pattern, iterations, async + cached
PROFILES = [
    ("compact", "compact", 17, 256, 3, "mixed", 3, False),
    ("expanded", "expanded", 17, 256, 3, "mixed", 3, False),
    ("large-compact", "compact", 256, 4096, 8, "mixed", 4, True),
    ("large-expanded", "expanded", 256, 7168, 8, "mixed", 8, True),
    ("skew-compact", "compact", 129, 1024, 3, "skew", 16, True),
    ("skew-expanded", "expanded", 129, 1024, 3, "skew", 16, True),
    ("masked-compact", "compact", 33, 256, 3, "masked", 4, True),
    ("masked-expanded", "expanded", 33, 256, 3, "masked", 4, True),
    ("uneven-compact", "compact", 65, 1024, 3, "uneven", 8, True),
    ("uneven-expanded", "expanded", 65, 1024, 3, "uneven", 8, True),
]


@pytest.mark.parametrize("profile", PROFILES, ids=[p[0] for p in PROFILES])
def test_delivery_profile(device, profile):
    _, layout, tokens, hidden, topk, pattern, iterations, fast = profile
    argv = ["--layout", layout, "--tokens", str(tokens), "--hidden", str(hidden), "--topk", str(topk), "--pattern", pattern,
            "--iterations", str(iterations), "--experts", "8"]
    if fast:
        argv += ["--async-op", "--cached"]
    report = moe.run(moe.parse_args(argv))
    assert report["layout"] == layout and report["world_size"] == 1
