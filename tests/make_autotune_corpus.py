"""Measure the lane's candidates on the MI355X and write
``tessera_amd/autotune_corpus.json`` (run on the GPU box:
``python tests/make_autotune_corpus.py [--out PATH]``).

The arbiter that verifies and times the candidates is the stand-in host of these
tests (``tests/standin_host.py``); inside Tessera the same call takes
``tessera.compiler.emit.candidate`` and ``tessera.compiler.fusion_core``."""
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
sys.path.insert(0, str(Path(__file__).resolve().parent))

import standin_host as host  # noqa: E402
from tessera_amd import autotune, lane  # noqa: E402


def main(argv) -> int:
    out = argv[argv.index("--out") + 1] if "--out" in argv else autotune.PACKAGED
    if not lane.available():
        print("gfx950 lane unavailable: the corpus is measured on the MI355X", file=sys.stderr)
        return 3
    corpus = autotune.measure_headline_corpus(host.CandidateHost(), host.regions)
    print(f"wrote {len(corpus)} records to {corpus.save(out)}")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
