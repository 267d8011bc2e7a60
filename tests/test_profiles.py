"""The measurement summaries under profiles/ say which tree they were taken at, and the one bench.py reads
numbers from (measured HBM traffic per GEMM launch) must have been taken with the GEMM kernels of this tree."""
import os

from fastconv_amd import provenance

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROFILES = os.path.join(ROOT, "profiles")


def test_every_summary_names_its_command_and_the_tree_it_was_taken_at():
    names = sorted(n for n in os.listdir(PROFILES) if n.endswith((".txt", ".md")))
    assert names
    for n in names:
        path = os.path.join(PROFILES, n)
        assert provenance.parse(path) is not None, "%s has no provenance line" % n
        text = open(path).read()
        assert "rocprofv3" in text or "bench.py" in text or "conv_test" in text, "%s does not give its command" % n
        assert os.path.getsize(path) < 64 * 1024, "%s is not a short summary" % n


def test_digest_follows_the_sources():
    everything = provenance.digest()
    assert len(everything) == 16 and everything == provenance.digest()
    assert provenance.digest(["wino_gemm.hip"]) != provenance.digest(["implicit_gemm.hip"])
    changed = provenance.digest(["wino_gemm.hip"], read=lambda n: b"something else")
    assert changed != provenance.digest(["wino_gemm.hip"])


def test_traffic_summary_was_measured_on_the_gemm_kernels_of_this_tree():
    """When wino_gemm.hip or implicit_gemm.hip change, profiles/gemm_hbm_traffic_pmc.txt has to be taken again
    (its commands are in its header); until then bench.py reports roofline.traffic as null."""
    path = os.path.join(PROFILES, "gemm_hbm_traffic_pmc.txt")
    commit, _, sources_digest, sources = provenance.parse(path)
    assert sources and sources_digest
    assert provenance.sources_current(path), (
        "%s changed since commit %s: measure the HBM traffic of the GEMM kernels again" % (", ".join(sources), commit))
