"""Access to tests/golden/reference_xml: MSCCL-IR emitted by msccl-tools' own compiler (data only)."""
import glob
import gzip
import os

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_xml")


def names():
    return sorted(os.path.basename(p)[:-len(".xml.gz")] for p in glob.glob(os.path.join(GOLDEN_DIR, "*.xml.gz")))


def load(name):
    with gzip.open(os.path.join(GOLDEN_DIR, name + ".xml.gz"), "rt") as f:
        return f.read()
