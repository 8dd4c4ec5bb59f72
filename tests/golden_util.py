"""Access to tests/golden/reference_xml and tests/golden/ncclize_xml: MSCCL-IR emitted by msccl-tools' own
compiler and by its second emitter, ncclize (data only)."""
import glob
import gzip
import os

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_xml")
NCCLIZE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ncclize_xml")


def names(directory=GOLDEN_DIR):
    return sorted(os.path.basename(p)[:-len(".xml.gz")] for p in glob.glob(os.path.join(directory, "*.xml.gz")))


def ncclize_names():
    return names(NCCLIZE_DIR)


def load(name):
    directory = NCCLIZE_DIR if name.startswith("ncclize_") else GOLDEN_DIR
    with gzip.open(os.path.join(directory, name + ".xml.gz"), "rt") as f:
        return f.read()
