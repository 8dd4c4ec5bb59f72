"""Access to tests/golden/reference_xml, tests/golden/reference_random_xml and tests/golden/ncclize_xml: MSCCL-IR
emitted by msccl-tools' own compiler and by its second emitter, ncclize (data only)."""
import glob
import gzip
import os

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_xml")
NCCLIZE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ncclize_xml")
RANDOM_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_random_xml")


def names(directory=GOLDEN_DIR):
    return sorted(os.path.basename(p)[:-len(".xml.gz")] for p in glob.glob(os.path.join(directory, "*.xml.gz")))


def ncclize_names():
    return names(NCCLIZE_DIR)


def random_names():
    """msccl-tools' compiler on random programs (fusion on): random_<seed>_fused, some of them malformed or racy on purpose."""
    return sorted(names(RANDOM_DIR), key=lambda n: int(n.split("_")[1]))


def load(name):
    directory = NCCLIZE_DIR if name.startswith("ncclize_") else RANDOM_DIR if name.startswith("random_") else GOLDEN_DIR
    with gzip.open(os.path.join(directory, name + ".xml.gz"), "rt") as f:
        return f.read()
