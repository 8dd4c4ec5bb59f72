"""msccl for MI355X: the MSCCLang tool-chain's run-time half.

`msccl.executor` runs MSCCL-IR XML on one MI355X through the HIP library libmscclx.so.
"""
__version__ = "0.1.0"
