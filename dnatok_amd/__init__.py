"""MI355X-native DNA tokenization backend (gfx950 HIP kernels behind a C ABI).

Public surface, named as in the reference it is a drop-in for:

    from dnatok_amd import DNATok, GPUTokBPEBackend, DnatokBpeKernel
    from dnatok_amd.dnatok_compat import NTv3Tokenizer, Evo2ByteTokenizer, CharTokenizer

plus the device-resident encoders in ``dnatok_amd.encoders``.
"""
__version__ = "0.1.0"

__all__ = ["DNATok", "GPUTokBPEBackend", "DnatokBpeKernel"]


def __getattr__(name):           # lazy: importing the package must not need torch or a GPU
    if name == "DNATok":
        from .dna_tokenizer import DNATok
        return DNATok
    if name == "GPUTokBPEBackend":
        from .gputok_bpe_backend import GPUTokBPEBackend
        return GPUTokBPEBackend
    if name == "DnatokBpeKernel":
        from .dnatok_bpe_kernel import DnatokBpeKernel
        return DnatokBpeKernel
    raise AttributeError(name)
