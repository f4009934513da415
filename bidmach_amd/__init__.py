"""MI355X-native skip-gram negative-sampling operators behind BIDMach's CUMACH word2vec API.

`bidmach_amd.cumach.CUMACH` mirrors the four static natives of the reference's
edu.berkeley.bid.CUMACH that the Word2Vec model calls; `bidmach_amd.word2vec.Word2Vec` mirrors the
minibatch step of BIDMach.networks.Word2Vec around them.  All arithmetic runs in the HIP
shared library built from bidmach_amd/csrc; there is no CPU fallback.
"""
from .cumach import CUMACH, W2VLibraryError, lib_path, load_library  # noqa: F401

__all__ = ["CUMACH", "W2VLibraryError", "lib_path", "load_library"]
