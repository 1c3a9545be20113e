"""Params blobs of the three-package GEMM example, packed from buffer addresses.

Stands on its own (no package imports) so that ``pipec launch --params <this file>:params_512`` can
load it as a plain file, the way the reference's examples hand a builder to ``pipec2 launch``."""
import struct


def params_blobs(addr: dict[str, int], m: int, n: int, k: int) -> dict[str, bytes]:
    """GsLoaderParams (40 B), GsMmaParams (16 B), GsEpilogueParams (24 B) of include/gs_abi.h."""
    return {
        "gs.loader": struct.pack("<QQQiiii", addr["a"], addr["bt"], addr["status"], m, n, k, 0),
        "gs.mma": struct.pack("<Qii", addr["status"], n, k),
        "gs.epilogue": struct.pack("<QQii", addr["bias"], addr["c"], m, n),
    }


def params_512(addr: dict[str, int]) -> dict[str, bytes]:
    """Builder for the 512 x 512 x 512 case with buffers named a, bt, bias, c, status."""
    return params_blobs(addr, 512, 512, 512)
