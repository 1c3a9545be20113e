"""Params blobs of the one-epilogue-many-producers example, packed from buffer addresses.

Stands on its own (no package imports) so that ``pipec launch --params <this file>:...`` can load it."""
import struct


def params_blobs(addr: dict[str, int], m: int, n: int, k: int, home: str) -> dict[str, bytes]:
    """GsLoaderParams (40 B, gemm_split/include/gs_abi.h), OeMmaParams (16 B), OeEpilogueParams (32 B)."""
    if home == "wide":
        return {
            "oe.loader.wide": struct.pack("<QQQiiii", addr["a"], addr["bt"], addr["status"], m, n, k, 0),
            "oe.mma.wide": struct.pack("<Qii", addr["status"], n, k),
            "oe.epilogue.wide": struct.pack("<QQQii", addr["bias"], addr["scale"], addr["c"], m, n),
        }
    if home == "full":
        return {
            "oe.mma.full": struct.pack("<QQQiiii", addr["a"], addr["bt"], addr["status"], m, n, k, 0),
            "oe.epilogue.full": struct.pack("<QQQii", addr["bias"], addr["scale"], addr["c"], m, n),
        }
    return {
        "gs.loader": struct.pack("<QQQiiii", addr["a"], addr["bt"], addr["status"], m, n, k, 0),
        f"oe.mma.{home}": struct.pack("<Qii", addr["status"], n, k),
        "oe.epilogue": struct.pack("<QQQii", addr["bias"], addr["scale"], addr["c"], m, n),
    }
