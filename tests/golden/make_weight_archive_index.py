"""Writes weight_archive_index_mul1_3bit.{bin,json}: the index region (bytes [0, index_bytes)) of
test/fixtures/exl3/mul1-3bit.llmopt, a data file the reference's tests hold, plus what a reader
must find in it.  Run once where /root/reference exists; the outputs are committed."""
import hashlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from llmopt_amd import weight_archive as wa  # noqa: E402

SOURCE = "/root/reference/test/fixtures/exl3/mul1-3bit.llmopt"


def main():
    data = open(SOURCE, "rb").read()
    index_bytes = int.from_bytes(data[16:24], "little")
    with open(os.path.join(HERE, "weight_archive_index_mul1_3bit.bin"), "wb") as handle:
        handle.write(data[:index_bytes])
    entries = wa.parse_index(data[:index_bytes], len(data))
    probe = next(e for e in entries if e.name == "weight.exl3")
    meta = {
        "source": "test/fixtures/exl3/mul1-3bit.llmopt (a data file the reference's tests hold): its index "
                  "region, bytes [0, index_bytes), unchanged",
        "file_size": len(data), "index_bytes": index_bytes,
        "archive_sha256": hashlib.sha256(data).hexdigest(),
        "payload_probe": {"name": probe.name, "bytes_hex": data[probe.offset:probe.offset + probe.byte_length].hex()},
        "entries": [{"name": e.name, "dtype": e.dtype, "shape": list(e.shape), "offset": e.offset,
                     "byte_length": e.byte_length} for e in entries]}
    with open(os.path.join(HERE, "weight_archive_index_mul1_3bit.json"), "w") as handle:
        json.dump(meta, handle, indent=1)


if __name__ == "__main__":
    main()
