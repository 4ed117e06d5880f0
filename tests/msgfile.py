"""Writer for the weight side-file of a compiled model (test infrastructure), after the layout of
fhe-cmplr/include/fhe/core/rt_data_def.h:62-84 and the writer in rt_data_writer.h:34-107: a 136-byte header, entries
from offset 4096 on padded to 2^align bytes, then the lookup table of 32-byte records."""
import struct

import numpy as np

PAGE = 4096


def write(path, entries, dtype=np.float32, align=5, model="model", uuid="XXXXXXXX-XXXX-XXXX-XXXX-XXXXXXXXXXXX"):
    """entries: list of (name, values, scale, level)."""
    ent_type = {np.float32: 0, np.float64: 1}[dtype]
    body, lut = bytearray(), []
    for i, (name, values, scale, level) in enumerate(entries):
        raw = np.asarray(values, dtype).tobytes()
        ofst = PAGE + len(body)
        body += raw + b"\0" * (-len(raw) % (1 << align))
        lut.append(struct.pack("<16sIIQ", name.encode(), i, len(raw), scale | (level << 8) | (ofst << 16)))
    hdr = struct.pack("<8sIHBBQQqq48s40s", b"!ANTFHE\0", 1, 0, ent_type, align, len(entries), PAGE + len(body), 0, 0,
                      model.encode(), uuid.encode())
    assert len(hdr) == 136
    with open(path, "wb") as f:
        f.write(hdr + b"\0" * (PAGE - len(hdr)) + bytes(body) + b"".join(lut))
