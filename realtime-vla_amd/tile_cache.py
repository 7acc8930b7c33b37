"""On-disk cache of the library's re-tiled weights.

The first rtvla_tiled_bytes bytes of the workspace after rtvla_prepare are a function of the checkpoint's weights, the
model kind, the layer counts, the number of flow steps and the tile layout version.  For Pi0 and DM0 only the re-tiled
matrices enter; for Pi05 the region also holds W diag(1 + scale) per (flow step, layer), and `scale` comes from the time
embedding table, the time MLP and the norm-modulation weights and biases, so the key has to cover every weight of the
checkpoint except the ones that are never tiled (token-embedding tables, prompt embeddings).  This module saves that
region once per checkpoint and, on later starts, memory-maps the file and copies it to the device instead of re-tiling.  The file is keyed by a
fingerprint of the weights computed on the device where they already are (exact integer sums, so it is
deterministic and costs one pass over the weights at memory bandwidth), not by a path or a time stamp.

    file = <dir>/<key>.rtvla-tiles :  64-byte little-endian header | the tiled region, byte for byte
    header: b"RTVLATIL" | u32 layout version | u16 model | u16 flow steps | u32 vision layers | u32 llm layers | u64 tiled bytes | 32-byte key
"""
import hashlib
import os
import struct

import torch

MAGIC = b"RTVLATIL"
HEADER = struct.Struct("<8sIHHIIQ32s")
assert HEADER.size == 64
# weights that never reach the tiled region: the prompt's embeddings and the token-embedding tables (about 1 GB each)
UNTILED_WEIGHTS = ("language_embeds", "embedding_weight", "vision_embed_tokens_w")


def fingerprint(weights):
    """sha256 over (name, dtype, shape, two exact checksums) of every tensor, in name order.  The checksums are the
    wrapping int64 sum of the tensor's 16-bit words and the sum weighted by (position mod 65521), which also moves when
    words are permuted; both are integer arithmetic, hence identical on any device."""
    h = hashlib.sha256()
    for name in sorted(weights):
        t = weights[name]
        h.update(name.encode()); h.update(str(t.dtype).encode()); h.update(str(tuple(t.shape)).encode())
        if t.numel() == 0:
            continue
        words = t.contiguous().view(torch.uint8).reshape(-1)
        if words.numel() % 2:
            words = torch.cat([words, words.new_zeros(1)])
        w = words.view(torch.int16).to(torch.int64)
        pos = torch.arange(w.numel(), device=w.device, dtype=torch.int64) % 65521
        h.update(struct.pack("<qq", int(w.sum().item()), int((w * pos).sum().item())))
    return h.digest()


class TileCache:
    def __init__(self, directory):
        self.directory = str(directory)

    def path(self, key):
        return os.path.join(self.directory, key.hex()[:40] + ".rtvla-tiles")

    def load_into(self, key, layout_version, model, num_steps, vision_layers, llm_layers, region):
        """Copy the cached region into `region` (a uint8 device tensor of exactly the tiled size).  False when there is
        no file for this key or its header does not match in every field."""
        path = self.path(key)
        n = region.numel()
        try:
            if os.path.getsize(path) != HEADER.size + n:
                return False
            with open(path, "rb") as f:
                magic, ver, mdl, steps, vl, ll, size, k = HEADER.unpack(f.read(HEADER.size))
        except (OSError, struct.error):
            return False
        if (magic, ver, mdl, steps, vl, ll, size, k) != (MAGIC, layout_version, model, num_steps, vision_layers, llm_layers, n, key):
            return False
        mapped = torch.from_file(path, shared=False, size=HEADER.size + n, dtype=torch.uint8)     # memory-mapped, read as it is copied
        region.copy_(mapped[HEADER.size:])
        return True

    def store(self, key, layout_version, model, num_steps, vision_layers, llm_layers, region):
        os.makedirs(self.directory, exist_ok=True)
        path = self.path(key)
        tmp = path + ".tmp.%d" % os.getpid()
        host = region.cpu()
        with open(tmp, "wb") as f:
            f.write(HEADER.pack(MAGIC, layout_version, model, num_steps, vision_layers, llm_layers, host.numel(), key))
            f.write(host.numpy().tobytes() if host.numel() < (1 << 28) else b"")
            if host.numel() >= (1 << 28):                      # large regions in pieces, without a second host copy
                step = 1 << 28
                for i in range(0, host.numel(), step):
                    f.write(host[i:i + step].numpy().tobytes())
        os.replace(tmp, path)                                   # atomic: readers see the old file or the whole new one
        return path
