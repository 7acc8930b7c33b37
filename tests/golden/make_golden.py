"""Writes the golden fixtures under tests/golden/ from the CPU oracle (oracle/) on seeded synthetic
checkpoints (realtime-vla_amd/synthetic.py).  The reference holds no vectors for this path and was
not imported or run to make these; they are regression pins for the oracle (they guard against the
oracle drifting, they are not an independent anchor: the oracle's independent pins are
tests/test_oracle_ops.py and tests/test_oracle_layers.py) and the targets the GPU parity tests
compare against.

    python tests/golden/make_golden.py small      # reduced-depth cases, seconds
    python tests/golden/make_golden.py full       # BASELINE configs C1..C4 at full size, minutes
"""
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "realtime-vla_amd"))

import synthetic as syn                     # noqa: E402
from oracle import pi0, pi05                # noqa: E402

SMALL = {
    # name: (model, seed, views, prompt_len, chunk, vision_layers, llm_layers, state_tokens, max_prompt_len, norms)
    "pi0_small": ("pi0", 7, 1, 4, 10, 2, 2, 0, None, "random"),
    "pi0_small_noprompt_c63": ("pi0", 8, 1, 0, 63, 1, 2, 0, None, "random"),
    "pi05_small": ("pi05", 9, 1, 4, 10, 2, 2, 3, 12, "random"),
}
FULL = {
    "c1": ("pi0", 1234, 1, 0, 50, 27, 18, 0, None, "ones"),
    "c2": ("pi0", 1234, 2, 20, 50, 27, 18, 0, None, "ones"),
    "c3": ("pi0", 1234, 3, 0, 63, 27, 18, 0, None, "ones"),
    "c4": ("pi05", 1234, 3, 20, 50, 27, 18, 32, None, "ones"),
    "headline": ("pi0", 1234, 3, 20, 50, 27, 18, 0, None, "random"),
}
TAPS = ["vision_embed", "vision_x/0", "encoder_x0", "encoder_x/0", "encoder_K/1", "encoder_V/1",
        "decoder_x/0/0", "decoder_x/9/1", "noise/0", "noise/9"]


def run_case(spec, device="cpu"):
    model, seed, views, plen, chunk, vl, ll, st, maxp, norms = spec
    if model == "pi0":
        ck = syn.pi0_checkpoint(seed, plen, device, vl, ll, norms=norms)
        img, state, noise = syn.observation(seed, views, chunk, device)
        ck = {k: v.cpu() for k, v in ck.items()}
        taps = {}
        out = pi0.forward(ck, img.cpu(), state.cpu(), noise.cpu(), taps=taps)
        out32 = pi0.forward(ck, img.cpu(), state.cpu(), noise.cpu(), bf16_boundaries=False)
    else:
        ck = syn.pi05_checkpoint(seed, plen, device, vl, ll, state_tokens=st, norms=norms)
        img, _, noise = syn.observation(seed, views, chunk, device)
        ck = {k: v.cpu() for k, v in ck.items()}
        taps = {}
        out = pi05.forward(ck, img.cpu(), noise.cpu(), max_prompt_len=maxp, taps=taps)
        out32 = pi05.forward(ck, img.cpu(), noise.cpu(), max_prompt_len=maxp, bf16_boundaries=False)
    return out, out32, taps


def main(which, only=None):
    cases = SMALL if which == "small" else FULL
    path = os.path.join(HERE, "golden_%s.pt" % which)
    blob = torch.load(path, weights_only=True) if only and os.path.exists(path) else {}      # `only`: add / refresh some cases
    for name, spec in cases.items():
        if only and name not in only:
            continue
        out, out32, taps = run_case(spec)
        blob[name + "/actions"] = out.to(torch.bfloat16)
        blob[name + "/actions_fp32"] = out32.clone()
        if which == "small":
            for t in TAPS:
                if t in taps:
                    blob[name + "/tap/" + t] = taps[t][:8].to(torch.bfloat16).clone()      # first rows only
        print(name, "mae(bf16 oracle, fp32 oracle) = %.5f" % (out - out32).abs().mean().item(), flush=True)
    torch.save(blob, path)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "small", sys.argv[2:])
