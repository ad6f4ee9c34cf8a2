"""Writes tests/golden/marlin_qqq_w4a8.npz: input/output vectors of the reference's W4A8 weight
quantiser and Marlin-QQQ packer, the one part of the path whose bit layout nothing but the
reference's own code pins.

Run once in the build container, where the reference checkout exists:
    python tests/golden/make_marlin_qqq_fixture.py /root/reference
It loads quamba/marlin_utils.py by file path (the file depends on numpy and torch only; the
package's __init__ is not executed) and stores plain arrays.  The tests read the .npz only.
"""
import importlib.util
import os
import sys

import numpy as np
import torch


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    path = os.path.join(ref_root, "quamba", "marlin_utils.py")
    spec = importlib.util.spec_from_file_location("ref_marlin_utils", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)

    out = {}
    g = torch.Generator().manual_seed(20240607)
    # per-group (group 128): K = 256, N = 128, with two outlier rows so that group scales differ
    w = torch.randn(256, 128, generator=g) * 0.05
    w[17] *= 6.0
    w[200] *= 3.0
    w = w.half()
    w_ref, q_w, s_group, s_channel = mod.get_w4a8_quantize_weights(w.clone(), 4, 128)
    out.update(g_w=w.numpy(), g_w_ref=w_ref.numpy(), g_q_w=q_w.numpy().astype(np.int32),
               g_s_group=s_group.numpy(), g_s_channel=s_channel.numpy())
    _, packed, ps_group, ps_channel = mod.w4a8_quantize(w.clone(), 4, 128)
    out.update(g_marlin_q_w=packed.numpy().astype(np.int32), g_marlin_s_group=ps_group.numpy(),
               g_marlin_s_channel=ps_channel.numpy())
    out_scales = torch.rand(128, generator=g) * 0.5 + 0.75
    _, packed, ps_group, ps_channel = mod.w4a8_quantize(w.clone(), 4, 128, out_scales=out_scales, pad_out=64)
    out.update(g_out_scales=out_scales.numpy(), gp_marlin_q_w=packed.numpy().astype(np.int32),
               gp_marlin_s_group=ps_group.numpy(), gp_marlin_s_channel=ps_channel.numpy())

    # per-channel (group -1): K = 128, N = 64
    w2 = (torch.randn(128, 64, generator=g) * 0.05).half()
    w_ref, q_w, s_group, s_channel = mod.get_w4a8_quantize_weights(w2.clone(), 4, -1)
    out.update(c_w=w2.numpy(), c_w_ref=w_ref.numpy(), c_q_w=q_w.numpy().astype(np.int32), c_s_channel=s_channel.numpy())
    _, packed, _, ps_channel = mod.w4a8_quantize(w2.clone(), 4, -1)
    out.update(c_marlin_q_w=packed.numpy().astype(np.int32), c_marlin_s_channel=ps_channel.numpy())

    # the permutations themselves
    out.update(perm_group=mod.get_w4a8_weight_perm(4, "per-group").numpy().astype(np.int32),
               perm_channel=mod.get_w4a8_weight_perm(4, "per-channel").numpy().astype(np.int32))
    sp, sps = mod.get_scale_perms()
    out.update(scale_perm=np.array(sp, np.int32), scale_perm_single=np.array(sps, np.int32))

    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "marlin_qqq_w4a8.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
