"""Writes the golden fixtures in this directory from DATA files shipped in the reference.

Run once in the build container:  python tests/golden/make_fixtures.py /root/reference
It reads only look-up-table text files (``app_mults/**/*_lutfp*.txt`` -- data, ``a b value`` lines);
no reference code is imported or executed.  Outputs:

  *.txt.gz                      verbatim gzip copies of four shipped table files (6-, 7-, 7-bit "+bp"
                                files and one plain 7-bit "_lutfp.txt" whose table header sits after
                                ABC warning lines) -- they pin the text format and the
                                forward-table -> gradient-table generator.
  lut8_resub_183.npz            the three tables of one shipped 8-bit "+bp" file as int32 arrays
                                (the text is 2.4 MB) plus its half window.
  manifest.json                 source path, size and half-window of every fixture.
"""
import gzip
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

COPIES = [
    ("app_mults/vert_trunc/mult6u/6_6_U_SP_WT_CL_GenMul_vertical_truncation_4cols_lutfp+bp_avg_2_2.txt", "lut6_vert_trunc_bp2.txt.gz", 6, 2),
    ("app_mults/resub_als/Mult_7_7_MED_63.6771_size_178_depth_23_lutfp+bp_avg_8_8.txt", "lut7_resub_63_bp8.txt.gz", 7, 8),
    ("app_mults/evo_selected/mult7u/mul7u_081_lutfp+bp_avg_16_16.txt", "lut7_evo_081_bp16.txt.gz", 7, 16),
    ("app_mults/vert_trunc/mult7u/7_7_U_SP_WT_CL_GenMul_vertical_truncation_6cols_lutfp.txt", "lut7_vert_trunc_fwdonly.txt.gz", 7, None),
]
NPZ = ("app_mults/resub_als/Mult_8_8_MED_183.376_size_209_depth_25_lutfp+bp_avg_16_16.txt", "lut8_resub_183.npz", 8, 16)


def main(ref_root):
    from oracle.lutgemm_oracle import parse_lut_file
    manifest = {}
    for rel, name, bits, hw in COPIES:
        src = os.path.join(ref_root, rel)
        data = open(src, "rb").read()
        with gzip.GzipFile(os.path.join(HERE, name), "wb", mtime=0) as f:
            f.write(data)
        manifest[name] = {"source": rel, "bytes": len(data), "bits": bits, "half_window": hw}
    rel, name, bits, hw = NPZ
    fwd, ga, gb = parse_lut_file(os.path.join(ref_root, rel), bits)
    np.savez_compressed(os.path.join(HERE, name), fwd=fwd.astype(np.int32), grad_a=ga.astype(np.int32),
                        grad_b=gb.astype(np.int32), half_window=np.int32(hw))
    manifest[name] = {"source": rel, "bits": bits, "half_window": hw}
    json.dump(manifest, open(os.path.join(HERE, "manifest.json"), "w"), indent=1, sort_keys=True)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
