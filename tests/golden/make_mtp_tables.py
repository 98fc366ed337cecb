"""Pack the MTP contraction tables of levels 6..22 into ai2pot_amd/_data/mtp_tables.npz.

The tables are data of MLIP-3 origin (https://gitlab.com/ashapeev/mlip-3), shipped by the
reference as text templates (source/descriptor/mtpr/MTP_templates/NN.almtp).  This script
parses those text files with this package's own parser and stores the four integer tables
of each level; it is run once, by hand, where the template directory exists:

    python tests/golden/make_mtp_tables.py /root/reference/source/descriptor/mtpr/MTP_templates
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from ai2pot_amd.mtp_param import parse_almtp, template_name  # noqa: E402


def main(src):
    out = {}
    for level in range(6, 24, 2):
        t = parse_almtp(os.path.join(src, template_name(level)))
        key = "L%02d" % level
        out[key + "_count"] = np.int32(t["alpha_moments_count"])
        out[key + "_basic"] = t["alpha_index_basic"].astype(np.int16)
        out[key + "_times"] = t["alpha_index_times"].astype(np.int16)
        out[key + "_mapping"] = t["alpha_moment_mapping"].astype(np.int16)
        print(level, t["alpha_moments_count"], t["alpha_index_basic"].shape,
              t["alpha_index_times"].shape, t["alpha_moment_mapping"].shape, t["nmus"])
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..", "ai2pot_amd", "_data", "mtp_tables.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main(sys.argv[1])
