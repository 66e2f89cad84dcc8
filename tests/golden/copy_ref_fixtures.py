"""Copies the expected-output files (.ref) of the reference's own GPU example tests that the
fixture tests replay into tests/golden/ref/. They are data files (printed tensors and scalars);
the scripts that produced them stay in the reference tree.

    python tests/golden/copy_ref_fixtures.py
"""
import os
import shutil

SRC = "/root/reference/examples/python/gpu/tensors"
NAMES = ["tensor_add_02", "ocean_min_01", "ocean_and_01", "ocean_or_01", "ocean_xor_01", "ocean_bitshift_01", "ocean_sign_01",
         "ocean_axis_reduce_04", "ocean_sum_02", "ocean_sumabs_01", "ocean_all_01", "ocean_maximumabs_02", "ocean_gemm_01",
         "ocean_fabs_01", "ocean_logical_01"]

if __name__ == "__main__":
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref")
    os.makedirs(dst, exist_ok=True)
    for n in NAMES:
        shutil.copyfile(os.path.join(SRC, n + ".ref"), os.path.join(dst, n + ".ref"))
    print("copied %d files" % len(NAMES))
