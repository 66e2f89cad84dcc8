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
         "ocean_fabs_01", "ocean_logical_01",
         "ocean_bitshift_02", "ocean_fabs_02", "ocean_gemm_10", "ocean_gemm_11", "ocean_linspace_03", "ocean_maximumabs_01", "ocean_not_01",
         "ocean_cast_01", "ocean_power_01", "ocean_power_02", "ocean_power_03", "ocean_sum_01", "ocean_unary_01", "tensor_add_01",
         "tensor_axis_norm2_01", "tensor_divide_01", "tensor_multiply_01", "tensor_subtract_01", "tensor_dtype_cast_01", "tensor_fill_01",
         "tensor_copy_03", "tensor_copy_04", "tensor_copy_06", "tensor_copy_07",
         "tensor_copy_01", "tensor_copy_02", "tensor_copy_05", "tensor_copy_09", "tensor_clone_01", "tensor_clone_02", "tensor_clone_03",
         "tensor_device_cast_01", "tensor_split_01"]
# the GPU file of tensor_fillnan_01 records a defect of the reference's GPU kernel (it fills every element,
# solid/src/core/gpu/template_fill.cu:72-79); the CPU twin holds the defined behaviour (only NaN is replaced)
CPU_TWINS = ["tensor_fillnan_01"]
# index operations: the GPU index example, and the CPU examples of find (absent from the reference's GPU module)
OTHER = [("/root/reference/examples/python/gpu/index/index_008.ref", "index_008.ref"),
         ("/root/reference/examples/python/cpu/tensors/ocean_find_01.ref", "ocean_find_01_cpu.ref"),
         ("/root/reference/examples/python/cpu/tensors/tensor_find_01.ref", "tensor_find_01_cpu.ref")]
# matrix products: transposition / conjugation modes for float, double, complex, int16 and bool (the GPU examples hold three)
OTHER += [("/root/reference/examples/python/cpu/tensors/%s.ref" % n, "%s_cpu.ref" % n)
          for n in ("ocean_gemm_02", "ocean_gemm_03", "ocean_gemm_07", "ocean_gemm_08a", "ocean_gemm_09a", "ocean_gemm_09b", "ocean_gemm_09c",
                    "ocean_gemm_09d", "ocean_multiply_01", "ocean_multiply_02")]
# reductions: axis sums / products with NaN variants, all / any / nnz along axes, p-norms
OTHER += [("/root/reference/examples/python/cpu/tensors/%s.ref" % n, "%s_cpu.ref" % n)
          for n in ("ocean_axis_reduce_01", "ocean_axis_reduce_02", "ocean_axis_sum_01", "ocean_axis_all_01", "ocean_axis_nnz_01", "ocean_norm_01", "ocean_norm_02")]
# division family on operands of either sign
OTHER += [("/root/reference/examples/python/cpu/tensors/%s.ref" % n, "%s_cpu.ref" % n)
          for n in ("ocean_divide_01", "ocean_floordivide_01", "ocean_truedivide_01", "ocean_fmod_01")]
# extremes with NaN and complex ordering; square root and negation over the types; integer power with a negative exponent
OTHER += [("/root/reference/examples/python/cpu/tensors/%s.ref" % n, "%s_cpu.ref" % n)
          for n in ("ocean_maximum_01", "ocean_minimum_01", "ocean_maximum_abs_01", "ocean_minimum_abs_01", "tensor_sqrt_01", "ocean_sqrt",
                    "tensor_negative_01", "tensor_negative_02", "ocean_power_04")]

if __name__ == "__main__":
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref")
    os.makedirs(dst, exist_ok=True)
    for n in NAMES:
        shutil.copyfile(os.path.join(SRC, n + ".ref"), os.path.join(dst, n + ".ref"))
    for n in CPU_TWINS:
        shutil.copyfile(os.path.join(SRC.replace("/gpu/", "/cpu/"), n + ".ref"), os.path.join(dst, n + "_cpu.ref"))
    for src, name in OTHER:
        shutil.copyfile(src, os.path.join(dst, name))
    print("copied %d files" % (len(NAMES) + len(CPU_TWINS) + len(OTHER)))
