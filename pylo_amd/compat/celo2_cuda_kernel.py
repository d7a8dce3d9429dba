"""``celo2_cuda_kernel`` of the reference (pylo/csrc/celo2_kernel.cu:284-357) on the HIP library."""

from ._call import check_sizes, pointers, run, shape_args


def celo2_kernel(g, p, m, v, fac_r, fac_c, row_factor, col_factor, second_moment, w_in, b_in, w_h, b_h,
                 w_out, b_out, step_out, exp_mult, dc, dr, vector_like):
    """Adds the sums of squared features into ``second_moment`` (30, zeroed by the caller) and writes
    ``step_out = o0 * exp(o1 * exp_mult)``; ``p`` is not modified."""
    who = "celo2_kernel"
    check_sizes(who, p, dc, dr, vector_like, 30,
                dict(g=(g, "n"), m=(m, "3n"), v=(v, "n"), fac_r=(fac_r, "row"), fac_c=(fac_c, "col"),
                     row_factor=(row_factor, "row"), col_factor=(col_factor, "col"),
                     second_moment=(second_moment, "stat"), step_out=(step_out, "n")),
                dict(w_in=(w_in, 240), b_in=(b_in, 8), w_h=(w_h, 64), b_h=(b_h, 8), w_out=(w_out, 24), b_out=(b_out, 3)))
    ptrs = pointers(who, p.device, p.dtype, g=g, p=p, m=m, v=v, fac_r=fac_r, fac_c=fac_c, row_factor=row_factor,
                    col_factor=col_factor, second_moment=second_moment, w_in=w_in, b_in=b_in, w_h=w_h, b_h=b_h,
                    w_out=w_out, b_out=b_out, step_out=step_out)
    shape, ndim = shape_args(p)
    run(who, "pylo_mi355_celo2_kernel", p, ptrs + [float(exp_mult), shape, ndim, int(dc), int(dr), int(vector_like)])
