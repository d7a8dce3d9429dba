"""``velo_cuda_kernel`` of the reference (pylo/csrc/velo_kernel.cu:370-462) on the HIP library."""

from ._call import check_sizes, pointers, run, shape_args


def velo_kernel_simple(grad, param, momentum, rms, row_factor, col_factor, fac_vec_row, fac_vec_col, second_moment,
                       input_weights, input_bias, hidden_weights, hidden_bias, output_weights, output_bias, lr,
                       step_mult, exp_mult, epsilon, weight_decay, dc, dr, vector_like):
    """Adds the sums of squared features into ``second_moment`` (30, zeroed by the caller) and updates
    ``param`` in place, weight decay included."""
    who = "velo_kernel_simple"
    check_sizes(who, param, dc, dr, vector_like, 30,
                dict(grad=(grad, "n"), momentum=(momentum, "3n"), rms=(rms, "n"), fac_vec_row=(fac_vec_row, "row"),
                     fac_vec_col=(fac_vec_col, "col"), row_factor=(row_factor, "row"), col_factor=(col_factor, "col"),
                     second_moment=(second_moment, "stat")),
                dict(input_weights=(input_weights, 120), input_bias=(input_bias, 4), hidden_weights=(hidden_weights, 16),
                     hidden_bias=(hidden_bias, 4), output_weights=(output_weights, 12), output_bias=(output_bias, 3)))
    ptrs = pointers(who, param.device, param.dtype, grad=grad, param=param, momentum=momentum, rms=rms, row_factor=row_factor,
                    col_factor=col_factor, fac_vec_row=fac_vec_row, fac_vec_col=fac_vec_col,
                    second_moment=second_moment, input_weights=input_weights, input_bias=input_bias,
                    hidden_weights=hidden_weights, hidden_bias=hidden_bias, output_weights=output_weights,
                    output_bias=output_bias)
    shape, ndim = shape_args(param)
    run(who, "pylo_mi355_velo_kernel_simple", param,
        ptrs + [float(lr), float(step_mult), float(exp_mult), float(epsilon), float(weight_decay),
                shape, ndim, int(dc), int(dr), int(vector_like)])
