"""``cuda_lo`` of the reference (pylo/csrc/learned_optimizer.cu:303-404) on the HIP library."""

from ._call import check_sizes, pointers, run, shape_args


def learned_optimizer_kernel(g, p, m, v, fac_r, fac_c, row_factor, col_factor, second_moment, input_weights,
                             input_bias, hidden_weights, hidden_bias, output_weights, output_bias, lr, step_mult,
                             exp_mult, epsilon, step, weight_decay, dc, dr, vector_like):
    """Adds the sums of squared features into ``second_moment`` (28 used, zeroed by the caller) and updates
    ``p`` in place.  ``weight_decay`` is accepted and unused, as in the reference."""
    who = "learned_optimizer_kernel"
    check_sizes(who, p, dc, dr, vector_like, 28,
                dict(g=(g, "n"), m=(m, "3n"), v=(v, "n"), fac_r=(fac_r, "row"), fac_c=(fac_c, "col"),
                     row_factor=(row_factor, "row"), col_factor=(col_factor, "col"),
                     second_moment=(second_moment, "stat")),
                dict(input_weights=(input_weights, 32 * 39), input_bias=(input_bias, 32),
                     hidden_weights=(hidden_weights, 32 * 32), hidden_bias=(hidden_bias, 32),
                     output_weights=(output_weights, 64), output_bias=(output_bias, 2)))
    ptrs = pointers(who, p.device, p.dtype, g=g, p=p, m=m, v=v, fac_r=fac_r, fac_c=fac_c, row_factor=row_factor,
                    col_factor=col_factor, second_moment=second_moment, input_weights=input_weights,
                    input_bias=input_bias, hidden_weights=hidden_weights, hidden_bias=hidden_bias,
                    output_weights=output_weights, output_bias=output_bias)
    shape, ndim = shape_args(p)
    run(who, "pylo_mi355_learned_optimizer_kernel", p,
        ptrs + [float(lr), float(step_mult), float(exp_mult), float(epsilon), float(step), float(weight_decay),
                shape, ndim, int(dc), int(dr), int(vector_like)])
