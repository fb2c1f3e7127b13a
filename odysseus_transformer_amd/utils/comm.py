"""Layout rule for the weight-gradient product (utils/comm.py:4-20 of the reference)."""


def prepare_input_tensors_for_wgrad_compute(grad_output, all_gathered_input):
    """dY made contiguous; a 3-D (b, s, h) pair is flattened to 2-D (b*s, h) for dY^T X."""
    grad_output = grad_output.contiguous()
    if grad_output.dim() == 3:
        b, s, h = grad_output.shape
        grad_output = grad_output.view(b * s, h)
        ib, is_, ih = all_gathered_input.shape
        all_gathered_input = all_gathered_input.view(ib * is_, ih)
    return grad_output, all_gathered_input
