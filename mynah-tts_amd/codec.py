"""The codec's residual layer as two sequences of backend calls.

`res_layer` issues what res_layer_device issues (src/graph.c:2423-2498): per branch a copy of the input, per block
copy, snake, conv, snake, conv, residual add, then the branch added to the output, and the sum scaled by a third at the
end.  `res_layer_fused` computes the same values, bit for bit, from a third of the launches: the element-wise operators
travel in the epilogue of the convolution before them (mynah_hip_conv1d_fused), and only a branch's first activation is a
pass of its own (snake_copy_dev).  `res_layer_batched` issues res_layer_fused's calls with the three branches' convolutions
of one block and position in one launch each (mynah_hip_conv1d_fused_batch): the branches do not depend on each other until
their last convolutions; those run side by side as well, each into its own rows, and one pass (rows_combine_dev) adds the
branches in order, scales and activates.  Same values again, bit for bit.

blocks[branch][block] = (alpha_in, (w_in, b_in), alpha_skip, (w_skip, b_skip), dilation); the branch's kernel size is the
weights' last dimension.  Buffers are device allocations of channels * length floats.
"""


def res_layer(backend, blocks, din, dout, channels, length, current, activated, residual, branch_out):
    n = channels * length
    for index, branch in enumerate(blocks):
        backend.copy_dev(current, din, n)
        for a_in, (w_in, b_in), a_skip, (w_skip, b_skip), dilation in branch:
            kernel = w_in.shape[2]
            backend.copy_dev(activated, current, n)
            backend.snake_dev(activated, a_in, channels, length, channels // 2)
            backend.conv1d(activated, residual, channels, channels, length, kernel, dilation, w_in, b_in)
            backend.snake_dev(residual, a_skip, channels, length, channels // 2)
            backend.conv1d(residual, branch_out, channels, channels, length, kernel, 1, w_skip, b_skip)
            backend.residual_inplace(current, branch_out, n)
        if index == 0:
            backend.copy_dev(dout, current, n)          # the reference adds to uploaded zeros (src/graph.c:2441,2492)
        else:
            backend.residual_inplace(dout, current, n)
    backend.scale_dev(dout, n, 1.0 / 3.0)


def res_layer_fused(backend, blocks, din, dout, channels, length, current, activated, residual, then_alpha=None):
    """then_alpha: the half-snake that the caller would apply to the layer's output next (decode_codec_resident's
    activation before the next stage's transposed conv or the post-conv), applied by the layer's last call."""
    for index, branch in enumerate(blocks):
        backend.snake_copy_dev(din, activated, branch[0][0], channels, length, channels // 2)
        for position, (a_in, (w_in, b_in), a_skip, (w_skip, b_skip), dilation) in enumerate(branch):
            kernel = w_in.shape[2]
            # input conv, its result activated for the skip conv
            backend.conv1d_fused(activated, residual, channels, channels, length, kernel, dilation, w_in, b_in, alpha=a_skip)
            before = din if position == 0 else current
            if position + 1 < len(branch):
                # skip conv + the block's residual add; the sum also leaves activated for the next block's input conv
                backend.conv1d_fused(residual, current, channels, channels, length, kernel, 1, w_skip, b_skip, residual=before,
                                     alpha=branch[position + 1][0], activated=activated)
            else:
                # the branch's last block adds the branch to the output, and the last branch scales the sum
                backend.conv1d_fused(residual, dout, channels, channels, length, kernel, 1, w_skip, b_skip, residual=before,
                                     residual2=None if index == 0 else dout,
                                     scale=1.0 / 3.0 if index + 1 == len(blocks) else 1.0,
                                     alpha=then_alpha if index + 1 == len(blocks) else None)


def res_layer_batched(backend, blocks, din, dout, channels, length, currents, activateds, residuals, then_alpha=None):
    """currents, activateds, residuals: one buffer per branch each (the branches run side by side)."""
    branches = len(blocks)
    # the input through every branch's first activation: one pass, one output per branch
    backend.rows_combine_dev([din], 1.0, activateds, [branch[0][0] for branch in blocks], channels, length)
    positions = len(blocks[0])
    for position in range(positions):
        # input convs of every branch, their results activated for the skip convs
        backend.conv1d_fused_batch([{"din": activateds[i], "dout": residuals[i], "kernel": blocks[i][position][1][0].shape[2],
                                     "dilation": blocks[i][position][4], "weight": blocks[i][position][1][0], "bias": blocks[i][position][1][1],
                                     "alpha": blocks[i][position][2]} for i in range(branches)], channels, channels, length)
        if position + 1 < positions:
            # skip convs + the blocks' residual adds; the sums also leave activated for the next blocks' input convs
            backend.conv1d_fused_batch([{"din": residuals[i], "dout": currents[i], "kernel": blocks[i][position][3][0].shape[2], "dilation": 1,
                                         "weight": blocks[i][position][3][0], "bias": blocks[i][position][3][1],
                                         "residual": din if position == 0 else currents[i], "alpha": blocks[i][position + 1][0],
                                         "activated": activateds[i]} for i in range(branches)], channels, channels, length)
        else:
            # the branches' last skip convs + residual adds side by side too (each into its own rows), then one pass that adds
            # the branches in branch order, scales the sum and applies the caller's activation: ((b0 + b1) + b2) * 1/3, which
            # is what the one-after-the-other form computes in its last convolutions' epilogues
            backend.conv1d_fused_batch([{"din": residuals[i], "dout": currents[i], "kernel": blocks[i][position][3][0].shape[2], "dilation": 1,
                                         "weight": blocks[i][position][3][0], "bias": blocks[i][position][3][1],
                                         "residual": din if position == 0 else currents[i]} for i in range(branches)], channels, channels, length)
            backend.rows_combine_dev(currents, 1.0 / branches, [dout], [then_alpha], channels, length)
