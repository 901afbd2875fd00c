[
[(('forward', 'norm_0-none-16-1024', 'norm_0-none-16-1024'), ('backward', 'linear_0-none-16-1024', 'linear_0-none-16-1024')),
 (('forward', 'linear_0-none-24-1024', 'linear_0-none-24-1024'), ('backward', 'rope_0-none-24-1024', 'activation_0-none-24-1024')),
 (('forward', 'rope_0-none-32-1024', 'activation_0-none-32-1024'), ('backward', 'attn_0-none-32-1024', 'linear_1-none-32-1024')),
 (('forward', 'attn_0-none-8-1024', 'linear_1-none-8-1024'), ('backward', 'norm_0-none-8-1024', 'norm_0-none-8-1024'))],
]
# One pipeline stage, four microbatches, per-microbatch grammar ((forward, attn, mlp), (backward, attn, mlp));
# each field is "<release slot>-<end>-<compute units reserved for the other nanobatch>-<block>".
# Written by hand for the 4-layer Llama-3.1-8B stack on one MI355X (MBS 2 x seq 8192, 2 nanobatches):
# the microbatches walk through early, middle and late release points and budgets of 8 to 32 of the
# 256 compute units, so that a run exercises every slot kind of the four partitions.
