[
[('forward', 'norm_0-none-12-1024', 'norm_0-none-18-1024'), ('backward', 'attn_0-none-21-1024', 'norm_0-none-15-1024', 'rope_0-none-30-1024', 'activation_0-none-15-1024'), ('forward', 'linear_0-none-27-1024', 'none-none-27-1024'), ('backward', 'norm_0-none-27-1024', 'linear_1-none-27-1024', '0--1-30-1024', '-1--1-15-1024')],
]
# hand-written: 1 pipeline stage, 2 microbatches, activation-checkpointing grammar
