[
[(('forward', 'norm_0-none-12-1024', 'linear_0-none-18-1024'), ('backward', 'rope_0-none-30-1024', 'activation_0-none-15-1024')),
 (('forward', 'rope_0-none-6-512', 'none-none-18-1024'), ('backward', 'attn_0-none-30-1024', 'norm_0-none-15-1024'))],
]
# hand-written: 1 pipeline stage, 2 microbatches, per-microbatch (forward, backward) pair grammar
