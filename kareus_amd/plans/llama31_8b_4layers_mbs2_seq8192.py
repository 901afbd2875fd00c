[
[(('forward', 'norm_0-none-0-1024', 'norm_0-none-0-1024'), ('backward', 'norm_0-none-0-1024', 'norm_0-none-0-1024')), (('forward', 'norm_0-none-0-1024', 'norm_0-none-0-1024'), ('backward', 'norm_0-none-0-1024', 'norm_0-none-0-1024')), (('forward', 'norm_0-none-0-1024', 'norm_0-none-0-1024'), ('backward', 'norm_0-none-0-1024', 'norm_0-none-0-1024')), (('forward', 'norm_0-none-0-1024', 'norm_0-none-0-1024'), ('backward', 'norm_0-none-0-1024', 'norm_0-none-0-1024'))],
]
# One pipeline stage, four microbatches, per-microbatch grammar ((forward, attn, mlp), (backward, attn, mlp));
# each field is "<release slot>-<end>-<compute units reserved for the other nanobatch>-<block>".
# The cheapest plan (iteration 0 of 9) that `python -m kareus_amd.profiling.plan_generator` made for the
# 4-layer Llama-3.1-8B stack on one MI355X (MBS 2 x seq 8192, 2 nanobatches, no recompute) from a sweep of
# the four partitions over every release slot and 0 or 16 reserved compute units:
#   python -m kareus_amd.profiling --partition <p> --hidden 4096 --q-heads 32 --kv-heads 8 --head-dim 128 \
#       --ffn 14336 --batch 2 --seq-len 8192 --nanobatches 2 --sm 0 16 --duration 0.6 --cooldown 0.3 --out logs/<p>.jsonl
#   python -m kareus_amd.profiling.profile_csv --log-dir logs --output profile_c5.csv --num-layers 4 \
#       --nanobatches 2 --no-activation-checkpointing --no-scale
#   python -m kareus_amd.profiling.plan_generator --inst-profile profile_c5.csv --output-dir plans \
#       --num-mbs 4 --unit-time 1e-4 --no-activation-checkpointing
# On one GPU the hand-over is a no-op, so handing compute units to it only costs the GEMMs a round of
# tiles and the earliest release is the cheapest: every slot reads norm_0 with no units reserved.
# Iteration 0 total cost: 296.2497956037519
# Iteration 0 total cost with P2P: 389.14259560375194
# Iteration 0 time: 0.32488834636468733
