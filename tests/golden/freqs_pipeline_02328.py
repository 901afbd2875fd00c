[
[('forward', 1410), ('forward', 900), ('backward', 1320), ('forward', 1320), ('backward', 1320), ('forward', 1320), ('backward', 1320), ('forward', 1320), ('backward', 1320), ('forward', 1320), ('backward', 1320), ('forward', 1320), ('backward', 1320), ('forward', 1290), ('backward', 1020), ('backward', 1410)],
[('forward', 1410), ('backward', 1410), ('forward', 1200), ('backward', 1200), ('forward', 1200), ('backward', 1200), ('forward', 1200), ('backward', 1200), ('forward', 1200), ('backward', 1200), ('forward', 1200), ('backward', 1200), ('forward', 1200), ('backward', 1200), ('forward', 1410), ('backward', 1410)],
]
# Iteration 2328 cost change: 1.0586643526687247
# Iteration 2328 total cost: 1798.1348593212274
# Iteration 2328 total cost with P2P: 2566.5348593212275
