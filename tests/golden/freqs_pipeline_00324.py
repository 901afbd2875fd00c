[
[('forward', 930), ('forward', 900), ('backward', 900), ('forward', 930), ('backward', 900), ('forward', 930), ('backward', 900), ('forward', 930), ('backward', 900), ('forward', 930), ('backward', 900), ('forward', 930), ('backward', 900), ('forward', 930), ('backward', 900), ('backward', 900)],
[('forward', 930), ('backward', 900), ('forward', 900), ('backward', 900), ('forward', 900), ('backward', 900), ('forward', 900), ('backward', 900), ('forward', 900), ('backward', 900), ('forward', 900), ('backward', 900), ('forward', 900), ('backward', 900), ('forward', 930), ('backward', 900)],
]
# Iteration 324 cost change: 0.0227579757019285
# Iteration 324 total cost: 1224.8441048803174
# Iteration 324 total cost with P2P: 2333.9241048803174
