"""Rotation frequencies with llama3 scaling as numbers, worked out once in float64 straight from
the rule (src/op/kernels/cpu/rope_kernel.cpp:121-139), by neither the plain implementation nor the
engine: f = theta^(-2p/hd), wl = 2 pi / f; wl >= orig/low: f / factor; wl > orig/high:
f ((1 - s)/factor + s) with s = (orig/wl - low)/(high - low); else f.

One of them by hand: the 1B constants (hd 64, theta 5e5, factor 32, low 1, high 4, orig 8192), pair
16: f = 1/sqrt(5e5) = 1.41421e-3, wl = 4442.88, s = (8192/4442.88 - 1)/3 = 0.281283,
f' = f (0.718717/32 + 0.281283) = 0.303743 f = 4.29557e-4.  With the blend the other way round
(s and 1 - s exchanged) it would be 0.7275 f.
"""

SCALING_B = {"factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 64}
SCALING_1B = {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
SCALING_8B = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}

# (head_dim, theta, scaling) -> {pair: (band, frequency)}
CASES = [
    (32, 500000.0, SCALING_B, {
        0: ("short", 1.0), 1: ("short", 0.44036660267178046), 2: ("middle", 0.09576297140341929),
        3: ("long", 0.021349275071441402), 4: ("long", 0.009401507732715983), 5: ("long", 0.004140110020248612)}),
    (64, 500000.0, SCALING_1B, {
        13: ("short", 0.004839421345719893), 14: ("short", 0.003211445994752591),
        15: ("middle", 0.0012905479282092638), 16: ("middle", 0.0004295567965593682),
        17: ("middle", 9.70828780262767e-05), 18: ("long", 1.9461638184831125e-05),
        19: ("long", 1.291476718704739e-05), 20: ("long", 8.570255489881478e-06)}),
    (128, 500000.0, SCALING_8B, {
        28: ("short", 0.003211445994752591), 29: ("middle", 0.002166570763503359),
        30: ("middle", 0.0013718935677611381), 31: ("middle", 0.0008567514129196321),
        32: ("middle", 0.0005248461609929546), 33: ("middle", 0.00031269375038406517),
        34: ("middle", 0.0001785078127679964), 35: ("long", 9.556212353964683e-05),
        36: ("long", 7.78465527393245e-05), 39: ("long", 4.208236768725526e-05)}),
]
