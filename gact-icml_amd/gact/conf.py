"""Global configuration of the activation-compression path.

Field names, defaults and optimisation levels follow gact/gact/conf.py:1-72 of the reference;
``rng_stream`` is the one addition.
"""


class QuantizationConfig:
    def __init__(self):
        # compress activations; False at optimisation level L0
        self.compress_activation = True

        # ---- general quantisation ----
        # average bits per activation element; with auto precision off every tensor uses this width
        self.bit = 4
        self.group_size = 256
        # skip tensors that were already saved in this iteration (keyed by sampled contents)
        self.check_dup = False

        # ---- auto precision ----
        self.auto_prec = True
        self.max_bit = 32          # widest allocation the greedy search starts from
        self.adapt_interval = 1000  # iterations between sensitivity refreshes
        self.work_dir = "./log/"
        self.log_interval = -1      # < 0 disables logging
        self.debug = False

        # Run the greedy allocation on the GPU (not in the reference): the sensitivities of an adaptation stay in
        # device memory, calc_precision runs there behind the probes, and one copy brings the widths back.
        # Same widths as the host routine.
        self.device_calc_precision = False

        # ---- memory management ----
        self.swap = False
        self.prefetch = False

        # ---- bool masks (not in the reference) ----
        # Current PyTorch saves dropout masks (and comparison masks) as bool, one byte per element, which the
        # reference's uint8 rule never sees.  They are packed to one bit per element, losslessly.
        self.compress_bool_masks = True

        # ---- seeds in device memory (not in the reference) ----
        # The iteration count that is added to every tensor's seed is read by the kernels from a word in device
        # memory instead of travelling as a launch argument.  Same noise; needed when the hooked pass is
        # recorded in a HIP graph, whose launch arguments are frozen at capture.
        self.device_seed = False

        # ---- stochastic-rounding noise (not in the reference) ----
        # "fast":          one Philox4x32-7 block per 32 elements: 16 draws of 8 bits, centred ((2h - 255)/512, so the
        #                  reference's "+ noise - 0.5" is one addition), each used once as c and once, half a group
        #                  further on, as -c.  The two elements of such a pair are not independent: their rounding
        #                  errors have covariance <= 0, which lowers the variance of a sum in which both carry
        #                  weights of the same sign and raises it (at most twofold) where the signs differ; over
        #                  weights of random sign it equals the independent stream's.
        # "reference":     the reference's stream (one Philox state per output byte, cuRAND uniform map)
        # "deterministic": u = 0.5 everywhere, i.e. round to nearest
        self.rng_stream = "fast"


config = QuantizationConfig()


def set_optimization_level(level):
    """gact/gact/conf.py:1-36."""
    if level == 'L0':
        config.compress_activation = False
    elif level == 'L1':      # fixed 4 bit
        config.auto_prec = False
        config.bit = 4
    elif level == 'L1.1':    # fixed 8 bit
        config.auto_prec = False
        config.bit = 8
    elif level == 'L1.2':    # fixed 2 bit
        config.auto_prec = False
        config.bit = 2
    elif level == 'L2':      # auto precision, 4 bit average
        config.auto_prec = True
        config.bit = 4
    elif level == 'L2.1':    # auto precision, 3 bit average
        config.auto_prec = True
        config.bit = 3
    elif level == 'L2.2':    # auto precision, 2 bit average
        config.auto_prec = True
        config.bit = 2
    elif level == 'L3':      # auto precision 4 bit + swap
        config.auto_prec = True
        config.bit = 4
        config.swap = True
        config.prefetch = True
    elif level == 'swap':    # swap only
        config.swap = True
        config.compress_activation = False
    elif level == 'L4bit-swap':
        config.bit = 4
        config.swap = True
        config.prefetch = True
        config.auto_prec = False
    else:
        raise ValueError("Invalid level: " + level)


def set_adapt_interval(i):
    config.adapt_interval = i
