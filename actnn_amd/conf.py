"""Global configuration of the compression path and the optimisation levels
(behaviour of the reference's actnn/actnn/conf.py:5-68, restated)."""
import ast
import os
import warnings


class QuantizationConfig:
    """One process-wide instance (`config`).  It must be set up before Q-layers are built:
    schemes read their bit budgets in their constructors (reference README.md:50-54)."""

    def __init__(self):
        self.reset()

    def reset(self):
        # what to compress and how (conf.py:40-52)
        self.compress_activation = True
        self.activation_compression_bits = [2, 8, 8]   # average bits per layer group
        self.pergroup = True                           # per-group min/max (else one range per tensor)
        self.perlayer = True                           # re-balance bits across layers each step
        self.initial_bits = 8                          # width the greedy allocation starts from
        self.stochastic = True
        self.training = True                           # toggled by QModule.train()/eval()
        self.group_size = 256
        self.use_gradient = False                      # per-sample gradient statistics (needs indices)
        self.adaptive_conv_scheme = True
        self.adaptive_bn_scheme = True
        self.simulate = False                          # pure-torch quantiser instead of the kernels
        self.enable_quantized_bn = True
        self.device_allocation = True                  # per-sample widths computed on the GPU when the batch fits
        self.fused_bn_backward = True                  # batch-norm backward reads the packed input directly
        self.share_relu_min_max = True                 # ReLU leaves its output's group min/max for the next layer
        self.share_grad_sqnorm = True                  # batch-norm backward leaves sum(dx^2) for the conv's set_scale
        self.fused_bn_pack = True                      # batch-norm forward writes the packed copy of its input
        # a layer's forward-side sequence (min/max or statistics -> widths -> pack) behind one library
        # call where the widths are made on the device: same kernels, less host time per layer
        self.fused_quantize = True
        # relu(bn(x)) in the batch norm's normalise + pack pass where a model hands the pair over
        # together (layers.bn_relu) and the shape allows it: bn(x) is never written
        self.fused_bn_relu = True
        self.fused_bn_relu_backward = True             # ... and its backward passes apply the ReLU's mask as they read
        self.fused_bn_add_relu = True                  # relu(bn(x) + identity) likewise (layers.bn_add_relu)
        # a residual block's input gradient: the closing ReLU's mask applied to the skip connection's
        # gradient as it is added to the one from the block's layers (layers.skip_connection)
        self.fused_skip_gradient = True
        # QLinear's weight gradient straight from the packed input (the dequantised input is never
        # written): True - where the fused kernel is the faster path, i.e. for the 2-bit fixed-width
        # stream; "always" - for every stream it takes (saves the full-precision copy at 0.7-0.9 ms
        # against 0.25 ms on [8192,4096] x [8192,4096] for the 4-bit and the mixed-width stream);
        # False - never
        self.fused_linear_grad_weight = True
        self.pool_index_nibbles = True                 # max-pool keeps its arg-max indices two per byte
        # memory management (conf.py:54-58)
        self.empty_cache_threshold = None
        self.pipeline_threshold = None
        self.cudnn_benchmark_conv2d = True
        self.swap = False
        # debugging (conf.py:60-66)
        self.debug_memory_model = ast.literal_eval(os.environ.get("DEBUG_MEM", "False"))
        self.debug_speed = ast.literal_eval(os.environ.get("DEBUG_SPEED", "False"))
        self.debug_memory_op_forward = False
        self.debug_memory_op_backward = False
        self.debug_remove_bn = False
        self.debug_remove_relu = False


config = QuantizationConfig()

_LEVELS = ("L0", "L1", "L2", "L3", "L3.1", "L4", "L5", "swap")


def set_optimization_level(level):
    """conf.py:5-36.  L0: masks only; L1: 4-bit conv inputs, BN left alone; L2: 4-bit everywhere;
    L3: 2-bit adaptive (the defaults); L3.1: + allocator hygiene and micro-batched conv backward;
    L4/L5: + packed tensors swapped to pinned host memory; swap: swapping without compression."""
    if level not in _LEVELS:
        raise ValueError("Invalid level: " + level)
    if level == "L0":
        config.compress_activation = False
        config.adaptive_conv_scheme = config.adaptive_bn_scheme = False
    elif level in ("L1", "L2"):
        config.activation_compression_bits = [4]
        config.adaptive_conv_scheme = config.adaptive_bn_scheme = False
        if level == "L1":
            config.enable_quantized_bn = False
    elif level == "L3.1":
        config.cudnn_benchmark_conv2d = False
        config.empty_cache_threshold = 0.2
        config.pipeline_threshold = 3 * 1024 ** 3
    elif level in ("L4", "L5"):
        config.swap = True
        if level == "L5":
            os.environ["PYTORCH_CACHE_THRESHOLD"] = "256000000"
            warnings.warn("L5's allocator defragmentation needs a patched PyTorch in the reference; "
                          "here it behaves like L4.")
    elif level == "swap":
        config.swap = True
        config.compress_activation = False
