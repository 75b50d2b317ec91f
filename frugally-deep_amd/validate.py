"""Checker for converted-JSON model files (the output of the reference's keras_export/convert_model.py).

`problems(text_or_dict)` walks a file the way the loader does (include/fdeep/model.hpp:226-267,
include/fdeep/import_model.hpp) but keeps going after the first finding, so an exporter or a hand-written writer gets
the whole list at once: missing top-level fields, layers of a class the device path does not run (those need a custom
layer creator), config keys the loader would dereference, parameter arrays that are absent or whose length does not
fit the layer's config, and connections that name unknown layers.  It never touches the GPU and runs no model code.
"""
import base64
import json

IDENTITY = {
    "Identity", "Dropout", "Masking", "ActivityRegularization", "AlphaDropout", "FixedDropout", "SpatialDropout1D",
    "SpatialDropout2D", "SpatialDropout3D", "GaussianDropout", "GaussianNoise", "RandomBrightness", "RandomContrast",
    "RandomCrop", "RandomFlip", "RandomHeight", "RandomRotation", "RandomTranslation", "RandomWidth", "RandomZoom",
    "RandomColorDegeneration", "RandomColorJitter", "RandomElasticTransform", "RandomErasing", "RandomGaussianBlur",
    "RandomGrayscale", "RandomHue", "RandomInvert", "RandomPerspective", "RandomPosterization", "RandomSaturation",
    "RandomSharpness", "RandomShear", "AugMix", "CutMix", "Equalization", "MaxNumBoundingBoxes", "MixUp", "Pipeline",
    "RandAugment", "Solarization",
}

ACTIVATION_LAYERS = {
    "LeakyReLU", "LeakyRelu", "ELU", "Elu", "Celu", "ReLU", "Relu6", "Exp", "Gelu", "Selu", "Silu", "Tanh", "TanhShrink",
    "Threshold", "Sigmoid", "HardShrink", "HardSigmoid", "HardTanh", "SoftShrink", "Softplus", "Softsign", "SparsePlus",
    "Squareplus", "LogSigmoid", "LogSoftmax", "Softmax",
}

# names accepted in an "activation" config entry or an Activation layer (import_model.hpp:1649-1700)
ACTIVATIONS = {
    "linear", "relu", "relu6", "gelu", "softmax", "log_softmax", "tanh", "sigmoid", "hard_sigmoid", "swish", "silu", "selu",
    "elu", "celu", "exponential", "softplus", "softsign", "leaky_relu", "hard_tanh", "hard_shrink", "soft_shrink",
    "tanh_shrink", "threshold", "log_sigmoid", "sparse_plus", "squareplus",
}

_CONV_KEYS = ("filters", "kernel_size", "strides", "dilation_rate", "padding", "use_bias")
_POOL_KEYS = ("pool_size", "strides", "padding")

# class -> config keys the loader reads without a default
REQUIRED_CONFIG = {
    "Conv1D": _CONV_KEYS, "Conv2D": _CONV_KEYS, "Conv1DTranspose": _CONV_KEYS, "Conv2DTranspose": _CONV_KEYS,
    "SeparableConv1D": _CONV_KEYS, "SeparableConv2D": _CONV_KEYS,
    "DepthwiseConv1D": ("kernel_size", "strides", "dilation_rate", "padding", "use_bias"),
    "DepthwiseConv2D": ("kernel_size", "strides", "dilation_rate", "padding", "use_bias"),
    "Dense": ("units", "use_bias"),
    "EinsumDense": ("equation", "output_shape"),
    "BatchNormalization": ("epsilon", "center", "scale", "axis"),
    "LayerNormalization": ("epsilon", "center", "scale", "axis"),
    "RMSNormalization": ("epsilon", "axis"),
    "Rescaling": ("scale", "offset"),
    "Normalization": ("axis",),
    "MaxPooling1D": _POOL_KEYS, "MaxPooling2D": _POOL_KEYS, "AveragePooling1D": _POOL_KEYS, "AveragePooling2D": _POOL_KEYS,
    "ZeroPadding1D": ("padding",), "ZeroPadding2D": ("padding",),
    "Cropping1D": ("cropping",), "Cropping2D": ("cropping",),
    "UpSampling1D": ("size",), "UpSampling2D": ("size", "interpolation"),
    "Permute": ("dims",), "Reshape": ("target_shape",), "Concatenate": ("axis",),
    "Embedding": ("input_dim", "output_dim"),
    "MultiHeadAttention": ("num_heads", "key_dim", "value_dim", "use_bias"),
    "GroupQueryAttention": ("head_dim", "num_query_heads", "num_key_value_heads", "use_bias"),
    "GroupedQueryAttention": ("head_dim", "num_query_heads", "num_key_value_heads", "use_bias"),
    "Activation": ("activation",),
}

NO_CONFIG_NEEDED = {
    "Add", "Multiply", "Subtract", "Average", "Maximum", "Minimum", "Flatten", "PReLU", "GlobalAveragePooling1D",
    "GlobalAveragePooling2D", "GlobalMaxPooling1D", "GlobalMaxPooling2D",
}

SUPPORTED = set(REQUIRED_CONFIG) | NO_CONFIG_NEEDED | IDENTITY | ACTIVATION_LAYERS | {"InputLayer", "Functional", "Model"}


def _float_count(chunks):
    """Number of fp32 values in a parameter (base64 chunks, keras_export/convert_model.py:190-192); None if not decodable."""
    if not isinstance(chunks, list) or not all(isinstance(c, str) for c in chunks):
        return None
    try:
        raw = base64.b64decode("".join(chunks), validate=True)
    except Exception:
        return None
    return len(raw) // 4 if len(raw) % 4 == 0 else None


def _pair(v):
    if isinstance(v, (int, float)):
        return 1, int(v)
    if isinstance(v, list) and len(v) == 1:
        return 1, int(v[0])
    return int(v[0]), int(v[1])


class _Walk:
    def __init__(self, params):
        self.params = params
        self.out = []

    def add(self, where, what):
        self.out.append("%s: %s" % (where, what))

    def count(self, where, owner, key, need=True):
        entry = self.params.get(owner)
        if not isinstance(entry, dict) or key not in entry:
            if need:
                self.add(where, "parameter '%s' missing under trainable_params['%s']" % (key, owner))
            return None
        n = _float_count(entry[key])
        if n is None:
            self.add(where, "parameter '%s' is not a list of base64 fp32 chunks" % key)
        elif any(len(c) > 1024 for c in entry[key]):
            self.add(where, "parameter '%s' has a chunk longer than 1024 characters" % key)
        return n

    def connections(self, where, node_list, known):
        """keras_history triples anywhere inside inbound_nodes (import_model.hpp:362-372, 1722-1740)."""
        def visit(v):
            if isinstance(v, dict):
                hist = v.get("config", {}).get("keras_history") if isinstance(v.get("config"), dict) else None
                if hist is not None:
                    if not (isinstance(hist, list) and len(hist) == 3 and isinstance(hist[0], str)):
                        self.add(where, "malformed keras_history %r" % (hist,))
                    elif hist[0] not in known:
                        self.add(where, "inbound layer '%s' does not exist" % hist[0])
                for x in v.values():
                    visit(x)
            elif isinstance(v, list):
                for x in v:
                    visit(x)
        visit(node_list)

    def endpoints(self, where, value, known):
        if isinstance(value, list) and len(value) == 3 and isinstance(value[0], str):
            value = [value]  # flat triple (import_model.hpp:352-360)
        if not isinstance(value, list) or not value:
            self.add(where, "must list at least one [layer, node, tensor] triple")
            return
        for t in value:
            if not (isinstance(t, list) and len(t) == 3 and isinstance(t[0], str)):
                self.add(where, "malformed entry %r" % (t,))
            elif t[0] not in known:
                self.add(where, "names unknown layer '%s'" % t[0])

    def model(self, where, cfg, prefix):
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            self.add(where, "config.layers must be a non-empty list")
            return
        names = [l.get("name") for l in layers if isinstance(l, dict)]
        known = set(n for n in names if isinstance(n, str))
        for n in known:
            if names.count(n) > 1:
                self.add(where, "layer name '%s' is used more than once" % n)
        for l in layers:
            if not isinstance(l, dict) or not isinstance(l.get("name"), str) or not isinstance(l.get("class_name"), str):
                self.add(where, "layer without name / class_name: %r" % (l,))
                continue
            self.layer("%s layer '%s' (%s)" % (where, l["name"], l["class_name"]), l, prefix, known)
        self.endpoints(where + " input_layers", cfg.get("input_layers"), known)
        self.endpoints(where + " output_layers", cfg.get("output_layers"), known)

    def layer(self, where, l, prefix, known):
        cls, name, cfg = l["class_name"], l["name"], l.get("config")
        owner = prefix + name
        if not isinstance(cfg, dict):
            self.add(where, "config missing")
            return
        if cls == "InputLayer":
            if l.get("inbound_nodes"):
                self.add(where, "an input layer must not have inbound nodes")
            if not isinstance(cfg.get("batch_shape", cfg.get("batch_input_shape")), list):
                self.add(where, "batch_shape missing")
            return
        if not l.get("inbound_nodes"):
            self.add(where, "no inbound nodes: the layer is never applied")
        self.connections(where, l.get("inbound_nodes"), known)
        if cls in ("Functional", "Model"):
            self.model(where, cfg, owner + "_")
            return
        if cls not in SUPPORTED:
            self.add(where, "class is not run on the device; register a custom layer creator for it")
            return
        for key in REQUIRED_CONFIG.get(cls, ()):
            if key not in cfg:
                self.add(where, "config key '%s' missing" % key)
                return
        act = cfg.get("activation")
        if cls != "Activation" and isinstance(act, dict):  # serialized activation object
            act = act.get("config", {}).get("name") if isinstance(act.get("config"), dict) else act.get("class_name")
        if isinstance(act, str) and act not in ACTIVATIONS:
            self.add(where, "activation '%s' is not known" % act)
        try:
            self.params_of(where, cls, cfg, owner)
        except (TypeError, ValueError, IndexError, KeyError) as e:
            self.add(where, "config not understood (%s: %s)" % (type(e).__name__, e))

    def params_of(self, where, cls, cfg, owner):
        if cls in ("Conv1D", "Conv2D", "Conv1DTranspose", "Conv2DTranspose"):
            kh, kw = _pair(cfg["kernel_size"])
            n = self.count(where, owner, "weights")
            if n is not None and (n == 0 or n % (kh * kw * int(cfg["filters"])) != 0):
                self.add(where, "%d weights do not divide into filters x kernel_size" % n)
            self.bias(where, owner, cfg, int(cfg["filters"]))
            if cfg["padding"] not in ("valid", "same", "causal"):
                self.add(where, "padding '%s' is not valid / same / causal" % cfg["padding"])
            if cls.endswith("Transpose") and cfg["padding"] == "causal":
                self.add(where, "a transposed convolution cannot use causal padding")
        elif cls in ("DepthwiseConv1D", "DepthwiseConv2D"):
            kh, kw = _pair(cfg["kernel_size"])
            n = self.count(where, owner, "slice_weights")
            if n is not None and (n == 0 or n % (kh * kw) != 0):
                self.add(where, "%d slice_weights do not divide into kernel_size" % n)
            if n:
                self.bias(where, owner, cfg, n // (kh * kw))
            if int(cfg.get("depth_multiplier", 1)) != 1:
                self.add(where, "depth_multiplier other than 1 is not supported")
        elif cls in ("SeparableConv1D", "SeparableConv2D"):
            kh, kw = _pair(cfg["kernel_size"])
            n = self.count(where, owner, "slice_weights")
            s = self.count(where, owner, "stack_weights")
            if n is not None and s is not None and n % (kh * kw) == 0 and s != (n // (kh * kw)) * int(cfg["filters"]):
                self.add(where, "stack_weights (%d) do not match depth x filters" % s)
            self.bias(where, owner, cfg, int(cfg["filters"]))
        elif cls == "Dense":
            n = self.count(where, owner, "weights")
            if n is not None and (n == 0 or n % int(cfg["units"]) != 0):
                self.add(where, "%d weights do not divide by units" % n)
            self.bias(where, owner, cfg, int(cfg["units"]))
        elif cls == "BatchNormalization":
            m, v = self.count(where, owner, "moving_mean"), self.count(where, owner, "moving_variance")
            if m is not None and v is not None and m != v:
                self.add(where, "moving_mean and moving_variance differ in length")
            for key, flag in (("gamma", "scale"), ("beta", "center")):
                g = self.count(where, owner, key, need=bool(cfg[flag]))
                if g is not None and m is not None and cfg[flag] and g != m:
                    self.add(where, "%s has %d values, moving_mean %d" % (key, g, m))
        elif cls == "Normalization":
            m, v = self.count(where, owner, "mean"), self.count(where, owner, "variance")
            if m is not None and v is not None and m != v:
                self.add(where, "mean and variance differ in length")
            ax = cfg["axis"]
            n_axes = len(ax) if isinstance(ax, (list, tuple)) else (0 if ax is None else 1)
            if n_axes > 1:
                self.add(where, "more than one Normalization axis")
            if n_axes == 0 and v is not None and v != 1:
                self.add(where, "axis-less Normalization needs exactly one mean / variance")
        elif cls == "LayerNormalization":
            for key, flag in (("gamma", "scale"), ("beta", "center")):
                self.count(where, owner, key, need=bool(cfg[flag]))
        elif cls == "RMSNormalization":
            self.count(where, owner, "scale")
        elif cls == "PReLU":
            self.count(where, owner, "alpha")
        elif cls == "Embedding":
            n = self.count(where, owner, "weights")
            if n is not None and n != int(cfg["input_dim"]) * int(cfg["output_dim"]):
                self.add(where, "%d weights, input_dim x output_dim is %d" % (n, int(cfg["input_dim"]) * int(cfg["output_dim"])))
        elif cls == "EinsumDense":
            self.count(where, owner, "kernel")
            if cfg.get("bias_axes"):
                self.count(where, owner, "bias")
            if "->" not in cfg["equation"] or "," not in cfg["equation"]:
                self.add(where, "equation '%s' is not of the form 'in,kernel->out'" % cfg["equation"])
        elif cls in ("MultiHeadAttention", "GroupQueryAttention", "GroupedQueryAttention"):
            entry = self.params.get(owner)
            if not isinstance(entry, dict) or "weights" not in entry:
                self.add(where, "parameter 'weights' missing under trainable_params['%s']" % owner)
                return
            if cls == "MultiHeadAttention":
                expected = 8 if cfg["use_bias"] else 4
            else:
                expected = (4 + (1 if cfg.get("use_gate") else 0)) * (2 if cfg["use_bias"] else 1)
            w = entry["weights"]
            if not isinstance(w, list) or len(w) != expected:
                self.add(where, "expected %d weight arrays, found %s" % (expected, len(w) if isinstance(w, list) else "none"))
            elif any(_float_count(x) is None for x in w):
                self.add(where, "weights hold an entry that is not a list of base64 fp32 chunks")
        elif cls in ("MaxPooling1D", "MaxPooling2D", "AveragePooling1D", "AveragePooling2D"):
            if cfg["padding"] not in ("valid", "same"):
                self.add(where, "padding '%s' is not valid / same" % cfg["padding"])
        elif cls == "UpSampling2D":
            if cfg["interpolation"] not in ("nearest", "bilinear"):
                self.add(where, "interpolation '%s' is not nearest / bilinear" % cfg["interpolation"])

    def bias(self, where, owner, cfg, expected):
        if cfg["use_bias"]:
            n = self.count(where, owner, "bias")
            if n is not None and n != expected:
                self.add(where, "bias has %d values, expected %d" % (n, expected))


def problems(model):
    """List of findings (empty = the file should load); `model` is the JSON text, bytes, or the parsed dict."""
    if isinstance(model, (bytes, bytearray)):
        model = model.decode("utf-8")
    if isinstance(model, str):
        try:
            model = json.loads(model)
        except ValueError as e:
            return ["file: not valid JSON (%s)" % e]
    if not isinstance(model, dict):
        return ["file: top level must be an object"]
    w = _Walk(model.get("trainable_params") if isinstance(model.get("trainable_params"), dict) else {})
    if model.get("image_data_format") != "channels_last":
        w.add("file", "image_data_format must be 'channels_last' (model.hpp:231-233)")
    for key in ("input_shapes", "output_shapes"):
        v = model.get(key)
        if not (isinstance(v, list) and v and all(isinstance(s, list) and 1 <= len(s) <= 5 for s in v)):
            w.add("file", "%s must be a non-empty list of shapes of rank 1..5" % key)
    if "trainable_params" in model and not isinstance(model["trainable_params"], dict):
        w.add("file", "trainable_params must be an object")
    arch = model.get("architecture")
    if not isinstance(arch, dict) or not isinstance(arch.get("config"), dict):
        w.add("file", "architecture.config missing")
        return w.out
    if arch.get("class_name") not in ("Functional", "Model", "Sequential"):
        w.add("file", "architecture.class_name '%s' is not a model class" % arch.get("class_name"))
    if arch.get("class_name") == "Sequential":
        w.add("file", "Sequential models must be converted to functional form by the exporter first")
        return w.out
    w.model("model", arch["config"], "")
    n_in, n_out = arch["config"].get("input_layers"), arch["config"].get("output_layers")

    def count(v):
        return 1 if isinstance(v, list) and len(v) == 3 and isinstance(v[0], str) else len(v) if isinstance(v, list) else 0
    if isinstance(model.get("input_shapes"), list) and count(n_in) != len(model["input_shapes"]):
        w.add("file", "%d input_shapes for %d input layers" % (len(model["input_shapes"]), count(n_in)))
    if isinstance(model.get("output_shapes"), list) and count(n_out) != len(model["output_shapes"]):
        w.add("file", "%d output_shapes for %d output layers" % (len(model["output_shapes"]), count(n_out)))
    return w.out
