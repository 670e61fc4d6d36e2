"""StableHLO module text for the windowed ops next to the hot path, in the forms the reference prints
them: `stablehlo.reduce_window` (generic form; built by src/Ops.jl:3967-4011 for pooling,
ext/ReactantNNlibExt/Ops.jl:1-32, and for cumsum/cumprod, src/TracedRArray.jl:1086-1108),
`stablehlo.convolution` (src/Ops.jl:1000-1073), `stablehlo.reverse` (kernel flip,
ext/ReactantNNlibExt/Implementations.jl:53-55), batch norm, the argmax reduce and gather.  Like
programs.py this stands in for the tracing front end: tests and the benchmark feed these modules to
the backend."""

INIT = {("add", True): "0.000000e+00", ("multiply", True): "1.000000e+00", ("maximum", True): "0xFF800000",
        ("minimum", True): "0x7F800000", ("add", False): "0", ("multiply", False): "1"}


def tt(shape, dt):
    return "tensor<" + "".join("%dx" % d for d in shape) + dt + ">"


def _init_literal(body, dt):
    if dt.startswith("f") or dt == "bf16":
        if body == "maximum":
            return {"f64": "0xFFF0000000000000", "f32": "0xFF800000", "bf16": "0xFF80", "f16": "0xFC00"}[dt]
        if body == "minimum":
            return {"f64": "0x7FF0000000000000", "f32": "0x7F800000", "bf16": "0x7F80", "f16": "0x7C00"}[dt]
        return INIT[(body, True)]
    if body == "maximum":
        return {"i32": "-2147483648", "i64": "-9223372036854775808"}[dt]
    if body == "minimum":
        return {"i32": "2147483647", "i64": "9223372036854775807"}[dt]
    return INIT[(body, False)]


def window_out_shape(shape, window, strides, padding, base_dil, win_dil):
    out = []
    for d, n in enumerate(shape):
        dil = n + max(n - 1, 0) * (base_dil[d] - 1)
        padded = dil + padding[d][0] + padding[d][1]
        span = (window[d] - 1) * win_dil[d] + 1
        out.append(0 if padded < span else (padded - span) // strides[d] + 1)
    return out


def reduce_window(shape, dt, body, window, strides=None, padding=None, base_dil=None, win_dil=None):
    r = len(shape)
    strides = strides or [1] * r
    padding = padding or [[0, 0]] * r
    base_dil = base_dil or [1] * r
    win_dil = win_dil or [1] * r
    out = window_out_shape(shape, window, strides, padding, base_dil, win_dil)
    arr = lambda v: "array<i64: " + ", ".join(str(x) for x in v) + ">"
    pad = "dense<[" + ", ".join("[%d, %d]" % (p[0], p[1]) for p in padding) + "]> : tensor<%dx2xi64>" % r
    ti, to, ts = tt(shape, dt), tt(out, dt), tt([], dt)
    return ("module {\n  func.func @main(%%arg0: %s) -> %s {\n"
            "    %%cst = stablehlo.constant dense<%s> : %s\n"
            "    %%0 = \"stablehlo.reduce_window\"(%%arg0, %%cst) <{base_dilations = %s, padding = %s, "
            "window_dilations = %s, window_dimensions = %s, window_strides = %s}> ({\n"
            "    ^bb0(%%arg1: %s, %%arg2: %s):\n"
            "      %%1 = stablehlo.%s %%arg1, %%arg2 : %s\n"
            "      stablehlo.return %%1 : %s\n"
            "    }) : (%s, %s) -> %s\n"
            "    return %%0 : %s\n  }\n}\n"
            % (ti, to, _init_literal(body, dt), ts, arr(base_dil), pad, arr(win_dil), arr(window), arr(strides),
               ts, ts, body, ts, ts, ti, ts, to, to)), out


def cumulative(shape, dt, dim, body="add", reverse=False):
    """What Base.cumsum / cumprod of a traced array print (src/TracedRArray.jl:1086-1108)."""
    r = len(shape)
    window = [1] * r
    window[dim] = shape[dim]
    padding = [[0, 0] for _ in range(r)]
    padding[dim] = [0, shape[dim] - 1] if reverse else [shape[dim] - 1, 0]
    return reduce_window(shape, dt, body, window, padding=padding)[0]


def conv_out_shape(x_sp, k_sp, strides, padding, lhs_dil, rhs_dil):
    out = []
    for d, n in enumerate(x_sp):
        dil = n + max(n - 1, 0) * (lhs_dil[d] - 1)
        padded = dil + padding[d][0] + padding[d][1]
        span = (k_sp[d] - 1) * rhs_dil[d] + 1
        out.append(0 if padded < span else (padded - span) // strides[d] + 1)
    return out


def convolution(x_shape, w_shape, dt, dims="[b, f, 1, 0]x[o, i, 1, 0]->[b, f, 1, 0]", strides=None, padding=None,
                lhs_dil=None, rhs_dil=None, groups=1, flip=False, generic=False, epilogue=None, batch_groups=1):
    """`dims` uses the textual dimension numbers; spatial dim s of the input has the size
    x_shape[position of s].  With `flip` the kernel's spatial dims are reversed first (NNlib's true
    convolution).  `epilogue="bias_relu"` adds a per-feature bias and a relu, the fused form LuxLib emits."""
    import re
    groups_txt = re.findall(r"\[([^\]]*)\]", dims)
    pos = []
    for gtxt in groups_txt:
        toks = [t.strip() for t in gtxt.split(",")]
        pos.append({t: k for k, t in enumerate(toks)})
    nsp = len(x_shape) - 2
    strides = strides or [1] * nsp
    padding = padding or [[0, 0]] * nsp
    lhs_dil = lhs_dil or [1] * nsp
    rhs_dil = rhs_dil or [1] * nsp
    x_sp = [x_shape[pos[0][str(s)]] for s in range(nsp)]
    k_sp = [w_shape[pos[1][str(s)]] for s in range(nsp)]
    o_sp = conv_out_shape(x_sp, k_sp, strides, padding, lhs_dil, rhs_dil)
    out = [0] * len(x_shape)
    out[pos[2]["b"]] = x_shape[pos[0]["b"]] // batch_groups
    out[pos[2]["f"]] = w_shape[pos[1]["o"]]
    for s in range(nsp):
        out[pos[2][str(s)]] = o_sp[s]
    tx, tw, to = tt(x_shape, dt), tt(w_shape, dt), tt(out, dt)
    lst = lambda v: "[" + ", ".join(str(x) for x in v) + "]"
    body = ""
    wname = "%arg1"
    if flip:
        rd = sorted(pos[1][str(s)] for s in range(nsp))
        body += "    %%w = stablehlo.reverse %%arg1, dims = %s : %s\n" % (lst(rd), tw)
        wname = "%w"
    if generic:
        arr = lambda v: "array<i64: " + ", ".join(str(x) for x in v) + ">"
        pad = "dense<[" + ", ".join("[%d, %d]" % (p[0], p[1]) for p in padding) + "]> : tensor<%dx2xi64>" % nsp
        body += ("    %%0 = \"stablehlo.convolution\"(%%arg0, %s) <{batch_group_count = %d : i64, dimension_numbers = "
                 "#stablehlo.conv<%s>, feature_group_count = %d : i64, lhs_dilation = %s, padding = %s, "
                 "precision_config = [#stablehlo<precision DEFAULT>, #stablehlo<precision DEFAULT>], rhs_dilation = %s, "
                 "window_strides = %s}> : (%s, %s) -> %s\n"
                 % (wname, batch_groups, dims, groups, arr(lhs_dil), pad, arr(rhs_dil), arr(strides), tx, tw, to))
    else:
        body += ("    %%0 = stablehlo.convolution(%%arg0, %s) dim_numbers = %s, window = {stride = %s, pad = %s, "
                 "lhs_dilate = %s, rhs_dilate = %s} {batch_group_count = %d : i64, feature_group_count = %d : i64, "
                 "precision_config = [#stablehlo<precision DEFAULT>, #stablehlo<precision DEFAULT>]} : (%s, %s) -> %s\n"
                 % (wname, dims, lst(strides), "[" + ", ".join(lst(p) for p in padding) + "]", lst(lhs_dil), lst(rhs_dil),
                    batch_groups, groups, tx, tw, to))
    args = "%%arg0: %s, %%arg1: %s" % (tx, tw)
    res = "%0"
    if epilogue == "bias_relu":
        nf = out[pos[2]["f"]]
        tb = tt([nf], dt)
        args += ", %%arg2: %s" % tb
        body += "    %%b = stablehlo.broadcast_in_dim %%arg2, dims = [%d] : (%s) -> %s\n" % (pos[2]["f"], tb, to)
        body += "    %%1 = stablehlo.add %%0, %%b : %s\n" % to
        body += "    %%z = stablehlo.constant dense<0.000000e+00> : %s\n" % to
        body += "    %%2 = stablehlo.maximum %%1, %%z : %s\n" % to
        res = "%2"
    return ("module {\n  func.func @main(%s) -> %s {\n%s    return %s : %s\n  }\n}\n" % (args, to, body, res, to)), out


def conv_chain(batch, channels, hw, layers, dt, k=3):
    """`layers` k x k convolutions (padding k // 2, unit strides) of `channels` -> `channels` features on `batch` images of
    hw x hw, each followed by a per-feature bias and a relu (the body of a VGG block as LuxLib fuses it); arguments: the
    images [batch, channels, hw, hw], then a filter [channels, channels, k, k] and a bias [channels] per layer."""
    t = tt([batch, channels, hw, hw], dt)
    tw = tt([channels, channels, k, k], dt)
    tb = tt([channels], dt)
    args = ["%%arg0: %s" % t]
    body = ""
    cur = "%arg0"
    for l in range(layers):
        w, b = "%%arg%d" % (1 + 2 * l), "%%arg%d" % (2 + 2 * l)
        args += ["%s: %s" % (w, tw), "%s: %s" % (b, tb)]
        body += ("    %%c%d = stablehlo.convolution(%s, %s) dim_numbers = [b, f, 1, 0]x[o, i, 1, 0]->[b, f, 1, 0], window = {stride = [1, 1], "
                 "pad = [[%d, %d], [%d, %d]], lhs_dilate = [1, 1], rhs_dilate = [1, 1]} {batch_group_count = 1 : i64, feature_group_count = 1 : i64, "
                 "precision_config = [#stablehlo<precision DEFAULT>, #stablehlo<precision DEFAULT>]} : (%s, %s) -> %s\n"
                 % (l, cur, w, k // 2, k // 2, k // 2, k // 2, t, tw, t))
        body += "    %%b%d = stablehlo.broadcast_in_dim %s, dims = [1] : (%s) -> %s\n" % (l, b, tb, t)
        body += "    %%a%d = stablehlo.add %%c%d, %%b%d : %s\n" % (l, l, l, t)
        body += "    %%z%d = stablehlo.constant dense<0.000000e+00> : %s\n" % (l, t)
        body += "    %%r%d = stablehlo.maximum %%a%d, %%z%d : %s\n" % (l, l, l, t)
        cur = "%%r%d" % l
    shapes = [[batch, channels, hw, hw]] + [[channels, channels, k, k], [channels]] * layers
    return ("module {\n  func.func @main(%s) -> %s {\n%s    return %s : %s\n  }\n}\n" % (", ".join(args), t, body, cur, t)), shapes


def batch_norm(shape, dt, feature_index, epsilon=1e-5, training=False):
    """`stablehlo.batch_norm_inference` / `batch_norm_training` in the generic form they print in
    (built by the reference's src/Ops.jl:4012-4092)."""
    tx, tf = tt(shape, dt), tt([shape[feature_index]], dt)
    if training:
        return ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s, %%arg2: %s) -> (%s, %s, %s) {\n"
                "    %%0:3 = \"stablehlo.batch_norm_training\"(%%arg0, %%arg1, %%arg2) <{epsilon = %e : f32, feature_index = %d : i64}> : "
                "(%s, %s, %s) -> (%s, %s, %s)\n    return %%0#0, %%0#1, %%0#2 : %s, %s, %s\n  }\n}\n"
                % (tx, tf, tf, tx, tf, tf, epsilon, feature_index, tx, tf, tf, tx, tf, tf, tx, tf, tf))
    return ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s, %%arg2: %s, %%arg3: %s, %%arg4: %s) -> %s {\n"
            "    %%0 = \"stablehlo.batch_norm_inference\"(%%arg0, %%arg1, %%arg2, %%arg3, %%arg4) <{epsilon = %e : f32, feature_index = %d : i64}> : "
            "(%s, %s, %s, %s, %s) -> %s\n    return %%0 : %s\n  }\n}\n"
            % (tx, tf, tf, tf, tf, tx, epsilon, feature_index, tx, tf, tf, tf, tf, tx, tx))


def vgg_block(batch=2, cin=3, cmid=8, hw=16, classes=10, dt="f32"):
    """conv3x3(pad 1) + batch norm (inference) + relu + maxpool 2x2 + conv3x3 + bias + relu +
    global mean pool + dense + softmax: the op sequence of the VGG forward pass of
    benchmark/nn/vision.jl:24-34 at toy sizes.  Arguments: x, w1, bn scale/offset/mean/var, w2, b2, wd, bd."""
    h2 = hw // 2
    X, W1, F1 = tt([batch, cin, hw, hw], dt), tt([cmid, cin, 3, 3], dt), tt([cmid], dt)
    A1 = tt([batch, cmid, hw, hw], dt)
    P1 = tt([batch, cmid, h2, h2], dt)
    W2, F2 = tt([2 * cmid, cmid, 3, 3], dt), tt([2 * cmid], dt)
    A2 = tt([batch, 2 * cmid, h2, h2], dt)
    G, WD, BD, OUT, S = tt([batch, 2 * cmid], dt), tt([2 * cmid, classes], dt), tt([classes], dt), tt([batch, classes], dt), tt([], dt)
    R = tt([batch], dt)
    conv = ("stablehlo.convolution(%s, %s) dim_numbers = [b, f, 1, 0]x[o, i, 1, 0]->[b, f, 1, 0], window = {stride = [1, 1], "
            "pad = [[1, 1], [1, 1]], rhs_dilate = [1, 1]} {batch_group_count = 1 : i64, feature_group_count = 1 : i64} : (%s, %s) -> %s")
    pool = ("\"stablehlo.reduce_window\"(%s, %s) <{base_dilations = array<i64: 1, 1, 1, 1>, padding = dense<0> : tensor<4x2xi64>, "
            "window_dilations = array<i64: 1, 1, 1, 1>, window_dimensions = array<i64: 1, 1, 2, 2>, window_strides = array<i64: 1, 1, 2, 2>}> ({\n"
            "    ^bb0(%%p: %s, %%q: %s):\n      %%m = stablehlo.maximum %%p, %%q : %s\n      stablehlo.return %%m : %s\n    }) : (%s, %s) -> %s")
    lines = [
        "%c1 = " + conv % ("%arg0", "%arg1", X, W1, A1),
        "%bn = \"stablehlo.batch_norm_inference\"(%c1, %arg2, %arg3, %arg4, %arg5) <{epsilon = 1.000000e-05 : f32, feature_index = 1 : i64}> : "
        "(" + ", ".join([A1, F1, F1, F1, F1]) + ") -> " + A1,
        "%z1 = stablehlo.constant dense<0.000000e+00> : " + A1,
        "%r1 = stablehlo.maximum %bn, %z1 : " + A1,
        "%ninf = stablehlo.constant dense<" + _init_literal("maximum", dt) + "> : " + S,
        "%p1 = " + pool % ("%r1", "%ninf", S, S, S, S, A1, S, P1),
        "%c2 = " + conv % ("%p1", "%arg6", P1, W2, A2),
        "%b2 = stablehlo.broadcast_in_dim %arg7, dims = [1] : (" + F2 + ") -> " + A2,
        "%a2 = stablehlo.add %c2, %b2 : " + A2,
        "%z2 = stablehlo.constant dense<0.000000e+00> : " + A2,
        "%r2 = stablehlo.maximum %a2, %z2 : " + A2,
        "%zero = stablehlo.constant dense<0.000000e+00> : " + S,
        "%gs = stablehlo.reduce(%r2 init: %zero) applies stablehlo.add across dimensions = [2, 3] : (" + A2 + ", " + S + ") -> " + G,
        "%cnt = stablehlo.constant dense<" + "%.6e" % float(h2 * h2) + "> : " + G,
        "%gm = stablehlo.divide %gs, %cnt : " + G,
        "%d = stablehlo.dot_general %gm, %arg8, contracting_dims = [1] x [0] : (" + G + ", " + WD + ") -> " + OUT,
        "%bd = stablehlo.broadcast_in_dim %arg9, dims = [1] : (" + BD + ") -> " + OUT,
        "%lg = stablehlo.add %d, %bd : " + OUT,
        "%mx = stablehlo.reduce(%lg init: %ninf) applies stablehlo.maximum across dimensions = [1] : (" + OUT + ", " + S + ") -> " + R,
        "%mxb = stablehlo.broadcast_in_dim %mx, dims = [0] : (" + R + ") -> " + OUT,
        "%sh = stablehlo.subtract %lg, %mxb : " + OUT,
        "%ex = stablehlo.exponential %sh : " + OUT,
        "%sm = stablehlo.reduce(%ex init: %zero) applies stablehlo.add across dimensions = [1] : (" + OUT + ", " + S + ") -> " + R,
        "%smb = stablehlo.broadcast_in_dim %sm, dims = [0] : (" + R + ") -> " + OUT,
        "%out = stablehlo.divide %ex, %smb : " + OUT,
    ]
    args = [X, W1, F1, F1, F1, F1, W2, F2, WD, BD]
    sig = ", ".join("%%arg%d: %s" % (k, t) for k, t in enumerate(args))
    shapes = [[batch, cin, hw, hw], [cmid, cin, 3, 3], [cmid], [cmid], [cmid], [cmid], [2 * cmid, cmid, 3, 3], [2 * cmid],
              [2 * cmid, classes], [classes]]
    return ("module {\n  func.func @main(%s) -> %s {\n    %s\n    return %%out : %s\n  }\n}\n" % (sig, OUT, "\n    ".join(lines), OUT)), shapes


VGG11_LAYERS = (64, "M", 128, "M", 256, 256, "M", 512, 512, "M", 512, 512, "M")


def vgg11(batch=4, hw=224, classes=1000, dt="f32", layers=VGG11_LAYERS, dense=4096, cin=3):
    """Forward pass of VGG-11 with batch norm in test mode, the model of benchmark/nn/vision.jl:24-34
    (`Vision.VGG(11; batchnorm=true)` on [224, 224, 3, 4]): per entry of `layers` a 3x3 convolution (padding 1, no bias) +
    batch_norm_inference + relu, or ("M") a 2x2 max pool; then flatten, two dense layers of `dense` features with relu and
    one of `classes` (logits).  Arguments: the images [batch, cin, hw, hw]; per convolution its filter and the batch
    norm's scale, offset, mean, variance; per dense layer its matrix [in, out] and its bias."""
    S = tt([], dt)
    conv = ("stablehlo.convolution(%s, %s) dim_numbers = [b, f, 1, 0]x[o, i, 1, 0]->[b, f, 1, 0], window = {stride = [1, 1], "
            "pad = [[1, 1], [1, 1]], rhs_dilate = [1, 1]} {batch_group_count = 1 : i64, feature_group_count = 1 : i64} : (%s, %s) -> %s")
    pool = ("\"stablehlo.reduce_window\"(%s, %%ninf) <{base_dilations = array<i64: 1, 1, 1, 1>, padding = dense<0> : tensor<4x2xi64>, "
            "window_dilations = array<i64: 1, 1, 1, 1>, window_dimensions = array<i64: 1, 1, 2, 2>, window_strides = array<i64: 1, 1, 2, 2>}> ({\n"
            "    ^bb0(%%p: %s, %%q: %s):\n      %%m = stablehlo.maximum %%p, %%q : %s\n      stablehlo.return %%m : %s\n    }) : (%s, %s) -> %s")
    lines = ["%ninf = stablehlo.constant dense<" + _init_literal("maximum", dt) + "> : " + S]
    args, shapes = [tt([batch, cin, hw, hw], dt)], [[batch, cin, hw, hw]]
    cur, c, h, flops = "%arg0", cin, hw, 0.0
    for k, l in enumerate(layers):
        T = tt([batch, c, h, h], dt)
        if l == "M":
            P = tt([batch, c, h // 2, h // 2], dt)
            lines.append("%%l%d = " % k + pool % (cur, S, S, S, S, T, S, P))
            h //= 2
        else:
            A, F = tt([batch, l, h, h], dt), tt([l], dt)
            a = len(args)
            args += [tt([l, c, 3, 3], dt), F, F, F, F]
            shapes += [[l, c, 3, 3], [l], [l], [l], [l]]
            lines.append("%%c%d = " % k + conv % (cur, "%%arg%d" % a, T, tt([l, c, 3, 3], dt), A))
            lines.append("%%n%d = \"stablehlo.batch_norm_inference\"(%%c%d, %%arg%d, %%arg%d, %%arg%d, %%arg%d) <{epsilon = 1.000000e-05 : f32, feature_index = 1 : i64}> : (%s) -> %s"
                         % (k, k, a + 1, a + 2, a + 3, a + 4, ", ".join([A, F, F, F, F]), A))
            lines.append("%%z%d = stablehlo.constant dense<0.000000e+00> : %s" % (k, A))
            lines.append("%%l%d = stablehlo.maximum %%n%d, %%z%d : %s" % (k, k, k, A))
            flops += 2.0 * batch * l * h * h * c * 9
            c = l
        cur = "%%l%d" % k
    feat = c * h * h
    lines.append("%%f = stablehlo.reshape %s : (%s) -> %s" % (cur, tt([batch, c, h, h], dt), tt([batch, feat], dt)))
    cur = "%f"
    for k, n in enumerate((dense, dense, classes)):
        X, W, Bv, O = tt([batch, feat], dt), tt([feat, n], dt), tt([n], dt), tt([batch, n], dt)
        a = len(args)
        args += [W, Bv]
        shapes += [[feat, n], [n]]
        lines.append("%%d%d = stablehlo.dot_general %s, %%arg%d, contracting_dims = [1] x [0] : (%s, %s) -> %s" % (k, cur, a, X, W, O))
        lines.append("%%bb%d = stablehlo.broadcast_in_dim %%arg%d, dims = [1] : (%s) -> %s" % (k, a + 1, Bv, O))
        lines.append("%%s%d = stablehlo.add %%d%d, %%bb%d : %s" % (k, k, k, O))
        cur = "%%s%d" % k
        if k < 2:
            lines.append("%%dz%d = stablehlo.constant dense<0.000000e+00> : %s" % (k, O))
            lines.append("%%e%d = stablehlo.maximum %%s%d, %%dz%d : %s" % (k, k, k, O))
            cur = "%%e%d" % k
        flops += 2.0 * batch * feat * n
        feat = n
    OUT = tt([batch, classes], dt)
    sig = ", ".join("%%arg%d: %s" % (k, t) for k, t in enumerate(args))
    text = "module {\n  func.func @main(%s) -> %s {\n    %s\n    return %s : %s\n  }\n}\n" % (sig, OUT, "\n    ".join(lines), cur, OUT)
    return text, shapes, flops


def resnet_stage(batch=2, channels=64, hw=16, blocks=2, dt="f32"):
    """`blocks` basic residual blocks on `batch` images of `channels` x hw x hw: 3x3 convolution (padding 1) + batch
    norm (test mode) + relu + 3x3 convolution + batch norm, the block's input added, relu (the identity blocks of a
    ResNet stage as Lux / Boltz build them).  Arguments: the images, then per block the two filters, each followed
    by its batch norm's scale, offset, mean, variance.  Returns (text, shapes, flops)."""
    T, W, F = tt([batch, channels, hw, hw], dt), tt([channels, channels, 3, 3], dt), tt([channels], dt)
    conv = ("stablehlo.convolution(%s, %s) dim_numbers = [b, f, 1, 0]x[o, i, 1, 0]->[b, f, 1, 0], window = {stride = [1, 1], "
            "pad = [[1, 1], [1, 1]], rhs_dilate = [1, 1]} {batch_group_count = 1 : i64, feature_group_count = 1 : i64} : (" + T + ", " + W + ") -> " + T)
    args, shapes, lines = [T], [[batch, channels, hw, hw]], ["%zero = stablehlo.constant dense<0.000000e+00> : " + T]
    cur = "%arg0"
    for b in range(blocks):
        inp = cur
        for half in range(2):
            a = len(args)
            args += [W, F, F, F, F]
            shapes += [[channels, channels, 3, 3]] + [[channels]] * 4
            k = "%d_%d" % (b, half)
            lines.append("%%c%s = " % k + conv % (cur, "%%arg%d" % a))
            lines.append("%%n%s = \"stablehlo.batch_norm_inference\"(%%c%s, %%arg%d, %%arg%d, %%arg%d, %%arg%d) <{epsilon = 1.000000e-05 : f32, feature_index = 1 : i64}> : (%s) -> %s"
                         % (k, k, a + 1, a + 2, a + 3, a + 4, ", ".join([T, F, F, F, F]), T))
            cur = "%%n%s" % k
            if half == 0:
                lines.append("%%r%s = stablehlo.maximum %s, %%zero : %s" % (k, cur, T))
                cur = "%%r%s" % k
        lines.append("%%s%d = stablehlo.add %s, %s : %s" % (b, cur, inp, T))
        lines.append("%%o%d = stablehlo.maximum %%s%d, %%zero : %s" % (b, b, T))
        cur = "%%o%d" % b
    sig = ", ".join("%%arg%d: %s" % (k, t) for k, t in enumerate(args))
    text = "module {\n  func.func @main(%s) -> %s {\n    %s\n    return %s : %s\n  }\n}\n" % (sig, T, "\n    ".join(lines), cur, T)
    return text, shapes, blocks * 2 * 2.0 * batch * channels * hw * hw * channels * 9


def attention_block(batch_heads=6, seq=40, dim=16, dt="f32"):
    """softmax(q k^T / sqrt(d)) v on [batch*heads, seq, dim] operands: the two batched products and the
    row softmax of NNlib.dot_product_attention, which the ViT of benchmark/nn/vision.jl:5-22 runs."""
    Q, SC, S, R = tt([batch_heads, seq, dim], dt), tt([batch_heads, seq, seq], dt), tt([], dt), tt([batch_heads, seq], dt)
    lines = [
        "%s0 = stablehlo.dot_general %arg0, %arg1, batching_dims = [0] x [0], contracting_dims = [2] x [2] : (" + Q + ", " + Q + ") -> " + SC,
        "%sc = stablehlo.constant dense<" + "%.9e" % (1.0 / dim ** 0.5) + "> : " + SC,
        "%s1 = stablehlo.multiply %s0, %sc : " + SC,
        "%ninf = stablehlo.constant dense<" + _init_literal("maximum", dt) + "> : " + S,
        "%zero = stablehlo.constant dense<0.000000e+00> : " + S,
        "%mx = stablehlo.reduce(%s1 init: %ninf) applies stablehlo.maximum across dimensions = [2] : (" + SC + ", " + S + ") -> " + R,
        "%mxb = stablehlo.broadcast_in_dim %mx, dims = [0, 1] : (" + R + ") -> " + SC,
        "%sh = stablehlo.subtract %s1, %mxb : " + SC,
        "%ex = stablehlo.exponential %sh : " + SC,
        "%sm = stablehlo.reduce(%ex init: %zero) applies stablehlo.add across dimensions = [2] : (" + SC + ", " + S + ") -> " + R,
        "%smb = stablehlo.broadcast_in_dim %sm, dims = [0, 1] : (" + R + ") -> " + SC,
        "%p = stablehlo.divide %ex, %smb : " + SC,
        "%out = stablehlo.dot_general %p, %arg2, batching_dims = [0] x [0], contracting_dims = [2] x [1] : (" + SC + ", " + Q + ") -> " + Q,
    ]
    sig = ", ".join("%%arg%d: %s" % (k, Q) for k in range(3))
    return ("module {\n  func.func @main(%s) -> %s {\n    %s\n    return %%out : %s\n  }\n}\n" % (sig, Q, "\n    ".join(lines), Q)), [[batch_heads, seq, dim]] * 3


def argreduce(shape, dt, dim, direction="GE", idt="i64", generic=False):
    """The variadic reduce that argmax / argmin / findmax print (reference src/Ops.jl:1571-1596):
    (value, index) pairs over `dim`, keeping the left pair when `a1 <direction> a2`.  Returns the
    module text; results are (values, zero-based indices)."""
    out = [s for d, s in enumerate(shape) if d != dim]
    tx, ti, tvo, tio = tt(shape, dt), tt(shape, idt), tt(out, dt), tt(out, idt)
    sv, si = tt([], dt), tt([], idt)
    vinit = _init_literal("maximum" if direction in ("GE", "GT") else "minimum", dt)
    if generic:
        red = ("    %%r:2 = \"stablehlo.reduce\"(%%arg0, %%io, %%cv, %%ci) <{dimensions = array<i64: %d>}> ({\n"
               "    ^bb0(%%a1: %s, %%i1: %s, %%a2: %s, %%i2: %s):\n" % (dim, sv, si, sv, si))
        tail = "    }) : (%s, %s, %s, %s) -> (%s, %s)\n" % (tx, ti, sv, si, tvo, tio)
    else:
        red = ("    %%r:2 = stablehlo.reduce(%%arg0 init: %%cv), (%%io init: %%ci) across dimensions = [%d] : (%s, %s, %s, %s) -> (%s, %s)\n"
               "     reducer(%%a1: %s, %%a2: %s) (%%i1: %s, %%i2: %s)  {\n" % (dim, tx, ti, sv, si, tvo, tio, sv, sv, si, si))
        tail = "    }\n"
    body = ("      %%c = stablehlo.compare %s, %%a1, %%a2 : (%s, %s) -> tensor<i1>\n"
            "      %%v = stablehlo.select %%c, %%a1, %%a2 : tensor<i1>, %s\n"
            "      %%i = stablehlo.select %%c, %%i1, %%i2 : tensor<i1>, %s\n"
            "      stablehlo.return %%v, %%i : %s, %s\n" % (direction, sv, sv, sv, si, sv, si))
    return ("module {\n  func.func @main(%%arg0: %s) -> (%s, %s) {\n"
            "    %%io = stablehlo.iota dim = %d : %s\n"
            "    %%cv = stablehlo.constant dense<%s> : %s\n"
            "    %%ci = stablehlo.constant dense<-1> : %s\n"
            "%s%s%s"
            "    return %%r#0, %%r#1 : %s, %s\n  }\n}\n"
            % (tx, tvo, tio, dim, ti, vinit, sv, si, red, body, tail, tvo, tio))


def gather(operand_shape, start_shape, out_shape, dt, offset_dims, collapsed_slice_dims, start_index_map, index_vector_dim,
           slice_sizes, operand_batching_dims=(), start_indices_batching_dims=(), idt="i64", one_based=False):
    """`stablehlo.gather` in the generic form it prints in.  With `one_based` the indices are
    decremented first, as the reference's Ops.gather does (src/Ops.jl:2313)."""
    to, ts, tr = tt(operand_shape, dt), tt(start_shape, idt), tt(out_shape, dt)
    lst = lambda v: "[" + ", ".join(str(x) for x in v) + "]"
    dn = "offset_dims = %s, collapsed_slice_dims = %s, " % (lst(offset_dims), lst(collapsed_slice_dims))
    if operand_batching_dims:
        dn += "operand_batching_dims = %s, start_indices_batching_dims = %s, " % (lst(operand_batching_dims), lst(start_indices_batching_dims))
    dn += "start_index_map = %s, index_vector_dim = %d" % (lst(start_index_map), index_vector_dim)
    pre, idx = "", "%arg1"
    if one_based:
        pre = ("    %%one = stablehlo.constant dense<1> : %s\n    %%idx = stablehlo.subtract %%arg1, %%one : %s\n" % (ts, ts))
        idx = "%idx"
    return ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n%s"
            "    %%0 = \"stablehlo.gather\"(%%arg0, %s) <{dimension_numbers = #stablehlo.gather<%s>, indices_are_sorted = false, "
            "slice_sizes = array<i64: %s>}> : (%s, %s) -> %s\n    return %%0 : %s\n  }\n}\n"
            % (to, ts, tr, pre, idx, dn, ", ".join(str(x) for x in slice_sizes), to, ts, tr, tr))


def scatter(operand_shape, index_shape, update_shape, dt, update_window_dims, inserted_window_dims, scatter_dims_to_operand_dims,
            index_vector_dim, body="assign", input_batching_dims=(), scatter_indices_batching_dims=(), idt="i64"):
    """`stablehlo.scatter` in the generic form it prints in (reference src/Ops.jl:2150-2268).  `body` is
    "assign" (the update replaces the element, what `setindex!` with index arrays prints) or the name of
    a binary op combining the element with the update ("add", "maximum", ...)."""
    to, ti, tu, ts = tt(operand_shape, dt), tt(index_shape, idt), tt(update_shape, dt), tt([], dt)
    lst = lambda v: "[" + ", ".join(str(x) for x in v) + "]"
    dn = "update_window_dims = %s, inserted_window_dims = %s, " % (lst(update_window_dims), lst(inserted_window_dims))
    if input_batching_dims:
        dn += "input_batching_dims = %s, scatter_indices_batching_dims = %s, " % (lst(input_batching_dims), lst(scatter_indices_batching_dims))
    dn += "scatter_dims_to_operand_dims = %s, index_vector_dim = %d" % (lst(scatter_dims_to_operand_dims), index_vector_dim)
    if body == "assign":
        region = "      stablehlo.return %%u : %s\n" % ts
    else:
        region = "      %%r = stablehlo.%s %%c, %%u : %s\n      stablehlo.return %%r : %s\n" % (body, ts, ts)
    return ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s, %%arg2: %s) -> %s {\n"
            "    %%0 = \"stablehlo.scatter\"(%%arg0, %%arg1, %%arg2) <{indices_are_sorted = false, scatter_dimension_numbers = "
            "#stablehlo.scatter<%s>, unique_indices = false}> ({\n    ^bb0(%%c: %s, %%u: %s):\n%s    }) : (%s, %s, %s) -> %s\n"
            "    return %%0 : %s\n  }\n}\n" % (to, ti, tu, to, dn, ts, ts, region, to, ti, tu, to, to))


def nnlib_scatter(op, dst_shape, src_shape, idx_shape, dt="f32"):
    """The module `NNlib.scatter!(op, dst, src, idx)` traces to for an integer index array
    (reference ext/ReactantNNlibExt/Implementations.jl:477-530 over src/Ops.jl:2204-2268): the index
    array gets a leading unit dim that holds the index vector, one is subtracted from it inside the
    module, the leading `ndims(src) - ndims(idx)` dims of `src` are the update window and the
    trailing dims of `dst` are indexed.  Arguments: dst, idx (i64, one-based), src.  `op` is "add",
    "subtract", "maximum", "minimum", "multiply", "divide" or "mean" (two additive scatters into
    zeros, then dst + sum / count where the count is not zero)."""
    nd, nw = len(dst_shape), len(src_shape) - len(idx_shape)
    ishape = [1] + list(idx_shape)
    to, ti, tu, ts = tt(dst_shape, dt), tt(ishape, "i64"), tt(src_shape, dt), tt([], dt)
    lst = lambda v: "[" + ", ".join(str(x) for x in v) + "]"
    dn = ("update_window_dims = %s, inserted_window_dims = %s, scatter_dims_to_operand_dims = %s, index_vector_dim = 0"
          % (lst(range(nw)), lst(range(nw, nd)), lst(range(nd - 1, nd))))

    def one(res, dst, upd, body):
        return ("    %s = \"stablehlo.scatter\"(%s, %%idx0, %s) <{indices_are_sorted = false, scatter_dimension_numbers = "
                "#stablehlo.scatter<%s>, unique_indices = false}> ({\n    ^bb0(%%c: %s, %%u: %s):\n"
                "      %%r = stablehlo.%s %%c, %%u : %s\n      stablehlo.return %%r : %s\n    }) : (%s, %s, %s) -> %s\n"
                % (res, dst, upd, dn, ts, ts, body, ts, ts, to, ti, tu, to))

    head = ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s, %%arg2: %s) -> %s {\n"
            "    %%one = stablehlo.constant dense<1> : %s\n    %%idx0 = stablehlo.subtract %%arg1, %%one : %s\n" % (to, ti, tu, to, ti, ti))
    if op != "mean":
        return head + one("%0", "%arg0", "%arg2", op) + "    return %%0 : %s\n  }\n}\n" % to
    tb = tt(dst_shape, "i1")
    return (head + "    %%z = stablehlo.constant dense<0.0> : %s\n    %%ones = stablehlo.constant dense<1.0> : %s\n" % (to, tu)
            + one("%ns", "%z", "%ones", "add") + one("%sum", "%z", "%arg2", "add")
            + "    %%isz = stablehlo.compare EQ, %%ns, %%z : (%s, %s) -> %s\n" % (to, to, tb)
            + "    %%q = stablehlo.divide %%sum, %%ns : %s\n" % to
            + "    %%sd = stablehlo.select %%isz, %%sum, %%q : %s, %s\n" % (tb, to)
            + "    %%0 = stablehlo.add %%arg0, %%sd : %s\n    return %%0 : %s\n  }\n}\n" % (to, to))


def select_and_scatter(x_shape, dt, window, strides=None, padding=None, direction="GE"):
    """`stablehlo.select_and_scatter` in the form the gradient of a pooling layer takes (what the
    reverse pass of `reduce_window` with a maximum body becomes): select = one compare of the two
    window elements, scatter = add, init 0.  Arguments: the pooled array and the gradient of the pooled
    result.  Returns (text, source shape)."""
    r = len(x_shape)
    strides = strides or [1] * r
    padding = padding or [[0, 0]] * r
    s_shape = window_out_shape(x_shape, window, strides, padding, [1] * r, [1] * r)
    tx, tsrc, t0, tb = tt(x_shape, dt), tt(s_shape, dt), tt([], dt), tt([], "i1")
    pad = "[" + ", ".join("[%d, %d]" % (p[0], p[1]) for p in padding) + "]"
    lst = lambda v: ", ".join(str(int(x)) for x in v)
    text = ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n"
            "    %%cst = stablehlo.constant dense<0.000000e+00> : %s\n"
            "    %%0 = \"stablehlo.select_and_scatter\"(%%arg0, %%arg1, %%cst) <{padding = dense<%s> : tensor<%dx2xi64>, "
            "window_dimensions = array<i64: %s>, window_strides = array<i64: %s>}> ({\n"
            "    ^bb0(%%a: %s, %%b: %s):\n      %%c = stablehlo.compare  %s, %%a, %%b,  FLOAT : (%s, %s) -> %s\n      stablehlo.return %%c : %s\n    }, {\n"
            "    ^bb0(%%a: %s, %%b: %s):\n      %%c = stablehlo.add %%a, %%b : %s\n      stablehlo.return %%c : %s\n    }) : (%s, %s, %s) -> %s\n"
            "    return %%0 : %s\n  }\n}\n"
            % (tx, tsrc, tx, t0, pad, r, lst(window), lst(strides), t0, t0, direction, t0, t0, tb, tb, t0, t0, t0, t0, tx, tsrc, t0, tx, tx))
    return text, s_shape
