"""Writes a synthetic YOLOv5n-architecture model in PNNX's on-disk format (`.pnnx.param` text + `.pnnx.bin`
store-only zip of raw float32 blobs), with random weights from a seed: depth multiple 0.33, width multiple 0.25,
BatchNorm already folded into the convolutions (what a PNNX export of a fused model holds), three detect stages.
There is no network and no checkpoint here, so this is the model the YOLOv5n forward configuration runs on.

The format follows what the reference's parser reads (src/pnnx/pnnx_parser.cpp:36-380): line 1 the magic 7767517,
line 2 `operators operands`, then one operator per line `type name n_in n_out inputs... outputs... key=value...`
with `@attr=(shape)f32` declaring a weight and `#i=(shape)f32` a blob shape; weights live in the zip as
`<node name>.<attr>`. The detect head uses the attribute names a PNNX export gives it (pnnx_0..pnnx_6, m.<i>.weight/bias,
see src/pnnx/operator_mapper.cpp:282-345)."""
import io
import zipfile

import numpy as np

ANCHORS = ((10, 13, 16, 30, 33, 23), (30, 61, 62, 45, 59, 119), (116, 90, 156, 198, 373, 326))
STRIDES = (8, 16, 32)


class _Builder:
    def __init__(self, seed, batch, size, num_classes):
        self.rng = np.random.default_rng(seed)
        self.lines, self.blobs, self.next_blob = [], {}, 0
        self.shape = {}
        self.batch, self.nc = batch, num_classes
        x = self.new_blob((batch, 3, size, size))
        self.lines.append("pnnx.Input pnnx_input_0 0 1 %s #0=%s" % (x, self.fmt(self.shape[x])))
        self.input = x

    @staticmethod
    def fmt(shape):
        return "(" + ",".join(str(int(s)) for s in shape) + ")f32"

    def new_blob(self, shape):
        name = str(self.next_blob)
        self.next_blob += 1
        self.shape[name] = tuple(int(s) for s in shape)
        return name

    def conv(self, name, x, c2, k=1, s=1, act=True):
        n, c1, h, w = self.shape[x]
        p = k // 2
        oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
        wt = (self.rng.standard_normal((c2, c1, k, k)) * np.sqrt(2.0 / (c1 * k * k))).astype(np.float32)
        bs = (self.rng.standard_normal(c2) * 0.1).astype(np.float32)
        self.blobs[name + ".conv.weight"], self.blobs[name + ".conv.bias"] = wt, bs
        y = self.new_blob((n, c2, oh, ow))
        self.lines.append(
            "nn.Conv2d %s.conv 1 1 %s %s bias=True dilation=(1,1) groups=1 in_channels=%d kernel_size=(%d,%d) "
            "out_channels=%d padding=(%d,%d) padding_mode=zeros stride=(%d,%d) @bias=%s @weight=%s #0=%s #1=%s"
            % (name, x, y, c1, k, k, c2, p, p, s, s, self.fmt((c2,)), self.fmt(wt.shape), self.fmt(self.shape[x]),
               self.fmt(self.shape[y])))
        if not act:
            return y
        z = self.new_blob(self.shape[y])
        self.lines.append("nn.SiLU %s.act 1 1 %s %s #0=%s #1=%s" % (name, y, z, self.fmt(self.shape[y]), self.fmt(self.shape[z])))
        return z

    def add(self, name, a, b):
        y = self.new_blob(self.shape[a])
        self.lines.append("pnnx.Expression %s 2 1 %s %s %s expr=add(@0,@1) #0=%s #1=%s #2=%s"
                          % (name, a, b, y, self.fmt(self.shape[a]), self.fmt(self.shape[b]), self.fmt(self.shape[y])))
        return y

    def cat(self, name, xs):
        n, _, h, w = self.shape[xs[0]]
        y = self.new_blob((n, sum(self.shape[x][1] for x in xs), h, w))
        shapes = " ".join("#%d=%s" % (i, self.fmt(self.shape[x])) for i, x in enumerate(xs + [y]))
        self.lines.append("torch.cat %s %d 1 %s %s dim=1 %s" % (name, len(xs), " ".join(xs), y, shapes))
        return y

    def maxpool(self, name, x, k):
        y = self.new_blob(self.shape[x])
        self.lines.append("nn.MaxPool2d %s 1 1 %s %s ceil_mode=False dilation=(1,1) kernel_size=(%d,%d) padding=(%d,%d) "
                          "return_indices=False stride=(1,1) #0=%s #1=%s"
                          % (name, x, y, k, k, k // 2, k // 2, self.fmt(self.shape[x]), self.fmt(self.shape[y])))
        return y

    def upsample(self, name, x):
        n, c, h, w = self.shape[x]
        y = self.new_blob((n, c, 2 * h, 2 * w))
        self.lines.append("nn.Upsample %s 1 1 %s %s mode=nearest scale_factor=(2.0,2.0) size=None #0=%s #1=%s"
                          % (name, x, y, self.fmt(self.shape[x]), self.fmt(self.shape[y])))
        return y

    def c3(self, name, x, c2, n=1, shortcut=True):
        c_ = c2 // 2
        a = self.conv(name + ".cv1", x, c_)
        for i in range(n):
            t = self.conv("%s.m.%d.cv1" % (name, i), a, c_)
            t = self.conv("%s.m.%d.cv2" % (name, i), t, c_, k=3)
            a = self.add("pnnx_expr_%s_%d" % (name.replace(".", "_"), i), a, t) if shortcut else t
        b = self.conv(name + ".cv2", x, c_)
        return self.conv(name + ".cv3", self.cat("torch.cat_" + name.replace(".", "_"), [a, b]), c2)

    def sppf(self, name, x, c2, k=5):
        c_ = self.shape[x][1] // 2
        a = self.conv(name + ".cv1", x, c_)
        y1 = self.maxpool(name + ".m", a, k)
        y2 = self.maxpool(name + ".m_1", y1, k)
        y3 = self.maxpool(name + ".m_2", y2, k)
        return self.conv(name + ".cv2", self.cat("torch.cat_" + name.replace(".", "_"), [a, y1, y2, y3]), c2)

    def detect(self, name, feats):
        na, ci = 3, self.nc + 5
        attrs, total = [], 0
        grid_names, anchor_names = ("pnnx_6", "pnnx_3", "pnnx_1"), ("pnnx_4", "pnnx_2", "pnnx_0")
        for i, f in enumerate(feats):
            n, c, h, w = self.shape[f]
            wt = (self.rng.standard_normal((na * ci, c, 1, 1)) * np.sqrt(1.0 / c)).astype(np.float32)
            bs = (self.rng.standard_normal(na * ci) * 0.5).astype(np.float32)
            yy, xx = np.meshgrid(np.arange(h, dtype=np.float32), np.arange(w, dtype=np.float32), indexing="ij")
            grid = np.broadcast_to(np.stack([xx, yy], -1) - np.float32(0.5), (1, na, h, w, 2)).astype(np.float32)
            anc = np.asarray(ANCHORS[i], np.float32).reshape(1, na, 1, 1, 2)
            anchor_grid = np.broadcast_to(anc, (1, na, h, w, 2)).astype(np.float32)
            for key, val in (("m.%d.weight" % i, wt), ("m.%d.bias" % i, bs), (grid_names[i], grid),
                             (anchor_names[i], anchor_grid)):
                self.blobs[name + "." + key] = np.ascontiguousarray(val)
                attrs.append("@%s=%s" % (key, self.fmt(val.shape)))
            total += na * h * w
        self.blobs[name + ".pnnx_5"] = np.asarray(STRIDES, np.float32)
        attrs.append("@pnnx_5=%s" % self.fmt((3,)))
        y = self.new_blob((self.batch, total, ci))
        shapes = " ".join("#%d=%s" % (i, self.fmt(self.shape[x])) for i, x in enumerate(feats + [y]))
        self.lines.append("models.yolo.Detect %s 3 1 %s %s %s %s" % (name, " ".join(feats), y, " ".join(sorted(attrs)), shapes))
        return y


def yolov5n(seed=0, batch=4, size=320, num_classes=80):
    """-> (param text, {member name: float32 array}, output shape). size must be a multiple of 32."""
    assert size % 32 == 0
    b = _Builder(seed, batch, size, num_classes)
    x = b.conv("model.0", b.input, 16, k=6, s=2)  # the 6x6 stem keeps pad 2 in YOLOv5
    # k // 2 = 3 for k = 6; YOLOv5's stem uses pad 2: patch the line just written
    b.lines[-2] = b.lines[-2].replace("padding=(3,3)", "padding=(2,2)")
    n, c, h, w = b.shape[x]
    fix = (size + 4 - 6) // 2 + 1
    for k in (str(int(x) - 1), x):
        b.shape[k] = (n, c, fix, fix)
    b.lines[-2] = b.lines[-2].rsplit(" #1=", 1)[0] + " #1=" + b.fmt(b.shape[x])
    b.lines[-1] = "nn.SiLU model.0.act 1 1 %s %s #0=%s #1=%s" % (str(int(x) - 1), x, b.fmt(b.shape[x]), b.fmt(b.shape[x]))
    x = b.conv("model.1", x, 32, k=3, s=2)
    x = b.c3("model.2", x, 32, n=1)
    x = b.conv("model.3", x, 64, k=3, s=2)
    p3 = b.c3("model.4", x, 64, n=2)
    x = b.conv("model.5", p3, 128, k=3, s=2)
    p4 = b.c3("model.6", x, 128, n=3)
    x = b.conv("model.7", p4, 256, k=3, s=2)
    x = b.c3("model.8", x, 256, n=1)
    x = b.sppf("model.9", x, 256)
    h10 = b.conv("model.10", x, 128)
    x = b.cat("torch.cat_12", [b.upsample("model.11", h10), p4])
    x = b.c3("model.13", x, 128, n=1, shortcut=False)
    h14 = b.conv("model.14", x, 64)
    x = b.cat("torch.cat_16", [b.upsample("model.15", h14), p3])
    o3 = b.c3("model.17", x, 64, n=1, shortcut=False)
    x = b.cat("torch.cat_19", [b.conv("model.18", o3, 64, k=3, s=2), h14])
    o4 = b.c3("model.20", x, 128, n=1, shortcut=False)
    x = b.cat("torch.cat_22", [b.conv("model.21", o4, 128, k=3, s=2), h10])
    o5 = b.c3("model.23", x, 256, n=1, shortcut=False)
    y = b.detect("model.24", [o3, o4, o5])
    b.lines.append("pnnx.Output pnnx_output_0 1 0 %s #0=%s" % (y, b.fmt(b.shape[y])))
    param = "7767517\n%d %d\n%s\n" % (len(b.lines), b.next_blob, "\n".join(b.lines))
    return param, b.blobs, b.shape[y]


def write(prefix, seed=0, batch=4, size=320, num_classes=80):
    """Writes <prefix>.pnnx.param and <prefix>.pnnx.bin; returns (param path, bin path, output shape)."""
    param, blobs, out_shape = yolov5n(seed, batch, size, num_classes)
    with open(prefix + ".pnnx.param", "w") as f:
        f.write(param)
    buf = io.BytesIO()
    with zipfile.ZipFile(buf, "w", zipfile.ZIP_STORED) as z:
        for name, arr in blobs.items():
            z.writestr(zipfile.ZipInfo(name), np.ascontiguousarray(arr, np.float32).tobytes())
    with open(prefix + ".pnnx.bin", "wb") as f:
        f.write(buf.getvalue())
    return prefix + ".pnnx.param", prefix + ".pnnx.bin", out_shape


def flops(batch=4, size=320, num_classes=80):
    """Multiply-add FLOPs (2 per MAC) of the convolutions of one forward pass."""
    param, _, _ = yolov5n(0, batch, size, num_classes)
    total = 0
    for line in param.splitlines():
        if line.startswith("nn.Conv2d"):
            kv = dict(t.split("=", 1) for t in line.split() if "=" in t)
            w = [int(v) for v in kv["@weight"].strip("()f32").rstrip(")f").split(",")] if False else \
                [int(v) for v in kv["@weight"][1:kv["@weight"].index(")")].split(",")]
            o = [int(v) for v in kv["#1"][1:kv["#1"].index(")")].split(",")]
            total += 2 * o[0] * o[2] * o[3] * w[0] * w[1] * w[2] * w[3]
    # detect heads: 1x1 convolutions on the three feature maps
    for line in param.splitlines():
        if line.startswith("models.yolo.Detect"):
            kv = dict(t.split("=", 1) for t in line.split() if "=" in t)
            for i in range(3):
                w = [int(v) for v in kv["@m.%d.weight" % i][1:kv["@m.%d.weight" % i].index(")")].split(",")]
                f = [int(v) for v in kv["#%d" % i][1:kv["#%d" % i].index(")")].split(",")]
                total += 2 * f[0] * f[2] * f[3] * w[0] * w[1]
    return total
