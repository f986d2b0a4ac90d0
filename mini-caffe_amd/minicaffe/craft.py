"""Network descriptions in Python and their prototxt rendering.

Plays the role of the reference's LayerCrafter (reference python/minicaffe/craft.py):
build a net as data, get prototxt text for CaffeNetCreateFromBuffer.

A spec is a list of layer dicts:
    {"name": ..., "type": ..., "bottom": [...], "top": [...],
     "<x>_param": {...},            # rendered verbatim into the prototxt
     "blobs": [np.ndarray, ...]}     # parameter values, in the layer's blob order
`to_prototxt` renders everything but the blobs; `load_weights` writes the blobs
into a created net through CaffeNetListParam + CaffeBlobData, which is how a
caller of the C ABI injects weights without a caffemodel file.
"""


class Enum(str):
    """A prototxt enum identifier (rendered without quotes)."""


def _render_value(v):
    if isinstance(v, Enum):
        return str(v)
    if isinstance(v, bool):
        return "true" if v else "false"
    if isinstance(v, str):
        return '"%s"' % v
    if isinstance(v, float):
        return repr(float(v))
    return str(v)


def _render_fields(d, indent):
    pad = " " * indent
    out = []
    for k, v in d.items():
        vals = v if isinstance(v, (list, tuple)) else [v]
        for item in vals:
            if isinstance(item, dict):
                out.append("%s%s {" % (pad, k))
                out.extend(_render_fields(item, indent + 2))
                out.append("%s}" % pad)
            else:
                out.append("%s%s: %s" % (pad, k, _render_value(item)))
    return out


def to_prototxt(spec, name="net"):
    lines = ['name: "%s"' % name]
    for layer in spec:
        lines.append("layer {")
        fields = {k: v for k, v in layer.items() if k != "blobs"}
        lines.extend(_render_fields(fields, 2))
        lines.append("}")
    return "\n".join(lines) + "\n"


def input_layer(tops_shapes, name="input"):
    tops = list(tops_shapes.keys())
    return {"name": name, "type": "Input", "top": tops,
            "input_param": {"shape": [{"dim": list(s)} for s in tops_shapes.values()]}}


def load_weights(net, spec):
    """Write every layer's blobs into the net's parameter blobs (in net order)."""
    params = net.param_list
    i = 0
    for layer in spec:
        for arr in layer.get("blobs", []):
            name, blob = params[i]
            assert name.startswith(layer["name"]), (name, layer["name"])
            assert list(blob.shape) == list(arr.shape), (name, blob.shape, arr.shape)
            if arr.size:
                blob.data[...] = arr
            i += 1
    assert i == len(params), "spec lists %d blobs, net has %d" % (i, len(params))


