"""Data ingest and weight files of the reference, on the Python host side.

parse_mnist_labels / parse_mnist_images / parse_cifar10 read the dataset files the way
tiny_dnn/io/mnist_parser.h and tiny_dnn/io/cifar10_parser.h do (same arguments, same float32
scaling arithmetic, same errors as ValueError); the arrays they return are what
tiny-cnn_amd.Feeder uploads batch by batch. save_weights / load_weights write and read the text
format of network::save(std::ostream&) (tiny_dnn/network.h:762-771,
tiny_dnn/layers/layer.h:361-385): every trainable vector of every layer in order, each value
with 8 significant digits followed by a blank.
"""
import numpy as np

F32 = np.float32


def _check_args(scale_min, scale_max, x_padding, y_padding):
    if x_padding < 0 or y_padding < 0:
        raise ValueError("padding size must not be negative")
    if scale_min >= scale_max:
        raise ValueError("scale_max must be greater than scale_min")


def _read(path):
    try:
        with open(path, "rb") as f:
            return np.frombuffer(f.read(), np.uint8)
    except OSError:
        raise ValueError("failed to open file:" + str(path))


def _be32(b, at):
    field = np.zeros(4, np.uint8)
    part = b[at:at + 4]
    field[:part.size] = part
    return int.from_bytes(field.tobytes(), "big")


def _padded(b, start, count):
    """`count` bytes from `start`; bytes past the end of the file read as 0 (a failed read
    leaves the reference's zero-initialised buffer untouched)."""
    out = np.zeros(count, np.uint8)
    part = b[start:start + count]
    out[:part.size] = part
    return out


def parse_mnist_labels(label_file):
    """mnist_parser.h:77-102 -> int64 [items]"""
    b = _read(label_file)
    magic, items = _be32(b, 0), _be32(b, 4)
    if magic != 0x00000801 or items <= 0:
        raise ValueError("MNIST label-file format error")
    return _padded(b, 8, items).astype(np.int64)


def parse_mnist_images(image_file, scale_min=-1.0, scale_max=1.0, x_padding=2, y_padding=2):
    """mnist_parser.h:26-75,121-147 -> float32 [items][(rows+2*y_padding)*(cols+2*x_padding)]:
    pixel p becomes (p/255)*(scale_max-scale_min)+scale_min, the border is scale_min."""
    _check_args(scale_min, scale_max, x_padding, y_padding)
    b = _read(image_file)
    magic, items, rows, cols = (_be32(b, 4 * i) for i in range(4))
    if magic != 0x00000803 or items <= 0:
        raise ValueError("MNIST label-file format error")
    lo, hi = F32(scale_min), F32(scale_max)
    px = _padded(b, 16, items * rows * cols).reshape(items, rows, cols).astype(F32)
    val = (px / F32(255)) * (hi - lo) + lo
    out = np.full((items, rows + 2 * y_padding, cols + 2 * x_padding), lo, F32)
    out[:, y_padding:y_padding + rows, x_padding:x_padding + cols] = val
    return out.reshape(items, -1)


def parse_cifar10(filename, scale_min=-1.0, scale_max=1.0, x_padding=0, y_padding=0):
    """cifar10_parser.h:38-86 -> (float32 [records][3*(32+2*y_padding)*(32+2*x_padding)],
    int64 labels); pixel c becomes scale_min + (scale_max-scale_min)*c/255; an incomplete last
    record is dropped."""
    _check_args(scale_min, scale_max, x_padding, y_padding)
    b = _read(filename)
    record = 1 + 3 * 32 * 32
    n = b.size // record
    rec = b[:n * record].reshape(n, record)
    lo, hi = F32(scale_min), F32(scale_max)
    val = lo + ((hi - lo) * rec[:, 1:].astype(F32)) / F32(255)
    out = np.full((n, 3, 32 + 2 * y_padding, 32 + 2 * x_padding), lo, F32)
    out[:, :, y_padding:y_padding + 32, x_padding:x_padding + 32] = val.reshape(n, 3, 32, 32)
    return out.reshape(n, -1), rec[:, 0].astype(np.int64)


# ------------------------------------------------------------------ weight files
def weights_to_text(vectors):
    """The stream network::save writes for these trainable vectors (in file order)."""
    return "".join("%.8g " % float(v) for vec in vectors for v in np.asarray(vec, F32).ravel())


def text_to_floats(text):
    """Every number of a weight file as float32 (what `is >> w` yields one by one)."""
    return np.array(text.split(), dtype=np.float64).astype(F32) if text.split() else np.zeros(0, F32)


def _file_length(layer, which, n):
    # an average-pooling layer's weight vector has pool_w*pool_h*channels entries in the
    # reference's files although only the first `channels` are read (average_pooling_layer.h:222-226)
    if layer.kind == 3 and which == 0:
        return n * layer.pool.pool_w * layer.pool.pool_h
    return n


def save_weights(net, path):
    vectors = []
    for i in range(net.n):
        for which in (0, 1, 2, 3):   # 2, 3: the running averages a batch-norm layer writes
            n = net.param_size(i, which)
            if not n:
                continue
            v = net.get_param(i, which)
            vectors.append(np.concatenate([v, np.zeros(_file_length(net.layers[i], which, n) - n, F32)]))
    with open(path, "w") as f:
        f.write(weights_to_text(vectors))


def load_weights(net, path):
    with open(path) as f:
        data = text_to_floats(f.read())
    at = 0
    for i in range(net.n):
        for which in (0, 1, 2, 3):   # 2, 3: the running averages a batch-norm layer writes
            n = net.param_size(i, which)
            if not n:
                continue
            length = _file_length(net.layers[i], which, n)
            if at + length > data.size:
                raise ValueError("load_weights: the file holds fewer weights than the network")
            net.set_param(i, which, data[at:at + n])
            at += length


# ------------------------------------------------------------------ cereal weight archives
# network::save(filename, content_type::weights, file_format::binary / portable_binary)
# (tiny_dnn/network.h:676-728, to_archive :787-799, nodes::save_weights tiny_dnn/nodes.h:203-214):
# for every layer in order, the layer's registered type name (serialize_prolog,
# tiny_dnn/util/serialization_helper.h:118-123; names in serialization_layer_list.h) as a string
# = u64 length + bytes, then every trainable vector (serialization_functions.h:747-754) as u64
# element count + float32 values. A portable_binary archive starts with one byte that says
# whether what follows is little-endian (cereal writes 1 on such a host). Batch-norm running
# averages are not trainable vectors and are not in these files.
ACT_TYPE_NAMES = {0: "tanh", 1: "relu", 2: "softmax", 3: "sigmoid", 4: "leaky_relu", 5: "elu",
                  6: "selu", 7: "softplus", 8: "softsign", 9: "asinh", 10: "tanh_scaled"}
LAYER_TYPE_NAMES = {0: "conv", 1: "fully_connected", 2: "maxpool", 3: "avepool", 5: "batchnorm",
                    6: "dropout"}


def archive_type_name(layer):
    """The name the reference registers for this layer's class."""
    return ACT_TYPE_NAMES[layer.act] if layer.kind == 4 else LAYER_TYPE_NAMES[layer.kind]


def weights_to_archive(type_names, vectors_per_layer, file_format="binary"):
    """The bytes of a weights-only archive: `type_names[i]` and the trainable vectors
    `vectors_per_layer[i]` (in file order, at their file length) of every layer."""
    if file_format not in ("binary", "portable_binary"):
        raise ValueError("weight archives are written as binary or portable_binary")
    out = [b"\x01"] if file_format == "portable_binary" else []
    for name, vectors in zip(type_names, vectors_per_layer):
        raw = name.encode()
        out.append(np.uint64(len(raw)).tobytes() + raw)
        for v in vectors:
            v = np.ascontiguousarray(v, dtype="<f4").ravel()
            out.append(np.uint64(v.size).tobytes() + v.tobytes())
    return b"".join(out)


def archive_to_weights(data, vector_counts, file_format="binary"):
    """[(type name, [float32 vectors])] of a weights-only archive whose i-th layer holds
    `vector_counts[i]` trainable vectors. Raises ValueError on a truncated file."""
    data = bytes(data)
    at, order = 0, "<"
    if file_format == "portable_binary":
        if not data:
            raise ValueError("archive is empty")
        order, at = ("<" if data[0] else ">"), 1
    elif file_format != "binary":
        raise ValueError("weight archives are read as binary or portable_binary")

    def take(n):
        nonlocal at
        if at + n > len(data):
            raise ValueError("archive ends inside a layer record")
        at += n
        return data[at - n:at]

    out = []
    for count in vector_counts:
        n = int(np.frombuffer(take(8), order + "u8")[0])
        name = take(n).decode()
        vectors = []
        for _ in range(count):
            m = int(np.frombuffer(take(8), order + "u8")[0])
            vectors.append(np.frombuffer(take(4 * m), order + "f4").astype(F32))
        out.append((name, vectors))
    return out


def save_weights_archive(net, path, file_format="binary"):
    names, vectors = [], []
    for i in range(net.n):
        names.append(archive_type_name(net.layers[i]))
        vs = []
        for which in (0, 1):
            n = net.param_size(i, which)
            if n:
                v = net.get_param(i, which)
                vs.append(np.concatenate([v, np.zeros(_file_length(net.layers[i], which, n) - n, F32)]))
        vectors.append(vs)
    with open(path, "wb") as f:
        f.write(weights_to_archive(names, vectors, file_format))


def load_weights_archive(net, path, file_format="binary"):
    counts = [sum(1 for which in (0, 1) if net.param_size(i, which)) for i in range(net.n)]
    with open(path, "rb") as f:
        layers = archive_to_weights(f.read(), counts, file_format)
    for i, (_, vectors) in enumerate(layers):
        k = 0
        for which in (0, 1):
            n = net.param_size(i, which)
            if not n:
                continue
            if vectors[k].size != _file_length(net.layers[i], which, n):
                raise ValueError(f"load_weights_archive: layer {i} holds {vectors[k].size} values, "
                                 f"the network's layer {_file_length(net.layers[i], which, n)}")
            net.set_param(i, which, vectors[k][:n])
            k += 1
