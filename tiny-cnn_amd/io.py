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
