"""Host side of the data-set readers and of the solver's driver (utilities/dataset.c:20-42,122-157,373-571,
drivers/kfac_trust_region_driver.cu:59-108,225-488): record files written here with known contents, read back
through the C entry points and compared with the arrangement numpy gives directly (per-channel transposition,
labels + 1), the closed form of the normalisation, and the reference's table of parameter-file names."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

from fitre_amd import lib as L
from fitre_amd.structs import CNN_MODEL, HOST_DATASET, KFAC_CURVATURE_INFO, TRUST_REGION_PARAMS

cnn = L.cnn


def records(rng, count, side, label_bytes, classes):
    """count records of `label_bytes` label bytes + 3 x side x side pixel bytes; returns (bytes, labels, pixels)."""
    px = rng.integers(0, 256, size=(count, 3, side, side), dtype=np.uint8)
    lab = rng.integers(0, classes, size=(count, label_bytes), dtype=np.uint8)
    return np.concatenate([lab, px.reshape(count, -1)], axis=1).tobytes(), lab, px


def as_array(ptr, n):
    return np.ctypeslib.as_array(ptr, shape=(n,)).copy()


def expect_images(px):
    """[image][channel][col * height + row], the reference's per-channel column-major image"""
    return px.astype(np.float32).transpose(0, 1, 3, 2).reshape(px.shape[0], -1)


def free_host(h):
    libc = C.CDLL(None)
    libc.free.argtypes = [C.c_void_p]
    for name in ("trainSetX", "trainSetY", "testSetX", "testSetY"):
        libc.free(C.cast(getattr(h, name), C.c_void_p))


@pytest.mark.parametrize("dataset,side,label_bytes,kept,classes,train_name,test_name,test_files", [
    (1, 32, 1, 0, 10, "data_batch_", "test_batch.bin", 1),
    (2, 32, 2, 1, 100, "train_", "test.bin", 1),
    (3, 64, 1, 0, 200, "train_", "test_", 2),
])
def test_record_files_are_read_into_column_major_images(tmp_path, dataset, side, label_bytes, kept, classes, train_name,
                                                        test_name, test_files):
    rng = np.random.default_rng(dataset)
    train_counts = [7, 5, 3]
    train = [records(rng, n, side, label_bytes, classes) for n in train_counts]
    for i, (blob, _, _) in enumerate(train):
        (tmp_path / ("%s%d.bin" % (train_name, i + 1))).write_bytes(blob)
    tests = [records(rng, 4 + i, side, label_bytes, classes) for i in range(test_files)]
    for i, (blob, _, _) in enumerate(tests):
        name = test_name if dataset != 3 else "%s%d.bin" % (test_name, i + 1)
        (tmp_path / name).write_bytes(blob)

    h = HOST_DATASET()
    d = (str(tmp_path) + "/").encode()
    cnn.readCIFARDataset(d, train_name.encode(), len(train), test_name.encode(), C.byref(h), None, 255, 64, dataset, side, side)
    feats = 3 * side * side
    total_test = sum(t[1].shape[0] for t in tests)
    assert (h.trainSizeX, h.trainSizeY, h.testSizeX, h.testSizeY) == (15, 15, total_test, total_test)
    assert h.features == feats and h.numClasses == classes
    got_x = as_array(h.trainSetX, 15 * feats).reshape(15, feats)
    got_y = as_array(h.trainSetY, 15)
    np.testing.assert_array_equal(got_x, np.concatenate([expect_images(t[2]) for t in train]))
    np.testing.assert_array_equal(got_y, np.concatenate([t[1][:, kept] for t in train]).astype(np.float32) + 1)
    nt = h.testSizeX
    np.testing.assert_array_equal(as_array(h.testSetX, nt * feats).reshape(nt, feats),
                                  np.concatenate([expect_images(t[2]) for t in tests]))
    np.testing.assert_array_equal(as_array(h.testSetY, nt), np.concatenate([t[1][:, kept] for t in tests]).astype(np.float32) + 1)
    # one cell by hand: image 2 of the first file, channel 1, row 3, column 9
    assert got_x[2, 1 * side * side + 9 * side + 3] == train[0][2][2, 1, 3, 9]
    free_host(h)


def test_a_trailing_partial_record_is_padded_with_zeros(tmp_path):
    rng = np.random.default_rng(9)
    blob, lab, px = records(rng, 3, 32, 1, 10)
    (tmp_path / "data_batch_1.bin").write_bytes(blob[:2 * 3073 + 1000])     # third record cut after 999 pixel bytes
    (tmp_path / "test_batch.bin").write_bytes(blob[:3073])
    h = HOST_DATASET()
    cnn.readCIFARDataset((str(tmp_path) + "/").encode(), b"data_batch_", 1, b"test_batch.bin", C.byref(h), None, 255, 64, 1, 32, 32)
    assert h.trainSizeX == 3 and h.testSizeX == 1
    got = as_array(h.trainSetX, 3 * 3072).reshape(3, 3072)
    cut = px[2].reshape(-1).copy()
    cut[999:] = 0
    np.testing.assert_array_equal(got[2], expect_images(cut.reshape(1, 3, 32, 32))[0])
    np.testing.assert_array_equal(got[:2], expect_images(px[:2]))
    free_host(h)


def test_a_missing_file_ends_the_process_with_a_message(tmp_path):
    code = ("import ctypes as C\nfrom fitre_amd import lib as L\nfrom fitre_amd.structs import HOST_DATASET\nh = HOST_DATASET()\n"
            "L.cnn.readCIFARDataset(%r, b'data_batch_', 1, b'test_batch.bin', C.byref(h), None, 255, 64, 1, 32, 32)\n"
            % (str(tmp_path) + "/").encode())
    run = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert run.returncode == 255 and "Error opening the dataset" in run.stderr, (run.returncode, run.stderr[-300:])


def test_layout_converters():
    rng = np.random.default_rng(2)
    src = rng.standard_normal((5, 7)).astype(np.float32)
    out = np.empty(35, np.float32)
    cnn.convertToColumnMajor(src.ctypes.data_as(C.c_void_p), 5, 7, out.ctypes.data_as(C.c_void_p))
    np.testing.assert_array_equal(out, src.T.reshape(-1))
    for height, width in ((4, 4), (3, 5)):      # square as in the reference; non-square: a true transposition
        img = rng.standard_normal((6, 3, height, width)).astype(np.float32)
        out = np.empty(img.size, np.float32)
        cnn.convertCIFARToColumnMajor(img.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), 6, 3, height, width)
        np.testing.assert_array_equal(out, img.transpose(0, 1, 3, 2).reshape(-1))


@pytest.mark.parametrize("dataset,mean,std", [
    (1, (0.4914, 0.4822, 0.4465), (0.2470, 0.2435, 0.2616)),
    (2, (0.5071, 0.4865, 0.4409), (0.2673, 0.2564, 0.2762)),
    (3, (0.4799, 0.4478, 0.3972), (0.2769, 0.2690, 0.2820)),
])
def test_image_normalisation(dataset, mean, std):
    rng = np.random.default_rng(4)
    x = rng.integers(0, 256, size=(3, 5, 4, 4)).astype(np.float32)       # [channel][image][cell]
    want = (x.astype(np.float64) / 255.0 - np.array(mean).reshape(3, 1, 1, 1)) / np.array(std).reshape(3, 1, 1, 1)
    got = x.copy()
    cnn.imageNormalization(got.ctypes.data_as(C.c_void_p), 5, 3, 4, 4, 255.0, dataset)
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-6)
    assert abs(got[0].mean() - want[0].mean()) < 1e-6


def test_parameter_file_names_follow_the_reference_table():
    cnn.fitreSetWeightsFolder(b"/w/")
    nets = {0: "lenet", 1: "alexnet", 2: "vgg11", 3: "vgg13", 4: "vgg16", 5: "vgg19"}
    folders = {1: "cifar10", 2: "cifar100", 3: "imagenet"}
    inits = {0: "default", 1: "kaiming", 2: "xavier"}
    buf = C.create_string_buffer(256)
    m = CNN_MODEL()
    for name, net in nets.items():
        for bias in (0, 1):
            for ds, folder in folders.items():
                for ini, word in inits.items():
                    m.name, m.bias = name, bias
                    assert cnn.kfacParamsFileName(C.byref(m), ds, ini, buf, 256) == 0
                    assert buf.value.decode() == "/w/%s/%s_%s%s.params" % (folder, net, word, "_bias" if bias else "")
    # spelled out from drivers/kfac_trust_region_driver.cu:372-376 and :263
    m.name, m.bias = 2, 1
    cnn.kfacParamsFileName(C.byref(m), 1, 1, buf, 256)
    assert buf.value == b"/w/cifar10/vgg11_kaiming_bias.params"
    m.name, m.bias = 0, 0
    cnn.kfacParamsFileName(C.byref(m), 2, 2, buf, 256)
    assert buf.value == b"/w/cifar100/lenet_xavier.params"
    for bad in ((9, 1, 0), (2, 0, 0), (2, 4, 0), (2, 1, 3), (2, 1, -1)):
        m.name = bad[0]
        assert cnn.kfacParamsFileName(C.byref(m), bad[1], bad[2], buf, 256) == -1
    m.name, m.bias = 2, 1
    assert cnn.kfacParamsFileName(C.byref(m), 1, 0, buf, 8) == -1           # buffer too small
    cnn.fitreSetWeightsFolder(None)
    assert cnn.kfacParamsFileName(C.byref(m), 1, 0, buf, 256) == 0
    assert buf.value == b"/scratch/gilbreth/skylasa/weights/cifar10/vgg11_default_bias.params"   # the reference's folder


def test_driver_defaults():
    tr = TRUST_REGION_PARAMS()
    cnn.initKFACTrustRegionParams(C.byref(tr), 50000)
    assert (tr.eta1, tr.gamma1, tr.delta, tr.maxDelta, tr.maxIters, tr.maxEpochs) == (np.float32(0.8), 2.0, 1.0, 100.0, 200, 1)
    assert tr.eta2 == np.float32(1e-4) and tr.gamma2 == np.float32(1.2) and tr.minDelta == np.float32(1e-6)
    assert tr.alpha == np.float32(0.01) and tr.curIteration == 0
    assert tr.lambda_ == 0.0 and tr.maxMatVecs == 2**31 - 1
    info = KFAC_CURVATURE_INFO()
    info.checkGrad = 7
    cnn.initKFACInfo(C.byref(info))
    assert (info.stats_decay, info.momentum, info.regLambda, info.dampGamma, info.checkGrad) == (
        np.float32(0.8), 0.0, np.float32(1e-3), 100.0, 1)
    assert info.OmegaZInv is None and list(info.OmegaZOffsets) == [0] * 20


def test_delimited_text_matrix(tmp_path):
    rng = np.random.default_rng(6)
    m = rng.standard_normal((7, 5)).astype(np.float32)
    lines = [", ".join("%.9g" % v for v in row) for row in m[:4]] + [" ".join("%.9g" % v for v in row) for row in m[4:]]
    path = tmp_path / "m.csv"
    path.write_text("\n".join(lines) + "\n\n9, 9, 9, 9, 9\n")          # the empty line ends the matrix
    data, rows, cols = C.POINTER(C.c_float)(), C.c_int(), C.c_int()
    cnn.readDelimitedMatrix(str(path).encode(), C.byref(data), C.byref(rows), C.byref(cols))
    assert (rows.value, cols.value) == (7, 5)
    np.testing.assert_array_equal(as_array(data, 35).reshape(7, 5), m)
    C.CDLL(None).free(C.cast(data, C.c_void_p))
    wide = tmp_path / "wide.csv"                                           # one line far beyond any fixed buffer
    row = np.arange(300000, dtype=np.float32)
    wide.write_text(",".join("%d" % v for v in row) + "\n")
    cnn.readDelimitedMatrix(str(wide).encode(), C.byref(data), C.byref(rows), C.byref(cols))
    assert (rows.value, cols.value) == (1, 300000)
    np.testing.assert_array_equal(as_array(data, 300000), row)


def test_delimited_text_matrix_reports_what_it_drops(tmp_path, capfd):
    """Rows after an empty line and rows of uneven length are named on stderr; a clean file draws neither message."""
    data, rows, cols = C.POINTER(C.c_float)(), C.c_int(), C.c_int()
    clean = tmp_path / "clean.csv"
    clean.write_text("1,2,3\n4,5,6\n\n")                                  # a trailing empty line drops nothing
    cnn.readDelimitedMatrix(str(clean).encode(), C.byref(data), C.byref(rows), C.byref(cols))
    err = capfd.readouterr().err
    assert (rows.value, cols.value) == (2, 3) and "readDelimitedMatrix" not in err
    C.CDLL(None).free(C.cast(data, C.c_void_p))
    cut = tmp_path / "cut.csv"
    cut.write_text("1,2,3\n4,5,6\n\n7,8,9\n")
    cnn.readDelimitedMatrix(str(cut).encode(), C.byref(data), C.byref(rows), C.byref(cols))
    err = capfd.readouterr().err
    assert (rows.value, cols.value) == (2, 3) and "stopped at the empty line after row 2" in err
    C.CDLL(None).free(C.cast(data, C.c_void_p))
    ragged = tmp_path / "ragged.csv"
    ragged.write_text("1,2,3\n4,5\n7,8,9\n")
    cnn.readDelimitedMatrix(str(ragged).encode(), C.byref(data), C.byref(rows), C.byref(cols))
    err = capfd.readouterr().err
    assert (rows.value, cols.value) == (3, 3) and "1 of 3 rows do not have the 3 values" in err
    np.testing.assert_array_equal(as_array(data, 9), [1, 2, 3, 4, 5, 0, 7, 8, 9])
    C.CDLL(None).free(C.cast(data, C.c_void_p))
