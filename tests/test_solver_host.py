"""Host-side pieces of the KFAC trust-region solver that need no GPU: the index shuffle
(device/gen_random.cu:76-98) and the arena sizing."""
import ctypes as C

import numpy as np

from fitre_amd import lib as L
from fitre_amd.structs import DEVICE_DATASET, KFAC_CURVATURE_INFO
from helpers import build_lenet

libc = C.CDLL(None)


def draw(m, n, seed):
    idx = (C.c_int * m)()
    libc.srand(seed)
    L.cnn.genRandomVector(idx, m, n)
    return np.array(idx[:])


def test_gen_random_vector_is_a_seeded_permutation():
    a = draw(1000, 1000, 1)
    assert sorted(a) == list(range(1000))
    assert (a != np.arange(1000)).sum() > 900                 # shuffled, not the identity
    np.testing.assert_array_equal(a, draw(1000, 1000, 1))     # srand fixes it
    assert (a != draw(1000, 1000, 2)).any()
    b = draw(37, 500, 3)                                      # a sample without repetition
    assert len(set(b)) == 37 and b.min() >= 0 and b.max() < 500
    assert draw(1, 1, 0).tolist() == [0]


def test_every_index_is_equally_likely_in_a_sample():
    counts = np.zeros(20)
    for seed in range(400):
        counts[draw(5, 20, seed)] += 1
    assert counts.min() > 60 and counts.max() < 140           # expectation 100 each


def test_arena_size_covers_the_persistent_buffers():
    model = build_lenet(32, bn=True)
    data = DEVICE_DATASET()
    data.trainSizeX, data.features, data.numClasses = 500, 3 * 32 * 32, 10
    info = KFAC_CURVATURE_INFO()
    info.inverseFreq = 1
    every = L.cnn.kfacTrustRegionMemRequired(C.byref(model), C.byref(data), C.byref(info))
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    layers = model.cLayers + model.lLayers
    persistent = (500 + info.OmegaZOffsets[layers] + info.LambdaGOffsets[layers] + 5 * model.pSize + 2 * model.zSize +
                  2 * 10 * 32)
    assert every > persistent + L.cnn.cnnHvMemRequired(C.byref(model)) + model.pSize
    info.inverseFreq = 10                                     # running averages of inputs, outputs and deltas
    assert L.cnn.kfacTrustRegionMemRequired(C.byref(model), C.byref(data), C.byref(info)) >= \
        every + 32 * 3 * 32 * 32 + 2 * model.zztSize
    assert L.cnn.kfacTrustRegionHostMemRequired(C.byref(data)) >= 500
