"""Re-encode the reference-held known-answer data that pins this hot path.

Run in the build container only (it reads /root/reference, which never
travels):   python tests/golden/make_fixtures.py

Source data: the .npy arrays the reference's own tests load in
tests/lava/lib/dl/netx/test_blocks.py:180-228 (LIF dense block, gts/dense),
:230-280 (RF_IZ complex input block, gts/complex_dense/{in,current}.npy) and
:282-332 (RF complex dense block, gts/complex_dense).  They are data, not
code; they are stored here bit-packed / narrowed so the three sets fit in
about 0.4 MB.  Nothing of the reference is imported or executed.
"""
import os
import numpy as np

SRC = '/root/reference/tests/lava/lib/dl/netx/gts/'
DST = os.path.dirname(os.path.abspath(__file__))


def bits(a):
    a = np.asarray(a)
    assert set(np.unique(a)) <= {0, 1}
    return np.packbits(a.astype(np.uint8), axis=-1)


def narrow(a, dtype):
    b = np.asarray(a).astype(dtype)
    assert np.array_equal(b.astype(np.float64), np.asarray(a, dtype=np.float64))
    return b


def main():
    d = SRC + 'dense/'
    np.savez_compressed(
        os.path.join(DST, 'netx_dense_lif.npz'),
        in_bits=bits(np.load(d + 'in.npy')),            # [200, 2000] input spikes
        weight=narrow(np.load(d + 'weight.npy'), np.int16),   # [256, 200]
        out_bits=bits(np.load(d + 'out.npy')),          # [256, 2000] output spikes
        num_steps=np.int64(2000))
    c = SRC + 'complex_dense/'
    np.savez_compressed(
        os.path.join(DST, 'netx_complex_dense_rf.npz'),
        in_bits=bits(np.load(c + 'in.npy')),            # [200, 2000]
        weight_real=narrow(np.load(c + 'weight_r.npy'), np.int8),    # [256, 200]
        weight_imag=narrow(np.load(c + 'weight_img.npy'), np.int8),  # [256, 200]
        out_bits=bits(np.load(c + 'out.npy')),          # [256, 2000] RF dense output spikes
        iz_out_bits=bits(np.load(c + 'current.npy')),   # [200, 2000] RF_IZ input-block output spikes
        num_steps=np.int64(2000))
    for f in ('netx_dense_lif.npz', 'netx_complex_dense_rf.npz'):
        print(f, os.path.getsize(os.path.join(DST, f)), 'bytes')


if __name__ == '__main__':
    main()
