"""Second, independently written restatement of the reordering compressor,
in plain Python lists, kept as close to the reference's data flow as Python
allows (csrc/SpMM_API.cu:235-351).  Slow; used on small matrices only, to
cross-check the C oracle and the product compressor on random tiles whose
answer nobody traced by hand."""
import numpy as np


def keeps(bits):
    mag = bits & 0x7FFF
    return mag != 0 and mag <= 0x7C00


def _argmin(banks):
    best = 0
    for i in range(1, 32):
        if len(banks[i]) < len(banks[best]):
            best = i
    return best


def _argmax(banks):
    best = 0
    for i in range(1, 32):
        if len(banks[i]) > len(banks[best]):
            best = i
    return best


def compress_reorder(a):
    a = np.asarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    m_total, k_total = a.shape
    assert m_total % 128 == 0 and k_total % 64 == 0
    stream, offsets, running = [], [0], 0
    for ti in range(m_total // 128):
        for tj in range(k_total // 64):
            tile = a[ti * 128:(ti + 1) * 128, tj * 64:(tj + 1) * 64]
            banks = [[] for _ in range(32)]
            zero_pos = [-1] * 32
            for m in range(128):
                for n in range(64):
                    col = n ^ ((m % 8) << 3)
                    bank = (col // 2) % 32
                    bits = int(tile[m, n])
                    if keeps(bits):
                        banks[bank].append(bits | ((m * 64 + col) << 16))
                    elif zero_pos[bank] == -1:
                        zero_pos[bank] = m * 64 + col
            count = sum(len(b) for b in banks)
            for _ in range((4 - count % 4) % 4):
                b = _argmin(banks)
                assert zero_pos[b] != -1
                banks[b].append(zero_pos[b] << 16)
                count += 1
            vectors = count // 4
            rep, rem = divmod(vectors, 32)
            tail = [[] for _ in range(32)]
            main = [[] for _ in range(32)]
            for v in range(4):
                for lane in range(rem):
                    tail[lane].append(banks[_argmax(banks)].pop())
            for r in range(rep):
                for v in range(4):
                    for lane in range(32):
                        main[lane].append(banks[_argmax(banks)].pop())
            out = [None] * count
            for r in range(rep):
                for v in range(4):
                    for lane in range(32):
                        out[r * 128 + lane * 4 + v] = main[lane].pop()
            base = rep * 128
            for v in range(4):
                for lane in range(rem):
                    out[base + lane * 4 + v] = tail[lane].pop()
            assert None not in out
            stream.extend(out)
            running += count
            offsets.append(running // 4)
    offsets.append(running // 4)
    return np.array(stream, dtype=np.uint32), np.array(offsets, dtype=np.int32)
