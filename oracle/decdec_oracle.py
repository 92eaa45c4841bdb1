"""CPU oracle for DecDEC's decode-time linear-layer path (NumPy).

TEST INFRASTRUCTURE ONLY.  This module restates, on the CPU, the arithmetic of
the reference's CUDA kernels so that the HIP kernels can be checked against
it.  Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it; the product path (``decdec_amd``) never does.

Every function cites the reference text it follows (paths relative to the
reference checkout).  How each one is pinned, independently of its own
formula, is listed here and exercised in ``tests/test_oracle_*.py``:

* ``bucket_floors``        closed form of dec.cu:117-137; pinned by invariants
                           (floor[0]==a, floor[31]==0, floor[16]==b*15/16
                           exactly, power-of-two scalings exact) and by the
                           independent soft-float C restatement
                           (oracle/decdec_oracle.c) agreeing bit for bit.
* ``select_channels``      dec.cu:78-182; pinned by a per-bucket brute force
                           written as the kernel's membership test, by the
                           set invariants of a bucket partition, and by the
                           special case thresholds=sorted|x| (the recipe of
                           decdec_extension/tests/test_dec.py:21) where the
                           selected set must equal torch.topk per chunk.
* ``dec_geometry``         dec_config.cu:34-115; pure integers, pinned by the
                           hand-evaluated table for the benchmark shapes.
* residual pack / unpack   cheatsheet.py:99-125 vs dec.cu:243-253 are mutually
                           inverse: round trip; k_chunk=1024 reduces DEC to a
                           dense GEMV (textbook routine: numpy matmul).
* ``quantize_residual``    cheatsheet.py:59-90; pinned by |e-q*s|<=s/2 unless
                           clamped and by brute force over the 32-scale grid.
* any-precision layout     anyprec.cu:297-329 (store addresses of
                           dequant_kbit_store) and anyprec.cu:411-475 (load
                           addresses of matmul_kbit_32) read independently:
                           ``anyprec_dequant`` follows the former,
                           ``anyprec_gemv_kernel_order`` the latter, and they
                           must agree; plus pack->unpack round trip.
* LUT-GEMM BCQ             qmodule.py:61-92 (pack) vs lutgemm.cu:87-142
                           (kernel) vs evaltools.py:546-580 (dequant): the
                           identity w = scale*(q-zero) must be reproduced.
* SqueezeLLM               sqllm.cu:64-113,152-166 vs evaltools.py:583-645;
                           3-bit 96-bit stream checked against Python big ints.

Parity unpinned (cannot be pinned without running the reference on NVIDIA
hardware): the run-specific order of entries inside one bucket of the
reference selector (an atomicAdd race, dec.cu:148) and the last-bit fp16
rounding of outputs (atomic order).  The oracle fixes the order as ascending
channel index, one of the outcomes the reference can produce.
"""
from __future__ import annotations

import numpy as np

CHUNK_SIZE = 1024          # macros.h:8
NUM_THRESHOLDS = 32        # macros.h:18
BIT_WIDTH = 4              # macros.h:10
NIBBLES_PER_ELEMENT = 8    # macros.h:16
WARP_SIZE_REF = 32         # macros.h:13 (only enters the geometry formulas)
THREADS_PER_BLOCK = 1024   # macros.h:11
MAX_MATRIX_COLS_PER_BLOCK = 256  # macros.h:14


# ----------------------------------------------------------------------------
# dtype helpers: fp16 is numpy's float16; bf16 is emulated on float32 storage
# ----------------------------------------------------------------------------
def bf16_round(v):
    """Round float32 values to the nearest bfloat16 (ties to even), kept as float32."""
    a = np.asarray(v, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    nan = np.isnan(a)
    lsb = (u >> 16) & 1
    u = (u + 0x7FFF + lsb) & 0xFFFF0000
    out = u.astype(np.uint32).view(np.float32)
    out = np.where(nan, np.float32(np.nan), out)
    return out.astype(np.float32)


def _rounder(dtype: str):
    if dtype == "fp16":
        return lambda v: np.asarray(v, dtype=np.float32).astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_round
    if dtype == "fp32":
        return lambda v: np.asarray(v, dtype=np.float32)
    raise ValueError(dtype)


def to_f32(x, dtype: str):
    """Values of ``dtype`` as float32 (bf16 inputs are float32 arrays already rounded)."""
    return np.asarray(x).astype(np.float32)


# ----------------------------------------------------------------------------
# A1: bucket selector
# ----------------------------------------------------------------------------
def bucket_floors(a, b, dtype: str = "fp16") -> np.ndarray:
    """The 32 bucket floors of the selector, as float32 holding ``dtype`` values.

    dec.cu:117-130.  For idx < 16:  a + T( F(T(b - a)) * idx / 15 )
                     for idx >= 16:     T( F(b) * (31 - idx) / 16 )
    where T rounds to the activation dtype, F widens to float32, and the
    multiply and the divide are float32 operations (integer operands are
    converted to float32 first, as C++ does for ``float * uint32_t``).
    """
    T = _rounder(dtype)
    a32 = np.float32(T(a))
    b32 = np.float32(T(b))
    floors = np.zeros(NUM_THRESHOLDS, dtype=np.float32)
    half = NUM_THRESHOLDS // 2
    diff = np.float32(T(np.float32(b32 - a32)))
    for idx in range(NUM_THRESHOLDS):
        if idx < half:
            step = np.float32(np.float32(diff * np.float32(idx)) / np.float32(half - 1))
            floors[idx] = T(np.float32(a32 + np.float32(T(step))))
        else:
            v = np.float32(np.float32(b32 * np.float32(NUM_THRESHOLDS - idx - 1))
                           / np.float32(NUM_THRESHOLDS - half))
            floors[idx] = T(v)
    return floors


def bucket_ceils(floors: np.ndarray) -> np.ndarray:
    """dec.cu:133-137: ceil[i] = floor[i-1], ceil[0] = +inf."""
    ceils = np.empty_like(floors)
    ceils[0] = np.inf
    ceils[1:] = floors[:-1]
    return ceils


def num_rows_to_fetch(k_chunk: int, K: int) -> int:
    """decdec.cu:50 / dec.cu:48."""
    return k_chunk * K // CHUNK_SIZE


def select_channels(x, thresholds, k_chunk: int, dtype: str = "fp16"):
    """Bucket top-k selection of one activation vector.

    dec.cu:78-182 with thresholds[0], thresholds[k-1] read as decdec.cu:66-67.
    Returns (selected_rows int32[num_chunks*k_chunk], selected_activations
    float32[...], filled bool[...]).  Entry c*k_chunk+pos is chunk c's pos-th
    pick (dec.cu:169-171); slots that the reference leaves untouched (a short
    last chunk, or fewer members than k_chunk when |x| is inf/NaN) have
    filled=False, rows=-1.  Order inside one bucket: ascending channel index.
    A channel is a member of bucket i iff floor[i] <= |x| < ceil[i]
    (dec.cu:145-146); the test is made per bucket, so with non-monotone floors
    a channel can be a member of several buckets, exactly as in the kernel.
    """
    x32 = to_f32(x, dtype).reshape(-1)
    K = x32.shape[0]
    k = num_rows_to_fetch(k_chunk, K)
    num_chunks = (K + CHUNK_SIZE - 1) // CHUNK_SIZE
    rows = np.full(num_chunks * max(k_chunk, 1), -1, dtype=np.int32)
    acts = np.zeros(num_chunks * max(k_chunk, 1), dtype=np.float32)
    filled = np.zeros(num_chunks * max(k_chunk, 1), dtype=bool)
    if k == 0:
        return rows, acts, filled
    th = to_f32(thresholds, dtype).reshape(-1)
    floors = bucket_floors(th[0], th[k - 1], dtype)
    ceils = bucket_ceils(floors)
    ax = np.abs(x32)
    for c in range(num_chunks):
        lo = c * CHUNK_SIZE
        hi = min(lo + CHUNK_SIZE, K)
        kc = k_chunk * (hi - lo) // CHUNK_SIZE          # dec.cu:84-86
        if kc == 0:
            continue
        seg = ax[lo:hi]
        # membership matrix [32, len]; comparisons on exactly representable values
        member = (seg[None, :] >= floors[:, None]) & (seg[None, :] < ceils[:, None])
        count = 0
        for i in range(NUM_THRESHOLDS):
            idxs = np.nonzero(member[i])[0]
            take = min(kc - count, idxs.shape[0])       # dec.cu:165-166
            if take > 0:
                sel = idxs[:take] + lo
                base = c * k_chunk + count               # dec.cu:169
                rows[base:base + take] = sel
                acts[base:base + take] = x32[sel]
                filled[base:base + take] = True
            count += take
            if count == kc:
                break
    return rows, acts, filled


def select_channels_bruteforce(x, thresholds, k_chunk: int, dtype: str = "fp16"):
    """Same result as select_channels, written as nested scalar loops that mirror
    the kernel's per-(bucket, channel) test (dec.cu:140-177).  Slow; tiny inputs."""
    T = _rounder(dtype)
    xs = [float(v) for v in to_f32(x, dtype).reshape(-1)]
    K = len(xs)
    k = k_chunk * K // CHUNK_SIZE
    num_chunks = -(-K // CHUNK_SIZE)
    rows = [-1] * (num_chunks * max(k_chunk, 1))
    if k == 0:
        return np.array(rows, dtype=np.int32)
    th = to_f32(thresholds, dtype).reshape(-1)
    a = float(th[0]); b = float(th[k - 1])
    fl = []
    for i in range(32):
        if i < 16:
            d = float(T(np.float32(b) - np.float32(a)))
            s = np.float32(np.float32(d) * np.float32(i)) / np.float32(15)
            fl.append(float(T(np.float32(a) + np.float32(T(s)))))
        else:
            fl.append(float(T(np.float32(np.float32(b) * np.float32(31 - i)) / np.float32(16))))
    for c in range(num_chunks):
        lo = c * CHUNK_SIZE; hi = min(lo + CHUNK_SIZE, K)
        kc = k_chunk * (hi - lo) // CHUNK_SIZE
        out = []
        for i in range(32):
            ce = float("inf") if i == 0 else fl[i - 1]
            for ch in range(lo, hi):
                v = abs(xs[ch])
                if len(out) < kc and v >= fl[i] and v < ce:
                    out.append(ch)
            if len(out) >= kc:
                break
        for p, ch in enumerate(out):
            rows[c * k_chunk + p] = ch
    return np.array(rows, dtype=np.int32)


# ----------------------------------------------------------------------------
# A3: launch geometry reported by read_dec_config
# ----------------------------------------------------------------------------
def _ceil_div(a, b):
    return (a + b - 1) // b


def dec_geometry(K: int, N: int, n_tb: int, k_chunk: int, itemsize: int = 2,
                 max_shared_memory: int = 65536) -> dict:
    """dec_config.cu:34-115 and :159-182 as integer arithmetic.  Keys are those of
    read_dec_config (dec_config.cu:343-351)."""
    total = N // NIBBLES_PER_ELEMENT
    cpt = _ceil_div(total, n_tb)
    cpt = _ceil_div(cpt, WARP_SIZE_REF) * WARP_SIZE_REF
    if cpt > MAX_MATRIX_COLS_PER_BLOCK:
        times = _ceil_div(cpt, MAX_MATRIX_COLS_PER_BLOCK)
        bx = total // n_tb // times
        bx = _ceil_div(bx, WARP_SIZE_REF) * WARP_SIZE_REF
        cpt = bx * times
    else:
        bx = cpt
    num_blocks = _ceil_div(total, cpt)
    by = THREADS_PER_BLOCK // bx
    num_chunks = _ceil_div(K, CHUNK_SIZE)
    grid = min(max(num_chunks, num_blocks), n_tb)
    rows_to_fetch = k_chunk * num_chunks                      # dec_config.cu:81 (note: not k)
    row_select = k_chunk * NUM_THRESHOLDS * 4 + CHUNK_SIZE * itemsize
    dec_req = (rows_to_fetch * 4 + NIBBLES_PER_ELEMENT * bx * by * itemsize
               + bx * NIBBLES_PER_ELEMENT * itemsize + rows_to_fetch * itemsize)
    static = 4 * NUM_THRESHOLDS
    dyn = max(row_select, dec_req)
    status = 0
    if dyn + static > max_shared_memory:
        dec_req = NIBBLES_PER_ELEMENT * bx * by * itemsize + bx * NIBBLES_PER_ELEMENT * itemsize
        dyn = max(row_select, dec_req)
        status = -1 if dyn + static > max_shared_memory else 1
    return {
        "num_chunks": num_chunks, "chunk_size": CHUNK_SIZE, "k_chunk": k_chunk,
        "channels_per_tb": cpt, "n_tb": grid, "block_dim_x": bx, "block_dim_y": by,
        "shared_memory_size": dyn, "reduced_shared_memory": int(status == 1),
        "shared_memory_status": status, "fetch_blocks": num_blocks,
    }


# ----------------------------------------------------------------------------
# A2: residual ("cheatsheet") format and DEC math
# ----------------------------------------------------------------------------
def _torch_linspace_f32(start, end, steps: int) -> np.ndarray:
    """float32 linspace with torch's two-sided evaluation (start + i*step for the
    first half, end - (steps-1-i)*step for the second)."""
    start = np.float32(start); end = np.float32(end)
    step = np.float32((end - start) / np.float32(steps - 1))
    out = np.empty(steps, dtype=np.float32)
    for i in range(steps):
        if i < steps // 2:
            out[i] = np.float32(start + np.float32(step * np.float32(i)))
        else:
            out[i] = np.float32(end - np.float32(step * np.float32(steps - i - 1)))
    return out


def quantize_residual(E: np.ndarray):
    """Per-output-row 4-bit quantisation of a residual E[N, K] (fp16 values).

    cheatsheet.py:59-90: 32 candidate scales linspace(max/7/32, max/7, 32) in
    float32, q = clamp(round(e/s), -7, 7), pick the minimum float32 MSE,
    scale stored as fp16.  Returns (q int8[N, K], scales float16[N]).
    """
    E16 = np.asarray(E, dtype=np.float16)
    N, K = E16.shape
    q = np.zeros((N, K), dtype=np.int8)
    scales = np.zeros(N, dtype=np.float16)
    grid = 32
    for n in range(N):
        e = E16[n]
        max_scale = np.float16(np.float16(np.max(np.abs(e))) / np.float16(7))   # fp16 / python int
        start = np.float32(np.float16(max_scale / np.float16(grid)))
        cand = _torch_linspace_f32(start, np.float32(max_scale), grid)
        with np.errstate(divide="ignore", invalid="ignore"):
            qc = np.clip(np.rint(e.astype(np.float32)[None, :] / cand[:, None]), -7, 7)
        rec = qc * cand[:, None]
        mse = np.mean((e.astype(np.float32)[None, :] - rec.astype(np.float32)) ** 2, axis=1,
                      dtype=np.float32)
        if np.all(np.isnan(mse)):
            best = 0
        else:
            best = int(np.nanargmin(mse))
        scales[n] = np.float16(cand[best])
        qrow = qc[best]
        q[n] = np.nan_to_num(qrow, nan=0.0).astype(np.int8)
    return q, scales


def pack_residual(q: np.ndarray, scales: np.ndarray):
    """cheatsheet.py:99-125.  q int[N, K] in [-7, 7], scales [N].
    cheatsheet[c, m] = sum_j ((q[8m+j, c] + 8) & 0xF) << 4j   (int32[K, N/8])
    reordered_scales[j*N/8 + m] = scales[8m + j].
    """
    N, K = q.shape
    assert N % 8 == 0, "row_count is not a multiple of 8, cannot pack nibbles"  # cheatsheet.py:46
    nib = (q.astype(np.int64) + 8) & 0xF                    # [N, K]
    nibT = nib.T.reshape(K, N // 8, 8)                      # [K, m, j]
    shifts = (4 * np.arange(8, dtype=np.int64))[None, None, :]
    words = np.sum(nibT << shifts, axis=2).astype(np.uint32)
    cheatsheet = words.view(np.int32).reshape(K, N // 8)
    reordered = np.asarray(scales).reshape(N // 8, 8).T.reshape(-1).copy()
    return cheatsheet, reordered


def unpack_residual(cheatsheet: np.ndarray, reordered_scales: np.ndarray) -> np.ndarray:
    """Dequantised residual R[K, N] in float64 as the kernel reads it.
    dec.cu:243-253: nibble j of word (c, m) -> output 8m+j, value (nib-8) * scale,
    scale = reordered_scales[j*N/8 + m] (dec.cu:222-225)."""
    K, M = cheatsheet.shape
    N = M * 8
    u = cheatsheet.view(np.uint32).astype(np.int64)
    shifts = (4 * np.arange(8, dtype=np.int64))[None, None, :]
    nib = (u[:, :, None] >> shifts) & 0xF                   # [K, M, 8]
    sc = np.asarray(reordered_scales).astype(np.float64).reshape(8, M).T  # [M, 8]
    R = (nib - 8).astype(np.float64) * sc[None, :, :]
    return R.reshape(K, N)


def dec_apply(x, cheatsheet, reordered_scales, rows) -> np.ndarray:
    """Exact (float64) DEC contribution:  out[n] = sum_{r in rows} R[r, n] * x[r].
    dec.cu:231-256 without the fp16 roundings.  ``rows`` may contain duplicates
    (each occurrence counts, as in the kernel) and -1 entries (skipped)."""
    x64 = np.asarray(x).astype(np.float64).reshape(-1)
    rows = np.asarray(rows).reshape(-1)
    rows = rows[rows >= 0]
    K, M = cheatsheet.shape
    u = cheatsheet.view(np.uint32)[rows].astype(np.int64)  # [k, M]
    shifts = (4 * np.arange(8, dtype=np.int64))[None, None, :]
    nib = ((u[:, :, None] >> shifts) & 0xF) - 8             # [k, M, 8]
    sc = np.asarray(reordered_scales).astype(np.float64).reshape(8, M).T
    contrib = np.einsum("kmj,k->mj", nib.astype(np.float64), x64[rows]) * sc
    return contrib.reshape(-1)


def dec_apply_reference_rounding(x, cheatsheet, reordered_scales, rows, block_dim_y: int):
    """DEC contribution with the reference's fp16 rounding sequence (dec.cu:248-275):
    per y-lane sequential ``acc += (nib*scale)*act`` in fp16 over rows y, y+by, ...,
    then a sequential fp16 sum over y.  Used only to show how far the reference's own
    arithmetic sits from the exact value."""
    x16 = np.asarray(x, dtype=np.float16).reshape(-1)
    rows = np.asarray(rows).reshape(-1)
    K, M = cheatsheet.shape
    N = M * 8
    sc = np.asarray(reordered_scales, dtype=np.float16).reshape(8, M).T.reshape(-1)   # [N] natural
    u = cheatsheet.view(np.uint32)
    shifts = (4 * np.arange(8, dtype=np.uint32))[None, :]
    partial = np.zeros((block_dim_y, N), dtype=np.float16)
    for i, r in enumerate(rows):
        if r < 0:
            continue
        y = i % block_dim_y
        nib = ((u[r][:, None] >> shifts) & 0xF).astype(np.int32).reshape(-1) - 8
        t = (nib.astype(np.float16) * sc).astype(np.float16)
        t = (t * x16[r]).astype(np.float16)
        partial[y] = (partial[y] + t).astype(np.float16)
    out = np.zeros(N, dtype=np.float16)
    for y in range(block_dim_y):
        out = (out + partial[y]).astype(np.float16)
    return out


# ----------------------------------------------------------------------------
# B1/B4: any-precision bitplanes
# ----------------------------------------------------------------------------
def _anyprec_channel_map(K: int):
    """For every channel c: (word index w within the row, bit position).
    anyprec.cu:297-329: chunk i of 1024 channels, lane t, word w = 32 i + t;
    the store address is 8*eff*j + 1024 i + 8 t + e for dq_w[4j + e/2][e%2], and
    the lookup walk (:314-324, with the nibble split of :53-63) gives element
    (j, e) <-> bit 31 - (8j + e).  eff = 32, or (K % 1024)/32 in a tail chunk."""
    assert K % 32 == 0
    word = np.zeros(K, dtype=np.int64)
    bit = np.zeros(K, dtype=np.int64)
    nfull = K // 1024
    for i in range(_ceil_div(K, 1024)):
        eff = 32 if i < nfull else (K % 1024) // 32
        for t in range(eff):
            for j in range(4):
                for e in range(8):
                    c = 1024 * i + 8 * eff * j + 8 * t + e
                    word[c] = 32 * i + t
                    bit[c] = 31 - (8 * j + e)
    return word, bit


def anyprec_pack(idx: np.ndarray, bits: int) -> np.ndarray:
    """idx uint[N, K] in [0, 2^bits) -> qweight int32[bits, N, K/32]; plane 0 is the MSB."""
    N, K = idx.shape
    word, bit = _anyprec_channel_map(K)
    chan_of = np.empty((K // 32, 32), dtype=np.int64)
    chan_of[word, bit] = np.arange(K)
    q = np.zeros((bits, N, K // 32), dtype=np.uint32)
    sh = np.arange(32, dtype=np.uint32)[None, None, :]
    for p in range(bits):
        pb = ((idx.astype(np.uint32) >> np.uint32(bits - 1 - p)) & np.uint32(1))  # [N, K]
        q[p] = np.bitwise_or.reduce(pb[:, chan_of] << sh, axis=2)
    return q.view(np.int32)


def anyprec_unpack(qweight: np.ndarray, bits: int) -> np.ndarray:
    """qweight int32[>=bits, N, K/32] -> idx uint8[N, K] (first ``bits`` planes only,
    decdec.cu:295)."""
    q = qweight.view(np.uint32)
    _, N, W = q.shape
    K = W * 32
    word, bit = _anyprec_channel_map(K)
    idx = np.zeros((N, K), dtype=np.uint32)
    for p in range(bits):
        b = (q[p][:, word] >> bit.astype(np.uint32)[None, :]) & np.uint32(1)
        idx |= b << np.uint32(bits - 1 - p)
    return idx.astype(np.uint16 if bits > 8 else np.uint8)


def anyprec_dequant(qweight: np.ndarray, lut: np.ndarray, bits: int) -> np.ndarray:
    """W[N, K] = lut[n, idx(n, c)]   (dequant_kbit_store, anyprec.cu:261-331)."""
    idx = anyprec_unpack(qweight, bits).astype(np.int64)
    return np.take_along_axis(np.asarray(lut), idx, axis=1)


def anyprec_gemv(x, qweight, lut, bits: int) -> np.ndarray:
    """Exact float64 value of out[n] = sum_c lut[n, idx(n,c)] * x[c]."""
    W = anyprec_dequant(qweight, lut, bits).astype(np.float64)
    return W @ np.asarray(x).astype(np.float64).reshape(-1)


def anyprec_gemv_kernel_order(x, qweight, lut, bits: int) -> np.ndarray:
    """Second, independent reading of the layout: follows matmul_kbit_32's *load*
    addresses (anyprec.cu:411-475) instead of dequant_kbit_store's store addresses.
    Lane t of chunk i reads x at float4 index eff*j + 128 i + t (8 halves each) and
    multiplies element e of group j with the LUT entry indexed by bit 31-(8j+e)."""
    q = qweight.view(np.uint32)
    _, N, Wn = q.shape
    K = Wn * 32
    x64 = np.asarray(x).astype(np.float64).reshape(-1)
    lut64 = np.asarray(lut).astype(np.float64)
    out = np.zeros(N, dtype=np.float64)
    nfull = K // 1024
    for i in range(_ceil_div(K, 1024)):
        eff = 32 if i < nfull else (K % 1024) // 32
        for t in range(eff):
            w = 32 * i + t
            planes = [q[p][:, w].astype(np.int64) for p in range(bits)]
            for j in range(4):
                base = 8 * (eff * j + 128 * i + t)
                for e in range(8):
                    pos = 31 - (8 * j + e)
                    idx = np.zeros(N, dtype=np.int64)
                    for p in range(bits):
                        idx |= ((planes[p] >> pos) & 1) << (bits - 1 - p)
                    out += lut64[np.arange(N), idx] * x64[base + e]
    return out


def uniform_quantize_rows(W: np.ndarray, bits: int):
    """Per-row uniform 2^bits-level quantiser used to synthesise any-precision /
    SqueezeLLM layers for tests and benches: LUT = linspace(min, max), nearest level.
    Not part of the reference (its quantisers are offline tools); returns
    (idx uint8[N,K], lut float16[N, 2^bits])."""
    W32 = np.asarray(W, dtype=np.float32)
    lo = W32.min(axis=1, keepdims=True)
    hi = W32.max(axis=1, keepdims=True)
    L = 1 << bits
    lut = (lo + (hi - lo) * (np.arange(L, dtype=np.float32)[None, :] / np.float32(L - 1)))
    lut16 = lut.astype(np.float16)
    step = np.maximum(hi - lo, 1e-12) / np.float32(L - 1)
    idx = np.clip(np.rint((W32 - lo) / step), 0, L - 1).astype(np.uint8)
    return idx, lut16


# ----------------------------------------------------------------------------
# B2: LUT-GEMM binary-coding quantisation
# ----------------------------------------------------------------------------
def awq_pseudo_quantize(W: np.ndarray, bits: int, group_size: int):
    """quantizer.py:216-258 (zero_point=True): per group of ``group_size`` input
    channels, scales=(max-min).clamp(1e-5)/(2^b-1), zeros=clamp(-round(min/scales)),
    q = clamp(round(w/scales)+zeros, 0, 2^b-1).  Returns (q int[N,K], scales[N,G],
    zeros[N,G]) in float32."""
    W32 = np.asarray(W, dtype=np.float32)
    N, K = W32.shape
    G = K // group_size
    w = W32.reshape(N * G, group_size)
    mx = w.max(axis=1, keepdims=True)
    mn = w.min(axis=1, keepdims=True)
    max_int = 2 ** bits - 1
    scales = np.maximum(mx - mn, np.float32(1e-5)) / np.float32(max_int)
    zeros = np.clip(-np.rint(mn / scales), 0, max_int)
    q = np.clip(np.rint(w / scales) + zeros, 0, max_int)
    return (q.reshape(N, K).astype(np.int32), scales.reshape(N, G).astype(np.float32),
            zeros.reshape(N, G).astype(np.float32))


def bcq_pack(q: np.ndarray, scales: np.ndarray, zeros: np.ndarray, bits: int):
    """qmodule.py:61-92 (convert_bcq_format).  q int[N,K]; scales, zeros [N,G].
    Returns (q_weight int32[K/32, bits, N], alpha float32[G, bits, N],
    q_bias float32[G, N]):  alpha[g,p,n] = scales/2 * 2^p,
    q_bias = sum_p alpha - scales*zeros, bit (c%32) of q_weight[c/32, p, n] = bit p of q."""
    N, K = q.shape
    half = scales / np.float32(2.0)
    alpha = half[:, :, None] * (2.0 ** np.arange(bits, dtype=np.float32))[None, None, :]  # [N,G,B]
    offset = alpha.sum(-1) - scales * zeros                                                # [N,G]
    binary = np.zeros((N, K, bits), dtype=np.int64)
    for p in range(bits):
        binary[:, :, p] = (q >> p) & 1
    b = binary.transpose(0, 2, 1).reshape(N, bits, K // 32, 32)
    words = np.sum(b << np.arange(32, dtype=np.int64)[None, None, None, :], axis=3)
    q_weight = words.astype(np.uint32).view(np.int32).transpose(2, 1, 0).copy()           # [K/32,B,N]
    return (q_weight, alpha.transpose(1, 2, 0).astype(np.float32).copy(),
            offset.T.astype(np.float32).copy())


def lutgemm_dequant(q_weight, alpha, q_bias, group_size: int) -> np.ndarray:
    """W[N, K] in float64: sum_p alpha[g,p,n] * (2*bit - 1) + q_bias[g,n]
    (evaltools.py:546-580; lutgemm.cu:113-142 computes the same sum tile by tile)."""
    qw = q_weight.view(np.uint32)
    KT, B, N = qw.shape
    K = KT * 32
    bits_ = ((qw[:, :, :, None] >> np.arange(32, dtype=np.uint32)[None, None, None, :]) & 1)
    bits_ = bits_.transpose(0, 3, 1, 2).reshape(K, B, N).astype(np.float64)   # [K,B,N]
    delta = bits_ * 2.0 - 1.0
    g = np.arange(K) // group_size
    a = np.asarray(alpha).astype(np.float64)[g]          # [K,B,N]
    qb = np.asarray(q_bias).astype(np.float64)[g]        # [K,N]
    return ((delta * a).sum(axis=1) + qb).T


def lutgemm_gemv(x, q_weight, alpha, q_bias, group_size: int) -> np.ndarray:
    return lutgemm_dequant(q_weight, alpha, q_bias, group_size) @ \
        np.asarray(x).astype(np.float64).reshape(-1)


# ----------------------------------------------------------------------------
# B3: SqueezeLLM
# ----------------------------------------------------------------------------
def sqllm_pack(idx: np.ndarray, bits: int) -> np.ndarray:
    """idx uint[N, K] -> mat int32[K*bits/32, N].
    4-bit: word c/8, field 4*(c%8) (sqllm.cu:152-166).  3-bit: 32 channels form a
    96-bit little-endian stream over 3 words, field at bit 3*(c%32) (sqllm.cu:64-113)."""
    N, K = idx.shape
    assert bits in (3, 4)
    if bits == 4:
        v = idx.astype(np.uint64).reshape(N, K // 8, 8)
        words = np.sum(v << (4 * np.arange(8, dtype=np.uint64))[None, None, :], axis=2)
        return words.astype(np.uint32).view(np.int32).T.copy()
    out = np.zeros((N, K // 32, 3), dtype=np.uint32)
    for j in range(32):
        pos = 3 * j
        w, off = divmod(pos, 32)
        val = idx.reshape(N, K // 32, 32)[:, :, j].astype(np.uint64)
        out[:, :, w] |= ((val << np.uint64(off)) & np.uint64(0xFFFFFFFF)).astype(np.uint32)
        if off + 3 > 32:
            out[:, :, w + 1] |= (val >> np.uint64(32 - off)).astype(np.uint32)
    return out.reshape(N, K // 32 * 3).view(np.int32).T.copy()


def sqllm_unpack(mat: np.ndarray, bits: int) -> np.ndarray:
    """mat int32[K*bits/32, N] -> idx uint8[N, K]."""
    m = mat.view(np.uint32).T.astype(np.uint64)      # [N, R]
    N, R = m.shape
    if bits == 4:
        f = (m[:, :, None] >> (4 * np.arange(8, dtype=np.uint64))[None, None, :]) & np.uint64(0xF)
        return f.reshape(N, R * 8).astype(np.uint8)
    g = m.reshape(N, R // 3, 3)
    idx = np.zeros((N, R // 3, 32), dtype=np.uint8)
    for j in range(32):
        pos = 3 * j
        w, off = divmod(pos, 32)
        val = g[:, :, w] >> np.uint64(off)
        if off + 3 > 32:
            val = val | (g[:, :, w + 1] << np.uint64(32 - off))
        idx[:, :, j] = (val & np.uint64(7)).astype(np.uint8)
    return idx.reshape(N, R // 3 * 32)


def sqllm_dequant(mat, lut, bits: int) -> np.ndarray:
    idx = sqllm_unpack(mat, bits).astype(np.int64)
    return np.take_along_axis(np.asarray(lut), idx, axis=1)


def sqllm_gemv(x, mat, lut, bits: int) -> np.ndarray:
    return sqllm_dequant(mat, lut, bits).astype(np.float64) @ \
        np.asarray(x).astype(np.float64).reshape(-1)


# ----------------------------------------------------------------------------
# Synthetic inputs of the benchmark recipe (shared by tests and bench)
# ----------------------------------------------------------------------------
def make_activation(K: int, rng: np.random.Generator, outlier_frac: float = 0.01,
                    outlier_scale: float = 20.0) -> np.ndarray:
    """x ~ N(0,1) fp16 with a random 1 % of channels scaled x20."""
    x = rng.standard_normal(K).astype(np.float32)
    n_out = max(1, int(round(K * outlier_frac)))
    pos = rng.choice(K, size=n_out, replace=False)
    x[pos] *= outlier_scale
    return x.astype(np.float16)


def calibrate_thresholds(K: int, rng: np.random.Generator, draws: int = 64) -> np.ndarray:
    """thresholds.py:162-175: element i = max over calibration vectors of the i-th largest |x|."""
    th = np.zeros(K, dtype=np.float32)
    for _ in range(draws):
        x = make_activation(K, rng).astype(np.float32)
        th = np.maximum(th, np.sort(np.abs(x))[::-1])
    return th.astype(np.float16)


def full_layer_reference(x, W_deq, cheatsheet, reordered_scales, rows) -> np.ndarray:
    """y = deq(Wq) x + R_hat[:, sel] x[sel] in float64."""
    y = np.asarray(W_deq).astype(np.float64) @ np.asarray(x).astype(np.float64).reshape(-1)
    return y + dec_apply(x, cheatsheet, reordered_scales, rows)
