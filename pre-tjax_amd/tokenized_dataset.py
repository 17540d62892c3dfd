"""Batch collation with the reference's tensor contract (tokenized_dataset.py:110-236 of
martin-kukla/pre-tjax) for callers of the kernel path, on any iterable of token lists --
no dataset download, no tokenizer.

A batch is the tuple ``(x, y_plus_one, x_mask, y_mask, yx_mask, x_indices, y_indices)`` of
numpy arrays stacked over the batch, exactly what ``train_gpt2_triton.py:287-292`` unpacks:

* ``y_plus_one`` int [B, T+1]: tokens, 0 = padding (the trainer feeds ``y[:, :-1]`` and
  scores ``y[:, 1:]``);
* ``y_mask`` [B, T, T]: lower triangular AND query-not-padding AND key-not-padding AND (with
  packing) same-document -- so a padded query's row is entirely zero;
* ``x_mask`` / ``yx_mask``: the encoder-side and cross masks of the same construction
  (unused by GPT-2, kept for the tuple layout); ``*_indices``: position inside the document.

``synthetic_items`` yields token lists of random lengths so that the collators, the padding
and the packing can be exercised (and benchmarked) without data.
"""
import numpy as np


def pad_and_trunc(toks, seq_len):
    """`toks` cut or zero-padded to exactly seq_len entries (tokenized_dataset.py:133)."""
    toks = list(toks)[:seq_len]
    return toks + [0] * (seq_len - len(toks))


def pack_batch(batch):
    """List of per-item tuples -> list of stacked arrays (tokenized_dataset.py:134)."""
    return [np.stack(column) for column in zip(*batch)]


def ones_block_diag(lens_dim0, lens_dim1):
    """Block-diagonal 0/1 matrix: block i is lens_dim0[i] x lens_dim1[i] (:147-155)."""
    out = np.zeros((int(sum(lens_dim0)), int(sum(lens_dim1))))
    r = c = 0
    for h, w in zip(lens_dim0, lens_dim1):
        out[r:r + h, c:c + w] = 1.0
        r, c = r + h, c + w
    return out


def create_packs(x_lens, y_lens):
    return ones_block_diag(x_lens, x_lens), ones_block_diag(y_lens, y_lens), ones_block_diag(y_lens, x_lens)


def create_indices(lens):
    return np.concatenate([np.arange(n) for n in lens])


def build_masks(x, y, x_packs=None, y_packs=None, yx_packs=None):
    """(x_mask [Tx,Tx], y_mask [Ty,Ty], yx_mask [Ty,Tx]) as float 0/1 arrays (:110-131)."""
    x_real = (x != 0).astype(np.float64)
    y_real = (y != 0).astype(np.float64)
    x_mask = np.outer(x_real, x_real)
    y_mask = np.tri(y.shape[0]) * np.outer(y_real, y_real)
    yx_mask = np.outer(y_real, x_real)
    if x_packs is not None:
        x_mask = x_mask * x_packs
    if y_packs is not None:
        y_mask = y_mask * y_packs
    if yx_packs is not None:
        yx_mask = yx_mask * yx_packs
    return x_mask, y_mask, yx_mask


def _fit_lens(lens, seq_len):
    """Document lengths made to sum to seq_len: the last one is cut, or a filler document
    covers the padded tail (:176-181)."""
    lens = list(lens)
    if sum(lens) > seq_len:
        lens[-1] = seq_len - sum(lens[:-1])
    else:
        lens.append(seq_len - sum(lens))
    return lens


def convert_batch_item(x, y, seq_len, x_lens=None, y_lens=None):
    """One batch row from token lists x, y (:165-192); `*_lens` = lengths of the documents
    packed into the row."""
    x = np.array(pad_and_trunc(x, seq_len))
    y_plus_one = np.array(pad_and_trunc(y, seq_len + 1))
    y = y_plus_one[:-1]
    if x_lens is not None:
        assert y_lens is not None
        x_lens, y_lens = _fit_lens(x_lens, seq_len), _fit_lens(y_lens, seq_len)
        packs = create_packs(x_lens, y_lens)
        x_idx, y_idx = create_indices(x_lens), create_indices(y_lens)
    else:
        packs = (None, None, None)
        x_idx, y_idx = np.arange(seq_len), np.arange(seq_len)
    return (x, y_plus_one) + build_masks(x, y, *packs) + (x_idx, y_idx)


def complete_last_batch(batch, batch_size, seq_len):
    """Fill a short batch with all-padding rows (:137-145)."""
    while len(batch) < batch_size:
        batch.append(convert_batch_item([], [], seq_len))
    return batch


def get_batched_examples(items, batch_size, seq_len, start_tok, end_tok, drop_last=True):
    """One document per row: y = [start] + item['y'] + [end], padded / cut (:193-204)."""
    batch = []
    for item in items:
        batch.append(convert_batch_item(item["x"], [start_tok] + list(item["y"]) + [end_tok], seq_len))
        if len(batch) == batch_size:
            yield pack_batch(batch)
            batch = []
    if batch and not drop_last:
        yield pack_batch(complete_last_batch(batch, batch_size, seq_len))


def get_batched_examples_packed(items, batch_size, seq_len, start_tok, end_tok, pack_frac=0.5):
    """Several documents per row: a document is appended to the current row while both of its
    sides are shorter than pack_frac * seq_len (:206-230)."""
    rows, x_lens, y_lens = [], [], []
    for item in items:
        ix, iy = list(item["x"]), [start_tok] + list(item["y"]) + [end_tok]
        if rows and len(rows[-1][0]) < seq_len * pack_frac and len(rows[-1][1]) < seq_len * pack_frac:
            rows[-1] = (rows[-1][0] + ix, rows[-1][1] + iy)
            x_lens[-1].append(len(ix))
            y_lens[-1].append(len(iy))
        else:
            rows.append((ix, iy))
            x_lens.append([len(ix)])
            y_lens.append([len(iy)])
        if len(rows) == batch_size:
            yield pack_batch([convert_batch_item(rx, ry, seq_len, xl, yl)
                              for (rx, ry), xl, yl in zip(rows, x_lens, y_lens)])
            rows, x_lens, y_lens = [], [], []


def synthetic_items(n_items, vocab_size, min_len, max_len, seed=0):
    """Token lists of random length in [min_len, max_len] with ids in [3, vocab_size) -- ids
    0, 1, 2 stay free for padding, start and end."""
    rng = np.random.default_rng(seed)
    for _ in range(n_items):
        n = int(rng.integers(min_len, max_len + 1))
        yield {"x": [], "y": rng.integers(3, vocab_size, size=n).tolist()}
