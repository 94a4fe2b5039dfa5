"""A step's work, flattened: rows of (request, next tokens) become flat integer arrays,
uploaded in one copy (reference atomserve/runner.py:87-158, 215-241).

A `Row` says: these tokens, at positions start.., for the request whose pages are
these tables; logits are wanted at these places among them.  Everything before `start`
is already in the cache.  Rows of any length mix freely in one step.
"""

from dataclasses import dataclass, field

import numpy as np
import torch

from atomserve_amd.cache.manager import RELEASED


@dataclass
class Row:
    """tokens: the new tokens, at positions start, start + 1, ...
    tables: the request's block table in each paged group; must cover every new position
    want:   indices into `tokens` whose next-token logits are asked for
    state_slot: the request's slot in the fixed-size state tables, or -1
    store:  False for a filler row whose keys must not be written anywhere
    """

    tokens: list
    start: int
    tables: list
    want: list = field(default_factory=list)
    state_slot: int = -1
    store: bool = True


def _leading_released(table: list) -> int:
    n = 0
    while n < len(table) and table[n] == RELEASED:
        n += 1
    return n


def slot_of(block_table: list, position: int, block_size: int) -> int:
    """Pool slot of the token at `position` (reference atomserve/runner.py:37-39)."""
    return block_table[position // block_size] * block_size + position % block_size


class PagedLayerView:
    """What an attention mixer sees of its cache in one step."""

    __slots__ = ("k_pages", "v_pages", "slots", "block_tables", "writes", "block_size")

    def __init__(self, k_pages, v_pages, slots, block_tables, writes, block_size):
        self.k_pages, self.v_pages, self.slots, self.block_tables = k_pages, v_pages, slots, block_tables
        self.writes, self.block_size = writes, block_size


class StateLayerView:
    """What a mixer with fixed-size state sees: its state table and each row's slot."""

    __slots__ = ("state", "row_slots", "writes")

    def __init__(self, state, row_slots, writes):
        self.state, self.row_slots, self.writes = state, row_slots, writes


class RowSplit:
    """A step's rows sorted as one kind of mixer asked (`Mixer.row_split` = (short, tile)):
    short_tokens [Ns] int32: the tokens of rows with at most `short` tokens, those that see most keys first;
    long_tiles [Nt, 4] int32: (first flat token, count, row, first position) per `tile` consecutive tokens
    of longer rows, those that see most keys first; max_short_context: host bound on the context of a
    short token; tile_keys: the keys that the tiles' last tokens see, added up (what the tiles' attention
    has to walk: a kernel may choose by it how to cut its work)."""

    def __init__(self, short: int, tile: int):
        if short < 0 or tile < 1:
            raise ValueError(f"a row split is (short >= 0, tile >= 1), not {(short, tile)}")
        self.short, self.tile = short, tile
        self.tokens, self.tiles, self.max_short_context, self.tile_keys = [], [], 0, 0
        self.short_tokens = self.long_tiles = None  # on the device once the step is packed
        self.num_short_tokens = self.num_long_tiles = 0


class StepBatch:
    """The flat batch of one step, on the device.

    token_ids, positions, tok_row [T] int32   (tok_row: which row a token belongs to)
    logits_rows [B'] int32                    flat indices of the wanted positions
    group_slots[g] [T], group_tables[g] [R, W_g] int32, per paged group
    all_tokens [T]: every token (in a decode step those with the longest contexts first);
    split((short, tile)): the rows sorted as a mixer asks (`RowSplit`), one for every distinct answer of
    the model's mixers (`row_splits`), so that mixers with different kernels share a step;
    row_first, row_len, row_start, row_slots [R] int32 (for mixers with per-request state)
    """

    def __init__(self, rows, block_size: int, num_paged_groups: int, vocab_size: int, device, pools=None,
                 staging=None, table_width: int = 0, max_context: int = 0, into=None, row_splits=()):  # fmt: skip
        """table_width, max_context: lower bounds that make the layout of a step independent of
        its rows (a step whose kernels were captured in a graph is replayed with new contents).
        into: an earlier batch of identical layout whose device buffer receives this one's arrays.
        row_splits: the distinct (short, tile) that the model's mixers ask for."""
        if not rows:
            raise ValueError("a step needs at least one row")
        bs = block_size
        self.splits = {tuple(key): RowSplit(*key) for key in row_splits}
        # A prompt's portion is hundreds of tokens: its fields are made as arrays; the single tokens of decoding
        # requests between such rows gather in lists, which become arrays when the next long row (or the end) comes.
        fields_of_tokens = 3 + num_paged_groups  # token ids, positions, rows, and a slot per group
        done = [[] for _ in range(fields_of_tokens)]  # arrays, in the order of the rows
        few = [[] for _ in range(fields_of_tokens)]  # what the short rows since the last array have added

        def settle():
            for arrays, values in zip(done, few):
                if values:
                    arrays.append(np.asarray(values, dtype=np.int32))
                    values.clear()

        want = []
        row_first, row_len, row_start, row_slots = [], [], [], []
        widths = [max(1, table_width)] * num_paged_groups
        flat = 0
        self.max_context = 0
        for r, row in enumerate(rows):
            n, end = len(row.tokens), row.start + len(row.tokens)
            if n < 1 or row.start < 0:
                raise ValueError(f"bad row: {n} tokens at position {row.start}")
            if n == 1 and len(row.tables) == num_paged_groups and all(w == 0 for w in row.want) \
                    and 0 <= row.tokens[0] < vocab_size:  # fmt: skip
                # A decoding request's one token, the common row of a step: the same checks and entries as
                # below, without their loops.
                start, page_at = row.start, row.start // bs
                for g, table in enumerate(row.tables):
                    if end > len(table) * bs:
                        raise ValueError(f"block table holds {len(table) * bs} slots, need {end}")
                    if table[page_at] == RELEASED:
                        raise ValueError("block table has given back a page that this row writes")
                    few[3 + g].append(table[page_at] * bs + start % bs if row.store else -1)
                    if page_at >= widths[g]:
                        widths[g] = page_at + 1
                few[0].append(row.tokens[0])
                few[1].append(start)
                few[2].append(r)
                want.extend([flat] * len(row.want))
                for split in self.splits.values():
                    if split.short >= 1:
                        split.tokens.append(flat)
                        if end > split.max_short_context:
                            split.max_short_context = end
                    else:
                        split.tiles.append((flat, 1, r, start))
                        split.tile_keys += end
                if end > self.max_context:
                    self.max_context = end
                row_first.append(flat)
                row_len.append(1)
                row_start.append(start)
                row_slots.append(row.state_slot)
                flat += 1
                continue
            if any(not 0 <= w < n for w in row.want):
                raise ValueError(f"bad row: wanted places {row.want} outside its {n} tokens")
            long = n > 64  # a prompt: checked and addressed as arrays, not token by token
            if long:
                ids = np.asarray(row.tokens, dtype=np.int64)
                bad = ids[(ids < 0) | (ids >= vocab_size)].tolist()
            else:
                bad = [t for t in row.tokens if not 0 <= t < vocab_size]
            if bad:
                raise ValueError(f"token id {bad[0]} is outside the vocabulary of {vocab_size}")
            if len(row.tables) != num_paged_groups:
                raise ValueError(f"row has {len(row.tables)} block tables, the model has {num_paged_groups} groups")
            if long:
                settle()
                places = np.arange(row.start, end, dtype=np.int64)
                done[0].append(ids.astype(np.int32))
                done[1].append(places.astype(np.int32))
                done[2].append(np.full(n, r, dtype=np.int32))
            else:
                few[0].extend(row.tokens)
                few[1].extend(range(row.start, end))
                few[2].extend([r] * n)
            for g, table in enumerate(row.tables):
                if end > len(table) * bs:
                    raise ValueError(f"block table holds {len(table) * bs} slots, need {end}")
                first_page, last_page = row.start // bs, (end - 1) // bs
                if any(table[b] == RELEASED for b in range(first_page, last_page + 1)):
                    raise ValueError("block table has given back a page that this row writes")
                if long and row.store:
                    pages = np.asarray(table[first_page : last_page + 1], dtype=np.int64)
                    done[3 + g].append((pages[places // bs - first_page] * bs + places % bs).astype(np.int32))
                elif long:
                    done[3 + g].append(np.full(n, -1, dtype=np.int32))
                elif row.store:
                    few[3 + g].extend(table[p // bs] * bs + p % bs for p in range(row.start, end))
                else:
                    few[3 + g].extend([-1] * n)
                widths[g] = max(widths[g], (end + bs - 1) // bs)
            want.extend(flat + w for w in row.want)
            for split in self.splits.values():
                if n <= split.short:
                    split.tokens.extend(range(flat, flat + n))
                    split.max_short_context = max(split.max_short_context, end)
                else:
                    for q0 in range(0, n, split.tile):
                        split.tiles.append((flat + q0, min(split.tile, n - q0), r, row.start + q0))
                        split.tile_keys += row.start + min(n, q0 + split.tile)
            self.max_context = max(self.max_context, end)
            row_first.append(flat)
            row_len.append(n)
            row_start.append(row.start)
            row_slots.append(row.state_slot)
            flat += n
        settle()
        tok, pos, trow, *slots = [arrays[0] if len(arrays) == 1 else np.concatenate(arrays) for arrays in done]

        # Work items of the prefill kernel, the ones that see most keys first: the kernel hands
        # them out in this order and pairs the longest with the shortest on a compute unit.
        for split in self.splits.values():
            split.tiles.sort(key=lambda t: -(t[3] + t[1]))
            split.tokens.sort(key=lambda t: -int(pos[t]))  # single queries too: the longest contexts first
            split.max_short_context = max(split.max_short_context, max_context if split.tokens else 0)
        self.max_context = max(self.max_context, max_context)
        T, R = flat, len(rows)
        tables = []
        for g in range(num_paged_groups):
            w = widths[g]
            arr = np.zeros((R, w), dtype=np.int32)
            for r, row in enumerate(rows):
                t = row.tables[g][:w]
                arr[r, : len(t)] = t
            arr[arr == RELEASED] = 0  # a page that was given back: its place names page 0, which nobody reads there
            tables.append(arr)

        # Every token; in a decode step those that see most keys first, the order in which the attention
        # kernel's workgroups take whole contexts (`advance` keeps it: the contexts grow together).
        every = range(T)
        if T == R and T > 1:
            every = np.argsort(-pos.astype(np.int64), kind="stable")
        fields = [("token_ids", tok), ("positions", pos), ("tok_row", trow), ("logits_rows", want),
                  ("all_tokens", every), ("row_first", row_first), ("row_len", row_len), ("row_start", row_start),
                  ("row_slots", row_slots)]  # fmt: skip
        for j, split in enumerate(self.splits.values()):
            fields.append((f"short{j}", split.tokens))
            fields.append((f"tiles{j}", [v for t in split.tiles for v in t]))
        for g in range(num_paged_groups):
            fields.append((f"slots{g}", slots[g]))
            fields.append((f"tables{g}", tables[g].reshape(-1)))
        arrays = [np.asarray(list(v) if not isinstance(v, np.ndarray) else v, dtype=np.int32) for _, v in fields]
        total = sum(a.size for a in arrays)
        sizes = [a.size for a in arrays]
        if into is not None and into.layout != sizes:
            raise ValueError("this step does not have the layout of the batch it should replace")
        if staging is not None:
            host = staging.take(total)
        else:
            host = torch.empty(total, dtype=torch.int32, pin_memory=torch.device(device).type == "cuda")
        if total:
            np.concatenate(arrays, out=host.numpy()[:total])
        if into is not None:
            dev = into.device_buffer
            dev.copy_(host[:total], non_blocking=True)
        else:
            dev = host[:total].to(device, non_blocking=True)
        if staging is not None:
            staging.sent()
        self._host = host  # alive until the copy has run
        self.device_buffer, self.layout = dev, sizes
        offset, parts, self._at = 0, {}, {}
        for (name, _), a in zip(fields, arrays):
            parts[name] = dev[offset : offset + a.size]
            self._at[name] = offset
            offset += a.size
        self._packed = np.concatenate(arrays) if total else np.zeros(0, dtype=np.int32)  # what `advance` edits
        # per group and row: the leading table entries that a window had given back when this was packed
        self._given_back = [[_leading_released(row.tables[g]) for row in rows] for g in range(num_paged_groups)]
        self._staging, self._widths, self._vocab = staging, widths, vocab_size

        self.num_tokens, self.num_rows = T, R
        self.decode_only = all(len(row.tokens) == 1 for row in rows)  # token t is row t
        self.token_ids, self.positions, self.tok_row = parts["token_ids"], parts["positions"], parts["tok_row"]
        self.logits_rows, self.num_logits = parts["logits_rows"], len(want)
        self.all_tokens = parts["all_tokens"]
        for j, split in enumerate(self.splits.values()):
            split.short_tokens, split.num_short_tokens = parts[f"short{j}"], len(split.tokens)
            split.long_tiles, split.num_long_tiles = parts[f"tiles{j}"].view(-1, 4), len(split.tiles)
        self.row_first, self.row_len = parts["row_first"], parts["row_len"]
        self.row_start, self.row_slots = parts["row_start"], parts["row_slots"]
        self.group_slots = [parts[f"slots{g}"] for g in range(num_paged_groups)]
        self.group_tables = [parts[f"tables{g}"].view(R, widths[g]) for g in range(num_paged_groups)]
        self.host_rows = rows
        self.block_size = bs
        self.pools = pools
        self.shared = {}  # per-step results that parts share (rotary tables, ...)

    def split(self, key) -> RowSplit:
        """The rows sorted as a mixer whose `row_split()` is `key` needs them."""
        found = self.splits.get(tuple(key))
        if found is None:
            raise ValueError(f"this step's rows are sorted for {sorted(self.splits)}, not for {tuple(key)}: "
                             "the step is packed with every split that the model's mixers ask for")  # fmt: skip
        return found

    def advance(self, rows) -> bool:
        """The next decode step of the same requests, in place: every row brings the one token
        that follows the row packed last, from the same block tables, so only the token, its
        position, its slots and the table entry of its page change.  Uploads and returns True,
        or returns False and changes nothing if `rows` are anything else (pack them anew)."""
        old_rows, bs = self.host_rows, self.block_size
        if len(rows) != len(old_rows) or self.num_tokens != len(old_rows):
            return False
        if any(split.num_long_tiles for split in self.splits.values()):
            return False  # a split without single queries lists positions per tile, which this does not move on
        for new, old in zip(rows, old_rows):
            if (len(new.tokens) != 1 or new.tables is not old.tables or new.store != old.store or new.want != old.want
                    or new.state_slot != old.state_slot or new.start != old.start + (1 if new.store else 0)):
                return False
            if not 0 <= new.tokens[0] < self._vocab:
                return False  # the full packing names the error
            for g, table in enumerate(new.tables):
                page = new.start // bs
                if page >= self._widths[g] or page >= len(table) or table[page] == RELEASED:
                    return False
        p, at = self._packed, self._at
        for r, row in enumerate(rows):
            p[at["token_ids"] + r] = row.tokens[0]
            p[at["positions"] + r] = row.start
            p[at["row_start"] + r] = row.start
            for g, table in enumerate(row.tables):
                page = row.start // bs
                p[at[f"slots{g}"] + r] = table[page] * bs + row.start % bs if row.store else -1
                p[at[f"tables{g}"] + r * self._widths[g] + page] = table[page]
                # pages that a window has given back since: their ids leave the device's table too
                # (the kernels skip them, but a tile at the window's edge may still touch one)
                gone = self._given_back[g][r]
                while gone < len(table) and gone < self._widths[g] and table[gone] == RELEASED:
                    p[at[f"tables{g}"] + r * self._widths[g] + gone] = 0
                    gone += 1
                self._given_back[g][r] = gone
        total = p.size
        if self._staging is not None:
            host = self._staging.take(total)
        else:
            host = torch.empty(total, dtype=torch.int32, pin_memory=self.device_buffer.is_cuda)
        host.numpy()[:total] = p
        self.device_buffer.copy_(host[:total], non_blocking=True)
        if self._staging is not None:
            self._staging.sent()
        self._host = host
        self.host_rows = rows
        self.shared = {}
        return True

    def cache_view(self, cache_id: int, writes: bool):
        """The view of cache `cache_id` for a mixer in this step; None for a mixer that keeps nothing."""
        found = self.pools.manager.group_of_cache.get(cache_id)
        if found is None:
            return None
        kind, gi, _ = found
        if kind == "paged":
            _, k_pages, v_pages = self.pools.pages(cache_id)
            return PagedLayerView(k_pages, v_pages, self.group_slots[gi], self.group_tables[gi], writes, self.block_size)
        _, state = self.pools.state_of(cache_id)
        return StateLayerView(state, self.row_slots, writes)


class Staging:
    """Two pinned host buffers used in turn for the step uploads; a buffer is reused only after
    the copy that read it has run."""

    def __init__(self, device):
        self.device = torch.device(device)
        self.buffers = [None, None]
        self.events = [None, None]
        self.turn = 0

    def take(self, count: int):
        i = self.turn
        if self.events[i] is not None:
            self.events[i].synchronize()
        if self.buffers[i] is None or self.buffers[i].numel() < count:
            self.buffers[i] = torch.empty(max(count, 4096), dtype=torch.int32, pin_memory=self.device.type == "cuda")
        return self.buffers[i]

    def sent(self) -> None:
        if self.device.type == "cuda":
            ev = torch.cuda.Event()
            ev.record()
            self.events[self.turn] = ev
        self.turn ^= 1
