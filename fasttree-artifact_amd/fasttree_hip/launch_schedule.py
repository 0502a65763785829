"""Launch schedule of the first decode stage on an MI355X: the planner's vnodes re-cut into
block programs.

The reference launches one thread block per (vnode, KV head) and leaves the order and the
placement to the hardware dispatcher (kernel_bench/fasttree.py:443-479, grid = (node_num,
head_num)).  On a part with 256 compute units a launch of a few hundred blocks of unequal
length ends when its most loaded compute unit does: with the planner's fixed KV split the
3-level tree of the headline benchmark puts 1.5 times the average work on some units.  The
functions here take the planner's lists (in the reference's order, kernel_bench/fasttree.py:
193-262) and return lists that describe the same computation -- every request still attends
every token of its root path exactly once, each (request, piece) pair through one scratch row
that the second stage merges -- arranged for the machine:

* The wide vnodes (more than 16 query rows) over one KV run are undone: the planner's KV chunks
  of a node are joined back into the node's run and its query tiles into the node's request
  list.  The run is then cut anew into row chunks of ``block_rows`` query rows (what one block
  of the kernel serves per pass) and, along the tokens, wherever a block program is full.
* A *block program* is a list of consecutive vnodes that one thread block serves, one after the
  other, for one KV head; there are at most ``block_slots // num_kv_heads`` of them per round
  and head, so that one round of programs is on the machine from the start.  Two layouts:

  - *resident* (where every (run, row chunk) gets a program of its own): the runs whose pieces
    would be the longest are cut into equal pieces until no more programs fit; one piece per
    program, longest first.  The programs are unequal, so they end one after the other, and
    the blocks of the narrow vnodes take the freed slots while the longest programs still
    compute: the scattered, read-once rows of the narrow vnodes are fetched under the matrix
    work of the wide ones (measured on the 3-level tree: a call on cold caches 9 us shorter
    than with packed programs, the same on warm caches, 17 % fewer scratch rows).
  - *packed* (any launch): programs of equal work (tile steps plus a start-up charge per vnode),
    either filled one after the other with the runs cut wherever a program is full, or -- when
    that leaves the fullest program about as full -- from runs cut into equal pieces that are
    dealt longest first to the least loaded program (measured on an irregular tree of 500
    requests: 6 % shorter, 12 % fewer vnodes).  All programs end together and the narrow
    vnodes follow.

  The resident layout is taken when it exists and its modelled duration is within
  :data:`RESIDENT_MARGIN` of the packed one's.
* Narrow vnodes (at most 16 query rows) keep the planner's chunks and are served one wave each.
  When the programs fill the machine there is no room for blocks of their own beside them, so
  they are dealt to the programs, longest first, in equal shares: a program serves its narrow
  vnodes with its four waves before its wide vnodes or after them.  The two blocks that share a
  compute unit get opposite orders, so the memory round trips of one block's narrow vnodes are
  filled by the matrix work of the other.  Narrow vnodes that would take a program longer than
  its wide vnodes stay in blocks of their own after the programs.

Nothing refers to a vnode by its position (the per-request lists name scratch rows), and the
kernels compute a vnode of any number of rows and tokens, so the arrangement changes the
schedule, not the result.  The lists this module returns are a complete plan on their own:
``fasttree_decode`` gives the same result with or without the program table.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List

import numpy as np

#: Query rows one block of the first-stage kernel serves per pass (4 waves x 32 rows).
BLOCK_ROWS = 128
#: Blocks and waves of the first-stage kernel one compute unit holds at a time (73 KB of LDS and
#: 241 registers per wave of a block of four).
BLOCKS_PER_CU = 2
WAVES_PER_CU = 8
#: Compute units assumed when no device can be asked (an MI355X has 256).
DEFAULT_COMPUTE_UNITS = 256
#: KV tokens of one tile step.
TILE_TOKENS = 32
#: Start-up and wind-down of one vnode inside a program, in tile steps (three dependent memory
#: round trips before the first step, the partial results after the last: about 6 us measured,
#: against 1.2 us per step of a block that shares its compute unit).
VNODE_STARTUP_TILES = 5.0
#: A narrow vnode on one wave, in the same unit: its start-up and one 32-token step.
NARROW_STARTUP_TILES = 3.8
NARROW_STEP_TILES = 0.85
#: What the merge of the waves that share one narrow vnode costs each of them (two block barriers
#: and an exchange of the state through LDS per halving), in the same unit.
NARROW_SHARE_TILES = 0.5
#: Microseconds per tile step of a block that shares its compute unit with another wide block,
#: and of one that does not (measured on the 3-level tree of the headline benchmark).
TILE_US_SHARED = 1.19
TILE_US_ALONE = 0.95
#: Bytes per microsecond the narrow vnodes stream at most on DEFAULT_COMPUTE_UNITS units (rows of
#: 2 * head_dim bytes at random slots); taken to scale with the number of units.
NARROW_BYTES_PER_US = 5.6e6
#: What a launch costs on top of its blocks' own time when launches are queued back to back on one
#: stream (measured: launches of 192 narrow vnodes, whose waves model at 5.5 us, repeat every 7.0 us).
#: Part of the reported duration only: it is the same for every layout of a launch, so the choice
#: between layouts does not see it.
LAUNCH_US = 1.5
#: A tile step of a piece of at most 64 query rows, relative to one of a full block.  The block's
#: waves then split the tokens of a super tile, but the super tile is loaded all the same: fitted on
#: the programs of an irregular tree of 500 requests, 1.21 against 1.44 us per tile step.
LIGHT_TILE_WEIGHT = 0.85
#: Waves of a block (each serves one narrow vnode at a time).
BLOCK_WAVES = 4
#: A launch is cut into equal programs only if every program gets at least this much work
#: (tile steps); smaller launches keep the planner's chunks, one vnode per program.
MIN_PROGRAM_TILES = 12.0
#: Most work (tile steps) one program may hold; larger launches run several rounds of programs.
MAX_PROGRAM_TILES = 160.0
#: Pieces are cut at multiples of this many tokens (two tiles: one trip of the kernel's loop) and
#: are not made shorter than MIN_PIECE_TOKENS.
CUT_TOKENS = 64
MIN_PIECE_TOKENS = 128
#: The resident layout is taken when its modelled duration is within this factor of the packed one's.
RESIDENT_MARGIN = 1.05
#: Of two program blocks on one compute unit the one launched later steps this much slower (its
#: waves are the younger on every SIMD and issue second): measured on the 3-level tree, 1.30 against
#: 1.13 us per tile step; and microseconds per tile step of the older one.
YOUNGER_BLOCK_SLOWDOWN = 1.15
TILE_US_OLDER = 1.10
#: Where pieces of the longest run have to be younger blocks, one piece of every row chunk is made
#: this much shorter than the others (1 / YOUNGER_BLOCK_SLOWDOWN: the two blocks of such a compute
#: unit then end together).  Measured on the 3-level tree against equal pieces: stage 1 59.0 ->
#: 56.2 us, wall per call 70.6 -> 67.3 us, cold call unchanged; 0.8 gives the same.
SHORT_PIECE_RATIO = 0.87
#: Equal pieces dealt to the programs are taken when the fullest program is within this factor of the
#: fullest of the programs filled one after the other.
DEALT_MARGIN = 1.06
#: A wide run of at most LIGHT_ROWS query rows and LIGHT_WORK query rows x KV tokens is served
#: with the narrow vnodes when the launch has more wide blocks than the machine runs at a time
#: (short runs under a few dozen rows are bound by memory latency, and the narrow path has eight
#: of them in flight per compute unit).
LIGHT_WORK = 4096
LIGHT_ROWS = 64
NARROW_ROWS = 16
#: Long narrow runs are cut (at multiples of a tile) while the launch's narrow vnodes would leave
#: more than a quarter of the wave slots idle: a wave walks its run tile by tile, one memory round
#: trip each, so a launch of a few long runs (a 1024-token prompt under 16 requests of a
#: 32-head model: 32 waves that matter) lasts as long as its longest walk.  Pieces are not made
#: shorter than this many tokens (every piece costs a start-up and a scratch row per request).
NARROW_MIN_PIECE_TOKENS = 128
NARROW_FILL = 0.75


class LaunchPhases(list):
    """``phase_node_nums`` as the decode call takes it (a list of two counts) that also carries
    the block programs of the launch: ``prog_table`` (int32 device tensor, four entries per
    program: first and end of its wide vnodes within the first phase, first and signed count of
    its narrow vnodes within the second; a negative count: served before the wide ones) or None,
    ``num_programs`` and ``narrow_in_programs`` (how many vnodes at the head of the second phase
    belong to programs)."""

    prog_table = None
    num_programs = 0
    narrow_in_programs = 0
    #: int32 device tensor of :func:`narrow_records` (64 entries per vnode of the second phase), or None
    narrow_table = None
    #: int32 device tensor of :func:`request_records` (16 entries per request), or None
    req_table = None
    #: int32 device tensor of :func:`program_records` (256 entries per program), or None
    prog_records = None
    #: what the schedule's model expects the first-stage launch to take, and the machine it was laid out for
    modelled_us = None
    num_cus = None
    block_slots = None


@dataclass
class LaunchSchedule:
    kv_offs: np.ndarray
    kv_lens: np.ndarray
    q_offs: np.ndarray
    q_lens: np.ndarray
    q_entries: np.ndarray        # request of every scratch row
    req_entries: np.ndarray      # scratch rows per request, back to back, then 32 x -1
    req_offs: np.ndarray
    req_lens: np.ndarray
    phase_node_nums: List[int]
    phase_node_offsets: List[int]
    prog_table: np.ndarray       # (num_programs, 4); see LaunchPhases
    narrow_in_programs: int
    program_tiles: np.ndarray    # modelled work of every program (for tests and reports)
    block_slots: int = BLOCKS_PER_CU * DEFAULT_COMPUTE_UNITS
    modelled_us: float = 0.0     # modelled duration of the launch
    num_cus: int = DEFAULT_COMPUTE_UNITS   # compute units the launch was laid out for

    @property
    def num_rows(self) -> int:
        return int(len(self.q_entries))

    @property
    def num_programs(self) -> int:
        return int(self.prog_table.shape[0])


#: Whether launch-order plans carry the records of :func:`narrow_records` (a switch for measurements).
USE_NARROW_RECORDS = True
#: Whether they carry the records of :func:`request_records` for the merge launch (likewise).
USE_REQUEST_RECORDS = True
#: Whether they carry the records of :func:`program_records` (likewise).
USE_PROGRAM_RECORDS = True
#: Entries of a narrow vnode's record, requests and token slots it holds (the kernels' layout).
NARROW_RECORD = 64
NARROW_RECORD_REQUESTS = 16
NARROW_RECORD_TOKENS = 32


def narrow_records(kv_entries, kv_offs, kv_lens, q_offs, q_lens, q_entries, first, count):
    """One record per vnode ``first .. first + count - 1`` of the lists (the narrow phase): what a
    wave needs to start on the vnode, in one place, so that it finds it in one memory round trip
    instead of two (the vnode's four list entries, then its slot indices and requests) before it
    can ask for K/V rows.  Entries: ``kv_off, kv_len, q_off, q_len``, the requests of the first 16
    scratch rows, the pool slots of the first 32 tokens (the last token repeated past the end of a
    shorter run), padding.  Returns an int32 array ``[count, 64]``."""
    kv_entries = np.asarray(kv_entries).reshape(-1)
    q_entries = np.asarray(q_entries).reshape(-1)
    table = np.zeros((int(count), NARROW_RECORD), dtype=np.int32)
    if count == 0:
        return table
    sl = slice(int(first), int(first) + int(count))
    ko, kl = np.asarray(kv_offs[sl], dtype=np.int64), np.asarray(kv_lens[sl], dtype=np.int64)
    qo, ql = np.asarray(q_offs[sl], dtype=np.int64), np.asarray(q_lens[sl], dtype=np.int64)
    table[:, 0], table[:, 1], table[:, 2], table[:, 3] = ko, kl, qo, ql
    rows = qo[:, None] + np.minimum(np.arange(NARROW_RECORD_REQUESTS)[None, :], np.maximum(ql[:, None] - 1, 0))
    table[:, 4:4 + NARROW_RECORD_REQUESTS] = np.where(ql[:, None] > 0, q_entries[np.minimum(rows, max(len(q_entries) - 1, 0))], 0) \
        if len(q_entries) else 0
    tokens = ko[:, None] + np.minimum(np.arange(NARROW_RECORD_TOKENS)[None, :], np.maximum(kl[:, None] - 1, 0))
    first_slot = 4 + NARROW_RECORD_REQUESTS
    table[:, first_slot:first_slot + NARROW_RECORD_TOKENS] = np.where(
        kl[:, None] > 0, kv_entries[np.minimum(tokens, max(len(kv_entries) - 1, 0))], 0) if len(kv_entries) else 0
    return table


#: Entries of a block program's record, where the requests and the token slots start in it, and how
#: many rows and tokens they cover (the kernels' layout).
PROGRAM_RECORD = 256
PROGRAM_RECORD_REQUESTS = 8
PROGRAM_RECORD_SLOTS = 136
PROGRAM_RECORD_ROWS = 128
PROGRAM_RECORD_TOKENS = 64


def program_records(kv_entries, kv_offs, kv_lens, q_offs, q_lens, q_entries, prog_table, first, group):
    """One record per block program: what its block needs to start on the program's first wide
    vnode, in one place, so that it can ask for query and K/V rows after one memory round trip
    (the record, fetched together with the table entry) instead of three (table entry, the
    vnode's list entries, its request and slot lists).  Entries: ``kv_off, kv_len, q_off, q_len`` of
    vnode ``first + prog_table[p][0]``; a flag (1: the program has a wide vnode of at most 128 query
    rows and the rest is filled in); from entry 8 the requests of its scratch rows; from entry 136
    the pool slots of its first 64 tokens (the last token repeated past the end of a shorter run).
    Returns an int32 array ``[num_programs, 256]``."""
    prog_table = np.asarray(prog_table, dtype=np.int64).reshape(-1, 4)
    kv_entries = np.asarray(kv_entries).reshape(-1)
    q_entries = np.asarray(q_entries).reshape(-1)
    table = np.zeros((len(prog_table), PROGRAM_RECORD), dtype=np.int32)
    if len(prog_table) == 0:
        return table
    has = prog_table[:, 1] > prog_table[:, 0]
    v = np.where(has, int(first) + prog_table[:, 0], 0)
    take = lambda x: np.asarray(x, dtype=np.int64).reshape(-1)[v] if len(x) else np.zeros(len(v), dtype=np.int64)
    ko, kl, qo, ql = take(kv_offs), take(kv_lens), take(q_offs), take(q_lens)
    ok = has & (ql * int(group) <= PROGRAM_RECORD_ROWS) & (ql > 0)
    table[:, 0], table[:, 1], table[:, 2], table[:, 3], table[:, 4] = ko, kl, qo, ql, ok
    if len(q_entries):
        rows = qo[:, None] + np.minimum(np.arange(PROGRAM_RECORD_ROWS)[None, :], np.maximum(ql[:, None] - 1, 0))
        table[:, PROGRAM_RECORD_REQUESTS:PROGRAM_RECORD_REQUESTS + PROGRAM_RECORD_ROWS] = np.where(
            ok[:, None], q_entries[np.minimum(rows, len(q_entries) - 1)], 0)
    if len(kv_entries):
        tokens = ko[:, None] + np.minimum(np.arange(PROGRAM_RECORD_TOKENS)[None, :], np.maximum(kl[:, None] - 1, 0))
        table[:, PROGRAM_RECORD_SLOTS:PROGRAM_RECORD_SLOTS + PROGRAM_RECORD_TOKENS] = np.where(
            (ok & (kl > 0))[:, None], kv_entries[np.minimum(tokens, len(kv_entries) - 1)], 0)
    table[~ok, 4] = 0
    return table


#: Entries of one request's record for the second stage: its number of scratch rows, where they
#: start in the per-request list, and the first REQUEST_RECORD - 2 of them.
REQUEST_RECORD = 16


def request_records(req_entries, req_offs, req_lens):
    """One record per request for the merge launch: ``req_lens[r], req_offs[r]`` and the first 14
    scratch rows of the request (zeros past its last), so that a block of that launch knows
    which partial rows to ask for after one memory round trip instead of two (length and offset,
    then the list).  Rows beyond the fourteenth are read from the list.  Returns an int32 array
    ``[len(req_offs), 16]``."""
    req_entries = np.asarray(req_entries).reshape(-1)
    offs, lens = np.asarray(req_offs, dtype=np.int64).reshape(-1), np.asarray(req_lens, dtype=np.int64).reshape(-1)
    table = np.zeros((len(offs), REQUEST_RECORD), dtype=np.int32)
    if len(offs) == 0:
        return table
    table[:, 0], table[:, 1] = lens, offs
    inside = REQUEST_RECORD - 2
    pos = offs[:, None] + np.arange(inside)[None, :]
    held = np.arange(inside)[None, :] < lens[:, None]
    if len(req_entries):
        table[:, 2:] = np.where(held, req_entries[np.minimum(pos, len(req_entries) - 1)], 0)
    return table


_CUS_OF_DEVICE = {}


def compute_units(device=None) -> int:
    """Compute units of ``device`` (a torch device, an index or None = the current one), as the
    runtime reports them (``multi_processor_count``, the attribute the kernels' launcher reads as
    well); :data:`DEFAULT_COMPUTE_UNITS` where no device is visible."""
    try:
        import torch

        if not torch.cuda.is_available():
            return DEFAULT_COMPUTE_UNITS
        dev = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        if dev.type != "cuda":
            return DEFAULT_COMPUTE_UNITS
        index = dev.index if dev.index is not None else torch.cuda.current_device()
        if index not in _CUS_OF_DEVICE:
            _CUS_OF_DEVICE[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
        return _CUS_OF_DEVICE[index]
    except Exception:
        return DEFAULT_COMPUTE_UNITS


def _tile_weight(rows: int) -> float:
    """Share of a block's time one tile step of a piece with ``rows`` query rows takes: the
    block's four waves form row groups of 32 rows; with half of them idle they split the tokens
    of a 64-token super tile instead (two ways: a super tile holds two tile steps)."""
    return 1.0 if rows > 64 else LIGHT_TILE_WEIGHT


def _row_chunks(n_requests: int, cap: int):
    """``n_requests`` cut into the fewest chunks of at most ``cap``, as even as possible (a last
    chunk of a few rows would leave most of a block's waves without rows)."""
    count = max(1, -(-n_requests // cap))
    base, extra = divmod(n_requests, count)
    lo = 0
    for i in range(count):
        size = base + (1 if i < extra else 0)
        yield lo, lo + size
        lo += size


def _runs_of(kv_offs, kv_lens, q_offs, q_lens, q_entries):
    """The (KV run, request list) pairs behind the planner's vnodes.

    Vnodes over one KV slice whose scratch rows adjoin are the query tiles of one chunk
    (kernel_bench/fasttree.py:212-231); chunks whose slices adjoin and whose requests are equal
    are the KV splits of one node (fasttree.py:199-210).  Returns a list of
    ``(kv_start, chunk_lens, requests)``: the run starts at ``kv_start`` of the flat KV index
    list and was cut by the planner into chunks of ``chunk_lens`` tokens.
    """
    n = len(kv_offs)
    order = np.lexsort((q_offs, kv_lens, kv_offs)).tolist()
    # (plain lists: the scan below touches every vnode once, and numpy scalars are slow at that)
    ko, kl, qo, ql = kv_offs.tolist(), kv_lens.tolist(), q_offs.tolist(), q_lens.tolist()
    chunks = []   # (kv_off, kv_len, requests)
    i = 0
    while i < n:
        v = order[i]
        first = qo[v]
        end = first + ql[v]
        j = i + 1
        while j < n:
            w = order[j]
            if ko[w] != ko[v] or kl[w] != kl[v] or qo[w] != end:
                break
            end += ql[w]
            j += 1
        chunks.append((ko[v], kl[v], q_entries[first:end]))   # (the tiles' rows adjoin: one slice)
        i = j
    # chain the chunks of one node: the next chunk starts where this one ends, same requests
    keys = [reqs.tobytes() for _, _, reqs in chunks]
    by_start = {}
    for idx, (off, length, reqs) in enumerate(chunks):
        by_start.setdefault((off, keys[idx]), []).append(idx)
    follower = [-1] * len(chunks)
    has_leader = [False] * len(chunks)
    for idx, (off, length, reqs) in enumerate(chunks):
        if length == 0:
            continue
        for cand in by_start.get((off + length, keys[idx]), ()):
            if cand != idx and not has_leader[cand]:
                follower[idx] = cand
                has_leader[cand] = True
                break
    runs = []
    for idx in range(len(chunks)):
        if has_leader[idx]:
            continue
        lens, cur = [], idx
        while cur >= 0:
            lens.append(chunks[cur][1])
            cur = follower[cur]
        runs.append((chunks[idx][0], lens, chunks[idx][2]))
    return runs


def block_programs(kv_offs, kv_lens, q_offs, q_lens, q_entries, batch_size, group, num_kv_heads, *,
                   block_rows=BLOCK_ROWS, block_slots=None, recut=None, embed=False, head_dim=128,
                   layout=None, cuts=None, num_cus=None) -> LaunchSchedule:
    """The planner's lists arranged as block programs (see the module docstring).

    ``layout`` forces "packed" or "resident" programs (None: by modelled duration); ``cuts``
    forces how packed programs are made, "sequential" (filled one after the other) or "dealt"
    (equal pieces dealt to the least loaded program); both are for experiments and tests.

    ``num_cus`` is the number of compute units the launch is laid out for (None: those of the
    current device, :func:`compute_units`); the block and wave slots follow from it.

    With ``block_slots=None`` the launch is laid out twice, for programs on every block slot of
    the machine (two per compute unit: the narrow vnodes then wait for the programs to end) and
    on half of them (one per compute unit: the narrow vnodes run beside the programs from the
    start, and a program that has its compute unit to itself steps faster), and the layout with
    the shorter modelled duration is returned.
    """
    kv_offs, kv_lens, q_offs, q_lens = (np.asarray(x, dtype=np.int64) for x in (kv_offs, kv_lens, q_offs, q_lens))
    q_entries = np.asarray(q_entries, dtype=np.int64)
    runs = _runs_of(kv_offs, kv_lens, q_offs, q_lens, q_entries)
    cus = max(1, int(num_cus)) if num_cus else compute_units()
    if block_slots is None:
        # (at head_dim 256 a compute unit holds one block of the kernel: 512-byte rows, 136 KB of LDS)
        layouts = (BLOCKS_PER_CU * cus, cus) if head_dim <= 128 else (cus,)
        both = [_block_programs(runs, batch_size, group, num_kv_heads, num_cus=cus,
                                block_rows=block_rows, block_slots=slots, recut=recut, embed=embed, head_dim=head_dim, layout=layout, cuts=cuts)
                for slots in layouts]
        return min(both, key=lambda layout: layout[0])[1]()     # (only the chosen layout's lists are built)
    return _block_programs(runs, batch_size, group, num_kv_heads, num_cus=cus,
                           block_rows=block_rows, block_slots=block_slots, recut=recut, embed=embed, head_dim=head_dim,
                           layout=layout, cuts=cuts)[1]()


def _cut_long_narrow_runs(narrow, group, heads, wave_slots):
    """Narrow vnodes ``(kv_off, kv_len, requests)`` with the longest runs halved, again and again,
    while the waves they take (one per 16 query rows and kv head) fill less than
    :data:`NARROW_FILL` of the wave slots and the halves keep :data:`NARROW_MIN_PIECE_TOKENS`."""
    import heapq

    def waves(v):
        return -(-len(v[2]) * group // NARROW_ROWS) * heads

    total = sum(waves(v) for v in narrow)
    heap = [(-v[1], i, v) for i, v in enumerate(narrow)]
    heapq.heapify(heap)
    serial = len(narrow)
    whole = []                                          # runs that cannot be halved any more
    while heap and total < NARROW_FILL * wave_slots and -heap[0][0] >= 2 * NARROW_MIN_PIECE_TOKENS:
        length, index, v = heapq.heappop(heap)
        length = -length
        first = (length // 2 + TILE_TOKENS - 1) // TILE_TOKENS * TILE_TOKENS
        if length - first < NARROW_MIN_PIECE_TOKENS:
            whole.append((-length, index, v))
            continue
        for off, take in ((v[0], first), (v[0] + first, length - first)):
            heapq.heappush(heap, (-take, serial, (off, take, v[2])))
            serial += 1
        total += waves(v)
    return [v for _, _, v in sorted(heap + whole, key=lambda item: item[1])]


def _resident_pieces(items, per_round, tiles, first_row):
    """The wide work as one program per piece, all of them on the machine from the start.

    Every (run, row chunk) item starts as one piece.  While the programs number at most
    ``per_round``, the run whose pieces are the longest is cut once more -- all its row chunks
    at the same tokens, multiples of :data:`CUT_TOKENS`, so that the blocks that stream one
    piece of the run do it side by side and share it in L2.  Returns ``(pieces, programs)``
    with the programs in order of decreasing work, or None when the items alone outnumber the
    programs of a round.
    """
    if not items or len(items) > per_round:
        return None
    runs = {}                                   # (kv_start, run length) -> item indices
    for i, (_, start, lens, _) in enumerate(items):
        runs.setdefault((start, sum(lens)), []).append(i)
    cuts = {key: 1 for key in runs}
    count = len(items)

    def piece_tiles(key):
        return max(items[i][0] for i in runs[key]) * tiles(-(-key[1] // cuts[key]))

    while True:
        key = max(runs, key=piece_tiles)
        if count + len(runs[key]) > per_round or key[1] // (cuts[key] + 1) < MIN_PIECE_TOKENS:
            break
        cuts[key] += 1
        count += len(runs[key])
    # The programs beyond the first `first_row` share their compute units with the longest ones
    # and, being the younger blocks there, step about YOUNGER_BLOCK_SLOWDOWN times slower.  When
    # pieces of the longest run would be among them, that run gets one shorter piece per row
    # chunk (SHORT_PIECE_RATIO of the others, which grow a little): sorted by length, the short
    # ones are the younger.
    longest = max(runs, key=piece_tiles)
    uneven = (SHORT_PIECE_RATIO < 1.0 and cuts[longest] >= 2 and count > first_row
              and cuts[longest] * len(runs[longest]) > first_row)
    pieces = []
    for (start, length), members in runs.items():
        n = cuts[(start, length)]
        units = -(-length // CUT_TOKENS)
        shares = [units // n + (1 if j < units % n else 0) for j in range(n)]
        if uneven and (start, length) == longest:
            short = max(MIN_PIECE_TOKENS // CUT_TOKENS, int(round(units * SHORT_PIECE_RATIO / (n - 1 + SHORT_PIECE_RATIO))))
            rest = units - short
            shares = [rest // (n - 1) + (1 if j < rest % (n - 1) else 0) for j in range(n - 1)] + [short]
        bounds, done = [], 0
        for share in shares:
            take = min(share * CUT_TOKENS, length - done)
            if take > 0:
                bounds.append((start + done, take))
                done += take
        for i in members:
            w, _, _, part = items[i]
            pieces += [(off, take, part, w * tiles(take) + VNODE_STARTUP_TILES) for off, take in bounds]
    order = sorted(range(len(pieces)), key=lambda i: -pieces[i][3])
    return pieces, [[i] for i in order]


def _block_programs(runs, batch_size, group, num_kv_heads, *,
                    block_rows, block_slots, recut, embed, head_dim, layout=None, cuts=None, num_cus=DEFAULT_COMPUTE_UNITS):
    """One layout of :func:`block_programs`, for ``block_slots`` programs at a time: its
    modelled duration and a function that builds its :class:`LaunchSchedule`.

    Takes the four per-vnode lists and the scratch-row list of kernel_bench/fasttree.py:193-231
    (any order), the number of requests, the GQA group size and the number of KV heads.
    ``recut`` forces (True) or forbids (False) cutting the wide runs anew; by default they are
    cut anew when every program of one round gets at least :data:`MIN_PROGRAM_TILES` of work.
    ``layout`` and ``cuts`` force one of the arrangements (see :func:`block_programs`).
    ``embed`` deals the narrow vnodes to the programs (None: when the runs were cut anew and no
    program's share outweighs its wide vnodes).  Off by default: measured, a program block that
    has its compute unit to itself steps only about a fifth faster, so narrow vnodes inside the
    programs run one after the other with the wide work all the same.
    """
    group = max(1, int(group))
    heads = max(1, int(num_kv_heads))
    machine_slots = BLOCKS_PER_CU * int(num_cus)      # blocks of the kernel the device holds at a time
    wave_slots = WAVES_PER_CU * int(num_cus)          # waves (narrow vnodes in flight)
    cap = max(1, int(block_rows) // group)            # requests per row chunk
    per_round = max(1, int(block_slots) // heads)     # programs per round and head

    wide_runs, narrow = [], []    # narrow: (kv_off, kv_len, requests) per planner chunk
    for start, lens, reqs in runs:
        rows = len(reqs) * group
        # (a run without tokens has no tile steps to schedule: it goes with the narrow vnodes, whose
        # waves write its empty partial results)
        if rows <= NARROW_ROWS or sum(lens) == 0:
            off = start
            for length in lens:
                narrow.append((off, length, reqs))
                off += length
        else:
            wide_runs.append((start, lens, reqs))
    # light wide runs go with the narrow vnodes when the wide blocks alone overfill the machine
    wide_blocks = sum(len(lens) * -(-len(reqs) * group // block_rows) for _, lens, reqs in wide_runs) * heads
    if wide_blocks > block_slots:
        kept = []
        for start, lens, reqs in wide_runs:
            rows = len(reqs) * group
            if rows <= LIGHT_ROWS and rows * max(lens) <= LIGHT_WORK:
                off = start
                for length in lens:
                    narrow.append((off, length, reqs))
                    off += length
            else:
                kept.append((start, lens, reqs))
        wide_runs = kept

    # ---- work items: (run, row chunk) with the run's planner chunks as possible cut points
    def tiles(tokens):
        return -(-tokens // TILE_TOKENS)

    items = []   # (weight per tile, kv_start, chunk_lens, requests of the row chunk)
    for start, lens, reqs in wide_runs:
        for lo, hi in _row_chunks(len(reqs), cap):
            part = reqs[lo:hi]
            items.append((_tile_weight(len(part) * group), start, lens, part))
    total = sum(w * tiles(sum(lens)) + VNODE_STARTUP_TILES for w, _, lens, _ in items)
    do_recut = (total / per_round >= MIN_PROGRAM_TILES) if recut is None else bool(recut)

    pieces = []      # (kv_off, kv_len, requests, work)
    programs = []    # list of lists of piece indices
    resident = None  # the same for the layout with a block of its own for every piece
    if items and do_recut:
        rounds = max(1, int(np.ceil(total / (per_round * MAX_PROGRAM_TILES))))
        nprog = per_round * rounds
        items.sort(key=lambda it: -(it[0] * tiles(sum(it[2]))))

        def fill(target):
            """Programs filled to `target` one after the other, runs cut where a program is full."""
            pieces, programs, current, load = [], [], [], 0.0
            for w, start, lens, part in items:
                run_len, done = sum(lens), 0
                while done < run_len:
                    left = run_len - done
                    last = len(programs) >= nprog - 1          # the last program takes whatever is left
                    room = target - load - VNODE_STARTUP_TILES  # tile steps of this weight that still fit
                    fit = (int(room / w) * TILE_TOKENS) // CUT_TOKENS * CUT_TOKENS if room > 0 else 0
                    if last or fit >= left or left - fit < MIN_PIECE_TOKENS:
                        take = left                              # the rest fits (or what would remain is too short)
                    elif fit >= MIN_PIECE_TOKENS:
                        take = fit                               # the program is full here
                    elif current:
                        programs.append((current, load))         # no room worth a piece: next program
                        current, load = [], 0.0
                        continue
                    else:
                        take = left
                    work = w * tiles(take) + VNODE_STARTUP_TILES
                    current.append(len(pieces))
                    pieces.append((start + done, take, part, work))
                    load += work
                    done += take
                    if load >= target - 0.5 * w and not last:
                        programs.append((current, load))
                        current, load = [], 0.0
            if current:
                programs.append((current, load))
            return pieces, programs

        # the smallest target (within a few percent) that the last program does not overshoot:
        # every cut adds a vnode and its start-up charge, so the first guess is a lower bound
        target = total / nprog
        for _ in range(60):
            pieces, filled = fill(target)
            if max(load for _, load in filled) <= 1.04 * target:
                break
            target *= 1.03
        programs = [prog for prog, _ in filled]

        def dealt(target):
            """Every row chunk of a run cut into the same equal pieces (the blocks that stream one
            token range of a run do it side by side and share it in L2), the pieces dealt to the
            programs longest first, each to the least loaded program."""
            pieces = []
            for w, start, lens, part in items:
                run_len = sum(lens)
                n = int(round(w * tiles(run_len) / max(1.0, target - VNODE_STARTUP_TILES)))
                n = max(1, min(n, run_len // MIN_PIECE_TOKENS))
                units, done = -(-run_len // CUT_TOKENS), 0
                for i in range(n):
                    take = min((units // n + (1 if i < units % n else 0)) * CUT_TOKENS, run_len - done)
                    if take > 0:
                        pieces.append((start + done, take, part, w * tiles(take) + VNODE_STARTUP_TILES))
                        done += take
            loads = [0.0] * nprog
            members = [[] for _ in range(nprog)]
            for i in sorted(range(len(pieces)), key=lambda i: -pieces[i][3]):
                p = min(range(nprog), key=loads.__getitem__)
                members[p].append(i)
                loads[p] += pieces[i][3]
            keep = sorted((p for p in range(nprog) if members[p]), key=lambda p: -loads[p])
            return pieces, [members[p] for p in keep], max(loads)

        if cuts != "sequential":
            d_pieces, d_programs, d_max = dealt(total / nprog)
            if cuts == "dealt" or d_max <= DEALT_MARGIN * max(load for _, load in filled):
                pieces, programs = d_pieces, d_programs
        if layout != "packed":
            resident = _resident_pieces(items, per_round, tiles, max(1, (machine_slots // 2) // heads))
    elif items:
        # The planner's chunks as they are, one vnode per program, longest first.  While the
        # launch would leave half of the machine idle, row chunks are halved (down to 64 rows):
        # the block's waves then split the tokens of the smaller chunk among them.
        rows_cap = int(block_rows)
        while rows_cap > 64:
            cap_now = max(1, rows_cap // group)
            blocks = sum(len(lens) * -(-len(reqs) // cap_now) for _, lens, reqs in wide_runs) * heads
            if 2 * blocks > block_slots:
                break
            rows_cap //= 2
        cap_now = max(1, rows_cap // group)
        for start, lens, reqs in wide_runs:
            for lo, hi in _row_chunks(len(reqs), cap_now):
                part = reqs[lo:hi]
                w = _tile_weight(len(part) * group)
                off = start
                for length in lens:
                    pieces.append((off, length, part, w * tiles(length) + VNODE_STARTUP_TILES))
                    off += length
        order = sorted(range(len(pieces)), key=lambda i: -pieces[i][3])
        programs = [[i] for i in order]

    narrow_all = _cut_long_narrow_runs(narrow, group, heads, wave_slots)

    def finish(pieces, programs, overlap=False):
        # ---- narrow vnodes, longest first; dealt to the programs when those fill the machine
        def narrow_work(v):
            return NARROW_STARTUP_TILES + NARROW_STEP_TILES * tiles(v[1]) * -(-len(v[2]) * group // NARROW_ROWS)

        narrow = sorted(narrow_all, key=lambda v: -narrow_work(v))
        program_tiles = [sum(pieces[i][3] for i in prog) for prog in programs]
        shares = [[] for _ in programs]
        embed_narrow = embed if embed is not None else (do_recut and bool(programs) and bool(narrow))
        if embed_narrow and programs and narrow:
            nprog = len(programs)
            for i, v in enumerate(narrow):
                lap, pos = divmod(i, nprog)
                shares[pos if lap % 2 == 0 else nprog - 1 - pos].append(v)
            # a program's waves serve its share together: the share takes as long as its largest wave load
            waves = BLOCK_WAVES
            share_tiles = [max(sum(narrow_work(v) for v in sh[w::waves]) for w in range(waves)) if sh else 0.0
                           for sh in shares]
            if embed is None and max(share_tiles) > min(program_tiles):
                shares = [[] for _ in programs]     # the narrow vnodes outweigh the programs: blocks of their own
            else:
                program_tiles = [t + s for t, s in zip(program_tiles, share_tiles)]
        embedded = [v for sh in shares for v in sh]
        taken = {id(v) for v in embedded}
        narrow = embedded + [v for v in narrow if id(v) not in taken]

        # ---- modelled duration of the launch (microseconds)
        shared = len(programs) * heads > machine_slots // 2        # two program blocks on some compute unit
        tile_us = TILE_US_SHARED if shared else TILE_US_ALONE
        if programs:
            waves_of_blocks = max(1.0, len(programs) * heads / float(block_slots))
            wide_us = max(max(program_tiles), sum(program_tiles) / len(programs) * waves_of_blocks) * tile_us
        else:
            wide_us = 0.0
        narrow_first = sum(len(sh) for sh in shares)
        trailing = narrow[narrow_first:]
        if trailing:
            # the kernel's launcher lets 2 or 4 waves share a vnode of the trailing blocks while that
            # leaves a quarter of the wave slots free; each then walks its share of the tiles
            items = sum(-(-len(v[2]) * group // NARROW_ROWS) for v in trailing) * heads
            share = 1
            while share < BLOCK_WAVES and 4 * items * 2 * share <= 3 * wave_slots:
                share *= 2

            def item_work(v):
                steps = -(-tiles(v[1]) // share) * -(-len(v[2]) * group // NARROW_ROWS)
                return NARROW_STARTUP_TILES + NARROW_STEP_TILES * steps + (NARROW_SHARE_TILES if share > 1 else 0.0)

            item_us = [item_work(v) * TILE_US_SHARED for v in trailing]
            narrow_bytes = sum(v[1] for v in trailing) * heads * 4 * head_dim
            # (a vnode holds `share` wave slots for as long as its waves walk their tiles)
            narrow_all_slots = max(sum(item_us) * heads * share / wave_slots, max(item_us),
                                   narrow_bytes / (NARROW_BYTES_PER_US * num_cus / DEFAULT_COMPUTE_UNITS))

            if overlap:
                # unequal programs end one after the other and the trailing blocks take their slots
                # while the longest still run: the launch lasts as long as its longest program, or
                # as long as all the work takes on all the slots
                first_row = max(1, (machine_slots // 2) // heads)    # programs that are the older block of their unit
                if shared:
                    longest_us = max(t * TILE_US_OLDER * (YOUNGER_BLOCK_SLOWDOWN if i >= first_row else 1.0)
                                     for i, t in enumerate(program_tiles))
                else:
                    longest_us = max(program_tiles) * tile_us
                modelled = max(longest_us,
                               sum(program_tiles) * heads / float(block_slots) * tile_us + narrow_all_slots)
            elif shared or not programs:
                modelled = wide_us + narrow_all_slots
            else:
                # programs on one block slot of every unit: the trailing blocks have the other half of
                # the wave slots while the programs run (and work at half their rate), all of them after
                modelled = max(wide_us, narrow_all_slots + wide_us / 2.0, max(item_us))
        else:
            modelled = wide_us

        def build() -> LaunchSchedule:
            # ---- the lists: wide pieces in program order, then the narrow vnodes
            new_kv_offs, new_kv_lens, new_q_offs, new_q_lens, rows_out = [], [], [], [], []
            prog_table = []
            row = 0

            def emit(off, length, reqs):
                nonlocal row
                new_kv_offs.append(off)
                new_kv_lens.append(length)
                new_q_offs.append(row)
                new_q_lens.append(len(reqs))
                rows_out.append(reqs)
                row += len(reqs)

            narrow_first = 0
            for p, prog in enumerate(programs):
                wide_first = len(new_kv_offs)
                for i in prog:
                    emit(*pieces[i][:3])
                # the two blocks of a compute unit (block b and b + 256) get opposite orders
                front = (p % per_round) < per_round // 2
                prog_table.append((wide_first, len(new_kv_offs), narrow_first, -len(shares[p]) if front else len(shares[p])))
                narrow_first += len(shares[p])
            n_wide = len(new_kv_offs)
            for off, length, reqs in narrow:
                emit(off, length, reqs)
            new_q_entries = np.concatenate(rows_out) if rows_out else np.zeros(0, dtype=np.int64)

            # scratch rows of every request, in row order (kernel_bench/fasttree.py:233-244)
            by_req = np.argsort(new_q_entries, kind="stable")
            req_lens = np.bincount(new_q_entries, minlength=int(batch_size)).astype(np.int64)[: int(batch_size)]
            req_offs = np.concatenate([[0], np.cumsum(req_lens)[:-1]]) if batch_size else np.zeros(0, dtype=np.int64)
            req_entries = np.concatenate([by_req, np.full(32, -1, dtype=np.int64)])

            i32 = lambda x: np.asarray(x, dtype=np.int32)
            return LaunchSchedule(
                kv_offs=i32(new_kv_offs), kv_lens=i32(new_kv_lens), q_offs=i32(new_q_offs), q_lens=i32(new_q_lens),
                q_entries=i32(new_q_entries), req_entries=i32(req_entries), req_offs=i32(req_offs), req_lens=i32(req_lens),
                phase_node_nums=[n_wide, len(new_kv_offs) - n_wide], phase_node_offsets=[0, n_wide],
                prog_table=i32(prog_table).reshape(-1, 4), narrow_in_programs=narrow_first,
                program_tiles=np.asarray(program_tiles, dtype=np.float64), block_slots=int(block_slots),
                modelled_us=float(modelled) + LAUNCH_US, num_cus=int(num_cus),
            )

        return float(modelled), build

    packed = finish(pieces, programs)
    if resident is not None:
        alone = finish(*resident, overlap=True)
        # preferred at about equal modelled duration: fewer vnodes (start-ups, scratch rows), and
        # the scattered rows of the trailing vnodes are fetched while wide blocks still compute
        if layout == "resident" or alone[0] <= RESIDENT_MARGIN * packed[0]:
            return alone
    return packed
