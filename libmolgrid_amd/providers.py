"""The data feed in front of the gridding path: example lists (``.types`` files), pre-typed atom
files (``.gninatypes``), ``.molcache2`` caches and the sampling schemes of the reference's
``ExampleProvider`` (include/libmolgrid/example_provider.h, exampleref_providers.h,
src/coord_cache.cpp, src/example_extractor.cpp).

Everything here runs on the host and produces ``Example`` objects for ``GridMaker``.  Molecule
files that need a chemistry toolkit (pdb, sdf, mol2, ...) are refused with an error; the reserved
file name ``none`` gives an empty coordinate set, as in the reference.
"""
import math
import mmap
import os
import pickle
import struct

import numpy as np

from . import gridding as _g
from .gridding import CoordinateSet, Example, ExampleVec
from .typers import AtomTyper, defaultGninaLigandTyper, defaultGninaReceptorTyper

_ATOM = np.dtype([("x", "<f4"), ("y", "<f4"), ("z", "<f4"), ("type", "<i4")])


class IterationScheme(object):
    Continuous, LargeEpoch, SmallEpoch = 0, 1, 2


_SETTINGS = [  # include/libmolgrid/example.h:24-45
    ("shuffle", False), ("balanced", False), ("stratify_receptor", False), ("labelpos", 0),
    ("stratify_pos", 1), ("stratify_abs", True), ("stratify_min", 0.0), ("stratify_max", 0.0),
    ("stratify_step", 0.0), ("group_batch_size", 1), ("max_group_size", 0),
    ("default_batch_size", 1), ("cache_structs", True), ("add_hydrogens", True),
    ("duplicate_first", False), ("num_copies", 1), ("make_vector_types", False),
    ("iteration_scheme", IterationScheme.Continuous), ("data_root", ""), ("recmolcache", ""),
    ("ligmolcache", ""),
]


class ExampleProviderSettings(object):
    def __init__(self, **kw):
        for name, default in _SETTINGS:
            setattr(self, name, default)
        self.update(kw)

    def update(self, kw):
        known = {name for name, _ in _SETTINGS}
        for k, v in kw.items():
            if k not in known:
                raise ValueError("Unknown example provider setting: " + k)
            setattr(self, k, v)

    def copy(self):
        return ExampleProviderSettings(**{name: getattr(self, name) for name, _ in _SETTINGS})


def _is_numeric(token):
    try:
        float(token)
        return True
    except ValueError:
        return False


class ExampleRef(object):
    """One line of a ``.types`` file: [group] labels... files... [# comment]
    (src/example.cpp:301-343)."""

    def __init__(self, line=None, numlabels=-1, hasgroup=False):
        self.files, self.labels, self.group, self.seqcont = [], [], -1, False
        if line is None:
            return
        tokens = line.split()
        if numlabels < 0:
            numlabels = 0
            for i, tok in enumerate(tokens):
                numlabels = i
                if not _is_numeric(tok):
                    break
            if hasgroup:
                numlabels -= 1
        pos = 0
        if hasgroup:
            self.group = int(float(tokens[0]))
            pos = 1
        self.labels = [float(t) for t in tokens[pos:pos + numlabels]]
        for tok in tokens[pos + numlabels:]:
            if tok.startswith("#"):
                break
            self.files.append(tok)
        if not self.files:
            raise ValueError("Missing molecular data in line: " + line)

    def copy(self):
        r = ExampleRef()
        r.files, r.labels, r.group, r.seqcont = list(self.files), list(self.labels), self.group, self.seqcont
        return r


# --------------------------------------------------------------------------------------------
# sampling schemes (include/libmolgrid/exampleref_providers.h, src/exampleref_providers.cpp)
# --------------------------------------------------------------------------------------------
def _shuffle(items):
    order = _g._rng.permutation(len(items))
    items[:] = [items[i] for i in order]


class ExampleRefProvider(object):
    def __init__(self, settings=None):
        self.cnt = 1   # epoch of the NEXT example

    def has_group(self):
        return False

    def check_batch_size(self, bsize):
        pass

    def populate(self, lines, numlabels=-1):
        for line in lines:
            line = line.strip()
            if line:
                self.addref(ExampleRef(line, numlabels, self.has_group()))
        return self.size()

    def get_small_epoch_num(self):
        return self.cnt // self.small_epoch_size()

    def get_large_epoch_num(self):
        return self.cnt // self.large_epoch_size()


class UniformExampleRefProvider(ExampleRefProvider):
    """One list, in file order or reshuffled at every pass; each example ``num_copies`` times."""

    def __init__(self, settings=None):
        super().__init__(settings)
        settings = settings or ExampleProviderSettings()
        self.all, self.current, self.current_copy, self.nlabels, self.epoch = [], 0, 0, 0, 0
        self.randomize, self.ncopies = bool(settings.shuffle), int(settings.num_copies)

    def addref(self, ref):
        self.all.append(ref)
        self.nlabels = len(ref.labels)

    def num_labels(self):
        return self.nlabels

    def setup(self):
        self.current = 0
        if self.randomize:
            _shuffle(self.all)
        if not self.all:
            raise ValueError("No valid examples found in training set.")

    def nextref(self):
        ref = self.all[self.current]
        if self.ncopies > 1:
            self.current_copy += 1
            if self.current_copy >= self.ncopies:
                self.current += 1
                self.current_copy = 0
        else:
            self.current += 1
        if self.current >= len(self.all):
            self.setup()
            self.epoch += 1
        self.cnt += 1
        return ref

    def size(self):
        return len(self.all)

    def __getitem__(self, idx):
        if idx >= len(self.all):
            raise ValueError("Invalid index: %d > %d" % (idx, len(self.all)))
        return self.all[idx]

    def get_small_epoch_num(self):
        return self.epoch

    def get_large_epoch_num(self):
        return self.epoch

    def small_epoch_size(self):
        return self.size()

    def large_epoch_size(self):
        return self.size()

    def reset(self):
        self.cnt, self.current, self.current_copy = 0, 0, 0


class BalancedExampleRefProvider(ExampleRefProvider):
    """Alternates between examples whose label at ``labelpos`` is non-zero and the others."""

    def __init__(self, settings=None):
        super().__init__(settings)
        settings = settings or ExampleProviderSettings()
        self.actives, self.decoys = UniformExampleRefProvider(settings), UniformExampleRefProvider(settings)
        self.current, self.labelpos = 0, int(settings.labelpos)

    def addref(self, ref):
        if self.labelpos >= len(ref.labels):
            raise ValueError("Example has no label at position %d but a label is required to "
                             "balance batches.  There are only %d labels"
                             % (self.labelpos, len(ref.labels)))
        (self.actives if ref.labels[self.labelpos] else self.decoys).addref(ref)

    def num_labels(self):
        return self.actives.num_labels()

    def setup(self):
        self.current = 0
        self.actives.setup()
        self.decoys.setup()

    def nextref(self):
        ref = self.actives.nextref() if self.current % 2 == 0 else self.decoys.nextref()
        self.current += 1
        self.cnt += 1
        return ref

    def size(self):
        return self.actives.size() + self.decoys.size()

    def num_actives(self):
        return self.actives.size()

    def num_decoys(self):
        return self.decoys.size()

    def small_epoch_size(self):
        return 2 * min(self.actives.size(), self.decoys.size())

    def large_epoch_size(self):
        return 2 * max(self.actives.size(), self.decoys.size())

    def reset(self):
        self.actives.reset()
        self.decoys.reset()
        self.current, self.cnt = 0, 0


class _Stratified(ExampleRefProvider):
    """Shared bookkeeping of the two stratifying providers: a list of sub-providers."""

    def num_labels(self):
        for p in self.examples:
            if p.size() > 0:
                return p.num_labels()
        return 0

    def size(self):
        return sum(p.size() for p in self.examples)

    def small_epoch_size(self):
        if not self.examples:
            raise ValueError("No valid stratified examples.")
        return min(p.small_epoch_size() for p in self.examples) * len(self.examples)

    def large_epoch_size(self):
        if not self.examples:
            raise ValueError("No valid stratified examples.")
        return max(p.large_epoch_size() for p in self.examples) * len(self.examples)


class ReceptorStratifiedExampleRefProvider(_Stratified):
    """Examples are grouped by receptor (first file); K examples are taken from each receptor in
    turn.  With a balanced sub-provider and K = 2 every receptor gives an active and a decoy."""

    def __init__(self, settings, make_sub, k=1):
        super().__init__(settings)
        self.settings, self.make_sub, self.k = settings, make_sub, k
        self.examples, self.recmap = [], {}
        self.currenti, self.currentk, self.randomize = 0, 0, bool(settings.shuffle)

    def addref(self, ref):
        if not ref.files:
            raise ValueError("Missing receptor from line")
        if ref.files[0] not in self.recmap:
            self.recmap[ref.files[0]] = len(self.examples)
            self.examples.append(self.make_sub(self.settings))
        self.examples[self.recmap[ref.files[0]]].addref(ref)

    def setup(self):
        if self.k <= 0:
            raise ValueError("Invalid sampling k for ReceptorStratifiedExampleRefProvider")
        self.currenti, self.currentk = 0, 0
        if self.k == 2 and self.examples and isinstance(self.examples[0], BalancedExampleRefProvider):
            # receptors without both actives and decoys are dropped
            self.examples = [p for p in self.examples if p.num_actives() > 0 and p.num_decoys() > 0]
        for p in self.examples:
            p.setup()
        if self.randomize:
            _shuffle(self.examples)

    def nextref(self):
        if not self.examples:
            raise ValueError("No valid stratified examples.")
        if self.currentk >= self.k:
            self.currentk = 0
            self.currenti += 1
        if self.currenti >= len(self.examples):
            self.currenti = 0
            if self.randomize:
                _shuffle(self.examples)
        if self.examples[self.currenti].size() == 0:
            raise RuntimeError("No valid sub-stratified examples.")
        ref = self.examples[self.currenti].nextref()
        self.currentk += 1
        self.cnt += 1
        return ref

    def reset(self):
        self.currenti, self.currentk, self.cnt = 0, 0, 0
        for p in self.examples:
            p.reset()


class ValueStratifiedExampleRefProvider(_Stratified):
    """Examples are binned by a label (its absolute value by default); the bins take turns."""

    def __init__(self, settings, make_sub):
        super().__init__(settings)
        self.max, self.min = float(settings.stratify_max), float(settings.stratify_min)
        self.step, self.use_abs = float(settings.stratify_step), bool(settings.stratify_abs)
        self.valpos = int(settings.stratify_pos)
        if self.valpos < 0:
            raise ValueError("Negative position for stratification value")
        if self.min == self.max:
            raise ValueError("Empty range for value stratification")
        maxbin = self._bin(self.max)
        if maxbin == 0:
            raise ValueError("Not enough bins for value stratification")
        self.examples = [make_sub(settings) for _ in range(maxbin + 1)]
        self.currenti = 0

    def _bin(self, val):
        if self.use_abs:
            val = abs(val)
        if val < self.min:
            val = self.min
        if val >= self.max:
            val = self.max - float(np.finfo(np.float32).eps)
        return int((val - self.min) / self.step)

    def addref(self, ref):
        if self.valpos >= len(ref.labels):
            raise ValueError("Invalid position for value stratification label")
        i = self._bin(ref.labels[self.valpos])
        if i >= len(self.examples):
            raise ValueError("Error with value stratification binning")
        self.examples[i].addref(ref)

    def setup(self):
        self.currenti = 0
        self.examples = [p for p in self.examples if p.size() > 0]
        for p in self.examples:
            p.setup()
        if not self.examples:
            raise ValueError("No examples in affinity stratification!")

    def nextref(self):
        ref = self.examples[self.currenti].nextref()
        self.currenti = (self.currenti + 1) % len(self.examples)
        self.cnt += 1
        return ref

    def reset(self):
        self.cnt, self.currenti = 0, 0
        for p in self.examples:
            p.reset()


class GroupedExampleRefProvider(ExampleRefProvider):
    """Time series: the first column of a line is its group; a batch holds the same frame of
    ``group_batch_size`` groups, successive batches walk through the frames, short groups are
    padded with empty examples whose labels are NaN."""

    def __init__(self, settings, make_sub):
        super().__init__(settings)
        self.examples = make_sub(settings)
        self.batch_size, self.maxgroupsize = int(settings.group_batch_size), int(settings.max_group_size)
        self.frame_groups = {}
        self.current_ts, self.current_group_index = 0, 0
        self.current_groups = [self.maxgroupsize] * self.batch_size

    def has_group(self):
        return True

    def check_batch_size(self, bsize):
        if bsize != self.batch_size:
            raise ValueError("Requested batch size %d does not match configured group batch "
                             "size %d" % (bsize, self.batch_size))

    def addref(self, ref):
        if ref.group not in self.frame_groups:
            self.examples.addref(ref)   # the sub-provider only selects the groups
            self.frame_groups[ref.group] = []
        self.frame_groups[ref.group].append(ref)

    def setup(self):
        self.examples.setup()

    def num_labels(self):
        return self.examples.num_labels()

    def nextref(self):
        if self.current_group_index >= len(self.current_groups):
            self.current_group_index = 0
            self.current_ts += 1
        if self.current_ts >= self.maxgroupsize:
            self.current_ts = 0
        if self.current_ts == 0:
            self.current_groups[self.current_group_index] = self.examples.nextref().group
        group = self.current_groups[self.current_group_index]
        series = self.frame_groups[group]
        if self.current_ts < len(series):
            ref = series[self.current_ts].copy()
        else:
            ref = series[-1].copy()
            ref.files = ["none"] * len(ref.files)
            ref.labels = [float("nan")] * len(ref.labels)
        ref.group = group
        ref.seqcont = self.current_ts > 0
        self.current_group_index += 1
        self.cnt += 1
        return ref

    def size(self):
        return self.examples.size()

    def small_epoch_size(self):
        return self.examples.small_epoch_size()

    def large_epoch_size(self):
        return self.examples.large_epoch_size()

    def reset(self):
        self.cnt, self.current_ts, self.current_group_index = 0, 0, 0
        self.examples.reset()


def create_provider(settings):
    """Value stratification > receptor stratification > balancing, optionally grouped
    (src/example_provider.cpp:96-211)."""
    balanced, strat_rec = bool(settings.balanced), bool(settings.stratify_receptor)
    strat_aff = settings.stratify_max != settings.stratify_min
    grouped = settings.max_group_size > 1

    if strat_rec and balanced:
        def inner(s):
            return ReceptorStratifiedExampleRefProvider(s, BalancedExampleRefProvider, 2)
    elif strat_rec:
        def inner(s):
            return ReceptorStratifiedExampleRefProvider(s, UniformExampleRefProvider, 1)
    elif balanced:
        inner = BalancedExampleRefProvider
    else:
        inner = UniformExampleRefProvider
    if strat_aff:
        base = inner

        def inner(s):   # noqa: F811
            return ValueStratifiedExampleRefProvider(s, base)
    if grouped and not (strat_rec and not balanced and not strat_aff):
        # (the reference does not group a receptor-stratified, unbalanced provider)
        return GroupedExampleRefProvider(settings, inner)
    return inner(settings)


# --------------------------------------------------------------------------------------------
# coordinates of one file (src/coord_cache.cpp)
# --------------------------------------------------------------------------------------------
class CoordCache(object):
    """Turns a file name into a typed CoordinateSet: from a ``.molcache2`` cache when the name is
    in it, from memory when it was read before, else from a ``.gninatypes`` file."""

    def __init__(self, typer=None, settings=None, molcache=""):
        settings = settings or ExampleProviderSettings()
        self.typer = typer if typer is not None else defaultGninaLigandTyper
        self.data_root, self.use_cache = settings.data_root, bool(settings.cache_structs)
        self.make_vector_types = bool(settings.make_vector_types)
        self.memcache, self.offsets, self.map = {}, {}, None
        if molcache:
            if not os.path.exists(molcache):
                molcache = os.path.join(self.data_root, molcache)
            try:
                f = open(molcache, "rb")
            except OSError:
                raise ValueError("Could not open file: " + molcache)
            with f:
                head = f.read(12)
                if len(head) < 12 or struct.unpack("<i", head[:4])[0] != -1:
                    raise ValueError(molcache + " is not a valid molcache2 file")
                start = struct.unpack("<Q", head[4:12])[0]
                self.map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
            # after the atom data: (name length, name, offset) records
            pos, size = start, len(self.map)
            while pos < size:
                n = self.map[pos]
                name = self.map[pos + 1:pos + 1 + n].decode()
                self.offsets[name] = struct.unpack_from("<Q", self.map, pos + 1 + n)[0]
                pos += 1 + n + 8

    def num_types(self):
        return self.typer.num_types()

    def get_type_names(self):
        return self.typer.get_type_names()

    def _typed(self, atoms, fname):
        """CoordinateSet of the pre-typed atoms the typer keeps."""
        if self.typer.is_vector_typer():
            raise ValueError("Vector typer used with pre-typed files")
        kinds = {}
        types = np.empty(len(atoms), np.float32)
        radii = np.empty(len(atoms), np.float32)
        for i, t in enumerate(atoms["type"].tolist()):
            if t not in kinds:
                kinds[t] = self.typer.get_int_type(t)
            types[i], radii[i] = kinds[t]
        keep = types >= 0
        coords = np.stack([atoms["x"], atoms["y"], atoms["z"]], axis=1)[keep]
        c = CoordinateSet(np.ascontiguousarray(coords, np.float32), types[keep], radii[keep],
                          self.typer.num_types())
        c.src = fname
        return c

    def set_coords(self, fname, coord):
        coord.copyInto(self.make_coords(fname))

    def make_coords(self, fname):
        if fname in self.offsets:
            off = self.offsets[fname]
            natoms = struct.unpack_from("<I", self.map, off)[0]
            atoms = np.frombuffer(self.map, _ATOM, natoms, off + 4)
            return self._typed(atoms, fname)
        if fname in self.memcache:
            return self.memcache[fname].clone()
        full = os.path.join(self.data_root, fname) if self.data_root else fname
        if fname.endswith(".gninatypes"):
            try:
                raw = np.fromfile(full, np.uint8)
            except OSError:
                raise ValueError("Could not read " + full)
            atoms = raw[:len(raw) // _ATOM.itemsize * _ATOM.itemsize].view(_ATOM)
            coord = self._typed(atoms, fname)
        elif fname.endswith("none"):
            coord = CoordinateSet()
            coord.max_type = self.typer.num_types()
        else:
            raise ValueError("Could not read %s: reading molecule files needs a chemistry toolkit; "
                             "this package reads .gninatypes files and .molcache2 caches" % full)
        if self.make_vector_types and hasattr(self.typer, "get_type_radii"):
            coord.make_vector_types(False, self.typer.get_type_radii())
        if self.use_cache:
            self.memcache[fname] = coord.clone()
        return coord

    def mem_cache_size(self):
        return len(self.memcache)

    def _dump(self):
        return {k: (v.coords.tonumpy(), v.type_index.tonumpy(), v.type_vector.tonumpy(),
                    v.radii.tonumpy(), v.max_type, v.src) for k, v in self.memcache.items()}

    def _restore(self, saved):
        for k, (coords, tindex, tvec, radii, max_type, src) in saved.items():
            c = CoordinateSet()
            c.coords, c.type_index = _g._managed(coords, 2), _g._managed(tindex, 1)
            c.type_vector, c.radii = _g._managed(tvec, 2), _g._managed(radii, 1)
            c.max_type, c.src = max_type, src
            self.memcache[k] = c


class ExampleExtractor(object):
    """One CoordCache per file position of a line, the last one repeated
    (src/example_extractor.cpp)."""

    def __init__(self, settings, typers, molcaches=()):
        if not typers:
            raise ValueError("Need at least one atom typer for example extractor")
        self.duplicate_poses = bool(settings.duplicate_first)
        molcaches = list(molcaches)
        if not molcaches:
            if settings.recmolcache:
                molcaches.append(settings.recmolcache)
            if settings.ligmolcache:
                while len(molcaches) < len(typers):
                    molcaches.append(settings.ligmolcache)
        self.coord_caches = [CoordCache(t, settings, molcaches[i] if i < len(molcaches) else "")
                             for i, t in enumerate(typers)]

    def _cache(self, i):
        return self.coord_caches[min(i, len(self.coord_caches) - 1)]

    def extract(self, ref):
        ex = Example()
        ex.labels, ex.group, ex.seqcont = list(ref.labels), ref.group, ref.seqcont
        n = len(ref.files)
        if not self.duplicate_poses or n < 3:
            ex.coord_sets = [self._cache(i).make_coords(f) for i, f in enumerate(ref.files)]
        else:   # the first set (receptor) is repeated in front of every other one
            rec = self._cache(0).make_coords(ref.files[0])
            ex.coord_sets = []
            for i in range(1, n):
                ex.coord_sets.append(rec if i == 1 else rec.clone())
                ex.coord_sets.append(self._cache(i).make_coords(ref.files[i]))
        return ex

    def _count_types(self, n):
        ret = sum(self._cache(i).num_types() for i in range(n))
        if self.duplicate_poses and len(self.coord_caches) > 2:
            ret += self.coord_caches[0].num_types() * (len(self.coord_caches) - 2)
        return ret

    def num_types(self, ref=None):
        return self._count_types(len(self.coord_caches) if ref is None else len(ref.files))

    def get_type_names(self):
        return ["%d_%s" % (i, name) for i, c in enumerate(self.coord_caches)
                for name in c.get_type_names()]

    def mem_caches_size(self):
        return sum(c.mem_cache_size() for c in self.coord_caches)


class ExampleProvider(object):
    """ExampleProvider([settings], [typer, ...], **settings) as in the reference's Python module:
    without typers the default receptor and ligand typers (14 channels each) are used."""

    def __init__(self, *args, **kw):
        args = list(args)
        settings = ExampleProviderSettings()
        if args and isinstance(args[0], ExampleProviderSettings):
            settings = args.pop(0).copy()
        settings.update(kw)
        for t in args:
            if not isinstance(t, AtomTyper):
                raise TypeError("ExampleProvider takes a settings object and atom typers")
        self.init_settings = settings
        self.provider = create_provider(settings)
        typers = args or [defaultGninaReceptorTyper, defaultGninaLigandTyper]
        molcaches = [settings.recmolcache, settings.ligmolcache] if not args else []
        self.extractor = ExampleExtractor(settings, typers, molcaches)
        self.last_epoch = 0

    def populate(self, file_name, num_labels=-1):
        names = [file_name] if isinstance(file_name, str) else list(file_name)
        for name in names:
            try:
                f = open(name)
            except OSError:
                raise ValueError("Could not open file " + name)
            with f:
                self.provider.populate(f, num_labels)
        self.provider.setup()

    def num_labels(self):
        return self.provider.num_labels()

    def settings(self):
        return self.init_settings

    def num_types(self):
        return self.extractor.num_types()

    def size(self):
        return self.provider.size()

    def get_type_names(self):
        return self.extractor.get_type_names()

    def next(self):
        return self.extractor.extract(self.provider.nextref())

    def next_batch(self, batch_size=0):
        if batch_size == 0:
            batch_size = int(self.init_settings.default_batch_size)
        self.provider.check_batch_size(batch_size)
        return ExampleVec(self.extractor.extract(self.provider.nextref())
                          for _ in range(batch_size))

    def skip(self, n):
        for _ in range(n):
            self.provider.nextref()

    def get_small_epoch_num(self):
        return self.provider.get_small_epoch_num()

    def get_large_epoch_num(self):
        return self.provider.get_large_epoch_num()

    def small_epoch_size(self):
        return self.provider.small_epoch_size()

    def large_epoch_size(self):
        return self.provider.large_epoch_size()

    def reset(self):
        self.provider.reset()

    def at_new_epoch(self):
        scheme = self.init_settings.iteration_scheme
        if scheme == IterationScheme.LargeEpoch:
            e = self.provider.get_large_epoch_num()
        elif scheme == IterationScheme.SmallEpoch:
            e = self.provider.get_small_epoch_num()
        else:
            return False
        if e != self.last_epoch:
            self.last_epoch = e
            return True
        return False

    def __iter__(self):
        return self

    def __next__(self):
        if self.at_new_epoch():
            raise StopIteration("End of epoch.")
        return self.next_batch()

    # the in-memory caches: this package's own format (the reference writes a boost archive)
    def mem_caches_size(self):
        return self.extractor.mem_caches_size()

    def save_mem_caches(self, file_name):
        with open(file_name, "wb") as f:
            pickle.dump([c._dump() for c in self.extractor.coord_caches], f)

    def load_mem_caches(self, file_name):
        with open(file_name, "rb") as f:
            saved = pickle.load(f)
        for c, s in zip(self.extractor.coord_caches, saved):
            c._restore(s)


class ExampleDataset(object):
    """The examples of a list by position, in file order (include/libmolgrid/example_dataset.h)."""

    def __init__(self, *args, **kw):
        args = list(args)
        settings = ExampleProviderSettings()
        if args and isinstance(args[0], ExampleProviderSettings):
            settings = args.pop(0).copy()
        settings.update(kw)
        self.init_settings = settings
        self.provider = UniformExampleRefProvider(ExampleProviderSettings())
        typers = args or [defaultGninaReceptorTyper, defaultGninaLigandTyper]
        molcaches = [settings.recmolcache, settings.ligmolcache] if not args else []
        self.extractor = ExampleExtractor(settings, typers, molcaches)

    def populate(self, file_name, num_labels=-1):
        names = [file_name] if isinstance(file_name, str) else list(file_name)
        for name in names:
            try:
                f = open(name)
            except OSError:
                raise ValueError("Could not open file " + name)
            with f:
                self.provider.populate(f, num_labels)

    def __len__(self):
        return self.provider.size()

    def size(self):
        return self.provider.size()

    def __getitem__(self, idx):
        n = self.provider.size()
        if idx < 0:
            idx += n
        if not 0 <= idx < n:
            raise IndexError("Invalid index: %d" % idx)
        return self.extractor.extract(self.provider[idx])

    def num_labels(self):
        return self.provider.num_labels()

    def settings(self):
        return self.init_settings

    def num_types(self):
        return self.extractor.num_types()

    def get_type_names(self):
        return self.extractor.get_type_names()


__all__ = ["IterationScheme", "ExampleProviderSettings", "ExampleRef", "ExampleProvider", "ExampleDataset",
           "ExampleExtractor", "CoordCache", "UniformExampleRefProvider",
           "BalancedExampleRefProvider", "ReceptorStratifiedExampleRefProvider",
           "ValueStratifiedExampleRefProvider", "GroupedExampleRefProvider"]
