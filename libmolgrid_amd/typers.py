"""Atom typers for pre-typed input (``.gninatypes`` files and ``.molcache2`` caches), with the
names and results of the reference's typers (include/libmolgrid/atom_typer.h, src/atom_typer.cpp).

A pre-typed atom carries the integer gnina ("smina") type that the reference's tools assigned when
the file was written; a typer turns that integer into a channel index and a radius
(``get_int_type``).  Typing atoms of a molecule file (``get_atom_type_index`` on a toolkit atom)
needs a chemistry toolkit and is not part of this package.
"""
import io

# gnina atom types: name, atomic number, covalent radius, XS radius
# (src/atom_typer.cpp:33-64; the AutoDock fields are not used by the index typers)
_GNINA_TYPES = [
    ("Hydrogen", 1, 0.37, 0.37),
    ("PolarHydrogen", 1, 0.37, 0.37),
    ("AliphaticCarbonXSHydrophobe", 6, 0.77, 1.9),
    ("AliphaticCarbonXSNonHydrophobe", 6, 0.77, 1.9),
    ("AromaticCarbonXSHydrophobe", 6, 0.77, 1.9),
    ("AromaticCarbonXSNonHydrophobe", 6, 0.77, 1.9),
    ("Nitrogen", 7, 0.75, 1.8),
    ("NitrogenXSDonor", 7, 0.75, 1.8),
    ("NitrogenXSDonorAcceptor", 7, 0.75, 1.8),
    ("NitrogenXSAcceptor", 7, 0.75, 1.8),
    ("Oxygen", 8, 0.73, 1.7),
    ("OxygenXSDonor", 8, 0.73, 1.7),
    ("OxygenXSDonorAcceptor", 8, 0.73, 1.7),
    ("OxygenXSAcceptor", 8, 0.73, 1.7),
    ("Sulfur", 16, 1.02, 2.0),
    ("SulfurAcceptor", 16, 1.02, 2.0),
    ("Phosphorus", 15, 1.06, 2.1),
    ("Fluorine", 9, 0.71, 1.5),
    ("Chlorine", 17, 0.99, 1.8),
    ("Bromine", 35, 1.14, 2.0),
    ("Iodine", 53, 1.33, 2.2),
    ("Magnesium", 12, 1.30, 1.2),
    ("Manganese", 25, 1.39, 1.2),
    ("Zinc", 30, 1.31, 1.2),
    ("Calcium", 20, 1.74, 1.2),
    ("Iron", 26, 1.25, 1.2),
    ("GenericMetal", 0, 1.75, 1.2),
    ("Boron", 5, 0.90, 1.92),
]
_GENERIC_METAL = 26

# Element names and covalent radii by atomic number (index 0: no element).  The reference takes
# them from its chemistry toolkit's element table, which is not available here; these are the
# published covalent radii that table is built from (Cordero et al., Dalton Trans. 2008), so the
# radii of the element typers are not pinned against the reference.
_ELEMENTS = [
    ("Xx", 0.0), ("Hydrogen", 0.31), ("Helium", 0.28), ("Lithium", 1.28), ("Beryllium", 0.96),
    ("Boron", 0.84), ("Carbon", 0.76), ("Nitrogen", 0.71), ("Oxygen", 0.66), ("Fluorine", 0.57),
    ("Neon", 0.58), ("Sodium", 1.66), ("Magnesium", 1.41), ("Aluminium", 1.21), ("Silicon", 1.11),
    ("Phosphorus", 1.07), ("Sulfur", 1.05), ("Chlorine", 1.02), ("Argon", 1.06),
    ("Potassium", 2.03), ("Calcium", 1.76), ("Scandium", 1.70), ("Titanium", 1.60),
    ("Vanadium", 1.53), ("Chromium", 1.39), ("Manganese", 1.39), ("Iron", 1.32), ("Cobalt", 1.26),
    ("Nickel", 1.24), ("Copper", 1.32), ("Zinc", 1.22), ("Gallium", 1.22), ("Germanium", 1.20),
    ("Arsenic", 1.19), ("Selenium", 1.20), ("Bromine", 1.20), ("Krypton", 1.16),
    ("Rubidium", 2.20), ("Strontium", 1.95), ("Yttrium", 1.90), ("Zirconium", 1.75),
    ("Niobium", 1.64), ("Molybdenum", 1.54), ("Technetium", 1.47), ("Ruthenium", 1.46),
    ("Rhodium", 1.42), ("Palladium", 1.39), ("Silver", 1.45), ("Cadmium", 1.44), ("Indium", 1.42),
    ("Tin", 1.39), ("Antimony", 1.39), ("Tellurium", 1.38), ("Iodine", 1.39), ("Xenon", 1.40),
    ("Caesium", 2.44), ("Barium", 2.15), ("Lanthanum", 2.07), ("Cerium", 2.04),
    ("Praseodymium", 2.03), ("Neodymium", 2.01), ("Promethium", 1.99), ("Samarium", 1.98),
    ("Europium", 1.98), ("Gadolinium", 1.96), ("Terbium", 1.94), ("Dysprosium", 1.92),
    ("Holmium", 1.92), ("Erbium", 1.89), ("Thulium", 1.90), ("Ytterbium", 1.87),
    ("Lutetium", 1.87), ("Hafnium", 1.75), ("Tantalum", 1.70), ("Tungsten", 1.62),
    ("Rhenium", 1.51), ("Osmium", 1.44), ("Iridium", 1.41), ("Platinum", 1.36), ("Gold", 1.36),
    ("Mercury", 1.32), ("Thallium", 1.45), ("Lead", 1.46), ("Bismuth", 1.48), ("Polonium", 1.40),
    ("Astatine", 1.50), ("Radon", 1.50), ("Francium", 2.60), ("Radium", 2.21), ("Actinium", 2.15),
    ("Thorium", 2.06), ("Protactinium", 2.00), ("Uranium", 1.96), ("Neptunium", 1.90),
    ("Plutonium", 1.87), ("Americium", 1.80), ("Curium", 1.69),
]


def _element(elem):
    if 0 <= elem < len(_ELEMENTS):
        return _ELEMENTS[elem]
    return (str(elem), 1.6)


class AtomTyper(object):
    def is_vector_typer(self):
        return False


class AtomIndexTyper(AtomTyper):
    """Base of the typers that give one channel index per atom."""

    def num_types(self):
        raise NotImplementedError

    def get_int_type(self, t):
        """(channel, radius) of a pre-typed atom; a negative channel drops the atom."""
        raise NotImplementedError

    def get_type_names(self):
        raise NotImplementedError

    def get_type_radii(self):
        raise NotImplementedError

    def get_atom_type_index(self, atom):
        raise NotImplementedError("typing an atom of a molecule needs a chemistry toolkit; "
                                  "only pre-typed input (get_int_type) is supported")


class GninaIndexTyper(AtomIndexTyper):
    """The 28 gnina types; radius is the XS radius or, on request, the covalent radius
    (src/atom_typer.cpp:66-200)."""
    NumTypes = len(_GNINA_TYPES)

    def __init__(self, use_covalent_radius=False):
        self.use_covalent = bool(use_covalent_radius)

    def num_types(self):
        return self.NumTypes

    def _radius(self, t):
        return _GNINA_TYPES[t][2] if self.use_covalent else _GNINA_TYPES[t][3]

    def get_int_type(self, t):
        ret = t if t < self.NumTypes else _GENERIC_METAL
        return ret, self._radius(ret)

    def get_type_names(self):
        return [r[0] for r in _GNINA_TYPES]

    def get_type_radii(self):
        return [self._radius(t) for t in range(self.NumTypes)]

    @staticmethod
    def gnina_type_name(t):
        return _GNINA_TYPES[t][0] if 0 <= t < len(_GNINA_TYPES) else "Unsupported"


class ElementIndexTyper(AtomIndexTyper):
    """Channel = atomic number, numbers from ``maxe`` on map to 0 (src/atom_typer.cpp:202-245)."""

    def __init__(self, maxe=84):
        self.last_elem = int(maxe)

    def num_types(self):
        return self.last_elem

    def get_int_type(self, elem):
        radius = _element(elem)[1]
        if elem >= self.last_elem:
            elem = 0
        return int(elem), radius

    def get_type_names(self):
        return ["GenericAtom"] + [_element(i)[0] for i in range(1, self.last_elem)]

    def get_type_radii(self):
        return [0.0] + [_element(i)[1] for i in range(1, self.last_elem)]


class NullIndexTyper(AtomIndexTyper):
    """No types at all: every atom is dropped (include/libmolgrid/atom_typer.h:246-266)."""

    def num_types(self):
        return 0

    def get_int_type(self, t):
        return -1, 0.0

    def get_type_names(self):
        return []

    def get_type_radii(self):
        return []


class _FileAtomMapper(object):
    """Each non-blank line of the map lists the old type names that share one new type
    (src/atom_typer.cpp:416-466)."""

    def __init__(self, source, old_names):
        if isinstance(source, str):
            try:
                stream = open(source)
            except OSError:
                raise ValueError("Could not open " + source)
        else:
            stream = source
        old = {name: i for i, name in enumerate(old_names)}
        self.old_to_new = [-1] * len(old_names)
        self.new_names = []
        for line in stream:
            names = line.split()
            if not names:
                continue
            new_type = len(self.new_names)
            self.new_names.append("_".join(names))
            for name in names:
                if name not in old:
                    raise ValueError("Invalid atom type " + name)
                self.old_to_new[old[name]] = new_type
        if isinstance(source, str):
            stream.close()

    def num_types(self):
        return len(self.new_names)

    def get_new_type(self, t):
        return self.old_to_new[t] if 0 <= t < len(self.old_to_new) else -1

    def get_type_names(self):
        return list(self.new_names)


class _SubsetAtomMapper(object):
    """Keep some old types (or merge lists of them), optionally with a catch-all for the rest
    (src/atom_typer.cpp:468-520)."""

    def __init__(self, subset, include_catchall, old_names):
        self.old_to_new = {}
        self.new_names = []
        for i, entry in enumerate(subset):
            olds = list(entry) if isinstance(entry, (list, tuple)) else [entry]
            for o in olds:
                self.old_to_new[int(o)] = i
            self.new_names.append("_".join(old_names[o] if o < len(old_names) else str(o)
                                           for o in olds))
        self.default_type = -1
        if include_catchall:
            self.default_type = len(subset)
            self.new_names.append("GenericAtom")

    def num_types(self):
        return len(self.new_names)

    def get_new_type(self, t):
        return self.old_to_new.get(t, self.default_type)

    def get_type_names(self):
        return list(self.new_names)


class _MappedIndexTyper(AtomIndexTyper):
    """A typer followed by a mapper; the radius of a new type is the mean of the radii of the old
    types it gathers (include/libmolgrid/atom_typer.h:315-372)."""

    def __init__(self, mapper, typer):
        self.mapper, self.typer = mapper, typer
        gathered = [[] for _ in range(mapper.num_types())]
        for old in range(typer.num_types()):
            t, r = typer.get_int_type(old)
            if t >= 0:
                new = mapper.get_new_type(t)
                if 0 <= new < len(gathered):
                    gathered[new].append(r)
        self.type_radii = [sum(g) / len(g) if g else float("nan") for g in gathered]

    def num_types(self):
        return self.mapper.num_types()

    def get_int_type(self, t):
        old, radius = self.typer.get_int_type(t)
        return self.mapper.get_new_type(old), radius

    def get_type_names(self):
        return self.mapper.get_type_names()

    def get_type_radii(self):
        return list(self.type_radii)


class FileMappedGninaTyper(_MappedIndexTyper):
    def __init__(self, source, use_covalent_radius=False):
        typer = GninaIndexTyper(use_covalent_radius)
        super().__init__(_FileAtomMapper(source, typer.get_type_names()), typer)


class FileMappedElementTyper(_MappedIndexTyper):
    def __init__(self, source, maxe=84):
        typer = ElementIndexTyper(maxe)
        super().__init__(_FileAtomMapper(source, typer.get_type_names()), typer)


class SubsettedGninaTyper(_MappedIndexTyper):
    def __init__(self, subset, catchall=True, use_covalent_radius=False):
        typer = GninaIndexTyper(use_covalent_radius)
        super().__init__(_SubsetAtomMapper(subset, catchall, typer.get_type_names()), typer)


class SubsettedElementTyper(_MappedIndexTyper):
    def __init__(self, subset, catchall=True, maxe=84):
        typer = ElementIndexTyper(maxe)
        super().__init__(_SubsetAtomMapper(subset, catchall, typer.get_type_names()), typer)


# the default receptor and ligand channels, 14 each (src/atom_typer.cpp:524-559)
_RECMAP = """AliphaticCarbonXSHydrophobe
AliphaticCarbonXSNonHydrophobe
AromaticCarbonXSHydrophobe
AromaticCarbonXSNonHydrophobe
Bromine Iodine Chlorine Fluorine
Nitrogen NitrogenXSAcceptor
NitrogenXSDonor NitrogenXSDonorAcceptor
Oxygen OxygenXSAcceptor
OxygenXSDonorAcceptor OxygenXSDonor
Sulfur SulfurAcceptor
Phosphorus
Calcium
Zinc
GenericMetal Boron Manganese Magnesium Iron
"""
_LIGMAP = """AliphaticCarbonXSHydrophobe
AliphaticCarbonXSNonHydrophobe
AromaticCarbonXSHydrophobe
AromaticCarbonXSNonHydrophobe
Bromine Iodine
Chlorine
Fluorine
Nitrogen NitrogenXSAcceptor
NitrogenXSDonor NitrogenXSDonorAcceptor
Oxygen OxygenXSAcceptor
OxygenXSDonorAcceptor OxygenXSDonor
Sulfur SulfurAcceptor
Phosphorus
GenericMetal Boron Manganese Magnesium Zinc Calcium Iron
"""
defaultGninaReceptorTyper = FileMappedGninaTyper(io.StringIO(_RECMAP))
defaultGninaLigandTyper = FileMappedGninaTyper(io.StringIO(_LIGMAP))

__all__ = ["AtomTyper", "AtomIndexTyper", "GninaIndexTyper", "ElementIndexTyper", "NullIndexTyper",
           "FileMappedGninaTyper", "FileMappedElementTyper", "SubsettedGninaTyper",
           "SubsettedElementTyper", "defaultGninaReceptorTyper", "defaultGninaLigandTyper"]
