"""One calling convention over the three address registries the tests compare:
the oracle restatement, the reference's own HybmVaManager (oracle/_ref) and the
product's VaManager behind the C ABI."""

NO_RANK = 0xFFFFFFFF


class OracleVa:
    name = "oracle"

    def __init__(self, o):
        self.o = o

    def clear(self):
        self.o.orc_va_clear()

    def add(self, gva, size, mem_type, lva, rank):
        return self.o.orc_va_add(gva, size, mem_type, lva, rank, NO_RANK)

    def add_external(self, gva, size, mem_type, lva, rank, imported=NO_RANK):
        return self.o.orc_va_add(gva, size, mem_type, lva, rank, imported)

    def remove(self, va):
        self.o.orc_va_remove(va)

    def gva_of_lva(self, a):
        return self.o.orc_va_gva_of_lva(a)

    def lva_of_gva(self, a):
        return self.o.orc_va_lva_of_gva(a)

    def is_gva(self, a):
        return bool(self.o.orc_va_is_gva(a))

    def is_known(self, a):
        return bool(self.o.orc_va_is_known(a))

    def mem_type(self, a):
        return self.o.orc_va_mem_type(a)

    def rank(self, a):
        return self.o.orc_va_rank(a)

    def infer(self, s, d):
        return self.o.orc_va_infer_direction(s, d)

    def reserve(self, rank, size, mem_type):
        return self.o.orc_va_reserve(size, mem_type)

    def unreserve(self, start):
        self.o.orc_va_unreserve(start)


class RefVa:
    name = "reference"

    def __init__(self, r):
        self.r = r

    def clear(self):
        self.r.ref_va_clear()

    def add(self, gva, size, mem_type, lva, rank):
        return self.r.ref_va_add(gva, size, mem_type, lva, rank)

    def add_external(self, gva, size, mem_type, lva, rank, imported=NO_RANK):
        return self.r.ref_va_add_external(gva, size, mem_type, lva, rank, imported)

    def remove(self, va):
        self.r.ref_va_remove(va)

    def gva_of_lva(self, a):
        return self.r.ref_va_gva_of_lva(a)

    def lva_of_gva(self, a):
        return self.r.ref_va_lva_of_gva(a)

    def is_gva(self, a):
        return bool(self.r.ref_va_is_gva(a))

    def is_known(self, a):
        return bool(self.r.ref_va_is_known(a))

    def mem_type(self, a):
        return self.r.ref_va_mem_type(a)

    def rank(self, a):
        return self.r.ref_va_rank(a)

    def infer(self, s, d):
        return self.r.ref_va_infer_direction(s, d)

    def reserve(self, rank, size, mem_type):
        return self.r.ref_va_reserve(rank, size, mem_type)

    def unreserve(self, start):
        self.r.ref_va_unreserve(start)


class ProductVa:
    name = "product"

    def __init__(self, lib):
        self.l = lib

    def clear(self):
        self.l.mf_va_clear()

    def add(self, gva, size, mem_type, lva, rank):
        return self.l.mf_va_add(gva, size, mem_type, lva, rank)

    def add_external(self, gva, size, mem_type, lva, rank, imported=NO_RANK):
        return self.l.mf_va_add_external(gva, size, mem_type, lva, rank, imported)

    def remove(self, va):
        self.l.mf_va_remove(va)

    def gva_of_lva(self, a):
        return self.l.mf_va_gva_of_lva(a)

    def lva_of_gva(self, a):
        return self.l.mf_va_lva_of_gva(a)

    def is_gva(self, a):
        return bool(self.l.mf_va_is_gva(a))

    def is_known(self, a):
        return bool(self.l.mf_va_is_known(a))

    def mem_type(self, a):
        return self.l.mf_va_mem_type(a)

    def rank(self, a):
        return self.l.mf_va_rank(a)

    def infer(self, s, d):
        return self.l.mf_va_infer_direction(s, d)

    def reserve(self, rank, size, mem_type):
        return self.l.mf_va_reserve(rank, size, mem_type)

    def unreserve(self, start):
        self.l.mf_va_unreserve(start)
