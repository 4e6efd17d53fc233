"""A plain statement of the cache bookkeeping and of the scheduler's policy, in a
few Python classes, for comparison with the host library step by step.

Policy (the reference's scheduler, /root/reference/src/paged_attention/scheduler.zig:
97-245, with the changes the engine documents): requests wait in arrival order;
each step serves running requests first, those that decode (one token left) before
those still in their prompt, each group in arrival order, every request with
min(tokens left, budget left, chunk size) tokens; when a request's pages do not
fit, the running request that arrived last gives everything back and returns to
the front of the line, until the pages fit or the request itself was the victim;
then waiting requests are admitted head of the line first while a slot, the budget,
the number of running requests and the pages for their first portion allow.  Pages:
LIFO free list (scheduler.zig's allocator, allocator.zig:72-86), a page index p of a
group's table is given back once every key in it lies behind the window.
"""

FREED = -1


class PlainOutOfPages(Exception):
    pass


class PlainCache:
    def __init__(self, windows, num_pages, page_size, num_slots):
        self.ps = page_size
        self.windows = list(windows)
        self.free = [list(range(num_pages - 1, -1, -1)) for _ in windows]   # pop() gives 0 first
        self.free_slots = list(range(num_slots - 1, -1, -1))
        self.req = {}        # id -> dict(slot, tokens, tables)

    def admit(self, r):
        self.req[r] = {"slot": self.free_slots.pop(), "tokens": 0,
                       "tables": [[] for _ in self.windows]}

    def needed(self, r, n):
        st = self.req[r]
        want = -(-(st["tokens"] + n) // self.ps)
        return [max(0, want - len(t)) for t in st["tables"]]

    def fits(self, r, n, promised):
        return all(need <= len(self.free[g]) - promised[g]
                   for g, need in enumerate(self.needed(r, n)))

    def reserve(self, r, n):
        need = self.needed(r, n)
        assert all(k <= len(self.free[g]) for g, k in enumerate(need))
        for g, k in enumerate(need):
            for _ in range(k):
                self.req[r]["tables"][g].append(self.free[g].pop())

    def commit(self, r, n):
        st = self.req[r]
        st["tokens"] += n
        for g, w in enumerate(self.windows):
            if w <= 0:
                continue
            first_needed = st["tokens"] - w + 1
            for p in range(min(max(first_needed, 0) // self.ps, len(st["tables"][g]))):
                if st["tables"][g][p] != FREED:
                    self.free[g].append(st["tables"][g][p])
                    st["tables"][g][p] = FREED

    def release(self, r):
        st = self.req.pop(r)
        for g, table in enumerate(st["tables"]):
            for page in table:
                if page != FREED:
                    self.free[g].append(page)
        self.free_slots.append(st["slot"])


class PlainScheduler:
    def __init__(self, cache, max_num_seqs, max_tokens, chunk, max_model_len=0):
        self.cache, self.max_num_seqs, self.max_tokens, self.chunk = cache, max_num_seqs, max_tokens, chunk
        self.max_model_len = max_model_len
        self.waiting, self.running, self.info = [], [], {}
        self.arrivals = 0
        self.preemptions = 0

    def add(self, r, prompt_len, max_new, eos=None):
        self.info[r] = {"prompt": prompt_len, "out": 0, "max_new": max_new, "eos": eos,
                        "number": self.arrivals, "computed": 0, "done": None}
        self.arrivals += 1
        if max_new == 0:
            self.info[r]["done"] = "length"
        else:
            self.waiting.append(r)

    def has_work(self):
        return bool(self.waiting or self.running)

    def _left(self, r):
        i = self.info[r]
        return i["prompt"] + i["out"] - i["computed"]

    def _preempt(self, v):
        self.cache.release(v)
        self.info[v]["computed"] = 0
        self.running.remove(v)
        self.waiting.insert(0, v)
        self.preemptions += 1

    def schedule(self):
        budget = self.max_tokens
        plan = []
        promised = [0] * len(self.cache.windows)
        order = sorted(self.running, key=lambda r: (self._left(r) != 1, self.info[r]["number"]))
        for r in order:
            if r not in self.running:
                continue
            if budget == 0:
                break
            n = min(self._left(r), budget, self.chunk)
            while not self.cache.fits(r, n, promised):
                victim = max(self.running, key=lambda x: self.info[x]["number"])
                if victim == r and len(self.running) == 1 and not plan:
                    raise PlainOutOfPages(r)
                for e in plan:
                    if e[0] == victim:
                        for g, k in enumerate(self.cache.needed(victim, e[2])):
                            promised[g] -= k
                        budget += e[2]
                        plan.remove(e)
                        break
                self._preempt(victim)
                if victim == r:
                    break
            if r not in self.running:
                continue
            for g, k in enumerate(self.cache.needed(r, n)):
                promised[g] += k
            i = self.info[r]
            plan.append((r, i["computed"], n, i["computed"] + n == i["prompt"] + i["out"]))
            budget -= n
        while (self.waiting and budget > 0 and len(self.running) < self.max_num_seqs
               and self.cache.free_slots):
            r = self.waiting[0]
            n = min(self._left(r), budget, self.chunk)
            self.cache.admit(r)
            if not self.cache.fits(r, n, promised):
                self.cache.release(r)
                if not self.running:
                    raise PlainOutOfPages(r)
                break
            self.waiting.pop(0)
            self.running.append(r)
            for g, k in enumerate(self.cache.needed(r, n)):
                promised[g] += k
            i = self.info[r]
            plan.append((r, 0, n, n == i["prompt"] + i["out"]))
            budget -= n
        return plan

    def update(self, plan, sampled):
        done = []
        for r, _, n, samples in plan:
            i = self.info[r]
            i["computed"] += n
            if not samples:
                continue
            i["out"] += 1
            if i["eos"] is not None and sampled[r] == i["eos"]:
                i["done"] = "eos"
            elif i["out"] >= i["max_new"]:
                i["done"] = "length"
            elif self.max_model_len and i["prompt"] + i["out"] >= self.max_model_len:
                i["done"] = "max_model_len"
            if i["done"]:
                self.cache.release(r)
                self.running.remove(r)
                done.append(r)
        return done
