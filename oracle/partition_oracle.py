"""numpy restatement of the reference's offline partitioner (csrc/partition/partition.cc).  TEST INFRASTRUCTURE ONLY.

The reference's loops carry OpenMP pragmas whose threads race on the shared counters, so its result with threads is
not a function of its input.  This restates the program its source is WITHOUT OpenMP: samples and embeddings are
visited in index order and every move is applied before the next decision.  All float arithmetic keeps the type and
order the C++ expressions have (float unless a double literal widens it); numpy float32 array operations are single
IEEE operations per element, so vectorising over the parts changes nothing.

Pure-python loops over samples and embeddings: meant for cases of up to ~10^5 samples x slots.

Where the reference reads past the end of soft_cnt_ (an embedding that occurs n_data times or more), the value read
here is 1, what the table saturates at.

Pinned by: tests/test_partition.py against the reference's own sources compiled without OpenMP (when that build is
present), against tests/golden/partition_*.npz made from that build, the generator against glibc's published first
outputs for srand(1) and the C library's rand() itself, and the soft-count table against its closed form.
"""
import numpy as np

F = np.float32


def glibc_rand(seed, count):
    """First `count` results of glibc rand() after srand(seed): TYPE_3 additive feedback o[i] = o[i-31] + o[i-3] over
    32-bit words, the state seeded by the minimal standard generator 16807 * x mod (2^31 - 1), 310 words discarded,
    each result the word shifted right once.  The reference draws its initial assignment from rand() and never seeds
    it (partition.cc:70,77), i.e. srand(1) in a fresh process."""
    seed = seed or 1
    o = [0] * (344 + count)
    s = seed if seed < 2 ** 31 else seed - 2 ** 32
    o[0] = s & 0xFFFFFFFF
    for i in range(1, 31):
        # int32 arithmetic of the seeding, C division truncating towards zero
        hi, lo = int(s / 127773), s - 127773 * int(s / 127773)
        s = 16807 * lo - 2836 * hi
        if s < 0:
            s += 2147483647
        o[i] = s & 0xFFFFFFFF
    for i in range(31, 34):
        o[i] = o[i - 31]
    for i in range(34, 344 + count):
        o[i] = (o[i - 31] + o[i - 3]) & 0xFFFFFFFF
    return np.array([v >> 1 for v in o[344:]], dtype=np.int64)


def soft_table(n_data, n_part, batch):
    """partition.cc:7-15,59-65: soft[i] = (1 - (1 - i/m)^batch) * m / batch for i < m = n_data // n_part, 1 from m on.
    The power is binary exponentiation in float."""
    m = n_data // n_part
    soft = np.ones(n_data, F)
    i = np.arange(m, dtype=F)
    base = (1.0 - (i / F(m)).astype(np.float64)).astype(F)
    ans, temp, n = np.ones(m, F), base.copy(), batch
    while n:
        if n & 1:
            ans = ans * temp
        n >>= 1
        temp = temp * temp
    soft[:m] = (F(1) - ans) * (F(m) / F(batch))
    return soft


def serial_sum(values):
    """float32 sum in index order from 0 (what `acc += v` in a C loop gives)."""
    values = np.asarray(values, F)
    return F(0) if values.size == 0 else np.add.accumulate(values, dtype=F)[-1]


class Partition:
    """State and methods of PartitionStruct (csrc/partition/partition.h:8-30)."""

    def __init__(self, data, comm_mat, n_part, batch_size, seed=1):
        data = np.ascontiguousarray(data, dtype=np.int32)
        self.data = data
        self.P, self.batch = int(n_part), int(batch_size)
        self.n_data, self.n_slot = data.shape
        self.n_embed = int(data.max()) + 1                                 # partition.cc:33-37
        self.comm = np.ascontiguousarray(comm_mat, dtype=F).reshape(self.P, self.P)
        self.soft = soft_table(self.n_data, self.P, self.batch)
        draws = glibc_rand(seed, self.n_data + self.n_embed)
        self.res_data = (draws[:self.n_data] % self.P).astype(np.int32)   # partition.cc:69-75
        self.res_embed = (draws[self.n_data:] % self.P).astype(np.int32)  # partition.cc:76-79
        self.cnt_data = np.bincount(self.res_data, minlength=self.P).astype(np.int64)
        self.cnt_embed = np.bincount(self.res_embed, minlength=self.P).astype(np.int64)
        # cnt[p, e]: samples of part p that use embedding e, counted once per slot
        self.cnt = np.zeros((self.P, self.n_embed), np.int64)
        np.add.at(self.cnt, (np.repeat(self.res_data, self.n_slot), data.reshape(-1)), 1)
        self.degree = np.bincount(data.reshape(-1), minlength=self.n_embed)
        self.alpha = F(-100.0 / (self.n_data // self.P))                  # partition.cc:82-83
        self.beta = F(-100.0 / (self.n_embed // self.P))
        self.scale = F(self.batch * self.P) / F(self.n_data)

    def _soft(self, idx):
        idx = np.asarray(idx)
        return np.where(idx < self.n_data, self.soft[np.minimum(idx, self.n_data - 1)], F(1)).astype(F)

    def refine_data(self):
        """partition.cc:89-120."""
        P, eye = self.P, np.eye(self.P, dtype=np.int64)
        for i in range(self.n_data):
            old = int(self.res_data[i])
            score = self.alpha * (self.cnt_data - eye[old]).astype(F)
            for e in self.data[i]:
                use = self.cnt[:, e] - eye[old]
                score = score - (self._soft(use + 1) - self._soft(use)) * self.comm[:, self.res_embed[e]]
            s = int(np.argmax(score))                                      # first of the largest, as partition.cc:17-24
            if s != old:
                self.cnt_data[old] -= 1
                self.cnt_data[s] += 1
                for e in self.data[i]:
                    self.cnt[s, e] += 1
                    self.cnt[old, e] -= 1
                self.res_data[i] = s

    def _embed_weight(self):
        """partition.cc:123-131: per owner part, soft counts of its embeddings as seen from every other part, summed
        over (seeing part, embedding) in that nesting order."""
        w = np.zeros(self.P, F)
        for p in range(self.P):
            mine = np.flatnonzero(self.res_embed == p)
            terms = [self._soft(self.cnt[i, mine]) for i in range(self.P) if i != p]
            w[p] = serial_sum(np.concatenate(terms)) if terms else F(0)
        return w * self.scale

    def refine_embed(self):
        """partition.cc:122-166."""
        P, eye = self.P, np.eye(self.P, dtype=np.int64)
        w = self._embed_weight()
        for i in range(self.n_embed):
            old = int(self.res_embed[i])
            # the reference counts in float: a count above 2^24 would stick there
            c = np.minimum(self.cnt[:, i], 1 << 24)
            seen = self._soft(c)
            own = float(self._soft(self.degree[i]))
            score = self.beta * (self.cnt_embed - eye[old]).astype(F)
            for j in range(P):
                score = score - self.comm[j, :] * seen[j]
                score[j] = F(float(score[j]) - 0.01 * float(w[j]) * own)  # the double literal widens this one
            s = int(np.argmax(score))
            if s != old:
                self.cnt_embed[old] -= 1
                self.cnt_embed[s] += 1
                self.res_embed[i] = s
                direct = self._soft(self.cnt[:, i])
                for j in range(P):
                    t = direct[j] * F(self.batch * P) / F(self.n_data)
                    if j != s:
                        w[s] = w[s] + t
                    if j != old:
                        w[old] = w[old] - t
        self.embed_weight = w

    def get_communication(self):
        """partition.cc:168-181: cost[i, p] = expected rows part i fetches from part p per batch round."""
        cost = np.zeros((self.P, self.P), F)
        for i in range(self.P):
            seen = self._soft(self.cnt[i])
            for p in range(self.P):
                cost[i, p] = serial_sum(seen[self.res_embed == p])
        return cost * self.scale

    def get_priority(self):
        """partition.cc:183-194, in double as the C++ promotes it, rounded to float once."""
        c = self.cnt.astype(np.float64)
        with np.errstate(divide="ignore", invalid="ignore"):
            pr = (self.comm[np.arange(self.P)[:, None], self.res_embed[None, :]].astype(np.float64) *
                  self._soft(self.cnt).astype(np.float64) ** 2) * (1.0 / self.degree[None, :] + 1.0 / c)
        return np.where(self.cnt == 0, 0.0, pr).astype(F)

    def get_result(self):
        return self.res_data.copy(), self.res_embed.copy()

    def get_data_cnt(self):
        return self.cnt_data.astype(np.int32)

    def get_embed_cnt(self):
        return self.cnt_embed.astype(np.int32)


def cache_lists(priority, res_embed):
    """What experimental/partition.py:53-57 keeps per part: the embeddings the part does not own, by descending
    priority.  numpy's default argsort leaves the order of equal priorities open; here (and in the library) equal
    priorities come in descending id, which is what a stable ascending sort read backwards gives."""
    out = []
    for i in range(priority.shape[0]):
        pr = priority[i].copy()
        owned = np.flatnonzero(res_embed == i)
        pr[owned] = -1
        out.append(np.argsort(pr, kind="stable")[len(owned):][::-1].astype(np.int32))
    return out
