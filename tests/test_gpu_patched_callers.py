"""`install_into_evox(patch_callers=True)` on the GPU, against a stand-in package whose classes follow the
reference's callers line by line: NSGA2.step (src/evox/algorithms/mo/nsga2.py:92-102), the cut of NSGA3.step
(nsga3.py:163-174) and of HypE.step (hype.py:130-138), EvalMonitor.get_pf_fitness / get_pf
(src/evox/workflows/eval_monitor.py:290-337).  Every patched caller must leave exactly the state that the unpatched
one leaves when both run on the HIP operators (the unpatched ones are compared with the CPU restatement in
test_gpu_nsga2_loop.py and test_gpu_parity.py)."""

import sys
import types

import pytest
import torch

import evox_amd
from evox_amd import compat

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _dtlz(x: torch.Tensor, n_objs: int) -> torch.Tensor:
    g = ((x[:, n_objs - 1:] - 0.5) ** 2).sum(dim=1, keepdim=True)
    theta = x[:, : n_objs - 1] * (torch.pi / 2)
    cols = []
    for k in range(n_objs):
        c = torch.ones(x.size(0), device=x.device)
        for t in range(n_objs - 1 - k):
            c = c * torch.cos(theta[:, t])
        if k > 0:
            c = c * torch.sin(theta[:, n_objs - 1 - k])
        cols.append(c)
    return ((1 + g) * torch.stack(cols, dim=1)).float().contiguous()


def _stand_in_package():
    mods = {}

    def module(name):
        if name not in mods:
            mods[name] = types.ModuleType(name)
            mods[name].__path__ = []
            parent, _, leaf = name.rpartition(".")
            if parent:
                setattr(module(parent), leaf, mods[name])
        return mods[name]

    def cpu_only(name):
        def original(*args, **kwargs):
            raise AssertionError(f"{name}: the call reached the package's own function")
        original.__name__ = name
        return original

    nsga2, nsga3, hype, monitor = (module(n) for n in ("evox.algorithms.mo.nsga2", "evox.algorithms.mo.nsga3",
                                                        "evox.algorithms.mo.hype", "evox.workflows.eval_monitor"))
    nsga2.nd_environmental_selection = cpu_only("nd_environmental_selection")
    nsga2.tournament_selection_multifit = cpu_only("tournament_selection_multifit")
    nsga2.clamp = lambda x, lb, ub: torch.minimum(torch.maximum(x, lb), ub)
    for m in (nsga3, hype, monitor):
        m.non_dominate_rank = cpu_only("non_dominate_rank")
    monitor.unique = lambda x: (None, torch.arange(x.size(0), device=x.device), None, None)  # utils.unique's index slot

    class NSGA2:
        def __init__(self, pop_size, dim, n_objs, seed):
            g = torch.Generator("cpu").manual_seed(seed)
            self.pop_size, self.n_objs = pop_size, n_objs
            self.lb, self.ub = torch.zeros(dim, device=DEV), torch.ones(dim, device=DEV)
            self.pop = torch.rand(pop_size, dim, generator=g).to(DEV)
            self.noise = [torch.randn(pop_size, dim, generator=g).to(DEV) * 0.05 for _ in range(16)]
            self.draws = [torch.randint(0, pop_size, (pop_size, 2), generator=g).to(DEV) for _ in range(16)]
            self.t = 0
            self.selection = self._select
            self.crossover = lambda parents: 0.5 * (parents + parents.roll(1, dims=0))
            self.mutation = lambda x, lb, ub: x + self.noise[self.t % 16]
            self.fit = self.evaluate(self.pop)
            _, _, self.rank, self.dis = nsga2.nd_environmental_selection(self.pop, self.fit, self.pop_size)  # nsga2.py:90

        def _select(self, n_round, fitnesses):
            keys = torch.stack(fitnesses, dim=1)
            return evox_amd.ops.tournament_pick(self.draws[self.t % 16], keys)

        def evaluate(self, x):
            return _dtlz(x, self.n_objs).to(x.dtype)

        def step(self):  # nsga2.py:92-102
            mating_pool = self.selection(self.pop_size, [-self.dis, self.rank])
            crossovered = self.crossover(self.pop[mating_pool])
            offspring = self.mutation(crossovered, self.lb, self.ub)
            offspring = nsga2.clamp(offspring, self.lb, self.ub)
            off_fit = self.evaluate(offspring)
            merge_pop = torch.cat([self.pop, offspring], dim=0)
            merge_fit = torch.cat([self.fit, off_fit], dim=0)
            self.pop, self.fit, self.rank, self.dis = nsga2.nd_environmental_selection(merge_pop, merge_fit, self.pop_size)

    class NSGA3:
        def __init__(self, pop_size):
            self.pop_size = pop_size

        def step(self, merge_fit):  # nsga3.py:169-174
            rank = nsga3.non_dominate_rank(merge_fit)
            worst_rank = torch.topk(rank, self.pop_size + 1, largest=False)[0][-1]
            candi_idx = torch.where(rank <= worst_rank)[0]
            return candi_idx, rank[candi_idx], worst_rank

    class HypE:
        def __init__(self, pop_size):
            self.pop_size = pop_size

        def step(self, merge_fit):  # hype.py:135-138, :143
            rank = hype.non_dominate_rank(merge_fit)
            order = torch.argsort(rank)
            worst_rank = rank[order[self.pop_size - 1]]
            mask = rank <= worst_rank
            dis = torch.where(mask, merge_fit.sum(dim=1), -torch.inf)
            combined = evox_amd.utils.lexsort([-dis, rank])[: self.pop_size]
            return mask, worst_rank, combined

    class EvalMonitor:
        multi_obj = True
        history_device = DEV

        def __init__(self, fitness, solutions):
            self.fitness_history = list(fitness)
            self._solutions = list(solutions)
            self.opt_direction = torch.tensor(-1)

        def get_solution_history(self):
            return self._solutions

        def get_pf_fitness(self, deduplicate=True):  # eval_monitor.py:297-303
            all_fitness = torch.cat(self.fitness_history, dim=0)
            if deduplicate:
                all_fitness = torch.unique(all_fitness, dim=0)
            rank = monitor.non_dominate_rank(all_fitness)
            return all_fitness[rank == 0] * self.opt_direction.to(self.history_device)

        def get_pf(self, deduplicate=True):  # eval_monitor.py:323-337
            all_solutions = torch.cat(self.get_solution_history(), dim=0)
            all_fitness = torch.cat(self.fitness_history, dim=0)
            if deduplicate:
                _, unique_index, _, _ = monitor.unique(all_solutions)
                all_solutions, all_fitness = all_solutions[unique_index], all_fitness[unique_index]
            rank = monitor.non_dominate_rank(all_fitness)
            opt_dir = self.opt_direction.to(self.history_device)
            return all_solutions[rank == 0], all_fitness[rank == 0] * opt_dir

    for cls, m in ((NSGA2, nsga2), (NSGA3, nsga3), (HypE, hype), (EvalMonitor, monitor)):
        cls.__module__ = m.__name__
        setattr(m, cls.__name__, cls)
    return mods


@pytest.fixture
def package(monkeypatch):
    mods = _stand_in_package()
    for n, m in mods.items():
        monkeypatch.setitem(sys.modules, n, m)
    yield mods
    compat.uninstall_from_evox()


def _patched_steps(mods):
    """NSGA-III's and HypE's steps take the merged fitness as an argument here, the patch wraps a step without
    arguments: a step of that shape around them."""
    for mod, name in (("evox.algorithms.mo.nsga3", "NSGA3"), ("evox.algorithms.mo.hype", "HypE")):
        cls = getattr(mods[mod], name)
        cls.cut = cls.step

        def step(self):
            return self.cut(self.merge_fit)

        cls.step = step


def test_patched_nsga2_step_leaves_the_same_state(package):
    NSGA2 = package["evox.algorithms.mo.nsga2"].NSGA2
    assert len(evox_amd.install_into_evox()) == 5  # the five module globals of the stand-in package
    plain = NSGA2(300, 10, 3, seed=5)
    states = []
    for _ in range(6):
        plain.step()
        plain.t += 1
        states.append([t.clone() for t in (plain.pop, plain.fit, plain.rank, plain.dis)])
    changed = evox_amd.install_into_evox(patch_callers=True)
    assert "evox.algorithms.mo.nsga2.NSGA2.step" in changed
    patched = NSGA2(300, 10, 3, seed=5)
    for want in states:
        patched.step()
        patched.t += 1
        for got, w in zip((patched.pop, patched.fit, patched.rank, patched.dis), want):
            assert torch.equal(got, w) and got.dtype == w.dtype


def test_patched_nsga2_step_with_float64_fitness(package):
    """A run under a float64 default dtype (float64 population and fitness): the two-part selection hands fitness
    that its kernels do not read to the selection of the concatenation, as the unpatched step does."""
    NSGA2 = package["evox.algorithms.mo.nsga2"].NSGA2
    torch.set_default_dtype(torch.float64)
    try:
        evox_amd.install_into_evox()
        plain = NSGA2(200, 8, 3, seed=9)
        assert plain.fit.dtype == torch.float64 and plain.dis.dtype == torch.float64
        states = []
        for _ in range(3):
            plain.step()
            plain.t += 1
            states.append([t.clone() for t in (plain.pop, plain.fit, plain.rank, plain.dis)])
        evox_amd.install_into_evox(patch_callers=True)
        patched = NSGA2(200, 8, 3, seed=9)
        for want in states:
            patched.step()
            patched.t += 1
            for got, w in zip((patched.pop, patched.fit, patched.rank, patched.dis), want):
                assert torch.equal(got, w) and got.dtype == w.dtype
    finally:
        torch.set_default_dtype(torch.float32)


@pytest.mark.parametrize("n,m,pop_size,seed", [(600, 3, 300, 1), (2000, 2, 1000, 2), (5000, 3, 2500, 3), (400, 8, 100, 4)])
def test_patched_cuts_of_nsga3_and_hype_read_the_same_from_truncated_ranks(package, n, m, pop_size, seed):
    _patched_steps(package)
    NSGA3, HypE = package["evox.algorithms.mo.nsga3"].NSGA3, package["evox.algorithms.mo.hype"].HypE
    f = torch.rand(n, m, generator=torch.Generator("cpu").manual_seed(seed)).to(DEV)
    if m == 2:
        f = (f * 16).round() / 16  # ties and duplicate rows
    evox_amd.install_into_evox()
    a3, hy = NSGA3(pop_size), HypE(pop_size)
    a3.merge_fit = hy.merge_fit = f
    want3, wanth = a3.step(), hy.step()
    evox_amd.install_into_evox(patch_callers=True)
    got3, goth = a3.step(), hy.step()
    for got, want in zip(got3 + goth, want3 + wanth):
        assert torch.equal(got, want)
    # the patched steps did stop early: behind the cut the ranks are unset
    with compat._rank_only_until(pop_size):
        cut = package["evox.algorithms.mo.hype"].non_dominate_rank(f)
    assert int((cut == evox_amd.ops.RANK_UNSET).sum()) == n - int(wanth[0].sum())
    assert compat._rank_until is None


def test_patched_monitor_takes_the_first_front_of_a_gpu_history(package):
    EvalMonitor = package["evox.workflows.eval_monitor"].EvalMonitor
    g = torch.Generator("cpu").manual_seed(9)
    fitness = [torch.rand(500, 3, generator=g).to(DEV) for _ in range(6)]
    fitness.append(fitness[0][:100].clone())  # duplicate rows in the history
    solutions = [torch.rand(f.size(0), 7, generator=g).to(DEV) for f in fitness]
    mon = EvalMonitor(fitness, solutions)
    evox_amd.install_into_evox()
    want_fit, want_fit_all, want_pf = mon.get_pf_fitness(), mon.get_pf_fitness(False), mon.get_pf()
    evox_amd.install_into_evox(patch_callers=True)
    assert torch.equal(mon.get_pf_fitness(), want_fit) and torch.equal(mon.get_pf_fitness(False), want_fit_all)
    got_pf = mon.get_pf()
    assert torch.equal(got_pf[0], want_pf[0]) and torch.equal(got_pf[1], want_pf[1])
    # a history on the CPU goes to the package's own method, untouched
    # a history on the CPU goes to the package's own method and function (the stand-in's refuses every call)
    cpu = EvalMonitor([f.cpu() for f in fitness], [s.cpu() for s in solutions])
    with pytest.raises(AssertionError, match="the package's own function"):
        cpu.get_pf_fitness()
