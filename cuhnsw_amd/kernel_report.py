"""Register budget of the search kernels, read off the compiler's own output.

The sorted-set search keeps its set in vector registers and is held to a fixed number of wavefronts per
SIMD; a register spilled INSIDE its hop loop (a scratch reload per hop, and the waits it drags in) costs
the pass 7 to 12 %, and whether the register allocator puts one there is decided by small changes anywhere
in the kernel.  This module compiles the kernels that matter on their own (a few seconds each), reads
hipcc's resource-usage remarks (registers, spills, scratch bytes, wavefronts per SIMD) and counts the
scratch-memory instructions that sit inside the hop loops (the innermost loops holding both the sorted-set
insert, `v_med3_f32`, and a fetch from global memory), from the control-flow graph of the emitted ISA.

  python -m cuhnsw_amd.kernel_report            # prints the table

cuhnsw_amd/build.py records the remarks of the library's own build, for every kernel in it, in
profiles/kernel_resources.json; tests/test_kernel_resources.py compiles the first-pass kernels with this module
and fails when one of them loses a wavefront per SIMD, spills more, or gains a scratch access inside its hop loop.
"""
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# the device-code flags of cuhnsw_amd/build.py
DEVICE_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-ffp-contract=off", "-Wno-unused-function",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# kernel instances the guard looks at: (template text, short name)
FIRST_PASS = [
    ("search_fast_kernel<DIST_DOT, 1, 5, false>(DevIndex, SearchArgs)", "search_fast_kernel<dot,1,5>"),
    ("search_fast_kernel<DIST_DOT, 1, 5, true>(DevIndex, SearchArgs)", "search_fast_kernel<dot,1,5,trails>"),
    ("search_fast_kernel<DIST_L2, 1, 5, false>(DevIndex, SearchArgs)", "search_fast_kernel<l2,1,5>"),
    ("search_fast_kernel<DIST_DOT, 2, 5, false>(DevIndex, SearchArgs)", "search_fast_kernel<dot,2,5>"),
    ("search_fast_kernel<DIST_L2, 2, 5, false>(DevIndex, SearchArgs)", "search_fast_kernel<l2,2,5>"),
    ("search_fast_kernel<DIST_L2, 2, 5, true>(DevIndex, SearchArgs)", "search_fast_kernel<l2,2,5,trails>"),
    ("search_fast_kernel<DIST_DOT, 1, 2, false>(DevIndex, SearchArgs)", "search_fast_kernel<dot,1,2>"),
    ("search_fast_kernel<DIST_DOT, 2, 8, false>(DevIndex, SearchArgs)", "search_fast_kernel<dot,2,8>"),
]
OTHERS = [
    ("search_kernel<DIST_DOT, 1, 5>(DevIndex, SearchArgs)", "search_kernel<dot,1,5>"),
    ("build_search_kernel<DIST_DOT, 1, 2>(DevIndex, BuildArgs)", "build_search_kernel<dot,1,2>"),
    ("build_search_kernel<DIST_L2, 2, 5>(DevIndex, BuildArgs)", "build_search_kernel<l2,2,5>"),
    ("reverse_kernel<DIST_DOT, 1>(DevIndex, BuildArgs)", "reverse_kernel<dot,1>"),
]

_REMARK = re.compile(r"remark:\s+(Function Name|TotalSGPRs|VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]|"
                     r"SGPRs Spill|VGPRs Spill|LDS Size \[bytes/block\]):\s+(\S+)")
_KEYS = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes_per_lane",
         "Occupancy [waves/SIMD]": "waves_per_simd", "SGPRs Spill": "sgpr_spills", "VGPRs Spill": "vgpr_spills",
         "LDS Size [bytes/block]": "static_lds_bytes"}


def parse_remarks(text):
  """{mangled kernel name: {vgprs, sgprs, spills, scratch, waves_per_simd, ...}} from -Rpass-analysis=kernel-resource-usage."""
  out, cur = {}, None
  for m in _REMARK.finditer(text):
    key, value = m.group(1), m.group(2)
    if key == "Function Name":
      cur = out.setdefault(value, {})
    elif cur is not None:
      cur[_KEYS[key]] = int(value)
  return out


def _blocks(body):
  """[(label, [instructions])] of one function's ISA text."""
  out, cur = [], None
  for line in body.split("\n"):
    t = line.strip()
    if not t or t.startswith(";") or t.startswith("//"):
      continue
    m = re.match(r"^(\.LBB\d+_\d+):", t)
    if m:
      cur = (m.group(1), [])
      out.append(cur)
      continue
    if t.startswith("."):
      continue
    if cur is None:
      cur = ("entry", [])
      out.append(cur)
    cur[1].append(t.split(";")[0].strip())
  return out


def loop_scratch_accesses(isa_text, mangled):
  """Scratch-memory instructions inside the hop loops (found as strongly connected components of the control-flow
  graph, nested), and in the whole kernel: (in_loops, total)."""
  start = isa_text.index("\n" + mangled + ":")
  body = isa_text[start:isa_text.index(".Lfunc_end", start)]
  blocks = _blocks(body)
  index = {label: i for i, (label, _) in enumerate(blocks)}
  succ = []
  for i, (_, ins) in enumerate(blocks):
    nxt = set()
    falls = True
    for t in ins:
      op = t.split()[0]
      if op.startswith("s_cbranch") or op == "s_branch":
        target = t.split()[-1]
        if target in index:
          nxt.add(index[target])
      if op in ("s_branch", "s_endpgm", "s_setpc_b64"):
        falls = False
    if falls and i + 1 < len(blocks):
      nxt.add(i + 1)
    succ.append(sorted(nxt))
  # Loop nest: strongly connected components, then again inside each component with the edges into its header
  # removed.  Depth 1 is the loop over the wavefront's queries; the hop loops are the deeper ones that hold
  # the sorted-set insert.
  def components(nodes, edges):
    """Tarjan, iterative, on the subgraph `nodes` (a set) with successor lists `edges`."""
    order, low, on, comps, stack = {}, {}, set(), [], []
    counter = 0
    for root in sorted(nodes):
      if root in order:
        continue
      work = [(root, 0)]
      while work:
        v, pi = work.pop()
        if pi == 0:
          order[v] = low[v] = counter
          counter += 1
          stack.append(v)
          on.add(v)
        nxt = [w for w in edges[v] if w in nodes]
        advanced = False
        for k in range(pi, len(nxt)):
          w = nxt[k]
          if w not in order:
            work.append((v, k + 1))
            work.append((w, 0))
            advanced = True
            break
          if w in on:
            low[v] = min(low[v], order[w])
        if advanced:
          continue
        if low[v] == order[v]:
          comp = set()
          while True:
            w = stack.pop()
            on.discard(w)
            comp.add(w)
            if w == v:
              break
          comps.append(comp)
        if work:
          parent = work[-1][0]
          low[parent] = min(low[parent], low[v])
    return comps

  # Hop loops: the innermost loops that hold both the sorted-set insert (v_med3_f32) and a fetch from global
  # memory (the link row, the vectors).  The loop over the wavefront's queries and any loop that merely
  # alternates between two hop loops contain such a loop and are not counted themselves; the loop over a hop's
  # offers holds the insert but fetches nothing.
  has_insert = [any(t.startswith("v_med3_f32") for t in ins) for _, ins in blocks]
  has_fetch = [any(t.startswith("global_load") for t in ins) for _, ins in blocks]
  hot_blocks = set()
  def nest(nodes, edges):
    """Marks the hop loops inside `nodes`; returns whether there was one."""
    found = False
    for comp in components(nodes, edges):
      if len(comp) == 1 and next(iter(comp)) not in edges[next(iter(comp))]:
        continue
      if not (any(has_insert[v] for v in comp) and any(has_fetch[v] for v in comp)):
        continue
      # headers: nodes of the component entered from outside it (or the first one)
      heads = {v for v in comp for u in range(len(blocks)) if u not in comp and v in succ[u]} or {min(comp)}
      inner = {v: [w for w in edges[v] if w not in heads] for v in comp}
      if not nest(comp, inner):
        hot_blocks.update(comp)
      found = True
    return found
  nest(set(range(len(blocks))), {i: succ[i] for i in range(len(blocks))})
  in_loops = total = 0
  for i, (_, ins) in enumerate(blocks):
    k = sum(1 for t in ins if t.startswith("scratch_"))
    total += k
    if i in hot_blocks:
      in_loops += k
  return in_loops, total


def compile_kernels(instances):
  """Compiles each kernel instance on its own; returns {short name: resource dict}."""
  out = {}
  with tempfile.TemporaryDirectory(prefix="cuhnsw_kr_") as tmp:
    for text, short in instances:
      src = os.path.join(tmp, "k.hip")
      asm = os.path.join(tmp, "k.s")
      with open(src, "w") as f:
        f.write('#include "kernels.h"\nusing namespace cuhnsw_amd;\ntemplate __global__ void cuhnsw_amd::%s;\n' % text)
      r = subprocess.run([HIPCC] + DEVICE_FLAGS + ["-I" + CSRC, "--cuda-device-only", "-S", "-x", "hip", src, "-o", asm,
                                                   "-Rpass-analysis=kernel-resource-usage"],
                         capture_output=True, text=True)
      if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (short, r.stderr[-2000:]))
      base = text.split("<")[0]
      mangled = [k for k in parse_remarks(r.stderr) if base in k]
      if len(mangled) != 1:
        raise RuntimeError("%s: expected one kernel named %s, found %r" % (short, base, mangled))
      info = dict(parse_remarks(r.stderr)[mangled[0]])
      with open(asm) as f:
        in_loops, total = loop_scratch_accesses(f.read(), mangled[0])
      info["scratch_instructions"] = total
      info["scratch_instructions_in_hop_loops"] = in_loops
      out[short] = info
  return out


def main():
  report = compile_kernels(FIRST_PASS + OTHERS)
  for name, r in report.items():
    print("%-34s VGPRs %3d  waves/SIMD %d  VGPR spills %3d  SGPR spills %3d  scratch %3d B/lane  scratch instrs %3d (in hop loops %d)" % (
        name, r["vgprs"], r["waves_per_simd"], r["vgpr_spills"], r["sgpr_spills"], r["scratch_bytes_per_lane"],
        r["scratch_instructions"], r["scratch_instructions_in_hop_loops"]))
  return 0


if __name__ == "__main__":
  sys.exit(main())
