"""Literal Python model of libstdc++ std::push_heap / std::pop_heap
(bits/stl_heap.h __push_heap / __adjust_heap) on (key, id) pairs compared by key only,
plus a lane-level model of the cooperative wavefront algorithm used on the GPU."""


def less(minq, a, b):
  return (a > b) if minq else (a < b)


def push_literal(a, v, minq=False):
  a.append(v)
  hole = len(a) - 1
  parent = (hole - 1) // 2
  while hole > 0 and less(minq, a[parent][0], v[0]):
    a[hole] = a[parent]
    hole = parent
    parent = (hole - 1) // 2
  a[hole] = v


def pop_literal(a, minq=False):
  if len(a) > 1:
    value = a[-1]
    ln = len(a) - 1
    hole = child = 0
    while child < (ln - 1) // 2:
      child = 2 * (child + 1)
      if less(minq, a[child][0], a[child - 1][0]):
        child -= 1
      a[hole] = a[child]
      hole = child
    if ln % 2 == 0 and child == (ln - 2) // 2:
      child = 2 * (child + 1)
      a[hole] = a[child - 1]
      hole = child - 1
    parent = (hole - 1) // 2
    while hole > 0 and less(minq, a[parent][0], value[0]):
      a[hole] = a[parent]
      hole = parent
      parent = (hole - 1) // 2
    a[hole] = value
  a.pop()


def _sift_up_coop(a, i, v, minq):
  reads, rises = {}, []
  for lane in range(64):
    q = ((i + 1) >> (lane + 1)) if lane < 31 else 0
    if q >= 1:
      reads[lane] = a[q - 1]
      rises.append(less(minq, a[q - 1][0], v[0]))
    else:
      rises.append(False)
  t = 0
  while rises[t]:
    t += 1
  writes = [(((i + 1) >> lane) - 1, reads[lane] if lane < t else v) for lane in range(t + 1)]
  for slot, e in writes:
    a[slot] = e


def push_coop(a, size, v, minq=False):
  if len(a) <= size:
    a.append(None)
  _sift_up_coop(a, size, v, minq)
  return size + 1


def pop_coop(a, size, minq=False):
  """The way down and the last entry's way up again in one pass: the way down stops at the first moved child that
  compares smaller than the last entry, which is written there; everything below stays as it was."""
  if size > 1:
    ln = size - 1
    value = a[ln]
    hole = 0
    while True:
      pos, left, right, has1, take_left = {}, {}, {}, {}, {}
      for lane in range(63):
        d = (lane + 1).bit_length() - 1
        p = ((hole + 1) << d) - 1 + (lane + 1 - (1 << d))
        pos[lane] = p
        c1 = 2 * p + 1
        has1[lane] = c1 < ln
        has2 = c1 + 1 < ln
        if has1[lane]:
          left[lane], right[lane] = a[c1], a[c1 + 1]
        take_left[lane] = has1[lane] and ((not has2) or less(minq, right[lane][0], left[lane][0]))
      # a node is on the hole's path iff every edge from the stage root down to it is the
      # chosen one (the kernels test this against one ballot mask per lane)
      def on_path(t):
        while t > 0:
          par = (t - 1) >> 1
          if not has1[par] or take_left[par] != (t % 2 == 1):
            return False
          t = par
        return True
      path = [t for t in range(63) if on_path(t)]
      child = {t: (left[t] if take_left[t] else right[t]) for t in path if has1[t]}
      rising = [t for t in path if has1[t] and less(minq, child[t][0], value[0])]
      if rising:
        first = min(rising)
        writes = [(pos[t], child[t] if t < first else value) for t in path if t <= first]
        for slot, e in writes:
          a[slot] = e
        break
      writes = [(pos[t], child[t]) for t in path if has1[t]]
      for slot, e in writes:
        a[slot] = e
      last = max(path)
      if not has1[last]:
        a[pos[last]] = value
        break
      hole = 2 * pos[last] + 2 - (1 if take_left[last] else 0)
  return size - 1
