import re, sys, collections
def regs_of(tok):
    m = re.match(r'v\[(\d+):(\d+)\]', tok)
    if m: return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r'v(\d+)$', tok)
    return {int(m.group(1))} if m else set()
def all_regs(line):
    s = set()
    for m in re.finditer(r'v\[(\d+):(\d+)\]', line): s |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r'\bv(\d+)\b', line): s.add(int(m.group(1)))
    return s
for path in sys.argv[1:]:
    text = open(path).read().split('\n')
    kernels = [i for i, l in enumerate(text) if re.match(r'^_ZN5ditto\S+:', l)]
    for ki, start in enumerate(kernels):
        end = kernels[ki + 1] if ki + 1 < len(kernels) else len(text)
        body = text[start:end]
        in_asm = False; tracked = set(); asm_lines = set()
        for i, l in enumerate(body):
            if '#ASMSTART' in l: in_asm = True; continue
            if '#ASMEND' in l: in_asm = False; continue
            if in_asm:
                asm_lines.add(i)
                if 'buffer_load_dwordx' in l and ' lds' not in l: tracked |= regs_of(l.split()[1].rstrip(','))
        if not tracked: continue
        uses = collections.Counter()
        for i, l in enumerate(body):
            if i in asm_lines or not l.startswith('\t') or l.strip().startswith(';'): continue
            if all_regs(l) & tracked: uses[l.split()[0]] += 1
        print(body[0][:80], 'async regs', len(tracked), dict(uses))
