"""Restates every Unary/BinaryGradientTester call in the tests of xyz-autodiff-cuda as an entry of
tester_suite_entries.inc (logic type, dimensions, name, case count, tolerance, delta, input range, with the
file and line of the call).  Run by hand where the reference is mounted; its output is committed."""
import re, glob, os
os.chdir('/root/reference')
out = []
files = sorted(glob.glob('tests/**/*.cu', recursive=True) + glob.glob('examples/**/tests/*.cu', recursive=True))
for f in files:
    s = open(f).read()
    for m in re.finditer(r'(?:using Logic = ([^;]+);\s*(?://[^\n]*\n\s*)*)?(?:xyz_autodiff::)?testing::(Unary|Binary)GradientTester<([^>]*(?:<[^>]*>[^>]*)*)>::(test\w*)\(([^;]*?)\);', s, re.S):
        ln = s[:m.start(2)].count('\n') + 1
        args = re.sub(r'//[^\n]*', '', m.group(5)); args = ' '.join(args.split())
        targs = ' '.join(m.group(3).split())
        logic = m.group(1)
        if logic is None and targs.startswith('Logic'):
            # the alias is defined further up in the same test body
            prev = s[:m.start()]
            logic = re.findall(r'using Logic = ([^;]+);', prev)[-1]
        body = []
        if targs.startswith('Logic'):
            body.append('        using Logic = %s;' % ' '.join(logic.split()))
        body.append('        add("%s:%d", testing::%sGradientTester<%s>::%s(%s));' % (f, ln, m.group(2), targs, m.group(4), args))
        out.append('    {\n' + '\n'.join(body) + '\n    }')
    for m in re.finditer(r'^TEST_(UNARY|BINARY)_GRADIENT\(([^\n]*)\)\s*$', s, re.M):
        ln = s[:m.start()].count('\n') + 1
        parts = [p.strip() for p in re.split(r',\s*(?![^<]*>)', m.group(2))]
        name = parts[-1]; logic = parts[0]; dims = ', '.join(parts[1:-1])
        kind = 'Unary' if m.group(1) == 'UNARY' else 'Binary'
        logic = {'MulLogic1D_t': 'op::MulLogic<VariableRef<1, double>, VariableRef<1, double>>', 'AddLogic1D_t': 'op::AddLogic<VariableRef<1, double>, VariableRef<1, double>>',
                 'MulLogic3D_t': 'op::MulLogic<VariableRef<3, double>, VariableRef<3, double>>', 'AddLogic3D_t': 'op::AddLogic<VariableRef<3, double>, VariableRef<3, double>>',
                 'MulLogic5D_t': 'op::MulLogic<VariableRef<5, double>, VariableRef<5, double>>', 'AddLogic5D_t': 'op::AddLogic<VariableRef<5, double>, VariableRef<5, double>>'}.get(logic, logic)
        out.append('    {\n        using Logic = %s;\n        add("%s:%d", testing::%sGradientTester<Logic, %s>::test("%s"));\n    }' % (logic, f, ln, kind, dims, name))
open('/root/repo/tests/native/tester_suite_entries.inc', 'w').write(
    '// One entry per Unary/BinaryGradientTester call in the tests of xyz-autodiff-cuda (cited at each entry): the same\n'
    '// logic type, dimensions, name, case count, tolerance, delta and input range.  Included by tester_suite.cuh.\n' + '\n'.join(out) + '\n')
print(len(out))
