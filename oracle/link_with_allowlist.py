"""Links a program whose reference sources name symbols this image cannot provide, and says which.

    python3 link_with_allowlist.py <link command ...>

The drop-in adapters are linked with the reference's own tensor, table and optimizer-base sources.
Optim::Create names the reference's four concrete optimizers, whose arithmetic (t/math.cc) needs
Eigen, which this image lacks; those symbols are never reached, because the adapters hand every
update to the device. The command is first run as it stands: every symbol the linker reports as
undefined must match ALLOWED, anything else is a real gap in the adapters and fails the build.
Only then is the command run again with the undefined symbols left open.
"""
import re
import subprocess
import sys

# the reference's concrete optimizers (ps/optim/{sgd,adagrad,adam,rmsprop}.cc) and its tensor
# arithmetic (t/math.cc): the files that need Eigen
ALLOWED = re.compile(r"kraken::(SGD|Adagrad|Adam|RMSprop)::|kraken::math::|vtable for kraken::(SGD|Adagrad|Adam|RMSprop)\b")


def undefined_symbols(stderr):
    return sorted(set(re.findall(r"undefined reference to `([^']+)'", stderr)))


def link(cmd):
    """-> (return code, message). cmd is the full compiler command line."""
    probe = subprocess.run(cmd, capture_output=True, text=True)
    if probe.returncode == 0:
        return 0, "linked with nothing left open"
    missing = undefined_symbols(probe.stderr)
    if not missing:
        return probe.returncode, probe.stderr[-3000:]
    stray = [s for s in missing if not ALLOWED.search(s)]
    if stray:
        return 1, "symbols outside the allow-list are undefined:\n  " + "\n  ".join(stray)
    final = subprocess.run(cmd + ["-Wl,--unresolved-symbols=ignore-all"], capture_output=True, text=True)
    return final.returncode, final.stderr[-3000:] if final.returncode else "%d symbols of the reference's Eigen-backed files left open" % len(missing)


if __name__ == "__main__":
    rc, msg = link(sys.argv[1:])
    print(msg, file=sys.stderr if rc else sys.stdout)
    sys.exit(rc)
