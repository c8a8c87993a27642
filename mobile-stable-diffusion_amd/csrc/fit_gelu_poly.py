import numpy as np
from scipy import special
np.set_printoptions(precision=17)
def fit(T, deg, iters=200):
    n = 4000
    t = np.linspace(1e-4, T, n)
    z = t/np.sqrt(2.0)
    f = np.log2(special.erfc(z))/t
    V = np.vander(t/T, deg+1, increasing=True)  # scaled for conditioning
    base_w = t
    lw = np.ones(n)
    for it in range(iters):
        w = base_w*np.sqrt(lw)
        coef, *_ = np.linalg.lstsq(V*w[:,None], f*w, rcond=None)
        err = np.abs((V@coef - f)*base_w)
        lw = lw*(err/err.max()+1e-3); lw/=lw.sum()/n
    coef = coef / T**np.arange(deg+1)
    return coef, err.max()*np.log(2)
for T in (5.0,5.5,6.0):
    for deg in (6,7,8,9):
        c, e = fit(T,deg)
        print(T,deg,"max rel err E: %.3e"%e)
