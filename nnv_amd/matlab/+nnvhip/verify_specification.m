function result = verify_specification(reachSet, property)
% Drop-in for NNV's verify_specification (engine/utils/verify_specification.m:36-80) on
% device-resident reach sets (nnvhip.Star / nnvhip.ImageStar, scalar or array).
%
%   result = 1 : no output set meets any half-space of the unsafe region (property holds)
%   result = 2 : some intersection is non-empty (unknown for an over-approximate reach)
%
% All (set, half-space) pairs are first bounded on the device without the constraint matrix
% (nnvhip_mex('halfspace_check', ...)).  A pair is sent to NNV's own LP (Star.isEmptySet) only
% when those bounds leave it undecided; C and d are then fetched once per set.

    if iscell(property)          % created from vnnlib (one or multiple HalfSpaces)
        property = property{1};
        property = property.Hg;
    end
    np = length(property);
    nr = length(reachSet);
    h = zeros(1, nr, 'uint64');
    for k = 1:nr
        S = reachSet(k);
        if isa(S, 'nnvhip.ImageStar'), S = S.toStar; end
        sets(k) = S; %#ok<AGROW>
        h(k) = S.dev.h;
    end
    G = []; g = []; rows = zeros(1, np);
    for c = 1:np
        G = [G; double(property(c).G)]; %#ok<AGROW>
        g = [g; double(property(c).g)]; %#ok<AGROW>
        rows(c) = size(property(c).G, 1);
    end
    verdict = nnvhip_mex('halfspace_check', h, G, g, rows);   % nr x np: 1 disjoint, 2 undecided, 3 inside

    host = cell(1, nr);          % lazily materialised NNV Star per set (dense C, d)
    result = 1;
    for c = 1:np                 % same visiting order as the reference: half-spaces outer, sets inner
        for k = 1:nr
            switch verdict(k, c)
                case 1
                    continue;    % lower bound of some row exceeds g: the LP is infeasible
                case 3
                    % the whole reach set satisfies the half-space.  A set made by reach from Star(lb,ub) is not
                    % empty; one that goes back to constraint rows of the caller's gets Star.isEmptySet
                    dims = nnvhip_mex('star_dims', h(k));
                    if dims(4) == 0
                        result = 2;
                        return;
                    end
                    if isempty(host{k}), host{k} = sets(k).gather(); end
                    if ~host{k}.isEmptySet
                        result = 2;
                        return;
                    end
                otherwise
                    if isempty(host{k}), host{k} = sets(k).gather(); end   % Star(V, C, d, pred_lb, pred_ub)
                    S = host{k}.intersectHalfSpace(double(property(c).G), double(property(c).g));
                    if ~isempty(S)
                        result = 2;
                        return;
                    end
            end
        end
    end
end
